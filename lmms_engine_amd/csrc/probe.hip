// Measurement kernels, no part of the optimizer step: loops of nothing but MFMAs on caller-supplied operands.
// They show what the matrix pipes sustain under the part's power management for a given instruction shape and
// operand content (random mantissas against constants), which is the ceiling the Newton-Schulz GEMMs are
// measured against and the reason they are built on v_mfma_f32_16x16x32_bf16.
#include "common.h"
#include "probe.h"

namespace {

// One workgroup of 8 waves per compute unit; a wave keeps 12 operand fragments and 128 accumulator registers,
// the footprint of a wave of the GEMM kernels, and issues 16 MFMAs of 32x32x16 (SHAPE 0) or 32 of 16x16x32
// (SHAPE 1) per iteration: 524288 FLOP per wave and iteration either way.
template <int SHAPE>
__global__ void __launch_bounds__(512) mfma_probe_kernel(const bf16x8* src, float* sink, int iters) {
    const int tid = threadIdx.x;
    bf16x8 fa[8], fb[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) fa[i] = src[((long)blockIdx.x * 12 + i) * 512 + tid];
#pragma unroll
    for (int i = 0; i < 4; ++i) fb[i] = src[((long)blockIdx.x * 12 + 8 + i) * 512 + tid];
    float s = 0.f;
    if (SHAPE == 0) {
        f32x16 acc[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks * 4 + i], fb[ks * 2 + j], acc[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    } else {
        f32x4 acc[8][4];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) s += acc[i][j][r];
    }
    sink[(long)blockIdx.x * 512 + tid] = s;
}

}  // namespace

hipError_t launch_mfma_probe(const void* operands, float* sink, int shape, int iters, hipStream_t stream) {
    dim3 grid(MUON_PROBE_BLOCKS), block(512);
    if (shape == 0) hipLaunchKernelGGL(mfma_probe_kernel<0>, grid, block, 0, stream, (const bf16x8*)operands, sink, iters);
    else if (shape == 1) hipLaunchKernelGGL(mfma_probe_kernel<1>, grid, block, 0, stream, (const bf16x8*)operands, sink, iters);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}
