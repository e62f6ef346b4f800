// Measurement kernels, no part of the optimizer step and no part of libmuon_hip.so: this file is built into a library of
// its own (libmuon_probe.so) that only the benchmark's operand-power legs load.  Loops of nothing but MFMAs on
// caller-supplied operands.
// They show what the matrix pipes sustain under the part's power management for a given instruction shape and
// operand content (random mantissas against constants), which is the ceiling the Newton-Schulz GEMMs are
// measured against and the reason they are built on v_mfma_f32_16x16x32_bf16.
#include "common.h"

#define MUON_PROBE_BLOCKS 256                            // workgroups: one per compute unit of a whole part
#define MUON_PROBE_FLOP_PER_ITER (256.0 * 8 * 16 * 32768.0)

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

// shape 0: v_mfma_f32_32x32x16_bf16, shape 1: v_mfma_f32_16x16x32_bf16.  `operands` holds 256 * 12 * 512 * 16 bytes of
// bf16 values chosen by the caller (random, constant ...), `sink` receives 256 * 512 floats; *flop is the work of the
// launch.  Returns a hipError_t (0 = launched) or -1 for bad arguments.  Time it with events on `stream`.
extern "C" __attribute__((visibility("default"))) int muon_probe_mfma(const void* operands, void* sink, int shape, int iters,
                                                                      double* flop, void* stream) {
    if (!operands || !sink || (shape != 0 && shape != 1) || iters <= 0) return -1;
    dim3 grid(MUON_PROBE_BLOCKS), block(512);
    hipStream_t s = (hipStream_t)stream;
    if (shape == 0) hipLaunchKernelGGL(mfma_probe_kernel<0>, grid, block, 0, s, (const bf16x8*)operands, (float*)sink, iters);
    else hipLaunchKernelGGL(mfma_probe_kernel<1>, grid, block, 0, s, (const bf16x8*)operands, (float*)sink, iters);
    if (flop) *flop = MUON_PROBE_FLOP_PER_ITER * iters;
    return (int)hipGetLastError();
}

// Streaming rate of plain kernels against the number of XCDs that take part (workgroup b sits on XCD b % 8; the others
// leave at once): what the memory system delivers for one read (mode 0), one read and one write in place (mode 1) and a
// copy (mode 2), the ceilings the elementwise kernels of the step are read against.
namespace {
template <int MODE>
__global__ void __launch_bounds__(256) stream_probe_kernel(f32x4* a, f32x4* b, long n4, int nx, float* sink) {
    const int xcd = blockIdx.x & 7;
    if (xcd >= nx) return;
    const long wg = (long)(blockIdx.x >> 3) * nx + xcd, nwg = (long)(gridDim.x >> 3) * nx;
    const long per = (n4 + nwg - 1) / nwg;
    const long lo = wg * per, hi = lo + per < n4 ? lo + per : n4;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (long i = lo + threadIdx.x; i < hi; i += 256) {
        const f32x4 v = a[i];
        if (MODE == 0) acc += v;
        else if (MODE == 1) a[i] = v * 1.0001f;
        else b[i] = v;
    }
    if (MODE == 0 && acc[0] + acc[1] + acc[2] + acc[3] == 12345.f) *sink = 1.f;  // keeps the loads alive
}
}  // namespace

// a, b: `bytes` of device memory each (a multiple of 16); mode 0, 1, 2 as above; xcds 1..8.  Returns a hipError_t or -1.
extern "C" __attribute__((visibility("default"))) int muon_probe_stream(void* a, void* b, long bytes, int mode, int xcds, void* sink,
                                                                        void* stream) {
    if (!a || !b || !sink || bytes <= 0 || bytes % 16 || mode < 0 || mode > 2 || xcds < 1 || xcds > 8) return -1;
    const long n4 = bytes / 16;
    dim3 grid(8 * 2048), block(256);
    hipStream_t s = (hipStream_t)stream;
    if (mode == 0) hipLaunchKernelGGL(stream_probe_kernel<0>, grid, block, 0, s, (f32x4*)a, (f32x4*)b, n4, xcds, (float*)sink);
    else if (mode == 1) hipLaunchKernelGGL(stream_probe_kernel<1>, grid, block, 0, s, (f32x4*)a, (f32x4*)b, n4, xcds, (float*)sink);
    else hipLaunchKernelGGL(stream_probe_kernel<2>, grid, block, 0, s, (f32x4*)a, (f32x4*)b, n4, xcds, (float*)sink);
    return (int)hipGetLastError();
}
