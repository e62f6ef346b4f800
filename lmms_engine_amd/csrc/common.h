// Shared device helpers for the gfx950 Muon kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// dtype codes shared with the C ABI (include/muon_hip.h)
#define MUON_HIP_F32 0
#define MUON_HIP_BF16 1

#define XCD_COUNT 8

// fp32 -> bf16, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950), and back.
__device__ __forceinline__ bf16_t f2bf(float f) { return (bf16_t)f; }
__device__ __forceinline__ float bf2f(bf16_t h) { return (float)h; }
// round through bf16 and return the fp32 value
__device__ __forceinline__ float rbf(float f) { return (float)((bf16_t)f); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Workgroups are dealt to the 8 XCDs round-robin by their linear id.  Give each XCD a
// contiguous range of logical ids instead, so tiles that share operands share an L2.
__device__ __forceinline__ int xcd_remap(int pid, int nblocks) {
    const int q = nblocks / XCD_COUNT, r = nblocks % XCD_COUNT;
    const int xcd = pid % XCD_COUNT, local = pid / XCD_COUNT;
    const int base = xcd * q + (xcd < r ? xcd : r);
    return base + local;
}
