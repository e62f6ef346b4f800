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

// Every matrix of the Newton-Schulz workspace is stored in blocks of 256 rows x BLK_COLS
// columns (rows of a block back to back): element (r, c) of a matrix with `cb` column blocks is at
//   ((r / 256) * cb + c / BLK_COLS) * BLK_ELEMS + (r % 256) * BLK_COLS + c % BLK_COLS.
// A k-tile of an operand panel is then one contiguous run of memory instead of 256 row pieces
// a row pitch apart, which is what DRAM pages, the L2 channels and the TLB all prefer.
#ifndef MUON_BLK_COLS
#define MUON_BLK_COLS 32
#endif
constexpr int BLK_ROWS = 256, BLK_COLS = MUON_BLK_COLS, BLK_SHIFT = BLK_COLS == 64 ? 6 : 5;
constexpr int BLK_ELEMS = BLK_ROWS * BLK_COLS;
static_assert(BLK_COLS == 32 || BLK_COLS == 64, "block width");

__host__ __device__ inline long blocked_offset(long r, long c, int cb) {
    return ((r >> 8) * cb + (c >> BLK_SHIFT)) * BLK_ELEMS + (r & 255) * BLK_COLS + (c & (BLK_COLS - 1));
}
// elements of a blocked rows x cols matrix (cols a multiple of BLK_COLS)
inline long blocked_elems(long rows, long cols) { return ((rows + BLK_ROWS - 1) / BLK_ROWS) * (cols / BLK_COLS) * BLK_ELEMS; }

// fp32 -> bf16, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950), and back.
__device__ __forceinline__ bf16_t f2bf(float f) { return (bf16_t)f; }
__device__ __forceinline__ float bf2f(bf16_t h) { return (float)h; }
// round through bf16 and return the fp32 value
__device__ __forceinline__ float rbf(float f) { return (float)((bf16_t)f); }

// Square roots and divisions: sqrtf(x) and __fdiv_rn(x, y) are correctly rounded in this build (hipcc's default
// -fhip-fp32-correctly-rounded-divide-sqrt), which is what torch's GPU kernels compute; __fsqrt_rn is the
// hardware approximation despite its name (it differs from the exact root in one result out of six) and is not used.

// A value that the reference holds in a tensor of its own: the compiler must round it where it stands and not
// contract the product behind it into the next addition (hipcc fuses across statements by default).
__device__ __forceinline__ float materialized(float x) {
    asm volatile("" : "+v"(x));
    return x;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Workgroups are dealt to the XCDs (2^xcd_shift of them) round-robin by their linear id.  Give each XCD runs of
// XCD_CHUNK consecutive logical ids instead (one round of its 32 CUs), so tiles that share operands
// share an L2, and deal those runs to the XCDs in turn, so that at any time all of them work on
// neighbouring tiles of the same matrix and the memory-side cache, which all XCDs share, serves
// the panels the others have already fetched.
#ifndef XCD_CHUNK
#define XCD_CHUNK 32
#endif
__device__ __forceinline__ int xcd_remap(int pid, int nblocks, int xcd_shift) {
    const int span = XCD_CHUNK << xcd_shift;  // one run for every XCD
    const int full = nblocks / span * span;
    if (pid >= full) return pid;
    const int xcd = pid & ((1 << xcd_shift) - 1), local = pid >> xcd_shift;
    return (((local / XCD_CHUNK) << xcd_shift) + xcd) * XCD_CHUNK + local % XCD_CHUNK;
}
