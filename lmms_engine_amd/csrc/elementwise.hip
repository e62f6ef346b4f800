// HBM-bound kernels of the Muon step on gfx950: momentum/Nesterov blend with Frobenius
// partial sums, normalisation into the blocked operand X, the scaled parameter
// update, and the AdamW fallback.  128-bit accesses on the aligned path, a scalar path
// otherwise.  All reductions are two-stage with a fixed order, so results are
// run-to-run bit identical (no float atomics).
//
// Arithmetic follows /root/reference/src/lmms_engine/utils/muon_utils.py:
//   momentum_norm : muon_update's lerp_ pair (:188-189) + X = G.bfloat16() (:138) + the
//                   sum of squares feeding X.norm (:146)
//   normalize     : X / (X.norm + 1e-7) (:146) and the rows>cols transpose (:139-140)
//   apply_update  : apply_scaling (:167-175) + param.mul_/add_ (:324-325)
//   adamw         : adam_update (:178-183) + the Adam branch (:468-477)
#include "common.h"
#include "elementwise.h"

namespace {

// Streaming variants (non-temporal) for tensors whose bytes are touched once per step.  They
// pay off for the update kernel (5.22 -> 5.55 TB/s) and cost the momentum kernel (5.16 -> 4.6),
// so each kernel picks per tensor.
template <typename V> __device__ __forceinline__ V nt_load(const V* p) { return __builtin_nontemporal_load(p); }
template <typename V> __device__ __forceinline__ void nt_store(V v, V* p) { __builtin_nontemporal_store(v, p); }

template <typename T> struct Ld;
template <> struct Ld<float> {
    template <bool NT = false>
    static __device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
        const f32x4 a = NT ? nt_load((const f32x4*)p) : *(const f32x4*)p;
        const f32x4 b = NT ? nt_load((const f32x4*)(p + 4)) : *(const f32x4*)(p + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
    }
    template <bool NT = false>
    static __device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
        f32x4 a, b;
#pragma unroll
        for (int i = 0; i < 4; ++i) { a[i] = v[i]; b[i] = v[4 + i]; }
        if (NT) { nt_store(a, (f32x4*)p); nt_store(b, (f32x4*)(p + 4)); }
        else { *(f32x4*)p = a; *(f32x4*)(p + 4) = b; }
    }
    static __device__ __forceinline__ float rnd(float x) { return x; }
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float x) { *p = x; }
};
template <> struct Ld<bf16_t> {
    template <bool NT = false>
    static __device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
        const bf16x8 a = NT ? nt_load((const bf16x8*)p) : *(const bf16x8*)p;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = bf2f(a[i]);
    }
    template <bool NT = false>
    static __device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
        bf16x8 a;
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = f2bf(v[i]);
        if (NT) nt_store(a, (bf16x8*)p);
        else *(bf16x8*)p = a;
    }
    static __device__ __forceinline__ float rnd(float x) { return rbf(x); }
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf2f(*p); }
    static __device__ __forceinline__ void store(bf16_t* p, float x) { *p = f2bf(x); }
};

// ATen's lerp with a scalar weight, one fma: |w| < 0.5 -> s + w (e - s), else
// e - (e - s)(1 - w).  wm1 = w - 1 (exact in fp32 for w in [0.5, 2]).
__device__ __forceinline__ float lerp_aten(float s, float e, float w, float wm1, bool small) {
    const float d = e - s;
    return small ? fmaf(w, d, s) : fmaf(wm1, d, e);
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

struct MomentumMath {
    float w1, w1m1, w2, w2m1;
    bool small1, small2, nesterov;
};

template <typename GT, typename MT>
__device__ __forceinline__ float momentum_one(float g, float m, const MomentumMath& mm, float& m_out) {
    const float mn = Ld<MT>::rnd(lerp_aten(m, g, mm.w1, mm.w1m1, mm.small1));
    m_out = mn;
    return mm.nesterov ? lerp_aten(g, mn, mm.w2, mm.w2m1, mm.small2) : mn;
}

template <typename GT, typename MT>
__global__ void __launch_bounds__(256)
momentum_norm_kernel(const void* const* g_ptrs, const void* const* m_ptrs, bf16_t* U, long strideU,
                     float* partials, long n, MomentumMath mm, int write_back) {
    __shared__ float red[4];
    const int b = blockIdx.y;
    GT* g = (GT*)g_ptrs[b];
    MT* m = (MT*)m_ptrs[b];
    bf16_t* u = U + b * strideU;
    float ss = 0.f;
    const bool vec = ((((uintptr_t)g) | ((uintptr_t)m)) & 15) == 0;
    const long n8 = vec ? n / 8 : 0;
    // Each block owns one contiguous run of the matrix (so the blocks resident at any time
    // stream neighbouring DRAM pages); two 8-element groups per thread and trip, all loads
    // issued before the arithmetic.  The launcher sizes the grid for one trip per block (4096 elements): measured on
    // every bucket of the benchmark sets, many short-lived blocks stream 3 to 5 % faster than blocks that loop four
    // times, and 11 % faster than the fourteen trips a single 28672 x 8192 matrix used to take under the old cap of
    // 4096 blocks per matrix (a plain in-place kernel shows the same: 5.98 TB/s at one 16-byte access per thread, 5.52 at
    // four, 4.27 at eight).
    const long per_block = ((n8 + gridDim.x - 1) / gridDim.x + 511) / 512 * 512;
    const long lo8 = (long)blockIdx.x * per_block, hi8 = lo8 + per_block < n8 ? lo8 + per_block : n8;
    for (long i8 = lo8 + threadIdx.x; i8 < hi8; i8 += 512) {
        const long j8 = i8 + 256;
        const bool two = j8 < hi8;
        float gv[2][8], mv[2][8], uv[2][8];
        Ld<GT>::load8(g + i8 * 8, gv[0]);
        Ld<MT>::load8(m + i8 * 8, mv[0]);
        if (two) {
            Ld<GT>::load8(g + j8 * 8, gv[1]);
            Ld<MT>::load8(m + j8 * 8, mv[1]);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h == 1 && !two) break;
            const long k8 = h ? j8 : i8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float mo;
                float uu = momentum_one<GT, MT>(gv[h][i], mv[h][i], mm, mo);
                mv[h][i] = mo;
                if (write_back) gv[h][i] = uu;
                uu = rbf(uu);
                uv[h][i] = uu;
                ss = fmaf(uu, uu, ss);
            }
            Ld<MT>::store8(m + k8 * 8, mv[h]);
            {
                bf16x8 ub;
#pragma unroll
                for (int i = 0; i < 8; ++i) ub[i] = f2bf(uv[h][i]);
                *(bf16x8*)(u + k8 * 8) = ub;  // re-read by the normalisation pass: keep it cacheable
            }
            if (write_back) Ld<GT>::store8(g + k8 * 8, gv[h]);
        }
    }
    // scalar tail (or everything when the pointers are not 16-byte aligned)
    for (long i = n8 * 8 + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        float mo;
        float uu = momentum_one<GT, MT>(Ld<GT>::load(g + i), Ld<MT>::load(m + i), mm, mo);
        Ld<MT>::store(m + i, mo);
        if (write_back) Ld<GT>::store(g + i, uu);
        uu = rbf(uu);
        u[i] = f2bf(uu);
        ss = fmaf(uu, uu, ss);
    }
    ss = block_sum_256(ss, red);
    if (threadIdx.x == 0) partials[(long)b * gridDim.x + blockIdx.x] = ss;
}

// Sum of squares of an existing bf16 (or fp32, rounded to bf16 first) matrix: the
// Frobenius stage of fast_newtonschulz when it is called on its own.  16-byte accesses when the
// matrix base and the batch strides allow it, scalars otherwise and for the last few elements.
template <typename GT>
__global__ void __launch_bounds__(256)
cast_norm_kernel(const GT* G, long strideG, bf16_t* U, long strideU, float* partials, long n) {
    __shared__ float red[4];
    const int b = blockIdx.y;
    const GT* g = G + b * strideG;
    bf16_t* u = U + b * strideU;
    float ss = 0.f;
    const bool vec = ((((uintptr_t)g) | ((uintptr_t)u)) & 15) == 0;
    const long n8 = vec ? n / 8 : 0;
    for (long i8 = (long)blockIdx.x * 256 + threadIdx.x; i8 < n8; i8 += (long)gridDim.x * 256) {
        float v[8];
        Ld<GT>::load8(g + i8 * 8, v);
        bf16x8 ub;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            ub[i] = f2bf(v[i]);
            const float uu = bf2f(ub[i]);
            ss = fmaf(uu, uu, ss);
        }
        *(bf16x8*)(u + i8 * 8) = ub;
    }
    for (long i = n8 * 8 + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const float uu = rbf(Ld<GT>::load(g + i));
        u[i] = f2bf(uu);
        ss = fmaf(uu, uu, ss);
    }
    ss = block_sum_256(ss, red);
    if (threadIdx.x == 0) partials[(long)b * gridDim.x + blockIdx.x] = ss;
}

// d = bf(bf(sqrt(sum)) + 1e-7) per matrix, from its partial sums in a fixed order.  The first workgroup also clears
// `clear_words` words at `clear` (the tile counters of the persistent GEMM kernels that follow on the stream).
__global__ void __launch_bounds__(256) frob_finalize_kernel(const float* partials, int nparts, float* denom,
                                                            unsigned* clear, int clear_words) {
    __shared__ float red[4];
    const int b = blockIdx.x;
    if (b == 0 && clear)
        for (int i = threadIdx.x; i < clear_words; i += 256) clear[i] = 0u;
    // eight partial sums in flight per thread (a matrix of 2^28 elements has 65536 of them), added in a fixed order
    const float* p = partials + (long)b * nparts;
    float s = 0.f;
    int i = threadIdx.x;
    for (; i + 7 * 256 < nparts; i += 8 * 256) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = p[i + k * 256];
        s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
    for (; i < nparts; i += 256) s += p[i];
    s = block_sum_256(s, red);
    if (threadIdx.x == 0) {
        const float nrm = rbf(sqrtf(s));
        denom[b] = rbf(nrm + 1e-7f);
    }
}

// The bf16 blend u (parameter layout, rows x cols) divided by d, written into the blocked X (M x K, zero padded to
// Mp x Kp).  Both kernels give a thread as little as one 16-byte load and one 16-byte store: measured on every bucket of
// the benchmark sets, tiles of 16 x 128 stream 8 % faster than the 64 x 128 tiles (four accesses each way per thread)
// they replace (5.7 to 5.8 against 5.3 TB/s), the same way a plain in-place kernel loses 8 % from one to four accesses.
//
// A parameter in X's orientation (rows <= cols): one tile of 16 rows x 128 columns per workgroup, straight through
// registers; in X, 16 rows of a column block lie back to back (1 KB runs).
__global__ void __launch_bounds__(256)
normalize_kernel(const bf16_t* U, long strideU, const float* denom, bf16_t* X, long strideX, int rows, int cols, int Kp) {
    constexpr int TR = 16, TC = 128;
    const int b = blockIdx.y;
    const float d = denom[b];
    const bf16_t* u = U + b * strideU;
    bf16_t* x = X + b * strideX;
    const int cbx = Kp / BLK_COLS;
    const int tiles_c = Kp / TC;
    const int r = (blockIdx.x / tiles_c) * TR + (threadIdx.x >> 4), c = (blockIdx.x % tiles_c) * TC + (threadIdx.x & 15) * 8;
    bf16x8 v;
    if (r < rows && (cols % 8) == 0 && c + 8 <= cols) {
        v = *(const bf16x8*)(u + (long)r * cols + c);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (r < rows && c + i < cols) ? u[(long)r * cols + c + i] : (bf16_t)0.f;
    }
    bf16x8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = f2bf(__fdiv_rn(bf2f(v[i]), d));
    *(bf16x8*)(x + blocked_offset(r, c, cbx)) = o;
}

// A parameter with rows > cols (X = u^T): a tile of TR rows x TC columns of u goes through an LDS transpose and leaves
// as TC rows of X, TR elements each (TR = 32: the 64-byte rows of one column block, TC of them back to back).
template <int TR, int TC>
__global__ void __launch_bounds__(256)
normalize_t_kernel(const bf16_t* U, long strideU, const float* denom, bf16_t* X, long strideX, int rows, int cols,
                   int Mp, int Kp) {
    constexpr int PITCH = TC + 8;
    constexpr int LCH = TC / 8, LROWS = 256 / LCH, LPASS = TR / LROWS;  // load: chunks per tile row, rows and passes
    constexpr int SCH = TR / 8, SROWS = 256 / SCH, SPASS = TC / SROWS;  // store: chunks per X row, X rows and passes
    static_assert(LPASS >= 1 && SPASS >= 1 && TR % 8 == 0 && TC % 8 == 0, "a whole number of passes");
    __shared__ __align__(16) bf16_t tile[TR][PITCH];
    const int b = blockIdx.y;
    const float d = denom[b];
    const bf16_t* u = U + b * strideU;
    bf16_t* x = X + b * strideX;
    const int cbx = Kp / BLK_COLS;
    const int tiles_c = Mp / TC;  // u's padded image is Kp rows x Mp columns
    const int r0 = (blockIdx.x / tiles_c) * TR, c0 = (blockIdx.x % tiles_c) * TC;
    const int tr = threadIdx.x / LCH, tc = (threadIdx.x % LCH) * 8;
    const bool vec = (cols % 8) == 0;
#pragma unroll
    for (int h = 0; h < LPASS; ++h) {
        const int r = r0 + tr + h * LROWS, c = c0 + tc;
        bf16x8 v;
        if (r < rows && vec && c + 8 <= cols) {
            v = *(const bf16x8*)(u + (long)r * cols + c);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = (r < rows && c + i < cols) ? u[(long)r * cols + c + i] : (bf16_t)0.f;
        }
        bf16x8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = f2bf(__fdiv_rn(bf2f(v[i]), d));
        *(bf16x8*)(&tile[tr + h * LROWS][tc]) = o;
    }
    __syncthreads();
    // X[c][r]: a thread gathers 8 consecutive r of one column of the tile
    const int fr = (threadIdx.x % SCH) * 8, fc0 = threadIdx.x / SCH;
#pragma unroll
    for (int h = 0; h < SPASS; ++h) {
        const int fc = fc0 + h * SROWS;
        bf16x8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = tile[fr + i][fc];
        *(bf16x8*)(x + blocked_offset(c0 + fc, r0 + fr, cbx)) = o;
    }
}

struct UpdateMath {
    float scale, decay, alpha;
};

template <typename PT>
__device__ __forceinline__ float update_one(float p, float o, const UpdateMath& um) {
    const float os = rbf(o * um.scale);
    const float pd = Ld<PT>::rnd(p * um.decay);
    return fmaf(um.alpha, os, pd);
}

// p <- p (1 - lr wd) - lr bf(O s); O is the NS output in the parameter's orientation, blocked
// with cbo column blocks.
template <typename PT>
__global__ void __launch_bounds__(256)
apply_update_kernel(const void* const* p_ptrs, const bf16_t* O, long strideO, int cbo, int rows, int cols,
                    UpdateMath um) {
    const int b = blockIdx.y;
    PT* p = (PT*)p_ptrs[b];
    const bf16_t* o = O + b * strideO;
    const bool vec = (cols % 8 == 0) && ((((uintptr_t)p) & 15) == 0);
    if (vec) {
        // Tiles of 16 rows x 128 columns, a thread per 8 columns: in O a tile is four runs of 1 KB (16 rows of a
        // column block lie back to back), in p sixteen row pieces that the next tile of the block continues.
        const int tiles_c = (cols + 127) / 128;
        const long ntiles = (long)((rows + 15) / 16) * tiles_c;
        const long per_block = (ntiles + gridDim.x - 1) / gridDim.x;
        const long t_lo = (long)blockIdx.x * per_block, t_hi = t_lo + per_block < ntiles ? t_lo + per_block : ntiles;
        const int tr = threadIdx.x >> 4, tc = (threadIdx.x & 15) * 8;
        for (long t = t_lo; t < t_hi; t += 2) {
            float pv[2][8], ov[2][8];
            long off[2];
            bool on[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const long tt = t + h;
                const int r = (int)(tt / tiles_c) * 16 + tr, c = (int)(tt % tiles_c) * 128 + tc;
                on[h] = tt < t_hi && r < rows && c < cols;
                off[h] = (long)r * cols + c;
                if (on[h]) {
                    Ld<PT>::template load8<true>(p + off[h], pv[h]);
                    Ld<bf16_t>::template load8<true>(o + blocked_offset(r, c, cbo), ov[h]);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (!on[h]) continue;
#pragma unroll
                for (int i = 0; i < 8; ++i) pv[h][i] = update_one<PT>(pv[h][i], ov[h][i], um);
                Ld<PT>::template store8<true>(p + off[h], pv[h]);
            }
        }
    } else {
        const long n = (long)rows * cols;
        for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
            const long r = i / cols;
            const int c = (int)(i - r * cols);
            Ld<PT>::store(p + i, update_one<PT>(Ld<PT>::load(p + i), bf2f(o[blocked_offset(r, c, cbo)]), um));
        }
    }
}

// The same for a parameter with rows > cols, whose update is X^T: one tile of 64 parameter rows x 128 parameter
// columns is read from X as 128 rows of 64 elements (8 KB runs of two blocks), transposed through LDS and applied
// to 256-byte (bf16) or 512-byte (fp32) pieces of the parameter's rows.
template <typename PT>
__global__ void __launch_bounds__(256)
apply_update_t_kernel(const void* const* p_ptrs, const bf16_t* O, long strideO, int cbo, int rows, int cols,
                      UpdateMath um) {
    constexpr int TR = 64, TC = 128, PITCH = TR + 8;
    __shared__ __align__(16) bf16_t tile[TC][PITCH];  // tile[c][r]
    const int b = blockIdx.y;
    PT* p = (PT*)p_ptrs[b];
    const bf16_t* o = O + b * strideO;
    const int tiles_c = (cols + TC - 1) / TC;
    const int r0 = (blockIdx.x / tiles_c) * TR, c0 = (blockIdx.x % tiles_c) * TC;
    // X rows c0..c0+127, columns r0..r0+63 (always inside the padded X): 8 chunks per row, 32 rows per pass
    const int xr = threadIdx.x >> 3, xc = (threadIdx.x & 7) * 8;
#pragma unroll
    for (int h = 0; h < 4; ++h)
        *(bf16x8*)(&tile[xr + h * 32][xc]) = *(const bf16x8*)(o + blocked_offset(c0 + xr + h * 32, r0 + xc, cbo));
    __syncthreads();
    const bool vec = (cols % 8 == 0) && ((((uintptr_t)p) & 15) == 0);
    const int pr = threadIdx.x >> 4, pc = (threadIdx.x & 15) * 8;  // 16 rows x 16 chunks per pass
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        const int r = r0 + pr + h * 16, c = c0 + pc;
        if (r >= rows || c >= cols) continue;
        float ov[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) ov[i] = bf2f(tile[pc + i][pr + h * 16]);
        PT* dst = p + (long)r * cols + c;
        if (vec) {
            float pv[8];
            Ld<PT>::template load8<true>(dst, pv);
#pragma unroll
            for (int i = 0; i < 8; ++i) pv[i] = update_one<PT>(pv[i], ov[i], um);
            Ld<PT>::template store8<true>(dst, pv);
        } else {
            for (int i = 0; i < 8 && c + i < cols; ++i) Ld<PT>::store(dst + i, update_one<PT>(Ld<PT>::load(dst + i), ov[i], um));
        }
    }
}

// A blocked matrix, or its transpose, into a dense row-major bf16 tensor (row pitch ld): the NS output of
// fast_newtonschulz called alone, and the result of a single GEMM.  One workgroup moves a tile of 64 output rows
// x 128 output columns: straight (16-byte pieces of rows of the blocked image) or, for the transpose, from 128
// rows x 64 columns of the blocked image through LDS.  Output rows leave as 16-byte vectors when the row pitch
// and the base allow it.
__global__ void __launch_bounds__(256)
unpack_kernel(bf16_t* out, long strideOut, int ld, const bf16_t* O, long strideO, int cbo, int rows, int cols,
              int transposed) {
    constexpr int TR = 64, TC = 128, PITCH = TR + 8;
    __shared__ __align__(16) bf16_t tile[TC][PITCH];  // transposed case: tile[c][r]
    const int b = blockIdx.y;
    bf16_t* dst = out + b * strideOut;
    const bf16_t* o = O + b * strideO;
    const int tiles_c = (cols + TC - 1) / TC;
    const int r0 = (blockIdx.x / tiles_c) * TR, c0 = (blockIdx.x % tiles_c) * TC;
    const bool vec = (ld % 8 == 0) && ((((uintptr_t)dst) & 15) == 0);
    const int pr = threadIdx.x >> 4, pc = (threadIdx.x & 15) * 8;  // 16 rows x 16 chunks per pass
    if (transposed) {
        // image rows c0..c0+127, columns r0..r0+63; the blocked image is padded to whole 128-tiles in both
        // directions, so these reads stay inside it
        const int xr = threadIdx.x >> 3, xc = (threadIdx.x & 7) * 8;
#pragma unroll
        for (int h = 0; h < 4; ++h)
            *(bf16x8*)(&tile[xr + h * 32][xc]) = *(const bf16x8*)(o + blocked_offset(c0 + xr + h * 32, r0 + xc, cbo));
        __syncthreads();
    }
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        const int r = r0 + pr + h * 16, c = c0 + pc;
        if (r >= rows || c >= cols) continue;
        bf16x8 v;
        if (transposed) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = tile[pc + i][pr + h * 16];
        } else {
            v = *(const bf16x8*)(o + blocked_offset(r, c, cbo));  // columns c..c+7 lie in one block row (c % 8 == 0)
        }
        bf16_t* d = dst + (long)r * ld + c;
        if (vec && c + 8 <= cols) {
            *(bf16x8*)d = v;
        } else {
            for (int i = 0; i < 8 && c + i < cols; ++i) d[i] = v[i];
        }
    }
}

// A dense row-major bf16 matrix (row pitch ld) into the blocked layout, zero padded to
// rows_p x cols_p; one thread per 8 consecutive columns of the blocked image.
__global__ void __launch_bounds__(256)
pack_kernel(const bf16_t* src, long strideSrc, int ld, int rows, int cols, bf16_t* dst, long strideDst, int rows_p,
            int cols_p) {
    const int b = blockIdx.y;
    const int cb = cols_p / BLK_COLS;
    const long n8 = (long)rows_p * (cols_p / 8);
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long)gridDim.x * 256) {
        const long r = i / (cols_p / 8);
        const int c = (int)(i - r * (cols_p / 8)) * 8;
        bf16x8 v;
        const bf16_t* sp = src + b * strideSrc + r * ld + c;
        if (r < rows && c + 8 <= cols && ((((uintptr_t)sp) & 15) == 0)) {
            v = *(const bf16x8*)sp;
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = (r < rows && c + k < cols) ? sp[k] : (bf16_t)0.f;
        }
        *(bf16x8*)(dst + b * strideDst + blocked_offset(r, c, cb)) = v;
    }
}

struct AdamMath {
    float w1, w1m1, w2, w2m1, r1, r2, eps, decay, alpha;  // r1, r2: reciprocals of the bias corrections
    bool small1, small2;
};

// adam_update (muon_utils.py:178-183) for one element, every in-place op rounded in the tensor dtype.  A tensor
// divided by a python scalar is evaluated on a GPU as a multiplication by the scalar's reciprocal (computed in
// double precision, narrowed to fp32).
template <typename T>
__device__ __forceinline__ float adam_moments(float gi, float& e1, float& e2, const AdamMath& am) {
    const float a = Ld<T>::rnd(lerp_aten(e1, gi, am.w1, am.w1m1, am.small1));
    const float g2 = materialized(Ld<T>::rnd(gi * gi));  // grad.square() is a tensor of its own
    const float bb = Ld<T>::rnd(lerp_aten(e2, g2, am.w2, am.w2m1, am.small2));
    e1 = a;
    e2 = bb;
    const float ac = Ld<T>::rnd(a * am.r1);
    const float bc = Ld<T>::rnd(bb * am.r2);
    const float den = Ld<T>::rnd(Ld<T>::rnd(sqrtf(bc)) + am.eps);
    return Ld<T>::rnd(__fdiv_rn(ac, den));
}

template <typename T>
__global__ void __launch_bounds__(256)
adamw_kernel(T* p, const T* g, T* e1, T* e2, long n, AdamMath am) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        float a = Ld<T>::load(e1 + i), bb = Ld<T>::load(e2 + i);
        const float upd = adam_moments<T>(Ld<T>::load(g + i), a, bb, am);
        Ld<T>::store(e1 + i, a);
        Ld<T>::store(e2 + i, bb);
        const float pd = Ld<T>::rnd(Ld<T>::load(p + i) * am.decay);
        Ld<T>::store(p + i, fmaf(am.alpha, upd, pd));
    }
}

// adam_update on its own: the moments move in place, the update goes to `out`.
template <typename T>
__global__ void __launch_bounds__(256)
adam_update_kernel(const T* g, T* e1, T* e2, T* out, long n, AdamMath am) {
    const bool vec = ((((uintptr_t)g) | ((uintptr_t)e1) | ((uintptr_t)e2) | ((uintptr_t)out)) & 15) == 0;
    const long n8 = vec ? n / 8 : 0;
    for (long i8 = (long)blockIdx.x * 256 + threadIdx.x; i8 < n8; i8 += (long)gridDim.x * 256) {
        float gv[8], av[8], bv[8], uv[8];
        Ld<T>::load8(g + i8 * 8, gv);
        Ld<T>::load8(e1 + i8 * 8, av);
        Ld<T>::load8(e2 + i8 * 8, bv);
#pragma unroll
        for (int k = 0; k < 8; ++k) uv[k] = adam_moments<T>(gv[k], av[k], bv[k], am);
        Ld<T>::store8(e1 + i8 * 8, av);
        Ld<T>::store8(e2 + i8 * 8, bv);
        Ld<T>::store8(out + i8 * 8, uv);
    }
    for (long i = n8 * 8 + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        float a = Ld<T>::load(e1 + i), bb = Ld<T>::load(e2 + i);
        const float upd = adam_moments<T>(Ld<T>::load(g + i), a, bb, am);
        Ld<T>::store(e1 + i, a);
        Ld<T>::store(e2 + i, bb);
        Ld<T>::store(out + i, upd);
    }
}

// x <- rnd(x * s): apply_scaling on its own (muon_utils.py:167-175).
template <typename T>
__global__ void __launch_bounds__(256) scale_kernel(T* x, long n, float s) {
    const bool vec = (((uintptr_t)x) & 15) == 0;
    const long n8 = vec ? n / 8 : 0;
    for (long i8 = (long)blockIdx.x * 256 + threadIdx.x; i8 < n8; i8 += (long)gridDim.x * 256) {
        float v[8];
        Ld<T>::load8(x + i8 * 8, v);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] *= s;
        Ld<T>::store8(x + i8 * 8, v);
    }
    for (long i = n8 * 8 + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        Ld<T>::store(x + i, Ld<T>::load(x + i) * s);
}

// p <- rnd(p * decay); p <- rnd(p + alpha * u): the decay and update lines on a dense update tensor u
// (muon_utils.py:406-407, the Muon branch of step_deepspeed, and :324-325).
template <typename PT, typename UT>
__global__ void __launch_bounds__(256) decay_update_kernel(PT* p, const UT* u, long n, float decay, float alpha) {
    const bool vec = ((((uintptr_t)p) | ((uintptr_t)u)) & 15) == 0;
    const long n8 = vec ? n / 8 : 0;
    for (long i8 = (long)blockIdx.x * 256 + threadIdx.x; i8 < n8; i8 += (long)gridDim.x * 256) {
        float pv[8], uv[8];
        Ld<PT>::load8(p + i8 * 8, pv);
        Ld<UT>::load8(u + i8 * 8, uv);
#pragma unroll
        for (int k = 0; k < 8; ++k) pv[k] = fmaf(alpha, uv[k], Ld<PT>::rnd(pv[k] * decay));
        Ld<PT>::store8(p + i8 * 8, pv);
    }
    for (long i = n8 * 8 + (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        Ld<PT>::store(p + i, fmaf(alpha, Ld<UT>::load(u + i), Ld<PT>::rnd(Ld<PT>::load(p + i) * decay)));
}

// Grids of the helper kernels: enough workgroups that each makes one or two trips of its loop (short-lived workgroups
// stream faster than a few thousand that loop), up to this many.
constexpr int kMaxBlocks = 1 << 20;

inline int blocks_for(long n, int per_block, int cap) {
    long b = (n + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (int)b;
}

inline void lerp_consts(double weight, float& w, float& wm1, bool& small) {
    w = (float)weight;
    wm1 = w - 1.0f;
    small = fabsf(w) < 0.5f;
}

}  // namespace

int momentum_parts(long n) { return blocks_for(n, MUON_PART_ELEMS, MUON_MAX_PARTS); }

hipError_t launch_momentum_norm(const void* const* g_ptrs, const void* const* m_ptrs, int g_dtype, int m_dtype,
                                bf16_t* U, long strideU, float* partials, int nparts, long n, int batch,
                                double beta, int nesterov, int write_back, hipStream_t stream) {
    MomentumMath mm;
    lerp_consts(1.0 - beta, mm.w1, mm.w1m1, mm.small1);
    lerp_consts(beta, mm.w2, mm.w2m1, mm.small2);
    mm.nesterov = nesterov != 0;
    if (!mm.nesterov) write_back = 0;  // without Nesterov the update is the momentum buffer and the gradient stays as it is
    dim3 grid(nparts, batch), block(256);
    if (g_dtype == MUON_HIP_F32 && m_dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((momentum_norm_kernel<float, float>), grid, block, 0, stream, g_ptrs, m_ptrs, U, strideU,
                           partials, n, mm, write_back);
    else if (g_dtype == MUON_HIP_BF16 && m_dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((momentum_norm_kernel<bf16_t, float>), grid, block, 0, stream, g_ptrs, m_ptrs, U, strideU,
                           partials, n, mm, write_back);
    else if (g_dtype == MUON_HIP_BF16 && m_dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((momentum_norm_kernel<bf16_t, bf16_t>), grid, block, 0, stream, g_ptrs, m_ptrs, U, strideU,
                           partials, n, mm, write_back);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_cast_norm(const void* G, long strideG, int g_dtype, bf16_t* U, long strideU, float* partials,
                            int nparts, long n, int batch, hipStream_t stream) {
    dim3 grid(nparts, batch), block(256);
    if (g_dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((cast_norm_kernel<float>), grid, block, 0, stream, (const float*)G, strideG, U, strideU,
                           partials, n);
    else if (g_dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((cast_norm_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)G, strideG, U, strideU,
                           partials, n);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_normalize(const bf16_t* U, long strideU, const float* partials, int nparts, float* denom, bf16_t* X,
                            long strideX, int rows, int cols, int Mp, int Kp, int batch, unsigned* clear, int clear_words,
                            hipStream_t stream) {
    hipLaunchKernelGGL(frob_finalize_kernel, dim3(batch), dim3(256), 0, stream, partials, nparts, denom, clear, clear_words);
    // u's padded image has whole 128-tiles in both directions (Mp and Kp are multiples of the GEMM tile edge)
    if (rows > cols) {
        // 32 x 128 measured best of {32, 64} x {64, 128}: 5.5 to 5.7 TB/s against 5.2 to 5.5 for 64 x 128
        constexpr int TR = 32, TC = 128;
        dim3 grid((Kp / TR) * (Mp / TC), batch), block(256);
        hipLaunchKernelGGL((normalize_t_kernel<TR, TC>), grid, block, 0, stream, U, strideU, denom, X, strideX, rows, cols, Mp, Kp);
    } else {
        dim3 grid((Mp / 16) * (Kp / 128), batch), block(256);
        hipLaunchKernelGGL(normalize_kernel, grid, block, 0, stream, U, strideU, denom, X, strideX, rows, cols, Kp);
    }
    return hipGetLastError();
}

// O is X (M x K, blocked with cbo column blocks): the update in the parameter's orientation when rows <= cols,
// its transpose otherwise.
hipError_t launch_apply_update(const void* const* p_ptrs, int p_dtype, const bf16_t* O, long strideO, int cbo,
                               int rows, int cols, int batch, double scale, double lr, double wd,
                               hipStream_t stream) {
    UpdateMath um;
    um.scale = (float)scale;
    um.decay = (float)(1.0 - lr * wd);
    um.alpha = (float)(-lr);
    dim3 block(256);
    if (rows > cols) {
        dim3 grid(((rows + 63) / 64) * ((cols + 127) / 128), batch);
        if (p_dtype == MUON_HIP_F32)
            hipLaunchKernelGGL((apply_update_t_kernel<float>), grid, block, 0, stream, p_ptrs, O, strideO, cbo, rows, cols, um);
        else if (p_dtype == MUON_HIP_BF16)
            hipLaunchKernelGGL((apply_update_t_kernel<bf16_t>), grid, block, 0, stream, p_ptrs, O, strideO, cbo, rows, cols, um);
        else
            return hipErrorInvalidValue;
        return hipGetLastError();
    }
    dim3 grid(blocks_for((long)rows * cols, 4096, kMaxBlocks), batch);
    if (p_dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((apply_update_kernel<float>), grid, block, 0, stream, p_ptrs, O, strideO, cbo, rows, cols, um);
    else if (p_dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((apply_update_kernel<bf16_t>), grid, block, 0, stream, p_ptrs, O, strideO, cbo, rows, cols,
                           um);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_unpack(bf16_t* out, long strideOut, int ld, const bf16_t* O, long strideO, int cbo, int rows,
                         int cols, bool transposed, int batch, hipStream_t stream) {
    dim3 grid(((rows + 63) / 64) * ((cols + 127) / 128), batch), block(256);
    hipLaunchKernelGGL(unpack_kernel, grid, block, 0, stream, out, strideOut, ld, O, strideO, cbo, rows, cols,
                       transposed ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_pack(const bf16_t* src, long strideSrc, int ld, int rows, int cols, bf16_t* dst, long strideDst,
                       int rows_p, int cols_p, int batch, hipStream_t stream) {
    dim3 grid(blocks_for((long)rows_p * cols_p / 8, 256 * 4, 4096), batch), block(256);
    hipLaunchKernelGGL(pack_kernel, grid, block, 0, stream, src, strideSrc, ld, rows, cols, dst, strideDst, rows_p, cols_p);
    return hipGetLastError();
}

namespace {
AdamMath adam_math(int step, double lr, double b1, double b2, double eps, double wd) {
    AdamMath am;
    lerp_consts(1.0 - b1, am.w1, am.w1m1, am.small1);
    lerp_consts(1.0 - b2, am.w2, am.w2m1, am.small2);
    // the reciprocal is taken in double precision and then narrowed, as ATen does for a python-scalar divisor
    am.r1 = (float)(1.0 / (1.0 - pow(b1, (double)step)));
    am.r2 = (float)(1.0 / (1.0 - pow(b2, (double)step)));
    am.eps = (float)eps;
    am.decay = (float)(1.0 - lr * wd);
    am.alpha = (float)(-lr);
    return am;
}
}  // namespace

hipError_t launch_adamw(void* p, const void* g, void* e1, void* e2, int dtype, long n, int step, double lr,
                        double b1, double b2, double eps, double wd, hipStream_t stream) {
    const AdamMath am = adam_math(step, lr, b1, b2, eps, wd);
    dim3 grid(blocks_for(n, 256 * 4, kMaxBlocks)), block(256);
    if (dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((adamw_kernel<float>), grid, block, 0, stream, (float*)p, (const float*)g, (float*)e1,
                           (float*)e2, n, am);
    else if (dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((adamw_kernel<bf16_t>), grid, block, 0, stream, (bf16_t*)p, (const bf16_t*)g, (bf16_t*)e1,
                           (bf16_t*)e2, n, am);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_adam_update(const void* g, void* e1, void* e2, void* out, int dtype, long n, int step, double b1,
                              double b2, double eps, hipStream_t stream) {
    const AdamMath am = adam_math(step, 0.0, b1, b2, eps, 0.0);
    dim3 grid(blocks_for(n, 256 * 8 * 2, kMaxBlocks)), block(256);
    if (dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((adam_update_kernel<float>), grid, block, 0, stream, (const float*)g, (float*)e1, (float*)e2,
                           (float*)out, n, am);
    else if (dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((adam_update_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)g, (bf16_t*)e1,
                           (bf16_t*)e2, (bf16_t*)out, n, am);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_scale(void* x, int dtype, long n, double s, hipStream_t stream) {
    dim3 grid(blocks_for(n, 256 * 8 * 2, kMaxBlocks)), block(256);
    if (dtype == MUON_HIP_F32) hipLaunchKernelGGL((scale_kernel<float>), grid, block, 0, stream, (float*)x, n, (float)s);
    else if (dtype == MUON_HIP_BF16) hipLaunchKernelGGL((scale_kernel<bf16_t>), grid, block, 0, stream, (bf16_t*)x, n, (float)s);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_decay_update(void* p, int p_dtype, const void* u, int u_dtype, long n, double lr, double wd,
                               hipStream_t stream) {
    const float decay = (float)(1.0 - lr * wd), alpha = (float)(-lr);
    dim3 grid(blocks_for(n, 256 * 8 * 2, kMaxBlocks)), block(256);
    if (p_dtype == MUON_HIP_F32 && u_dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((decay_update_kernel<float, float>), grid, block, 0, stream, (float*)p, (const float*)u, n, decay, alpha);
    else if (p_dtype == MUON_HIP_F32 && u_dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((decay_update_kernel<float, bf16_t>), grid, block, 0, stream, (float*)p, (const bf16_t*)u, n, decay, alpha);
    else if (p_dtype == MUON_HIP_BF16 && u_dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((decay_update_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (bf16_t*)p, (const bf16_t*)u, n, decay, alpha);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}
