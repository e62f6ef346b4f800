// Multi-tensor memory-bound kernels: one launch walks a whole list of tensors.
//
//   adamw_multi      : adam_update + the Adam branch of step_fsdp (muon_utils.py:178-183,
//                      :468-477) for every tensor of a parameter group
//   sqnorm / norms   : the norm torch's _get_total_norm computes for
//                      fsdp2_clip_grad_norm_ (utils/fsdp2_utils.py:234-255): per-tensor norms
//                      rounded to the tensor dtype, then the norm of those norms, for any order torch's
//                      vector_norm takes: 2, 1, 0 (count of non-zeros), +inf / -inf (largest / smallest magnitude,
//                      a NaN anywhere makes the result NaN, as torch's max and min do), and (sum |x|^p)^(1/p) otherwise
//   clip_scale_multi : _clip_grads_with_norm_: g *= clamp(max_norm / (total + 1e-6), max=1)
//
// A tensor list is cut into chunks of MUON_MULTI_CHUNK elements; chunk_start[t] is the index of
// tensor t's first chunk (chunk_start[n] = number of chunks = grid size).  A block finds its
// tensor by bisection and handles one chunk: 16-byte vectors when every base pointer of the
// tensor is 16-byte aligned, scalars otherwise and for the last few elements.
#include "multi_tensor.h"
#include <type_traits>

namespace {

template <typename T> struct Mt;
template <> struct Mt<float> {
    static __device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
        const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
    }
    static __device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
        f32x4 a, b;
#pragma unroll
        for (int i = 0; i < 4; ++i) { a[i] = v[i]; b[i] = v[4 + i]; }
        *(f32x4*)p = a;
        *(f32x4*)(p + 4) = b;
    }
    static __device__ __forceinline__ float rnd(float x) { return x; }
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float x) { *p = x; }
};
template <> struct Mt<bf16_t> {
    static __device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
        const bf16x8 a = *(const bf16x8*)p;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = bf2f(a[i]);
    }
    static __device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
        bf16x8 a;
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = f2bf(v[i]);
        *(bf16x8*)p = a;
    }
    static __device__ __forceinline__ float rnd(float x) { return rbf(x); }
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf2f(*p); }
    static __device__ __forceinline__ void store(bf16_t* p, float x) { *p = f2bf(x); }
};

__device__ __forceinline__ float rnd_dtype(float x, int dtype) { return dtype == MUON_HIP_BF16 ? rbf(x) : x; }

// tensor index t with chunk_start[t] <= chunk < chunk_start[t + 1]
__device__ __forceinline__ int find_tensor(const long* chunk_start, int n, long chunk) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (chunk_start[mid] <= chunk) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

struct ChunkRange {
    int t;
    long begin, len;  // element offset in the tensor, elements in this chunk
};

// The range of workgroup blockIdx.x when every chunk is shared by SUB workgroups (a power of two): chunk blockIdx.x / SUB,
// piece blockIdx.x % SUB of it.  The kernels that read and write (AdamW, the clip scaling) run four workgroups per chunk, one
// trip of 4096 elements each: measured, short-lived workgroups stream 3 to 6 % faster there than one workgroup making four
// trips; the read-only norm kernel is faster with one workgroup per chunk (fewer partial sums).
template <int SUB = 1>
__device__ __forceinline__ ChunkRange my_chunk(const long* numel, const long* chunk_start, int n) {
    constexpr long PIECE = MUON_MULTI_CHUNK / SUB;
    const long chunk = blockIdx.x / SUB, piece = blockIdx.x % SUB;
    ChunkRange r;
    r.t = find_tensor(chunk_start, n, chunk);
    r.begin = (chunk - chunk_start[r.t]) * MUON_MULTI_CHUNK + piece * PIECE;
    const long left = numel[r.t] - r.begin;
    r.len = left < 0 ? 0 : left < PIECE ? left : PIECE;
    return r;
}
constexpr int RW_SUB = 4;  // workgroups per chunk of the read-and-write kernels

__device__ __forceinline__ float lerp_aten(float s, float e, float w, float wm1, bool small) {
    const float d = e - s;
    return small ? fmaf(w, d, s) : fmaf(wm1, d, e);
}

struct AdamConst {
    float w1, w1m1, w2, w2m1, eps, decay, alpha;
    bool small1, small2;
};

template <typename T>
__device__ __forceinline__ void adam_one(float& p, float g, float& e1, float& e2, const AdamConst& am, float r1, float r2) {
    const float a = Mt<T>::rnd(lerp_aten(e1, g, am.w1, am.w1m1, am.small1));
    const float g2 = materialized(Mt<T>::rnd(g * g));  // grad.square() is a tensor of its own
    const float bb = Mt<T>::rnd(lerp_aten(e2, g2, am.w2, am.w2m1, am.small2));
    e1 = a;
    e2 = bb;
    // a tensor divided by a python scalar is a multiplication by the scalar's reciprocal on a GPU
    const float ac = Mt<T>::rnd(a * r1);
    const float bc = Mt<T>::rnd(bb * r2);
    const float den = Mt<T>::rnd(Mt<T>::rnd(sqrtf(bc)) + am.eps);
    const float upd = Mt<T>::rnd(__fdiv_rn(ac, den));
    const float pd = Mt<T>::rnd(p * am.decay);
    p = fmaf(am.alpha, upd, pd);  // stored through Mt<T>::store*, which rounds
}

template <typename T>
__global__ void __launch_bounds__(256)
adamw_multi_kernel(const void* const* p_ptrs, const void* const* g_ptrs, const void* const* e1_ptrs,
                   const void* const* e2_ptrs, const long* numel, const long* chunk_start, const double* bias1,
                   const double* bias2, int n, AdamConst am) {
    const ChunkRange r = my_chunk<RW_SUB>(numel, chunk_start, n);
    T* p = (T*)p_ptrs[r.t] + r.begin;
    const T* g = (const T*)g_ptrs[r.t] + r.begin;
    T* e1 = (T*)e1_ptrs[r.t] + r.begin;
    T* e2 = (T*)e2_ptrs[r.t] + r.begin;
    const float r1 = (float)(1.0 / bias1[r.t]), r2 = (float)(1.0 / bias2[r.t]);  // double reciprocal, then narrowed
    const bool vec = ((((uintptr_t)p) | ((uintptr_t)g) | ((uintptr_t)e1) | ((uintptr_t)e2)) & 15) == 0;
    const long n8 = vec ? r.len / 8 : 0;
    for (long i = threadIdx.x; i < n8; i += 256) {
        float pv[8], gv[8], av[8], bv[8];
        Mt<T>::load8(p + i * 8, pv);
        Mt<T>::load8(g + i * 8, gv);
        Mt<T>::load8(e1 + i * 8, av);
        Mt<T>::load8(e2 + i * 8, bv);
#pragma unroll
        for (int k = 0; k < 8; ++k) adam_one<T>(pv[k], gv[k], av[k], bv[k], am, r1, r2);
        Mt<T>::store8(e1 + i * 8, av);
        Mt<T>::store8(e2 + i * 8, bv);
        Mt<T>::store8(p + i * 8, pv);
    }
    for (long i = n8 * 8 + threadIdx.x; i < r.len; i += 256) {
        float pv = Mt<T>::load(p + i), av = Mt<T>::load(e1 + i), bv = Mt<T>::load(e2 + i);
        adam_one<T>(pv, Mt<T>::load(g + i), av, bv, am, r1, r2);
        Mt<T>::store(e1 + i, av);
        Mt<T>::store(e2 + i, bv);
        Mt<T>::store(p + i, pv);
    }
}

__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// Largest / smallest of two magnitudes; a NaN on either side wins (fmaxf and fminf would drop it).
__device__ __forceinline__ float nan_max(float a, float b) { return (a != a) ? a : (b != b) ? b : fmaxf(a, b); }
__device__ __forceinline__ float nan_min(float a, float b) { return (a != a) ? a : (b != b) ? b : fminf(a, b); }

// The reductions of torch's norm kernels (aten/src/ATen/native/cuda/ReduceNormKernel.cu and SharedReduceOps.h), by order:
// what one element adds to the running value, how two running values combine, and what turns the total into the norm.
enum NormKind { NORM_TWO, NORM_INF, NORM_ONE, NORM_ZERO, NORM_NEG_INF, NORM_P };

template <int KIND> struct NormOp {
    static constexpr bool kSum = KIND != NORM_INF && KIND != NORM_NEG_INF;
    static __device__ __forceinline__ float identity() { return KIND == NORM_NEG_INF ? __builtin_inff() : 0.f; }
    static __device__ __forceinline__ float reduce(float acc, float v, float p) {
        if constexpr (KIND == NORM_TWO) return fmaf(v, v, acc);
        else if constexpr (KIND == NORM_INF) return nan_max(acc, fabsf(v));
        else if constexpr (KIND == NORM_NEG_INF) return nan_min(acc, fabsf(v));
        else if constexpr (KIND == NORM_ONE) return acc + fabsf(v);
        else if constexpr (KIND == NORM_ZERO) return acc + (v == 0.f ? 0.f : 1.f);
        else return acc + powf(fabsf(v), p);
    }
    static __device__ __forceinline__ float combine(float a, float b) {
        if constexpr (KIND == NORM_INF) return nan_max(a, b);
        else if constexpr (KIND == NORM_NEG_INF) return nan_min(a, b);
        else return a + b;
    }
    static __device__ __forceinline__ float project(float acc, float p) {
        if constexpr (KIND == NORM_TWO) return sqrtf(acc);
        else if constexpr (KIND == NORM_P) return powf(acc, __fdiv_rn(1.0f, p));
        else return acc;
    }
};

template <int KIND>
__device__ __forceinline__ float block_reduce_256(float v, float* red) {
    if constexpr (NormOp<KIND>::kSum) {
        return block_sum_256(v, red);
    } else {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v = NormOp<KIND>::combine(v, __shfl_xor(v, off, 64));
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        __syncthreads();
        if (lane == 0) red[wave] = v;
        __syncthreads();
        return NormOp<KIND>::combine(NormOp<KIND>::combine(red[0], red[1]), NormOp<KIND>::combine(red[2], red[3]));
    }
}

// The running value of one chunk (sum of squares, of magnitudes, of powers, the count of non-zeros, or the extreme magnitude).
template <typename T, int KIND>
__global__ void __launch_bounds__(256)
sqnorm_multi_kernel(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n, float p, float* partials) {
    __shared__ float red[4];
    const ChunkRange r = my_chunk(numel, chunk_start, n);
    const T* g = (const T*)g_ptrs[r.t] + r.begin;
    const bool vec = (((uintptr_t)g) & 15) == 0;
    const long n8 = vec ? r.len / 8 : 0;
    float ss = NormOp<KIND>::identity();
    for (long i = threadIdx.x; i < n8; i += 256) {
        float v[8];
        Mt<T>::load8(g + i * 8, v);
#pragma unroll
        for (int k = 0; k < 8; ++k) ss = NormOp<KIND>::reduce(ss, v[k], p);
    }
    for (long i = n8 * 8 + threadIdx.x; i < r.len; i += 256) ss = NormOp<KIND>::reduce(ss, Mt<T>::load(g + i), p);
    ss = block_reduce_256<KIND>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = ss;
}

// One block per tensor: its partial results in a fixed order -> norm, rounded to the tensor dtype.
template <int KIND>
__global__ void __launch_bounds__(256)
tensor_norm_kernel(const float* partials, const long* chunk_start, int dtype, float p, float* norms) {
    __shared__ float red[4];
    const int t = blockIdx.x;
    float ss = NormOp<KIND>::identity();
    for (long c = chunk_start[t] + threadIdx.x; c < chunk_start[t + 1]; c += 256) ss = NormOp<KIND>::combine(ss, partials[c]);
    ss = block_reduce_256<KIND>(ss, red);
    if (threadIdx.x == 0) norms[t] = rnd_dtype(NormOp<KIND>::project(ss, p), dtype);
}

// One block: norm of the per-tensor norms, rounded to the result dtype; written as fp32 (for the
// scaling kernel) and in the result dtype (the tensor the caller returns).
template <int KIND>
__global__ void __launch_bounds__(256)
total_norm_kernel(const float* norms, int n, int dtype, float p, float* total_f32, void* total_typed) {
    __shared__ float red[4];
    float ss = NormOp<KIND>::identity();
    for (int t = threadIdx.x; t < n; t += 256) ss = NormOp<KIND>::reduce(ss, norms[t], p);
    ss = block_reduce_256<KIND>(ss, red);
    if (threadIdx.x == 0) {
        const float tn = rnd_dtype(NormOp<KIND>::project(ss, p), dtype);
        *total_f32 = tn;
        if (dtype == MUON_HIP_BF16) *(bf16_t*)total_typed = f2bf(tn);
        else *(float*)total_typed = tn;
    }
}

// torch evaluates max_norm / (total + 1e-6) as (total + 1e-6).reciprocal() * max_norm, every
// step rounded to the norm's dtype, then clamps at 1.
__device__ __forceinline__ float clip_coef(float total, int norm_dtype, float max_norm) {
    const float s = rnd_dtype(total + 1e-6f, norm_dtype);
    const float r = rnd_dtype(__fdiv_rn(1.0f, s), norm_dtype);
    const float c = rnd_dtype(r * max_norm, norm_dtype);
    return c > 1.0f ? 1.0f : c;  // a NaN coefficient stays NaN, as torch.clamp leaves it
}

template <typename T>
__global__ void __launch_bounds__(256)
clip_scale_multi_kernel(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n,
                        const float* total_f32, int norm_dtype, float max_norm) {
    const float coef = clip_coef(*total_f32, norm_dtype, max_norm);
    const ChunkRange r = my_chunk<RW_SUB>(numel, chunk_start, n);
    T* g = (T*)g_ptrs[r.t] + r.begin;
    const bool vec = (((uintptr_t)g) & 15) == 0;
    const long n8 = vec ? r.len / 8 : 0;
    for (long i = threadIdx.x; i < n8; i += 256) {
        float v[8];
        Mt<T>::load8(g + i * 8, v);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] *= coef;
        Mt<T>::store8(g + i * 8, v);
    }
    for (long i = n8 * 8 + threadIdx.x; i < r.len; i += 256) Mt<T>::store(g + i, Mt<T>::load(g + i) * coef);
}

inline void lerp_consts(double weight, float& w, float& wm1, bool& small) {
    w = (float)weight;
    wm1 = w - 1.0f;
    small = fabsf(w) < 0.5f;
}

}  // namespace

hipError_t launch_adamw_multi(const MultiTensorList& l, const void* const* g_ptrs, const void* const* e1_ptrs,
                              const void* const* e2_ptrs, const double* bias1, const double* bias2, int dtype,
                              double lr, double b1, double b2, double eps, double wd, hipStream_t stream) {
    AdamConst am;
    lerp_consts(1.0 - b1, am.w1, am.w1m1, am.small1);
    lerp_consts(1.0 - b2, am.w2, am.w2m1, am.small2);
    am.eps = (float)eps;
    am.decay = (float)(1.0 - lr * wd);
    am.alpha = (float)(-lr);
    dim3 grid((unsigned)(l.chunks * RW_SUB)), block(256);
    if (dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((adamw_multi_kernel<float>), grid, block, 0, stream, l.ptrs, g_ptrs, e1_ptrs, e2_ptrs, l.numel,
                           l.chunk_start, bias1, bias2, l.n, am);
    else if (dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((adamw_multi_kernel<bf16_t>), grid, block, 0, stream, l.ptrs, g_ptrs, e1_ptrs, e2_ptrs, l.numel,
                           l.chunk_start, bias1, bias2, l.n, am);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

namespace {
int norm_kind_of(double norm_type) {
    if (norm_type == 2.0) return NORM_TWO;
    if (norm_type == 1.0) return NORM_ONE;
    if (norm_type == 0.0) return NORM_ZERO;
    if (norm_type == (double)__builtin_inff()) return NORM_INF;
    if (norm_type == -(double)__builtin_inff()) return NORM_NEG_INF;
    return NORM_P;
}

// f(std::integral_constant<int, KIND>) for the kind of `norm_type`
template <typename F> void with_norm_kind(double norm_type, F&& f) {
    switch (norm_kind_of(norm_type)) {
        case NORM_TWO: f(std::integral_constant<int, NORM_TWO>()); break;
        case NORM_INF: f(std::integral_constant<int, NORM_INF>()); break;
        case NORM_ONE: f(std::integral_constant<int, NORM_ONE>()); break;
        case NORM_ZERO: f(std::integral_constant<int, NORM_ZERO>()); break;
        case NORM_NEG_INF: f(std::integral_constant<int, NORM_NEG_INF>()); break;
        default: f(std::integral_constant<int, NORM_P>()); break;
    }
}
}  // namespace

hipError_t launch_tensor_norms(const MultiTensorList& l, int dtype, double norm_type, float* partials, float* norms,
                               hipStream_t stream) {
    dim3 grid((unsigned)l.chunks), block(256);
    if (dtype != MUON_HIP_F32 && dtype != MUON_HIP_BF16) return hipErrorInvalidValue;
    if (norm_type != norm_type) return hipErrorInvalidValue;
    const float p = (float)norm_type;  // torch narrows the order to the accumulation type
    hipError_t e = hipSuccess;
    with_norm_kind(norm_type, [&](auto kind) {
        constexpr int KIND = decltype(kind)::value;
        if (dtype == MUON_HIP_F32)
            hipLaunchKernelGGL((sqnorm_multi_kernel<float, KIND>), grid, block, 0, stream, l.ptrs, l.numel, l.chunk_start, l.n, p, partials);
        else
            hipLaunchKernelGGL((sqnorm_multi_kernel<bf16_t, KIND>), grid, block, 0, stream, l.ptrs, l.numel, l.chunk_start, l.n, p, partials);
        e = hipGetLastError();
        if (e != hipSuccess) return;
        hipLaunchKernelGGL((tensor_norm_kernel<KIND>), dim3((unsigned)l.n), block, 0, stream, partials, l.chunk_start, dtype, p, norms);
        e = hipGetLastError();
    });
    return e;
}

hipError_t launch_total_norm(const float* norms, int n, int dtype, double norm_type, float* total_f32, void* total_typed,
                             hipStream_t stream) {
    if (norm_type != norm_type) return hipErrorInvalidValue;
    const float p = (float)norm_type;
    with_norm_kind(norm_type, [&](auto kind) {
        constexpr int KIND = decltype(kind)::value;
        hipLaunchKernelGGL((total_norm_kernel<KIND>), dim3(1), dim3(256), 0, stream, norms, n, dtype, p, total_f32, total_typed);
    });
    return hipGetLastError();
}

hipError_t launch_clip_scale_multi(const MultiTensorList& l, int dtype, const float* total_f32, int norm_dtype,
                                   double max_norm, hipStream_t stream) {
    dim3 grid((unsigned)(l.chunks * RW_SUB)), block(256);
    if (dtype == MUON_HIP_F32)
        hipLaunchKernelGGL((clip_scale_multi_kernel<float>), grid, block, 0, stream, l.ptrs, l.numel, l.chunk_start, l.n,
                           total_f32, norm_dtype, (float)max_norm);
    else if (dtype == MUON_HIP_BF16)
        hipLaunchKernelGGL((clip_scale_multi_kernel<bf16_t>), grid, block, 0, stream, l.ptrs, l.numel, l.chunk_start, l.n,
                           total_f32, norm_dtype, (float)max_norm);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}
