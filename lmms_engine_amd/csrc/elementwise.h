// Host launchers for the memory-bound kernels (see elementwise.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "common.h"

#define MUON_PART_ELEMS 4096   // elements per Frobenius partial sum = per workgroup of the momentum kernel
#define MUON_MAX_PARTS 65536   // partial sums per matrix, at most (larger matrices put more elements into each)

int momentum_parts(long n);
hipError_t launch_momentum_norm(const void* const* g_ptrs, const void* const* m_ptrs, int g_dtype, int m_dtype,
                                bf16_t* U, long strideU, float* partials, int nparts, long n, int batch,
                                double beta, int nesterov, int write_back, hipStream_t stream);
hipError_t launch_cast_norm(const void* G, long strideG, int g_dtype, bf16_t* U, long strideU, float* partials,
                            int nparts, long n, int batch, hipStream_t stream);
hipError_t launch_normalize(const bf16_t* U, long strideU, const float* partials, int nparts, float* denom, bf16_t* X,
                            long strideX, int rows, int cols, int Mp, int Kp, int batch, unsigned* clear, int clear_words,
                            hipStream_t stream);
hipError_t launch_apply_update(const void* const* p_ptrs, int p_dtype, const bf16_t* O, long strideO, int cbo,
                               int rows, int cols, int batch, double scale, double lr, double wd,
                               hipStream_t stream);
hipError_t launch_unpack(bf16_t* out, long strideOut, int ld, const bf16_t* O, long strideO, int cbo, int rows,
                         int cols, bool transposed, int batch, hipStream_t stream);
hipError_t launch_pack(const bf16_t* src, long strideSrc, int ld, int rows, int cols, bf16_t* dst, long strideDst,
                       int rows_p, int cols_p, int batch, hipStream_t stream);
hipError_t launch_adamw(void* p, const void* g, void* e1, void* e2, int dtype, long n, int step, double lr,
                        double b1, double b2, double eps, double wd, hipStream_t stream);
hipError_t launch_adam_update(const void* g, void* e1, void* e2, void* out, int dtype, long n, int step, double b1,
                              double b2, double eps, hipStream_t stream);
hipError_t launch_scale(void* x, int dtype, long n, double s, hipStream_t stream);
hipError_t launch_decay_update(void* p, int p_dtype, const void* u, int u_dtype, long n, double lr, double wd,
                               hipStream_t stream);
