/* C ABI of libmuon_hip.so: the Muon optimizer step of lmms-engine on one MI355X (gfx950).
 *
 * The reference path is pure Python (src/lmms_engine/utils/muon_utils.py); its "FFI" is the
 * set of torch / Triton calls that file makes.  Each entry point below replaces one group of
 * those calls, cited as muon_utils.py:LINE.  A Python caller binds them with ctypes
 * (lmms_engine_amd/_abi.py); any other host can bind the same symbols.
 *
 * Conventions
 *  - Plain C types only.  Device pointers are borrowed for the duration of the call; the
 *    library never allocates, frees or retains device memory.
 *  - `stream` is a hipStream_t (0 = the null stream).  Every call only enqueues work on it
 *    and returns without synchronising the host.
 *  - Return value: 0 on success, a positive hipError_t when the runtime failed, a negative
 *    MUON_HIP_E* code when an argument was rejected.  muon_hip_last_error() describes the
 *    last failure on the calling thread.
 *  - dtype codes: MUON_HIP_F32 = 0, MUON_HIP_BF16 = 1.
 *  - A parameter is `rows x cols`, row-major, contiguous.  M = min(rows, cols),
 *    K = max(rows, cols); "transposed" means rows > cols (muon_utils.py:139-140).
 *  - Batched entry points work on `batch` matrices of one shape.  Optimizer tensors are
 *    reached through device-resident pointer tables (`const void* const*`, `batch` entries).
 *  - The Newton-Schulz operands live, in a blocked layout (below), in a caller-allocated workspace of
 *    muon_hip_workspace_bytes() bytes, 256-byte aligned, which the entry points partition
 *    identically; its contents between calls are private to the library.
 *  - Concurrency.  The library keeps no device state of its own (the one exception is
 *    muon_hip_grad_norms_static, which says so).  Everything a call shares between its kernels lives in
 *    the caller's workspace, the tile counters of the persistent GEMM kernels included (the
 *    normalisation stage clears them, every persistent launch leaves them zero).  Calls that use
 *    different workspaces may run at the same time on different streams, also a replayed HIP graph beside
 *    eager calls; calls that share a workspace (or a counter buffer of the single-GEMM entry points) must
 *    be ordered on one stream, as for any other buffer both would write.
 */
#ifndef MUON_HIP_H
#define MUON_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUON_HIP_F32 0
#define MUON_HIP_BF16 1

#define MUON_HIP_EINVAL (-1)  /* bad argument (null pointer, non-positive size, unknown dtype/config) */
#define MUON_HIP_ESHAPE (-2)  /* shape is not a whole number of tiles / exceeds a launch limit */

/* kernel ids for muon_hip_timing_read */
#define MUON_HIP_K_MOMENTUM 0
#define MUON_HIP_K_NORMALIZE 1
#define MUON_HIP_K_SYRK 2
#define MUON_HIP_K_SYMPOLY 3
#define MUON_HIP_K_BX 4
#define MUON_HIP_K_UPDATE 5
#define MUON_HIP_K_ADAMW 6
#define MUON_HIP_K_ADAMW_MULTI 7
#define MUON_HIP_K_GRAD_NORM 8
#define MUON_HIP_K_CLIP_SCALE 9
#define MUON_HIP_K_BX_UPDATE 10 /* the a.X + B.X launch that carries the parameter update in its epilogue */
#define MUON_HIP_K_COUNT 11

/* GEMM kernel variants; MUON_HIP_CFG_AUTO picks per kernel and shape.  All feed LDS with direct
 * global->LDS loads (global_load_lds_dwordx4), software pipelined behind the MFMAs. */
#define MUON_HIP_CFG_AUTO (-1)
#define MUON_HIP_CFG_128_PIPE 0      /* 128x128 tile, 4 waves, 64-column k-tiles, two LDS stages */
#define MUON_HIP_CFG_256_PIPE 1      /* 256x256 tile, 8 waves, the same pipeline */
#define MUON_HIP_CFG_256_PINGPONG 2  /* 256x256 tile, two groups of 4 waves alternating memory / MFMA phases */
#define MUON_HIP_CFG_128_PINGPONG 3  /* 128x128 tile, the same eight-wave kernel, two workgroups per compute unit */
#define MUON_HIP_CFG_256_PERSIST 4   /* the ping-pong loop as a persistent kernel: a workgroup per compute unit walks 256x256 tiles,
                                        the next tile's first loads land behind an epilogue that needs no LDS.  Taken by launches
                                        of more than one round of tiles: a.X + B.X, and the symmetric products with reductions
                                        of at most 2048; everything else runs MUON_HIP_CFG_256_PINGPONG */
#define MUON_HIP_CFG_COUNT 5

int muon_hip_version(void);
const char* muon_hip_last_error(void);

/* Padded operand geometry for a rows x cols parameter: M, K as above, Mp/Kp the zero-padded
 * sizes the GEMM kernels work on, tile the square tile edge.  Any out pointer may be null. */
int muon_hip_geometry(int rows, int cols, int* M, int* K, int* Mp, int* Kp, int* tile);

/* Bytes of workspace one bucket of `batch` rows x cols matrices needs. */
size_t muon_hip_workspace_bytes(int rows, int cols, int batch);

/* Force one tile configuration for every later call (MUON_HIP_CFG_AUTO restores the default).
 * Affects geometry and workspace size; meant for benchmarking sweeps. */
int muon_hip_set_gemm_config(int cfg);

/* ---- stage entry points (workspace based) ------------------------------------------- */

/* muon_update's momentum stage, muon_utils.py:188-189, fused with X = G.bfloat16() (:138)
 * and the sum of squares behind X.norm (:146):
 *   m <- lerp(m, g, 1-beta);  u <- nesterov ? lerp(g, m, beta) : m;  workspace.U <- bf16(u)
 * g is read through g_ptrs (dtype g_dtype), m updated in place through m_ptrs (m_dtype).
 * Supported (g, m) dtypes: (f32, f32), (bf16, bf16) as the reference, and (bf16, f32).
 * write_back_grad != 0 also stores u into g, as the reference's in-place lerp_ does. */
int muon_hip_momentum_norm(const void* const* g_ptrs, const void* const* m_ptrs, int g_dtype, int m_dtype,
                           void* workspace, int rows, int cols, int batch, double beta, int nesterov,
                           int write_back_grad, void* stream);

/* The same first stage for fast_newtonschulz called on its own (muon_utils.py:138,146):
 * G is a dense [batch][rows][cols] tensor; workspace.U <- bf16(G) plus the partial sums. */
int muon_hip_cast_norm(const void* G, int g_dtype, void* workspace, int rows, int cols, int batch, void* stream);

/* The normalisation of fast_newtonschulz on its own, muon_utils.py:139-146, on what the first stage left in
 * the workspace:  d = bf16(bf16(||U||_F) + 1e-7) from the partial sums (fixed order);  X <- bf16(U / d), written
 * in the blocked operand layout, transposed when rows > cols (:139-140).  muon_hip_ns_grouped starts with it;
 * muon_hip_ns_output(steps = 0) returns the normalised matrix. */
int muon_hip_normalize(void* workspace, int rows, int cols, int batch, void* stream);

/* fast_newtonschulz, muon_utils.py:139-156, on what the first stage left in the workspace:
 * normalise by bf16(bf16(||X||_F) + 1e-7), then `steps` iterations of
 *   A = X Xt; B = b A + c A A; X = a X + B X
 * with the reference's bf16 rounding points.  The result stays in the workspace. */
int muon_hip_ns_grouped(void* workspace, int rows, int cols, int batch, int steps, double a, double b, double c,
                        void* stream);

/* apply_scaling (muon_utils.py:167-175) and the parameter update (:324-325):
 *   o = bf16(O * scale);  p <- p * (1 - lr*wd);  p <- p + (-lr) * o
 * O is the result muon_hip_ns_grouped(steps) left in the workspace.  `scale` is the python
 * double the reference multiplies by (0.2*sqrt(max(rows, cols)) or sqrt(max(1, rows/cols))). */
int muon_hip_apply_update(const void* const* p_ptrs, int p_dtype, void* workspace, int rows, int cols, int batch,
                          int steps, double scale, double lr, double weight_decay, void* stream);

/* Copies the NS result out of the workspace into a dense bf16 [batch][rows][cols] tensor:
 * the return value of fast_newtonschulz (muon_utils.py:154-156). */
int muon_hip_ns_output(void* workspace, int rows, int cols, int batch, int steps, void* out, void* stream);

/* The whole Muon step for one bucket: SingelDeviceWork.start (muon_utils.py:315-325) for
 * `batch` same-shape parameters in one grouped dispatch per stage.  With ns_steps >= 1 the scaling,
 * decay and update lines (:167-175, :324-325) run in the epilogue of the last B.X product, so the
 * final X' is neither written nor read back (results equal muon_hip_momentum_norm + muon_hip_ns_grouped
 * + muon_hip_apply_update bit for bit); the workspace then does not hold the last iterate. */
int muon_hip_step_grouped(const void* const* p_ptrs, const void* const* g_ptrs, const void* const* m_ptrs,
                          int p_dtype, int g_dtype, int m_dtype, void* workspace, int rows, int cols, int batch,
                          double lr, double weight_decay, double beta, int nesterov, int ns_steps, double scale,
                          double a, double b, double c, int write_back_grad, void* stream);

/* ---- blocked matrices and single GEMM entry points ---------------------------------------
 * The Newton-Schulz operands are kept in blocks of 256 rows x 32 columns (16 KB, 64-byte
 * rows back to back): element (r, c) of a matrix with cb = cols / 32 column blocks is at
 *     ((r / 256) * cb + c / 32) * 8192 + (r % 256) * 32 + c % 32
 * so that every 32-column k-tile of an operand panel is one contiguous run of memory.  A blocked
 * rows x cols matrix (cols a multiple of 32) takes muon_hip_blocked_elems(rows, cols) elements;
 * matrix b of a batch starts b times that many elements after the first. */
long muon_hip_blocked_elems(int rows, int cols);

/* Row-major bf16 (row pitch ld, matrices src_stride elements apart) -> blocked rows_p x cols_p,
 * zero padded; and back (only rows x cols are written). */
int muon_hip_pack_bf16(const void* src, long src_stride, int ld, int rows, int cols, void* dst, int rows_p, int cols_p,
                       int batch, void* stream);
int muon_hip_unpack_bf16(const void* src, int rows_p, int cols_p, void* dst, long dst_stride, int ld, int rows, int cols,
                         int batch, void* stream);

/* The three products on explicit blocked buffers already padded to whole tiles (Mp, Kp multiples
 * of the configuration's tile edge).  `counters` is either null or MUON_HIP_PPX_COUNTER_BYTES of device
 * memory, 64-byte aligned and zero before its first use: the tile counters that the persistent kernel
 * (MUON_HIP_CFG_256_PERSIST) needs.  Every launch leaves the buffer zero again; launches that share it must
 * be ordered on one stream.  With a null pointer the one-tile kernels run instead (same results bit for bit). */
#define MUON_HIP_PPX_COUNTER_BYTES 576

/* A (Mp x Mp) = bf16(X Xt) for X (Mp x Kp): matmul_transpose_assign + mmt_kernel,
 * muon_utils.py:95-119 and :28-92.  Upper tiles computed, mirrored below the diagonal. */
int muon_hip_syrk_bf16(const void* X, void* A, int Mp, int Kp, int batch, int cfg, void* counters, void* stream);

/* B = bf16(bf16(b*A) + bf16(c*bf16(A A))) for symmetric A (Mp x Mp): muon_utils.py:150-151. */
int muon_hip_sympoly_bf16(const void* A, void* B, int Mp, int batch, double b, double c, int cfg, void* counters,
                          void* stream);

/* X' = bf16(bf16(a*X) + bf16(B X)): muon_utils.py:152.  B (Mp x Mp) symmetric, X and Xout (Mp x Kp) distinct
 * buffers.  The reduction runs down the columns of X, which the kernel reads from LDS with gfx950's
 * transposing read, so no transposed copy of X exists anywhere. */
int muon_hip_bx_axpy_bf16(const void* B, const void* X, void* Xout, int Mp, int Kp, int batch, double a, int cfg,
                          void* counters, void* stream);

/* ---- AdamW fallback ------------------------------------------------------------------ */

/* adam_update + the Adam branch of step_fsdp, muon_utils.py:178-183 and :468-477, for one
 * tensor of n elements; p, g, exp_avg, exp_avg_sq share `dtype`; `step` is already incremented. */
int muon_hip_adamw(void* p, const void* g, void* exp_avg, void* exp_avg_sq, int dtype, long n, int step, double lr,
                   double beta1, double beta2, double eps, double weight_decay, void* stream);

/* adam_update on its own, muon_utils.py:178-183: exp_avg and exp_avg_sq move in place, the bias-corrected
 * update exp_avg_c / (sqrt(exp_avg_sq_c) + eps) is written to `out` (n elements of `dtype`, may not alias). */
int muon_hip_adam_update(const void* g, void* exp_avg, void* exp_avg_sq, void* out, int dtype, long n, int step,
                         double beta1, double beta2, double eps, void* stream);

/* apply_scaling on its own, muon_utils.py:167-175: x <- x * scale in place, one rounding in x's dtype. */
int muon_hip_scale(void* x, int dtype, long n, double scale, void* stream);

/* The decay and update lines on a dense update tensor, muon_utils.py:406-407 (the Muon branch of
 * step_deepspeed, where DeepSpeed has already put the orthogonalised update into p.grad) and :324-325:
 *   p <- p * (1 - lr*wd);  p <- p + (-lr) * u
 * (p, u) dtypes: (f32, f32), (bf16, bf16), (f32, bf16). */
int muon_hip_decay_update(void* p, int p_dtype, const void* u, int u_dtype, long n, double lr, double weight_decay,
                          void* stream);

/* ---- multi-tensor kernels ---------------------------------------------------------------
 * One launch walks a list of n tensors of one dtype.  The list is described by device arrays:
 * base pointers (`const void* const*`, n entries), element counts `numel` (n longs) and
 * `chunk_start` (n + 1 longs): tensors are cut into chunks of MUON_HIP_MULTI_CHUNK elements,
 * chunk_start[t] is the index of tensor t's first chunk and chunk_start[n] == chunks, the total
 * (one workgroup per chunk).  The caller builds these arrays; the library cannot check them. */
#define MUON_HIP_MULTI_CHUNK 16384

/* The Adam branch of step_fsdp over a whole parameter group in one launch: adam_update
 * (muon_utils.py:178-183) then decay and update (:473-477), i.e. muon_hip_adamw for every tensor
 * of the list.  bias1[t] = 1 - beta1**step_t and bias2[t] = 1 - beta2**step_t (device doubles,
 * steps already incremented: each parameter keeps its own step, muon_utils.py:471). */
int muon_hip_adamw_multi(const void* const* p_ptrs, const void* const* g_ptrs, const void* const* exp_avg_ptrs,
                         const void* const* exp_avg_sq_ptrs, const long* numel, const long* chunk_start,
                         const double* bias1, const double* bias2, int n, long chunks, int dtype, double lr,
                         double beta1, double beta2, double eps, double weight_decay, void* stream);

/* Gradient clipping, the step before optimizer.step(): fsdp2_clip_grad_norm_ on one device
 * (utils/fsdp2_utils.py:234-255) is torch's _get_total_norm + _clip_grads_with_norm_.  `norm_type` is the
 * reference's argument of that name, with the meanings torch.linalg.vector_norm gives it: 2 (the default), 1,
 * 0 (the count of non-zeros), +inf / -inf (the largest / smallest magnitude; a NaN anywhere makes the result NaN,
 * as torch's max and min do) and any other order p as (sum |x|^p)^(1/p) in fp32.  NaN is rejected.
 * muon_hip_grad_norms: norms[t] = ||g_t|| accumulated in fp32 and rounded to the tensors' dtype,
 *   as fp32 values (the per-tensor norms of torch._foreach_norm); `partials` is scratch of
 *   `chunks` floats.
 * muon_hip_total_norm: the norm of n such norms (lists of several dtypes concatenated by the
 *   caller), rounded to `dtype`, written as fp32 to *total_f32 and in `dtype` to *total_typed.
 * muon_hip_clip_scale: g_t *= min(1, max_norm / (total + 1e-6)) for every tensor of the list,
 *   the coefficient evaluated as torch does, (total + 1e-6).reciprocal() * max_norm in the
 *   norm's dtype `norm_dtype`, read from device memory so that no host synchronisation is needed. */
int muon_hip_grad_norms(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n, long chunks,
                        int dtype, double norm_type, float* partials, float* norms, void* stream);
int muon_hip_total_norm(const float* norms, int n, int dtype, double norm_type, float* total_f32, void* total_typed,
                        void* stream);

/* muon_hip_grad_norms without the `partials` argument.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory for the scratch buffer (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  The partial sums go to an array of MUON_HIP_STATIC_MAX_CHUNKS
 * floats (4 MiB) built into the library, one copy per device, held until the process ends; more chunks than
 * that are rejected with MUON_HIP_ESHAPE.  The call allocates and frees nothing.  All calls on one device share
 * the array, so calls that may overlap on one device (different streams, different threads) race: serialise
 * them.  The first call on a device looks the array's address up and must not run under stream capture. */
#define MUON_HIP_STATIC_MAX_CHUNKS (1 << 20)
int muon_hip_grad_norms_static(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n,
                               long chunks, int dtype, double norm_type, float* norms, void* stream);
int muon_hip_clip_scale(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n, long chunks,
                        int dtype, const float* total_f32, int norm_dtype, double max_norm, void* stream);

/* Shape of the current device as the launchers see it, read from the runtime once per device: compute units
 * (a round of 256x256 tiles is one per compute unit) and XCDs (compute units / 32 on gfx950, whole XCDs per
 * partition).  No counterpart in the reference.  Either pointer may be null. */
int muon_hip_device_shape(int* compute_units, int* xcds);

/* ---- per-kernel timing ----------------------------------------------------------------
 * No counterpart in the reference.  When enabled, every kernel launch is bracketed by a pair
 * of HIP events on its own stream; muon_hip_timing_read waits for them and returns the summed
 * duration and launch count of one kernel id since timing was enabled.  The events come from a pool:
 * muon_hip_timing_reserve(n), called while timing is off, makes sure n pairs exist (enabling creates
 * 4096 if there are fewer), so that a timed launch creates nothing and takes no lock.  Launches beyond
 * the pool, and launches on a stream that is being captured into a graph, run untimed;
 * muon_hip_timing_untimed() counts them since timing was enabled. */
int muon_hip_timing_reserve(long launches);
int muon_hip_timing_enable(int on);
int muon_hip_timing_read(int kernel_id, double* total_ms, long* launches);
long muon_hip_timing_untimed(void);

#ifdef __cplusplus
}
#endif
#endif /* MUON_HIP_H */
