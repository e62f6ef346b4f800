// C ABI of libmuon_hip.so (declared in include/muon_hip.h): argument checks, workspace
// partitioning, the grouped launch sequence of one Muon step, and per-kernel event timing.
#include <stdarg.h>
#include <stdio.h>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

// The library is built with hidden visibility; the entry points declared in the public header are what it exports.
#pragma GCC visibility push(default)
#include "../../include/muon_hip.h"
#pragma GCC visibility pop
#include "common.h"
#include "elementwise.h"
#include "gemm_nt.h"
#include "multi_tensor.h"

namespace {

thread_local char g_err[512] = "";
std::atomic<int> g_forced_cfg{MUON_HIP_CFG_AUTO};  // benchmarking override, read once per call

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
}

// ---- timing ------------------------------------------------------------------------
// Event pairs come from a pool that muon_hip_timing_reserve fills ahead of the region to be measured, so that a timed
// launch costs two hipEventRecord calls and one atomic increment: no event is created and no lock is taken while the
// clock runs.  A launch that finds the pool empty goes untimed and is counted in g_untimed.
struct EventPair {
    hipEvent_t start, stop;
    int kid;
};
std::mutex g_tmu;                    // guards the pool's growth and the read-out, never a launch
std::atomic<bool> g_timing{false};
// The pool grows in chunks that are never moved or freed, so a launch may index it while another thread adds a chunk.
constexpr size_t kPoolChunk = 4096, kPoolChunks = 256, kMaxPool = kPoolChunk * kPoolChunks;
EventPair* g_chunks[kPoolChunks] = {};
std::atomic<size_t> g_pool_size{0};  // pairs that exist
std::atomic<size_t> g_used{0};       // pairs handed out since timing was enabled
std::atomic<long> g_untimed{0};
inline EventPair& pool_at(size_t i) { return g_chunks[i / kPoolChunk][i % kPoolChunk]; }

int grow_pool(size_t want) {  // under g_tmu
    if (want > kMaxPool) want = kMaxPool;
    for (size_t i = g_pool_size.load(std::memory_order_relaxed); i < want; ++i) {
        if (i % kPoolChunk == 0 && !g_chunks[i / kPoolChunk]) g_chunks[i / kPoolChunk] = new EventPair[kPoolChunk]();
        EventPair& p = pool_at(i);
        if (hipError_t e = hipEventCreate(&p.start); e != hipSuccess) return hip_fail(e, "hipEventCreate");
        if (hipError_t e = hipEventCreate(&p.stop); e != hipSuccess) {
            (void)hipEventDestroy(p.start);
            return hip_fail(e, "hipEventCreate");
        }
        g_pool_size.store(i + 1, std::memory_order_release);
    }
    return 0;
}

struct Timed {
    EventPair* ev;
    hipStream_t s;
    Timed(int kid, hipStream_t st) : ev(nullptr), s(st) {
        if (!g_timing.load(std::memory_order_acquire)) return;
        // a launch that is being recorded into a graph has no time of its own: its events would become graph nodes
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            g_untimed.fetch_add(1, std::memory_order_relaxed);
            return;
        }
        const size_t i = g_used.fetch_add(1, std::memory_order_relaxed);
        if (i >= g_pool_size.load(std::memory_order_acquire)) {
            g_untimed.fetch_add(1, std::memory_order_relaxed);
            return;
        }
        ev = &pool_at(i);
        ev->kid = kid;
        if (hipEventRecord(ev->start, s) != hipSuccess) ev->kid = -1;
    }
    ~Timed() {
        if (ev && ev->kid >= 0 && hipEventRecord(ev->stop, s) != hipSuccess) ev->kid = -1;
    }
};

// ---- geometry / workspace ------------------------------------------------------------
struct Plan {
    int rows, cols, batch, M, K, Mp, Kp, tile, cfg, nparts;
    bool transposed;
    long n, strideU, strideX, strideA;  // elements per matrix: U dense, the others blocked
    size_t offX[2], offA, offB, offParts, offDenom, offPpx, total;
};

inline long round_up(long v, long m) { return (v + m - 1) / m * m; }

// Tile edge for a matrix whose short side is M: 256 when M is a whole number of 256-tiles.
bool use_tile256(int M) { return M % 256 == 0 && M >= 512; }

// Configuration per kernel, from a sweep of every variant over the benchmark shapes: the ping-pong kernel
// everywhere, on 256-tiles where they fill the machine and on 128-tiles (two workgroups per compute unit) for
// short sides that are no whole number of 256-tiles and for the symmetric products of matrices up to 512 rows.
int pick_cfg(int M, int epi = EPI_BX, int kdim = 0) {
    const int forced = g_forced_cfg.load(std::memory_order_relaxed);
    if (forced != MUON_HIP_CFG_AUTO) return forced;
    (void)kdim;
    if (!use_tile256(M)) return GEMM_CFG_128_PINGPONG;
    if (epi != EPI_BX && M <= 512) return GEMM_CFG_128_PINGPONG;
    // The persistent kernel where the launcher takes it: a.X + B.X, and the symmetric products with reductions of at
    // most 2048 (past that a tile is long enough that what the persistent kernel removes around it no longer shows in
    // a step that runs at the power limit); launches of at most one round of tiles and those that carry the parameter
    // update run the one-tile ping-pong kernel.
    return GEMM_CFG_256_PERSIST;
}

int make_plan(int rows, int cols, int batch, Plan& p) {
    if (rows <= 0 || cols <= 0 || batch <= 0) return fail(MUON_HIP_EINVAL, "rows, cols and batch must be positive");
    if (batch > 65535) return fail(MUON_HIP_ESHAPE, "batch %d exceeds 65535 matrices per call", batch);
    p.rows = rows;
    p.cols = cols;
    p.batch = batch;
    p.transposed = rows > cols;
    p.M = rows < cols ? rows : cols;
    p.K = rows < cols ? cols : rows;
    p.cfg = pick_cfg(p.M);
    p.tile = gemm_cfg_tile(p.cfg);
    if (p.tile == 0) return fail(MUON_HIP_EINVAL, "unknown GEMM configuration %d", p.cfg);
    p.Mp = (int)round_up(p.M, p.tile);
    p.Kp = (int)round_up(p.K, p.tile);
    p.n = (long)rows * cols;
    p.strideU = round_up(p.n, 8);
    p.strideX = blocked_elems(p.Mp, p.Kp);
    p.strideA = blocked_elems(p.Mp, p.Mp);
    p.nparts = momentum_parts(p.n);
    const long T = p.Mp / p.tile, TN = p.Kp / p.tile;
    if (T * TN * batch > 0x7fffffffL) return fail(MUON_HIP_ESHAPE, "too many tiles for one launch");
    size_t off = 0;
    auto seg = [&](size_t bytes) {
        size_t o = off;
        off += (size_t)round_up((long)bytes, 256);
        return o;
    };
    const size_t xb = (size_t)batch * p.strideX * 2;
    const size_t ab = (size_t)batch * p.strideA * 2;
    p.offX[0] = seg(xb);
    p.offX[1] = seg(xb);  // doubles as U (the blend in the parameter's layout) before the first iteration
    p.offA = seg(ab);
    p.offB = seg(ab);
    p.offParts = seg((size_t)batch * p.nparts * sizeof(float));
    p.offDenom = seg((size_t)batch * sizeof(float));
    p.offPpx = seg(GEMM_PPX_COUNTER_BYTES);  // tile counters of the persistent kernels: cleared by the normalisation stage
    p.total = off;
    return 0;
}

inline bf16_t* wsp(void* ws, size_t off) { return (bf16_t*)((char*)ws + off); }
inline unsigned* ws_ppx(void* ws, const Plan& p) { return (unsigned*)((char*)ws + p.offPpx); }

int check_ws(const void* ws) {
    if (!ws) return fail(MUON_HIP_EINVAL, "workspace is null");
    if (((uintptr_t)ws) & 255) return fail(MUON_HIP_EINVAL, "workspace must be 256-byte aligned");
    return 0;
}

int check_counters(const void* counters) {
    if (((uintptr_t)counters) & 63) return fail(MUON_HIP_EINVAL, "the counter buffer must be 64-byte aligned");
    return 0;
}

int check_gemm(int cfg, int Mp, int Kp, int batch, int& tile) {
    tile = gemm_cfg_tile(cfg);
    if (tile == 0) return fail(MUON_HIP_EINVAL, "unknown GEMM configuration %d", cfg);
    if (Mp <= 0 || Kp <= 0 || batch <= 0) return fail(MUON_HIP_EINVAL, "sizes must be positive");
    if (Mp % tile || Kp % tile) return fail(MUON_HIP_ESHAPE, "Mp=%d, Kp=%d must be multiples of the %d tile", Mp, Kp, tile);
    const long T = Mp / tile, TN = Kp / tile;
    if (T * TN * batch > 0x7fffffffL) return fail(MUON_HIP_ESHAPE, "too many tiles for one launch");
    return 0;
}

// The three products on blocked buffers; matrix b of a batch starts at b * blocked_elems(rows, cols).
int do_syrk(int cfg, const bf16_t* X, bf16_t* A, int Mp, int Kp, int batch, unsigned* ppx, hipStream_t s) {
    GemmArgs g = {};
    const int tile = gemm_cfg_tile(cfg), T = Mp / tile;
    g.P = g.Q = X;
    g.strideP = g.strideQ = blocked_elems(Mp, Kp);
    g.kdim = Kp;
    g.tiles_m = g.tiles_n = T;
    g.tiles_per_mat = T * (T + 1) / 2;
    g.batch = batch;
    g.C = g.Ct = A;
    g.strideC = g.strideCt = blocked_elems(Mp, Mp);
    g.cbC = g.cbCt = Mp / BLK_COLS;
    g.ppx = ppx;
    Timed t(MUON_HIP_K_SYRK, s);
    hipError_t e = launch_gemm_nt(cfg, EPI_SYRK, g, s);
    return e == hipSuccess ? 0 : hip_fail(e, "syrk launch");
}

int do_sympoly(int cfg, const bf16_t* A, bf16_t* B, int Mp, int batch, double b, double c, unsigned* ppx, hipStream_t s) {
    GemmArgs g = {};
    const int tile = gemm_cfg_tile(cfg), T = Mp / tile;
    g.P = g.Q = A;
    g.strideP = g.strideQ = blocked_elems(Mp, Mp);
    g.kdim = Mp;
    g.tiles_m = g.tiles_n = T;
    g.tiles_per_mat = T * (T + 1) / 2;
    g.batch = batch;
    g.C = g.Ct = B;
    g.strideC = g.strideCt = blocked_elems(Mp, Mp);
    g.cbC = g.cbCt = Mp / BLK_COLS;
    g.Et = A;
    g.strideEt = blocked_elems(Mp, Mp);
    g.cbEt = Mp / BLK_COLS;
    g.s0 = (float)b;
    g.s1 = (float)c;
    g.ppx = ppx;
    Timed t(MUON_HIP_K_SYMPOLY, s);
    hipError_t e = launch_gemm_nt(cfg, EPI_SYMPOLY, g, s);
    return e == hipSuccess ? 0 : hip_fail(e, "sympoly launch");
}

// Parameter update folded into the last B.X of a step (the parameter is X's image when rows <= cols, its transpose otherwise).
struct FoldUpdate {
    const void* const* p_ptrs;
    int p_dtype, rows, cols;
    double scale, lr, weight_decay;
};

int do_bx(int cfg, const bf16_t* B, const bf16_t* X, bf16_t* Xout, int Mp, int Kp, int batch, double a, unsigned* ppx,
          hipStream_t s, const FoldUpdate* fold = nullptr) {
    GemmArgs g = {};
    const int tile = gemm_cfg_tile(cfg);
    g.P = B;
    g.strideP = blocked_elems(Mp, Mp);
    g.Q = X;
    g.strideQ = blocked_elems(Mp, Kp);
    g.cbQ = Kp / BLK_COLS;
    g.kdim = Mp;
    g.tiles_m = Mp / tile;
    g.tiles_n = Kp / tile;
    g.tiles_per_mat = g.tiles_m * g.tiles_n;
    g.batch = batch;
    g.C = Xout;
    g.strideC = blocked_elems(Mp, Kp);
    g.cbC = Kp / BLK_COLS;
    g.Et = X;
    g.strideEt = blocked_elems(Mp, Kp);
    g.cbEt = Kp / BLK_COLS;
    g.s0 = (float)a;
    if (fold) {
        g.upd_ptrs = fold->p_ptrs;
        g.upd_dtype = fold->p_dtype;
        g.upd_rows = fold->rows;
        g.upd_cols = fold->cols;
        g.upd_scale = (float)fold->scale;
        g.upd_decay = (float)(1.0 - fold->lr * fold->weight_decay);
        g.upd_alpha = (float)(-fold->lr);
    }
    g.ppx = ppx;
    Timed t(fold ? MUON_HIP_K_BX_UPDATE : MUON_HIP_K_BX, s);
    hipError_t e = launch_gemm_nt(cfg, !fold ? EPI_BX : fold->rows <= fold->cols ? EPI_BX_UPD : EPI_BX_UPD_T, g, s);
    return e == hipSuccess ? 0 : hip_fail(e, "bx launch");
}

int dtype_ok(int d) { return d == MUON_HIP_F32 || d == MUON_HIP_BF16; }

}  // namespace

extern "C" {

int muon_hip_version(void) { return 100; }

const char* muon_hip_last_error(void) { return g_err; }

int muon_hip_set_gemm_config(int cfg) {
    if (cfg != MUON_HIP_CFG_AUTO && gemm_cfg_tile(cfg) == 0) return fail(MUON_HIP_EINVAL, "unknown GEMM configuration %d", cfg);
    g_forced_cfg.store(cfg, std::memory_order_relaxed);
    return 0;
}

int muon_hip_geometry(int rows, int cols, int* M, int* K, int* Mp, int* Kp, int* tile) {
    Plan p;
    if (int rc = make_plan(rows, cols, 1, p)) return rc;
    if (M) *M = p.M;
    if (K) *K = p.K;
    if (Mp) *Mp = p.Mp;
    if (Kp) *Kp = p.Kp;
    if (tile) *tile = p.tile;
    return 0;
}

size_t muon_hip_workspace_bytes(int rows, int cols, int batch) {
    Plan p;
    if (make_plan(rows, cols, batch, p)) return 0;
    return p.total;
}

int muon_hip_momentum_norm(const void* const* g_ptrs, const void* const* m_ptrs, int g_dtype, int m_dtype,
                           void* workspace, int rows, int cols, int batch, double beta, int nesterov,
                           int write_back_grad, void* stream) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    if (!g_ptrs || !m_ptrs) return fail(MUON_HIP_EINVAL, "pointer table is null");
    const bool combo = (g_dtype == MUON_HIP_F32 && m_dtype == MUON_HIP_F32) ||
                       (g_dtype == MUON_HIP_BF16 && (m_dtype == MUON_HIP_F32 || m_dtype == MUON_HIP_BF16));
    if (!combo) return fail(MUON_HIP_EINVAL, "unsupported (grad, momentum) dtypes (%d, %d)", g_dtype, m_dtype);
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_MOMENTUM, s);
    hipError_t e = launch_momentum_norm(g_ptrs, m_ptrs, g_dtype, m_dtype, wsp(workspace, p.offX[1]), p.strideU,
                                        (float*)((char*)workspace + p.offParts), p.nparts, p.n, batch, beta, nesterov,
                                        write_back_grad, s);
    return e == hipSuccess ? 0 : hip_fail(e, "momentum_norm launch");
}

int muon_hip_cast_norm(const void* G, int g_dtype, void* workspace, int rows, int cols, int batch, void* stream) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    if (!G || !dtype_ok(g_dtype)) return fail(MUON_HIP_EINVAL, "bad input tensor or dtype");
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_MOMENTUM, s);
    hipError_t e = launch_cast_norm(G, p.n, g_dtype, wsp(workspace, p.offX[1]), p.strideU,
                                    (float*)((char*)workspace + p.offParts), p.nparts, p.n, batch, s);
    return e == hipSuccess ? 0 : hip_fail(e, "cast_norm launch");
}

int muon_hip_normalize(void* workspace, int rows, int cols, int batch, void* stream) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_NORMALIZE, s);
    hipError_t e = launch_normalize(wsp(workspace, p.offX[1]), p.strideU, (const float*)((char*)workspace + p.offParts),
                                    p.nparts, (float*)((char*)workspace + p.offDenom), wsp(workspace, p.offX[0]),
                                    p.strideX, rows, cols, p.Mp, p.Kp, batch, ws_ppx(workspace, p),
                                    (int)(GEMM_PPX_COUNTER_BYTES / sizeof(unsigned)), s);
    return e == hipSuccess ? 0 : hip_fail(e, "normalize launch");
}

}  // extern "C"

namespace {
// normalise, then `steps` iterations; with `fold` the last B.X applies the parameter update instead of writing X'
int ns_chain(void* workspace, int rows, int cols, int batch, int steps, double a, double b, double c, void* stream,
             const FoldUpdate* fold) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    if (steps < 0) return fail(MUON_HIP_EINVAL, "steps must be >= 0");
    if (int rc = muon_hip_normalize(workspace, rows, cols, batch, stream)) return rc;
    hipStream_t s = (hipStream_t)stream;
    bf16_t* X[2] = {wsp(workspace, p.offX[0]), wsp(workspace, p.offX[1])};
    bf16_t* A = wsp(workspace, p.offA);
    bf16_t* B = wsp(workspace, p.offB);
    unsigned* ppx = ws_ppx(workspace, p);  // zero: muon_hip_normalize has just cleared them
    int cur = 0;
    for (int it = 0; it < steps; ++it) {
        if (int rc = do_syrk(pick_cfg(p.M, EPI_SYRK, p.Kp), X[cur], A, p.Mp, p.Kp, batch, ppx, s)) return rc;
        if (int rc = do_sympoly(pick_cfg(p.M, EPI_SYMPOLY), A, B, p.Mp, batch, b, c, ppx, s)) return rc;
        if (int rc = do_bx(pick_cfg(p.M, EPI_BX), B, X[cur], X[cur ^ 1], p.Mp, p.Kp, batch, a, ppx, s,
                           it == steps - 1 ? fold : nullptr))
            return rc;
        cur ^= 1;
    }
    return 0;
}
}  // namespace

extern "C" {

int muon_hip_ns_grouped(void* workspace, int rows, int cols, int batch, int steps, double a, double b, double c,
                        void* stream) {
    return ns_chain(workspace, rows, cols, batch, steps, a, b, c, stream, nullptr);
}

int muon_hip_apply_update(const void* const* p_ptrs, int p_dtype, void* workspace, int rows, int cols, int batch,
                          int steps, double scale, double lr, double weight_decay, void* stream) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    if (!p_ptrs || !dtype_ok(p_dtype) || steps < 0) return fail(MUON_HIP_EINVAL, "bad pointer table, dtype or steps");
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* O = wsp(workspace, p.offX[steps & 1]);  // X (M x K): the parameter's image, or its transpose when rows > cols
    Timed t(MUON_HIP_K_UPDATE, s);
    hipError_t e = launch_apply_update(p_ptrs, p_dtype, O, p.strideX, p.Kp / BLK_COLS, rows, cols, batch, scale, lr,
                                       weight_decay, s);
    return e == hipSuccess ? 0 : hip_fail(e, "apply_update launch");
}

int muon_hip_ns_output(void* workspace, int rows, int cols, int batch, int steps, void* out, void* stream) {
    Plan p;
    if (int rc = make_plan(rows, cols, batch, p)) return rc;
    if (int rc = check_ws(workspace)) return rc;
    if (!out || steps < 0) return fail(MUON_HIP_EINVAL, "bad output pointer or steps");
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* O = wsp(workspace, p.offX[steps & 1]);
    hipError_t e = launch_unpack((bf16_t*)out, p.n, cols, O, p.strideX, p.Kp / BLK_COLS, rows, cols, p.transposed, batch, s);
    return e == hipSuccess ? 0 : hip_fail(e, "ns_output launch");
}

int muon_hip_step_grouped(const void* const* p_ptrs, const void* const* g_ptrs, const void* const* m_ptrs,
                          int p_dtype, int g_dtype, int m_dtype, void* workspace, int rows, int cols, int batch,
                          double lr, double weight_decay, double beta, int nesterov, int ns_steps, double scale,
                          double a, double b, double c, int write_back_grad, void* stream) {
    if (int rc = muon_hip_momentum_norm(g_ptrs, m_ptrs, g_dtype, m_dtype, workspace, rows, cols, batch, beta, nesterov,
                                        write_back_grad, stream))
        return rc;
    // The parameter is updated by the epilogue of the last B.X (for rows > cols through a transposing gather out of
    // LDS): the final X' is then neither written nor read back.  Without an iteration there is no such product.
    if (ns_steps >= 1) {
        if (!p_ptrs || !dtype_ok(p_dtype)) return fail(MUON_HIP_EINVAL, "bad pointer table, dtype or steps");
        const FoldUpdate fold{p_ptrs, p_dtype, rows, cols, scale, lr, weight_decay};
        return ns_chain(workspace, rows, cols, batch, ns_steps, a, b, c, stream, &fold);
    }
    if (int rc = muon_hip_ns_grouped(workspace, rows, cols, batch, ns_steps, a, b, c, stream)) return rc;
    return muon_hip_apply_update(p_ptrs, p_dtype, workspace, rows, cols, batch, ns_steps, scale, lr, weight_decay,
                                 stream);
}

long muon_hip_blocked_elems(int rows, int cols) {
    if (rows <= 0 || cols <= 0 || cols % BLK_COLS) {
        fail(MUON_HIP_ESHAPE, "a blocked matrix needs positive sizes and a multiple of 32 columns (got %d x %d)", rows, cols);
        return 0;
    }
    return blocked_elems(rows, cols);
}

int muon_hip_pack_bf16(const void* src, long src_stride, int ld, int rows, int cols, void* dst, int rows_p, int cols_p,
                       int batch, void* stream) {
    if (!src || !dst || batch <= 0) return fail(MUON_HIP_EINVAL, "null tensor or empty batch");
    if (rows <= 0 || cols <= 0 || rows > rows_p || cols > cols_p || ld < cols || cols_p % BLK_COLS || batch > 65535)
        return fail(MUON_HIP_ESHAPE, "pack: need 0 < rows <= rows_p, 0 < cols <= cols_p, ld >= cols, cols_p %% 32 == 0");
    hipError_t e = launch_pack((const bf16_t*)src, src_stride, ld, rows, cols, (bf16_t*)dst, blocked_elems(rows_p, cols_p),
                               rows_p, cols_p, batch, (hipStream_t)stream);
    return e == hipSuccess ? 0 : hip_fail(e, "pack launch");
}

int muon_hip_unpack_bf16(const void* src, int rows_p, int cols_p, void* dst, long dst_stride, int ld, int rows, int cols,
                         int batch, void* stream) {
    if (!src || !dst || batch <= 0) return fail(MUON_HIP_EINVAL, "null tensor or empty batch");
    if (rows <= 0 || cols <= 0 || rows > rows_p || cols > cols_p || ld < cols || cols_p % BLK_COLS || batch > 65535)
        return fail(MUON_HIP_ESHAPE, "unpack: need 0 < rows <= rows_p, 0 < cols <= cols_p, ld >= cols, cols_p %% 32 == 0");
    hipError_t e = launch_unpack((bf16_t*)dst, dst_stride, ld, (const bf16_t*)src, blocked_elems(rows_p, cols_p),
                                 cols_p / BLK_COLS, rows, cols, false, batch, (hipStream_t)stream);
    return e == hipSuccess ? 0 : hip_fail(e, "unpack launch");
}

int muon_hip_syrk_bf16(const void* X, void* A, int Mp, int Kp, int batch, int cfg, void* counters, void* stream) {
    if (cfg == MUON_HIP_CFG_AUTO) cfg = pick_cfg(Mp, EPI_SYRK, Kp);
    int tile;
    if (int rc = check_gemm(cfg, Mp, Kp, batch, tile)) return rc;
    if (!X || !A) return fail(MUON_HIP_EINVAL, "null operand");
    if (int rc = check_counters(counters)) return rc;
    return do_syrk(cfg, (const bf16_t*)X, (bf16_t*)A, Mp, Kp, batch, (unsigned*)counters, (hipStream_t)stream);
}

int muon_hip_sympoly_bf16(const void* A, void* B, int Mp, int batch, double b, double c, int cfg, void* counters,
                          void* stream) {
    if (cfg == MUON_HIP_CFG_AUTO) cfg = pick_cfg(Mp, EPI_SYMPOLY);
    int tile;
    if (int rc = check_gemm(cfg, Mp, Mp, batch, tile)) return rc;
    if (!A || !B || A == B) return fail(MUON_HIP_EINVAL, "null or aliased operand");
    if (int rc = check_counters(counters)) return rc;
    return do_sympoly(cfg, (const bf16_t*)A, (bf16_t*)B, Mp, batch, b, c, (unsigned*)counters, (hipStream_t)stream);
}

int muon_hip_bx_axpy_bf16(const void* B, const void* X, void* Xout, int Mp, int Kp, int batch, double a, int cfg,
                          void* counters, void* stream) {
    if (cfg == MUON_HIP_CFG_AUTO) cfg = pick_cfg(Mp, EPI_BX);
    int tile;
    if (int rc = check_gemm(cfg, Mp, Kp, batch, tile)) return rc;
    if (!B || !X || !Xout) return fail(MUON_HIP_EINVAL, "null operand");
    if (Xout == X) return fail(MUON_HIP_EINVAL, "Xout must not alias X");
    if (int rc = check_counters(counters)) return rc;
    return do_bx(cfg, (const bf16_t*)B, (const bf16_t*)X, (bf16_t*)Xout, Mp, Kp, batch, a, (unsigned*)counters, (hipStream_t)stream);
}

int muon_hip_adamw(void* p, const void* g, void* exp_avg, void* exp_avg_sq, int dtype, long n, int step, double lr,
                   double beta1, double beta2, double eps, double weight_decay, void* stream) {
    if (!p || !g || !exp_avg || !exp_avg_sq) return fail(MUON_HIP_EINVAL, "null tensor");
    if (!dtype_ok(dtype) || n < 0 || step < 1) return fail(MUON_HIP_EINVAL, "bad dtype, size or step");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_ADAMW, s);
    hipError_t e = launch_adamw(p, g, exp_avg, exp_avg_sq, dtype, n, step, lr, beta1, beta2, eps, weight_decay, s);
    return e == hipSuccess ? 0 : hip_fail(e, "adamw launch");
}

int muon_hip_adam_update(const void* g, void* exp_avg, void* exp_avg_sq, void* out, int dtype, long n, int step,
                         double beta1, double beta2, double eps, void* stream) {
    if (!g || !exp_avg || !exp_avg_sq || !out) return fail(MUON_HIP_EINVAL, "null tensor");
    if (!dtype_ok(dtype) || n < 0 || step < 1) return fail(MUON_HIP_EINVAL, "bad dtype, size or step");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_ADAMW, s);
    hipError_t e = launch_adam_update(g, exp_avg, exp_avg_sq, out, dtype, n, step, beta1, beta2, eps, s);
    return e == hipSuccess ? 0 : hip_fail(e, "adam_update launch");
}

int muon_hip_scale(void* x, int dtype, long n, double scale, void* stream) {
    if (!x) return fail(MUON_HIP_EINVAL, "null tensor");
    if (!dtype_ok(dtype) || n < 0) return fail(MUON_HIP_EINVAL, "bad dtype or size");
    if (n == 0) return 0;
    hipError_t e = launch_scale(x, dtype, n, scale, (hipStream_t)stream);
    return e == hipSuccess ? 0 : hip_fail(e, "scale launch");
}

int muon_hip_decay_update(void* p, int p_dtype, const void* u, int u_dtype, long n, double lr, double weight_decay,
                          void* stream) {
    if (!p || !u) return fail(MUON_HIP_EINVAL, "null tensor");
    if (!dtype_ok(p_dtype) || !dtype_ok(u_dtype) || n < 0) return fail(MUON_HIP_EINVAL, "bad dtype or size");
    if (p_dtype == MUON_HIP_BF16 && u_dtype == MUON_HIP_F32)
        return fail(MUON_HIP_EINVAL, "an fp32 update for a bf16 parameter is not supported");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_UPDATE, s);
    hipError_t e = launch_decay_update(p, p_dtype, u, u_dtype, n, lr, weight_decay, s);
    return e == hipSuccess ? 0 : hip_fail(e, "decay_update launch");
}

namespace {
int check_norm_type(double norm_type) {
    if (norm_type != norm_type) return fail(MUON_HIP_EINVAL, "norm_type is NaN");
    return 0;
}
int check_list(const void* ptrs, const long* numel, const long* chunk_start, int n, long chunks, int dtype) {
    if (!ptrs || !numel || !chunk_start) return fail(MUON_HIP_EINVAL, "null tensor-list array");
    if (n <= 0 || chunks <= 0) return fail(MUON_HIP_EINVAL, "a tensor list needs at least one tensor and one chunk");
    if (chunks > 0x1fffffffL) return fail(MUON_HIP_ESHAPE, "%ld chunks exceed one launch", chunks);  // up to four workgroups each
    if (!dtype_ok(dtype)) return fail(MUON_HIP_EINVAL, "unknown dtype %d", dtype);
    return 0;
}
}  // namespace

int muon_hip_adamw_multi(const void* const* p_ptrs, const void* const* g_ptrs, const void* const* exp_avg_ptrs,
                         const void* const* exp_avg_sq_ptrs, const long* numel, const long* chunk_start,
                         const double* bias1, const double* bias2, int n, long chunks, int dtype, double lr,
                         double beta1, double beta2, double eps, double weight_decay, void* stream) {
    if (int rc = check_list(p_ptrs, numel, chunk_start, n, chunks, dtype)) return rc;
    if (!g_ptrs || !exp_avg_ptrs || !exp_avg_sq_ptrs || !bias1 || !bias2) return fail(MUON_HIP_EINVAL, "null table");
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_ADAMW_MULTI, s);
    const MultiTensorList l{p_ptrs, numel, chunk_start, n, chunks};
    hipError_t e = launch_adamw_multi(l, g_ptrs, exp_avg_ptrs, exp_avg_sq_ptrs, bias1, bias2, dtype, lr, beta1, beta2,
                                      eps, weight_decay, s);
    return e == hipSuccess ? 0 : hip_fail(e, "adamw_multi launch");
}

int muon_hip_grad_norms(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n, long chunks,
                        int dtype, double norm_type, float* partials, float* norms, void* stream) {
    if (int rc = check_list(g_ptrs, numel, chunk_start, n, chunks, dtype)) return rc;
    if (int rc = check_norm_type(norm_type)) return rc;
    if (!partials || !norms) return fail(MUON_HIP_EINVAL, "null output");
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_GRAD_NORM, s);
    const MultiTensorList l{g_ptrs, numel, chunk_start, n, chunks};
    hipError_t e = launch_tensor_norms(l, dtype, norm_type, partials, norms, s);
    return e == hipSuccess ? 0 : hip_fail(e, "grad_norms launch");
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// Partial sums of muon_hip_grad_norms_static live in this array instead of a caller buffer.  Each device the
// library runs on holds its own copy at its own address, looked up once per device.
static __device__ __align__(256) float scratch[MUON_HIP_STATIC_MAX_CHUNKS];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (0 on failure, with the error recorded).
int scratch_for_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(MUON_HIP_EINVAL, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!ptr) return fail(MUON_HIP_EINVAL, "hipGetSymbolAddress returned a null address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

int muon_hip_grad_norms_static(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n,
                               long chunks, int dtype, double norm_type, float* norms, void* stream) {
    if (int rc = check_list(g_ptrs, numel, chunk_start, n, chunks, dtype)) return rc;
    if (int rc = check_norm_type(norm_type)) return rc;
    if (!norms) return fail(MUON_HIP_EINVAL, "null output");
    if (chunks > (long)MUON_HIP_STATIC_MAX_CHUNKS)
        return fail(MUON_HIP_ESHAPE, "%ld chunks exceed the %ld the built-in scratch array holds; use muon_hip_grad_norms "
                    "with a caller buffer", chunks, (long)MUON_HIP_STATIC_MAX_CHUNKS);
    float* partials = nullptr;
    if (int rc = scratch_for_current_device(&partials)) return rc;
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_GRAD_NORM, s);
    const MultiTensorList l{g_ptrs, numel, chunk_start, n, chunks};
    // every partial the second kernel reads is written by the first: nothing has to start at zero
    hipError_t e = launch_tensor_norms(l, dtype, norm_type, partials, norms, s);
    return e == hipSuccess ? 0 : hip_fail(e, "grad_norms launch");
}

int muon_hip_total_norm(const float* norms, int n, int dtype, double norm_type, float* total_f32, void* total_typed,
                        void* stream) {
    if (!norms || !total_f32 || !total_typed || n <= 0 || !dtype_ok(dtype))
        return fail(MUON_HIP_EINVAL, "null pointer, empty list or unknown dtype");
    if (int rc = check_norm_type(norm_type)) return rc;
    hipError_t e = launch_total_norm(norms, n, dtype, norm_type, total_f32, total_typed,
                                     (hipStream_t)stream);
    return e == hipSuccess ? 0 : hip_fail(e, "total_norm launch");
}

int muon_hip_clip_scale(const void* const* g_ptrs, const long* numel, const long* chunk_start, int n, long chunks,
                        int dtype, const float* total_f32, int norm_dtype, double max_norm, void* stream) {
    if (int rc = check_list(g_ptrs, numel, chunk_start, n, chunks, dtype)) return rc;
    if (!total_f32 || !dtype_ok(norm_dtype)) return fail(MUON_HIP_EINVAL, "null total or unknown norm dtype");
    hipStream_t s = (hipStream_t)stream;
    Timed t(MUON_HIP_K_CLIP_SCALE, s);
    const MultiTensorList l{g_ptrs, numel, chunk_start, n, chunks};
    hipError_t e = launch_clip_scale_multi(l, dtype, total_f32, norm_dtype, max_norm, s);
    return e == hipSuccess ? 0 : hip_fail(e, "clip_scale launch");
}

int muon_hip_device_shape(int* compute_units, int* xcds) {
    MachineShape ms;
    if (hipError_t e = machine_shape(ms); e != hipSuccess) return hip_fail(e, "device attributes");
    if (compute_units) *compute_units = ms.cus;
    if (xcds) *xcds = 1 << ms.xcd_shift;
    return 0;
}

int muon_hip_timing_reserve(long launches) {
    if (launches < 0 || (size_t)launches > kMaxPool) return fail(MUON_HIP_EINVAL, "0 to %ld launches can be reserved", (long)kMaxPool);
    if (g_timing.load(std::memory_order_acquire)) return fail(MUON_HIP_EINVAL, "reserve events while timing is off");
    std::lock_guard<std::mutex> lk(g_tmu);
    return grow_pool((size_t)launches);
}

int muon_hip_timing_enable(int on) {
    std::lock_guard<std::mutex> lk(g_tmu);
    g_timing.store(false, std::memory_order_release);
    if (on) {
        if (int rc = grow_pool(kPoolChunk)) return rc;  // at least one chunk (a no-op once it exists)
        g_used.store(0, std::memory_order_relaxed);  // the pairs of the last measurement are recorded over
        g_untimed.store(0, std::memory_order_relaxed);
        g_timing.store(true, std::memory_order_release);
    }
    return 0;
}

int muon_hip_timing_read(int kernel_id, double* total_ms, long* launches) {
    if (kernel_id < 0 || kernel_id >= MUON_HIP_K_COUNT || !total_ms || !launches)
        return fail(MUON_HIP_EINVAL, "bad kernel id or null output");
    std::lock_guard<std::mutex> lk(g_tmu);
    const size_t used = std::min(g_used.load(std::memory_order_acquire), g_pool_size.load(std::memory_order_acquire));
    double tot = 0.0;
    long cnt = 0;
    for (size_t i = 0; i < used; ++i) {
        const EventPair& p = pool_at(i);
        if (p.kid != kernel_id) continue;
        hipError_t e = hipEventSynchronize(p.stop);
        if (e != hipSuccess) return hip_fail(e, "event synchronize");
        float ms = 0.f;
        e = hipEventElapsedTime(&ms, p.start, p.stop);
        if (e != hipSuccess) return hip_fail(e, "event elapsed");
        tot += ms;
        ++cnt;
    }
    *total_ms = tot;
    *launches = cnt;
    return 0;
}

long muon_hip_timing_untimed(void) { return g_untimed.load(std::memory_order_relaxed); }

}  // extern "C"
