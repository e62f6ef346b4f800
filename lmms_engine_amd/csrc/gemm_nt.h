// Host-side description of one batched NT GEMM launch (see gemm_nt.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "common.h"

// EPI_BX_UPD is EPI_BX with the parameter update folded into the epilogue (GemmArgs::upd_*) instead of writing X';
// EPI_BX_UPD_T is the same for a parameter that is the transpose of X (rows > cols)
enum { EPI_SYRK = 0, EPI_SYMPOLY = 1, EPI_BX = 2, EPI_BX_UPD = 3, EPI_BX_UPD_T = 4 };
constexpr bool epi_is_bx(int e) { return e == EPI_BX || e == EPI_BX_UPD || e == EPI_BX_UPD_T; }
// how the B.X epilogue finishes: 0 writes X', 1 updates a parameter in the orientation of X, 2 a transposed one
constexpr int epi_fold_mode(int e) { return e == EPI_BX_UPD ? 1 : e == EPI_BX_UPD_T ? 2 : 0; }
enum {
    GEMM_CFG_128_PIPE = 0,      // 128x128 tile, 4 waves, 64-column k-tiles in two LDS stages
    GEMM_CFG_256_PIPE = 1,      // 256x256 tile, 8 waves, the same pipeline
    GEMM_CFG_256_PINGPONG = 2,  // 256x256 tile, 8 waves in two alternating groups, four stages of 32 columns
    GEMM_CFG_128_PINGPONG = 3,  // 128x128 tile, the same eight-wave kernel, two workgroups per compute unit
    GEMM_CFG_256_PERSIST = 4,   // the ping-pong loop as a persistent kernel (a workgroup per compute unit walks tiles, the next
                                // tile's first loads land behind an epilogue without LDS): a.X + B.X, and the symmetric
                                // products with reductions up to 2048; launches of at most one round and the launches that
                                // carry the parameter update run GEMM_CFG_256_PINGPONG
    GEMM_CFG_COUNT = 5
};

struct GemmArgs {
    const bf16_t* P;        // left operand: rows x kdim, blocked
    const bf16_t* Q;        // right operand, blocked: rows x kdim (SYRK, SYMPOLY) or kdim x columns (BX)
    long strideP, strideQ;  // elements between matrices of the batch
    int cbQ;                // BX: column blocks of Q
    int kdim;               // reduction length, a multiple of 128
    int tiles_m, tiles_n;   // tile grid of one matrix (triangular kernels: tiles_m == tiles_n)
    int tiles_per_mat;      // tiles_m*(tiles_m+1)/2 for the symmetric kernels, tiles_m*tiles_n for BX
    int batch;
    bf16_t* C;              // out[i][j], blocked with cbC column blocks
    long strideC;
    int cbC;
    bf16_t* Ct;             // symmetric kernels: out[j][i], the same buffer as C; BX: unused
    long strideCt;
    int cbCt;
    const bf16_t* Et;       // elementwise source, blocked: A read as Et[j][i] (symmetric), or X read as Et[i][j] (BX)
    long strideEt;
    int cbEt;
    float s0, s1;           // SYMPOLY: (b, c); BX: (a, -)
    // BX, optional: fold apply_scaling and the parameter update into the epilogue instead of writing X'
    // (EPI_BX_UPD: the parameter is X's image, rows <= cols; EPI_BX_UPD_T: its transpose, rows > cols)
    const void* const* upd_ptrs;  // device table of parameter base pointers, one per matrix; null = write X'
    int upd_dtype;                // MUON_HIP_F32 or MUON_HIP_BF16
    int upd_rows, upd_cols;       // the parameter's own (unpadded) shape
    float upd_scale, upd_decay, upd_alpha;  // python-double scale, 1 - lr*wd and -lr, as fp32
    int big_blocks;         // set by the launcher: workgroups that compute whole 256x256 tiles (split-tail kernel)
    unsigned* ppx;          // tile counters of the persistent kernel (GEMM_PPX_COUNTER_BYTES, zero between launches);
                            // null: the launcher takes the one-tile kernels instead
    int xcd_shift;          // set by the launcher: log2 of the XCD count of the device
};

// Tile counters of one persistent launch: a 64-byte line per XCD (tiles handed out beyond the two static rounds) and one
// for the workgroups that have left.  A launch finds them zero and leaves them zero (the last workgroup out resets them),
// so launches that share a buffer must be ordered on one stream.
constexpr int GEMM_MAX_XCDS = 8;
constexpr size_t GEMM_PPX_COUNTER_BYTES = (GEMM_MAX_XCDS + 1) * 16 * sizeof(unsigned);

// Shape of the current device, read once per device: compute units (one 256x256 workgroup each per round of tiles) and
// XCDs.  gfx950 dies carry 32 active compute units per XCD, and a partition of the part exposes whole XCDs, so the XCD
// count is the compute-unit count over 32; workgroups are dealt to the XCDs round-robin by their linear id.
struct MachineShape {
    int cus, xcd_shift;
};
hipError_t machine_shape(MachineShape& ms);

int gemm_cfg_tile(int cfg);
hipError_t launch_gemm_nt(int cfg, int epi, const GemmArgs& g, hipStream_t stream);
