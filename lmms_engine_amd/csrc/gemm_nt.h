// Host-side description of one batched NT GEMM launch (see gemm_nt.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "common.h"

enum { EPI_SYRK = 0, EPI_SYMPOLY = 1, EPI_BX = 2 };
enum {
    GEMM_CFG_128x128_W4 = 0,
    GEMM_CFG_256x256_W4 = 1,
    GEMM_CFG_256x256_W8 = 2,
    GEMM_CFG_128x128_W4_DLDS = 3,
    GEMM_CFG_256x256_W4_DLDS = 4,
    GEMM_CFG_256x256_W8_DLDS = 5,
    GEMM_CFG_128x128_W4_PIPE = 6,
    GEMM_CFG_256x256_W4_PIPE = 7,
    GEMM_CFG_256x256_W8_PIPE = 8,
    GEMM_CFG_128x128_W4_PIPE4 = 9,
    GEMM_CFG_256x256_W4_PIPE4 = 10,
    GEMM_CFG_256x256_W8_PIPE4 = 11,
    GEMM_CFG_256x256_W8_PINGPONG = 12,
    GEMM_CFG_256x256_W8_PINGPONG5 = 13,
    GEMM_CFG_COUNT = 14
};

struct GemmArgs {
    const bf16_t* P;   // left operand rows (reduction contiguous)
    const bf16_t* Q;   // right operand rows (reduction contiguous)
    long strideP, strideQ;  // elements between matrices of the batch
    int ldp, ldq;           // elements between rows
    int kdim;               // reduction length, a multiple of 64
    int tiles_m, tiles_n;   // tile grid of one matrix (triangular kernels: tiles_m == tiles_n)
    int tiles_per_mat;      // tiles_m*(tiles_m+1)/2 for the symmetric kernels, tiles_m*tiles_n for BX
    int batch;
    bf16_t* C;    // out[i][j]; may be null for BX
    long strideC;
    int ldc;
    bf16_t* Ct;   // out[j][i]; the same buffer as C for the symmetric kernels; may be null for BX
    long strideCt;
    int ldct;
    const bf16_t* Et;  // elementwise source read as Et[j][i]: A (symmetric) or Xt
    long strideEt;
    int ldet;
    float s0, s1;  // SYMPOLY: (b, c); BX: (a, -)
    int stagger;   // cycles by which XCD x delays its first tile (x * stagger); 0 = off
};

int gemm_cfg_tile(int cfg);
hipError_t launch_gemm_nt(int cfg, int epi, const GemmArgs& g, hipStream_t stream);
