// NT GEMM family for the Newton-Schulz chain on gfx950 (v_mfma_f32_32x32x16_bf16).
//
// All three products of one NS iteration are "row times row" contractions of bf16
// operands whose reduction dimension is contiguous:
//   SYRK     A  = bf(X Xt)                         P = Q = X   (M x K)
//   SYMPOLY  B  = bf(bf(b A) + bf(c bf(A A)))      P = Q = A   (M x M, symmetric so A A = A At)
//   BX       X' = bf(bf(a X) + bf(B X))            P = B (M x M), Q = Xt (K x M)
// BX reads the transposed copy Xt as its second operand and writes both X' and X't, so no
// operand ever needs a transposing load.  SYRK/SYMPOLY compute only tiles on or above the
// diagonal and mirror them, which makes the result symmetric bit for bit.
//
// Every bf16 rounding point of the reference's torch expressions
// (/root/reference/src/lmms_engine/utils/muon_utils.py:149-152) is applied in registers.
//
// Operands are zero padded by the caller to whole tiles, so there is no masking here; the
// host launcher checks that the shapes it is given are whole tiles before launching.
#include <type_traits>

#include "common.h"
#include "gemm_nt.h"

namespace {

constexpr int BK = 64;          // bf16 elements per k-tile: one 128-byte LDS row
constexpr int ROW_BYTES = 128;

// Upper-triangle tile order in row groups of GM: inside a group, column by column, so the
// ~32 tiles an XCD works on at a time touch few distinct row panels.
template <int GM>
__device__ __forceinline__ void tri_decode(int t, int T, int& ti, int& tj) {
    int r0 = 0;
    for (;;) {
        const int gm = (T - r0 < GM) ? (T - r0) : GM;
        const int cnt = gm * (T - r0) - gm * (gm - 1) / 2;
        if (t < cnt || r0 + gm >= T) {
            const int tri = gm * (gm + 1) / 2;
            if (t < tri) {
                int c = 0;  // column c of the leading gm x gm triangle holds c+1 tiles
                while (t >= c + 1) { t -= c + 1; ++c; }
                ti = r0 + t;
                tj = r0 + c;
            } else {
                t -= tri;
                tj = r0 + gm + t / gm;
                ti = r0 + t % gm;
            }
            return;
        }
        t -= cnt;
        r0 += gm;
    }
}

template <int GM>
__device__ __forceinline__ void rect_decode(int t, int TM, int TN, int& ti, int& tj) {
    const int per_group = GM * TN;
    const int gidx = t / per_group;
    const int first = gidx * GM;
    const int gm = (TM - first < GM) ? (TM - first) : GM;
    const int r = t - gidx * per_group;
    ti = first + r % gm;
    tj = r / gm;
}

struct TileCoord {
    int bidx, ti, tj;
};

// A pointer that is the same in every lane, moved into scalar registers.
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const T*)(((unsigned long long)hi << 32) | lo);
}

// Every tile takes the same time, so without help all CUs reach their epilogues together and
// the write-back arrives at HBM as one burst per round while the MFMAs idle.  Delaying the
// first tile of XCD x by x/8 of a tile time keeps the eight XCDs out of phase for the rest of
// the launch, so each XCD's burst drains while the others compute.
__device__ __forceinline__ void stagger_first_round(const GemmArgs& g) {
    if (g.stagger > 0 && blockIdx.x < 256) {
        const long long wait = (long long)(blockIdx.x % XCD_COUNT) * g.stagger;
        const long long t0 = clock64();
        while (clock64() - t0 < wait) __builtin_amdgcn_s_sleep(32);
    }
}

template <int EPI>
__device__ __forceinline__ TileCoord decode_tile(const GemmArgs& g) {
    stagger_first_round(g);
    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    TileCoord tc;
    tc.bidx = logical / g.tiles_per_mat;
    const int t = logical - tc.bidx * g.tiles_per_mat;
    if (EPI == EPI_BX) rect_decode<4>(t, g.tiles_m, g.tiles_n, tc.ti, tc.tj);
    else tri_decode<4>(t, g.tiles_m, tc.ti, tc.tj);
    return tc;
}

// Lane (lane&31) owns column j; registers 4q..4q+3 are rows 8q + 4*(lane>>5) + 0..3.
template <int BM, int BN, int WGM, int WGN, int EPI>
__device__ __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc,
                                         f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32]) {
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN, hi = lane >> 5;
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bool diag = (EPI != EPI_BX) && (tc.ti == tc.tj);
    bf16_t* C = g.C ? g.C + tc.bidx * g.strideC : nullptr;
    bf16_t* Ct = g.Ct ? g.Ct + tc.bidx * g.strideCt : nullptr;
    const bf16_t* Et = g.Et ? g.Et + tc.bidx * g.strideEt : nullptr;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const long gj = n0 + wn * WTN + j * 32 + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const long gi = m0 + wm * WTM + i * 32 + q * 8 + hi * 4;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = rbf(acc[i][j][q * 4 + r]);
                if (EPI != EPI_SYRK) {
                    const bf16x4 e = *(const bf16x4*)(Et + gj * g.ldet + gi);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (EPI == EPI_SYMPOLY) v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + rbf(g.s1 * v[r]));
                        else v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + v[r]);
                    }
                }
                bf16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = f2bf(v[r]);
                if (diag) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (gi + r <= gj) {
                            C[(gi + r) * g.ldc + gj] = o[r];
                            C[gj * g.ldc + gi + r] = o[r];
                        }
                    }
                } else {
                    if (C) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) C[(gi + r) * g.ldc + gj] = o[r];
                    }
                    if (Ct) *(bf16x4*)(Ct + gj * g.ldct + gi) = o;
                }
            }
        }
    }
}

// The same epilogue staged through LDS (free once the main loop is over) so that global
// traffic is 16-byte vectors: the tile is kept as Tt[n][m] (n = local column, m = local row of
// the accumulator tile), row stride BM*2+16 bytes.  The elementwise source Et has exactly that
// orientation, so it is loaded into Tt with coalesced reads, each lane then replaces its own
// 8-byte pieces by the rounded results, and the tile leaves as rows of Ct (straight) and rows
// of C (gathered down the columns of Tt).  Diagonal tiles of the symmetric kernels write the
// full tile once: acc(i,j) and acc(j,i) are sums of the same exact products in the same order.
template <int BM, int BN>
constexpr int epilogue_lds_bytes() { return BN * (BM * 2 + 16); }

#ifdef EXP_TRACE_EPI
__device__ long long* g_epi_trace;
#define EPI_POINT(n) do { if (threadIdx.x == 0) g_epi_trace[(long)blockIdx.x * 8 + (n)] = clock64(); } while (0)
#else
#define EPI_POINT(n) do {} while (0)
#endif

template <int BM, int BN, int WGM, int WGN, int EPI>
__device__ __forceinline__ void epilogue_lds(const GemmArgs& g, const TileCoord& tc,
                                             f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32], unsigned char* smem) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int S = BM * 2 + 16;
    constexpr int CPR = BM / 8;  // 16-byte chunks per Tt row
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN, hi = lane >> 5;
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bool diag = (EPI != EPI_BX) && (tc.ti == tc.tj);
    bf16_t* C = g.C ? g.C + tc.bidx * g.strideC : nullptr;
    bf16_t* Ct = g.Ct ? g.Ct + tc.bidx * g.strideCt : nullptr;
    EPI_POINT(0);
    __syncthreads();  // every wave is done reading the operand stages
    EPI_POINT(1);
    if (EPI != EPI_SYRK) {
        const bf16_t* Et = g.Et + tc.bidx * g.strideEt + n0 * g.ldet + m0;
#pragma unroll 4
        for (int c = tid; c < BN * CPR; c += NT) {
            const int n = c / CPR, k = c % CPR;
            *(u32x4*)(smem + n * S + k * 16) = *(const u32x4*)(Et + (long)n * g.ldet + k * 8);
        }
        __syncthreads();
    }
    EPI_POINT(2);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int n = wn * WTN + j * 32 + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = wm * WTM + i * 32 + q * 8 + hi * 4;
                unsigned char* p = smem + n * S + m * 2;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = rbf(acc[i][j][q * 4 + r]);
                if (EPI != EPI_SYRK) {
                    const bf16x4 e = *(const bf16x4*)p;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (EPI == EPI_SYMPOLY) v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + rbf(g.s1 * v[r]));
                        else v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + v[r]);
                    }
                }
                bf16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = f2bf(v[r]);
                *(bf16x4*)p = o;
            }
        }
    }
    EPI_POINT(3);
    __syncthreads();
    EPI_POINT(4);
    if (Ct) {
        bf16_t* dst = Ct + n0 * g.ldct + m0;
#pragma unroll 4
        for (int c = tid; c < BN * CPR; c += NT) {
            const int n = c / CPR, k = c % CPR;
            *(u32x4*)(dst + (long)n * g.ldct + k * 8) = *(const u32x4*)(smem + n * S + k * 16);
        }
    }
    EPI_POINT(5);
    if (C && !diag) {
        bf16_t* dst = C + m0 * g.ldc + n0;
#pragma unroll 2
        for (int idx = tid; idx < BM * (BN / 8); idx += NT) {
            const int m = idx % BM, c = idx / BM;  // consecutive lanes walk down a column of C
            bf16x8 o;
#pragma unroll
            for (int r = 0; r < 8; ++r) o[r] = *(const bf16_t*)(smem + (c * 8 + r) * S + m * 2);
            *(bf16x8*)(dst + (long)m * g.ldc + c * 8) = o;
        }
    }
    EPI_POINT(6);
#ifdef EXP_TRACE_EPI
    __builtin_amdgcn_s_waitcnt(0x0F70);
    EPI_POINT(7);
#endif
}

// Epilogue with both output orientations coalesced.  Stage 1 (all waves): the elementwise
// source Et comes through LDS as Et[n][m] with 16-byte loads, each lane picks its 8-byte pieces
// and keeps the rounded results of all its fragments in registers.  Stage 2, one half of the
// columns at a time (LDS cannot hold both orientations of a whole tile): the owners drop their
// items into Tt[n][m] (the orientation of Ct) and T[m][n] (the orientation of C), and
// everybody copies whole rows out with 16-byte stores.
template <int BM, int BN>
constexpr int epilogue_lds2_bytes() {
    constexpr int halves = (BN / 2) * (BM * 2 + 16) + BM * (BN + 16), whole = BN * (BM * 2 + 16);
    return halves > whole ? halves : whole;
}

template <int BM, int BN, int WGM, int WGN, int EPI>
__device__ __forceinline__ void epilogue_lds2(const GemmArgs& g, const TileCoord& tc,
                                              f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32], unsigned char* smem) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int HN = BN / 2;             // columns per half
    constexpr int S1 = BM * 2 + 16;        // Tt row pitch (bytes)
    constexpr int S2 = HN * 2 + 16;        // T row pitch (bytes)
    constexpr int T_OFF = HN * S1;
    constexpr int CPR1 = BM / 8, CPR2 = HN / 8;  // 16-byte chunks per row
    constexpr int NL1 = HN * CPR1 / NT, NL2 = BM * CPR2 / NT;
    static_assert(WTN <= HN && HN % WTN == 0, "a wave's columns lie in one half");
    static_assert((HN * CPR1) % NT == 0 && (BM * CPR2) % NT == 0, "row copies divide evenly");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN, hi = lane >> 5;
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bool diag = (EPI != EPI_BX) && (tc.ti == tc.tj);
    bf16_t* C = (g.C && !diag) ? g.C + tc.bidx * g.strideC + m0 * g.ldc + n0 : nullptr;
    bf16_t* Ct = g.Ct ? g.Ct + tc.bidx * g.strideCt + n0 * g.ldct + m0 : nullptr;
    unsigned char* Tt = smem;
    unsigned char* T = smem + T_OFF;

    // Stage 1, every wave at once: results of all fragments, rounded, packed 4 rows per item.
    bf16x4 res[FM][FN][4];
    EPI_POINT(0);
    __syncthreads();  // the operand stages are no longer read
    EPI_POINT(1);
    if (EPI != EPI_SYRK) {
        // the whole Et tile goes through LDS as Et[n][m] (pitch S1) with coalesced 16-byte loads
        const bf16_t* Et = g.Et + tc.bidx * g.strideEt + n0 * g.ldet + m0;
        constexpr int NLE = BN * CPR1 / NT;
#pragma unroll
        for (int b = 0; b < NLE; b += 16) {
            u32x4 ev[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int c = tid + (b + u) * NT, n = c / CPR1, k = c % CPR1;
                if (b + u < NLE) ev[u] = *(const u32x4*)(Et + (long)n * g.ldet + k * 8);
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int c = tid + (b + u) * NT, n = c / CPR1, k = c % CPR1;
                if (b + u < NLE) *(u32x4*)(smem + n * S1 + k * 16) = ev[u];
            }
        }
        __syncthreads();
    }
    EPI_POINT(2);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int n = wn * WTN + j * 32 + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = wm * WTM + i * 32 + q * 8 + hi * 4;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = rbf(acc[i][j][q * 4 + r]);
                if (EPI != EPI_SYRK) {
                    const bf16x4 e = *(const bf16x4*)(smem + n * S1 + m * 2);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (EPI == EPI_SYMPOLY) v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + rbf(g.s1 * v[r]));
                        else v[r] = rbf(rbf(g.s0 * bf2f(e[r])) + v[r]);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) res[i][j][q][r] = f2bf(v[r]);
            }
        }
    }
    EPI_POINT(3);
    // Stage 2, one half of the columns at a time: owners drop their items into Tt and T, then
    // everybody copies whole rows out.
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        __syncthreads();  // Et tile (h == 0) or the previous half (h == 1) is no longer read
        if ((wn * WTN) / HN == h) {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int n = (wn * WTN) % HN + j * 32 + (lane & 31);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int m = wm * WTM + i * 32 + q * 8 + hi * 4;
                        if (Ct) *(bf16x4*)(Tt + n * S1 + m * 2) = res[i][j][q];
                        if (C) {
#pragma unroll
                            for (int r = 0; r < 4; ++r) *(bf16_t*)(T + (m + r) * S2 + n * 2) = res[i][j][q][r];
                        }
                    }
                }
            }
        }
        __syncthreads();
        if (h == 0) EPI_POINT(4);
        if (Ct) {
#pragma unroll
            for (int u = 0; u < NL1; ++u) {
                const int c = tid + u * NT, n = c / CPR1, k = c % CPR1;
                *(u32x4*)(Ct + (long)(h * HN + n) * g.ldct + k * 8) = *(const u32x4*)(Tt + n * S1 + k * 16);
            }
        }
        if (h == 0) EPI_POINT(5);
        if (C) {
#pragma unroll
            for (int u = 0; u < NL2; ++u) {
                const int c = tid + u * NT, m = c / CPR2, k = c % CPR2;
                *(u32x4*)(C + (long)m * g.ldc + h * HN + k * 8) = *(const u32x4*)(T + m * S2 + k * 16);
            }
        }
        if (h == 0) EPI_POINT(6);
        if (h == 1) EPI_POINT(7);
    }
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// Epilogue with one LDS copy of the tile and both output orientations written as 16-byte
// vectors.  The tile lives in LDS as Tt[n][m] (n = local column, m = local row of the
// accumulator tile), the orientation of Ct and of the elementwise source Et: Et is loaded
// into it with coalesced reads, every lane replaces its own 8-byte pieces (4 consecutive m of
// one n, exactly what an accumulator lane holds) by the rounded results, and after one barrier
// rows of Tt leave as rows of Ct, while rows of C are gathered with ds_read_b64_tr_b16: in a
// group of 16 lanes, lane i receives element i%4 of the 8-byte pieces addressed by lanes
// i/4, 4+i/4, 8+i/4, 12+i/4, so pointing lane j at row n0+j/4, pieces m0+4*(j%4).. hands lane
// i the four values Tt[n0..n0+3][m0+i], i.e. 8 bytes of row m0+i of C.
#ifndef EPI3_PITCH_PAD
#define EPI3_PITCH_PAD 16
#endif
template <int BM, int BN>
constexpr int epilogue_lds3_bytes() { return BN * (BM * 2 + EPI3_PITCH_PAD); }

typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ s16x4 lds_read_tr16(const unsigned char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(lds_void_ptr)p);
}

template <int BM, int BN, int WGM, int WGN, int EPI>
__device__ __forceinline__ void epilogue_lds3(const GemmArgs& g, const TileCoord& tc,
                                              f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32], unsigned char* smem) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int S = BM * 2 + EPI3_PITCH_PAD;  // Tt row pitch (bytes)
    constexpr int CPR = BM / 8;                 // 16-byte chunks per Tt row
    constexpr int NLE = BN * CPR / NT;          // 16-byte chunks per thread for a whole tile
    static_assert((BN * CPR) % NT == 0, "even split");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN, hi = lane >> 5;
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bool diag = (EPI != EPI_BX) && (tc.ti == tc.tj);
    bf16_t* C = (g.C && !diag) ? g.C + tc.bidx * g.strideC + m0 * g.ldc + n0 : nullptr;
    bf16_t* Ct = g.Ct ? g.Ct + tc.bidx * g.strideCt + n0 * g.ldct + m0 : nullptr;
    EPI_POINT(0);
    __syncthreads();  // the operand stages are no longer read
    EPI_POINT(1);
    if (EPI != EPI_SYRK) {
        const bf16_t* Et = g.Et + tc.bidx * g.strideEt + n0 * g.ldet + m0;
#pragma unroll
        for (int b = 0; b < NLE; b += 16) {
            u32x4 ev[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int c = tid + (b + u) * NT, n = c / CPR, k = c % CPR;
                if (b + u < NLE) ev[u] = *(const u32x4*)(Et + (long)n * g.ldet + k * 8);
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int c = tid + (b + u) * NT, n = c / CPR, k = c % CPR;
                if (b + u < NLE) *(u32x4*)(smem + n * S + k * 16) = ev[u];
            }
        }
        __syncthreads();
    }
    EPI_POINT(2);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        // all LDS reads of a fragment row first: in one loop the compiler must assume that each
        // write may alias the next read and the chain becomes one LDS latency per item
        bf16x4 e[FN][4];
        if (EPI != EPI_SYRK) {
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    e[j][q] = *(const bf16x4*)(smem + (wn * WTN + j * 32 + (lane & 31)) * S +
                                               (wm * WTM + i * 32 + q * 8 + hi * 4) * 2);
        }
        bf16x4 o[FN][4];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = rbf(acc[i][j][q * 4 + r]);
                    if (EPI == EPI_SYMPOLY) v = rbf(rbf(g.s0 * bf2f(e[j][q][r])) + rbf(g.s1 * v));
                    if (EPI == EPI_BX) v = rbf(rbf(g.s0 * bf2f(e[j][q][r])) + v);
                    o[j][q][r] = f2bf(v);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *(bf16x4*)(smem + (wn * WTN + j * 32 + (lane & 31)) * S + (wm * WTM + i * 32 + q * 8 + hi * 4) * 2) =
                    o[j][q];
    }
    EPI_POINT(3);
    __syncthreads();
    EPI_POINT(4);
    if (Ct) {
#pragma unroll
        for (int u = 0; u < NLE; ++u) {
            const int c = tid + u * NT, n = c / CPR, k = c % CPR;
            *(u32x4*)(Ct + (long)n * g.ldct + k * 8) = *(const u32x4*)(smem + n * S + k * 16);
        }
    }
    EPI_POINT(5);
    if (C) {
        // lane j = 4r+s of a group addresses row n0 + 8s + r (then + 4), pieces m = 4c..4c+3: lane i = 4s+e
        // receives Tt[n0+8s .. n0+8s+7][4c+e], 16 bytes of row 4c+e of C.  A group writes 4 rows x 64
        // contiguous bytes and the four groups of a wave sit side by side: 4 rows x 256 bytes per store.
        const int grp = lane >> 4, i16 = lane & 15;
        const unsigned char* src = smem + ((i16 & 3) * 8 + (i16 >> 2) + grp * 32) * S;
        bf16_t* dst = C + (long)(i16 & 3) * g.ldc + grp * 32 + (i16 >> 2) * 8;
        constexpr int NSTRIP = BN / 128, NQUAD = BM / 4, NW = NT / 64;
        constexpr int NUNIT = NSTRIP * NQUAD / NW;
        static_assert(BN % 128 == 0 && (NSTRIP * NQUAD) % NW == 0, "whole 128-column strips per wave");
#pragma unroll 8
        for (int u = 0; u < NUNIT; ++u) {
            const int wu = wave + u * NW, strip = wu % NSTRIP, c = wu / NSTRIP;
            const unsigned char* q = src + strip * 128 * S + c * 8;
            const s16x4 lo = lds_read_tr16(q), hi4 = lds_read_tr16(q + 4 * S);
            short __attribute__((ext_vector_type(8))) o = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            *(decltype(o)*)(dst + (long)c * 4 * g.ldc + strip * 128) = o;
        }
    }
    EPI_POINT(6);
#ifdef EXP_TRACE_EPI
    __builtin_amdgcn_s_waitcnt(0x0F70);
    EPI_POINT(7);
#endif
}

#ifdef EXP_EPI_LDS2
#define EPILOGUE epilogue_lds2
#define EPILOGUE_BYTES epilogue_lds2_bytes
#else
#define EPILOGUE epilogue_lds3
#define EPILOGUE_BYTES epilogue_lds3_bytes
#endif

// ---- variant 1: global -> registers -> LDS, two LDS stages, one barrier per k-tile -------
template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_kernel(const GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE = A_BYTES + B_BYTES;
    constexpr int CA = BM * 8 / NT, CB = BN * 8 / NT;  // 16-byte chunks per thread per k-tile
    constexpr int RSTEP = NT / 8;                      // rows between a thread's chunks
    static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tiling");
    static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0 && RSTEP % 16 == 0, "staging");
    static_assert(EPI == EPI_BX || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bf16_t* Pb = g.P + tc.bidx * g.strideP + m0 * g.ldp;
    const bf16_t* Qb = g.Q + tc.bidx * g.strideQ + n0 * g.ldq;

    const int lrow = tid >> 3, lc = tid & 7;
    const bf16_t* pa = Pb + (long)lrow * g.ldp + lc * 8;
    const bf16_t* pb = Qb + (long)lrow * g.ldq + lc * 8;
    // 16-byte chunk c of row r lives at r*128 + ((c ^ ((r>>1)&7)) << 4): the 16 rows one
    // ds_read_b128 phase touches then cover all 64 banks once.
    const int lds_w = lrow * ROW_BYTES + ((lc ^ ((lrow >> 1) & 7)) << 4);
    u32x4 ra[CA], rb[CB];

    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < CA; ++i) ra[i] = *(const u32x4*)(pa + (long)i * RSTEP * g.ldp + k0);
#pragma unroll
        for (int i = 0; i < CB; ++i) rb[i] = *(const u32x4*)(pb + (long)i * RSTEP * g.ldq + k0);
    };
    auto lstore = [&](int stage) {
        unsigned char* s = smem + stage * STAGE + lds_w;
#pragma unroll
        for (int i = 0; i < CA; ++i) *(u32x4*)(s + i * RSTEP * ROW_BYTES) = ra[i];
#pragma unroll
        for (int i = 0; i < CB; ++i) *(u32x4*)(s + A_BYTES + i * RSTEP * ROW_BYTES) = rb[i];
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int sw = (lane >> 1) & 7, hi = lane >> 5;
    const int a_off = (wm * WTM + (lane & 31)) * ROW_BYTES;
    const int b_off = A_BYTES + (wn * WTN + (lane & 31)) * ROW_BYTES;

    const int nk = g.kdim / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) gload((kt + 1) * BK);
        const unsigned char* st = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int co = (((ks << 1) | hi) ^ sw) << 4;
            bf16x8 af[FM], bq[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) af[i] = *(const bf16x8*)(st + a_off + i * 32 * ROW_BYTES + co);
#pragma unroll
            for (int j = 0; j < FN; ++j) bq[j] = *(const bf16x8*)(st + b_off + j * 32 * ROW_BYTES + co);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bq[j], acc[i][j], 0, 0, 0);
        }
        if (more) lstore((kt + 1) & 1);
        __syncthreads();
    }
#ifdef EXP_NO_EPI
    float ssum = 0.f;
    for (int i = 0; i < FM; ++i) for (int j = 0; j < FN; ++j) for (int r = 0; r < 16; ++r) ssum += acc[i][j][r];
    if (ssum == 123.456f) g.C[threadIdx.x] = f2bf(ssum);
#elif defined(EXP_DIRECT_EPI)
    epilogue<BM, BN, WGM, WGN, EPI>(g, tc, acc);
#else
    EPILOGUE<BM, BN, WGM, WGN, EPI>(g, tc, acc, smem);
#endif
}

// ---- variant 2: global -> LDS directly (global_load_lds_dwordx4), two LDS stages ---------
// One wave-level load instruction fills 1 KB of LDS in lane order, i.e. 8 rows of the tile;
// the XOR swizzle is applied on the global side: lane L fetches the chunk whose swizzled
// position is L&7.  Loads for k-tile t+2 are issued as soon as every wave has finished
// reading k-tile t, and are waited for (vmcnt) one whole tile of MFMA work later.
typedef const __attribute__((address_space(1))) void* glb_void_ptr;

#define WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)
// s_waitcnt with only vmcnt set: vmcnt is split over bits [3:0] and [15:14] (N < 64)
#define WAIT_VM(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))

template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_dlds_kernel(const GemmArgs g) {
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;  // 1 KB load instructions per wave per k-tile
    constexpr int KS = BK / 16;
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "dma split");
    static_assert(LA + LB < 64, "vmcnt immediate");
    static_assert(EPI == EPI_BX || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bf16_t* Pb = g.P + tc.bidx * g.strideP + m0 * g.ldp;
    const bf16_t* Qb = g.Q + tc.bidx * g.strideQ + n0 * g.ldq;

    // Wave w fills rows [w*8*LA, +8*LA) of A and [w*8*LB, +8*LB) of B, 8 rows per instruction.
    // Row r keeps chunk c at position c ^ ((r>>1)&7); lane L lands on position L&7 of row
    // r = 8*group + (L>>3), so it fetches chunk (L&7) ^ (4*(group&1) + (L>>4)).
    const int drow = lane >> 3;
    const bf16_t* pa = Pb + (long)(wave * 8 * LA + drow) * g.ldp;
    const bf16_t* pb = Qb + (long)(wave * 8 * LB + drow) * g.ldq;
    const int lds_a = wave * 8 * LA * ROW_BYTES;
    const int lds_b = A_BYTES + wave * 8 * LB * ROW_BYTES;
    const int ch_even = ((lane & 7) ^ (drow >> 1)) * 8, ch_odd = ((lane & 7) ^ (4 | (drow >> 1))) * 8;

    auto issue = [&](int stage, int k0) {
        unsigned char* s = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const int ch = ((wave * LA + i) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pa + (long)i * 8 * g.ldp + k0 + ch),
                                             (lds_void_ptr)(s + lds_a + i * 8 * ROW_BYTES), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            const int ch = ((wave * LB + i) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pb + (long)i * 8 * g.ldq + k0 + ch),
                                             (lds_void_ptr)(s + lds_b + i * 8 * ROW_BYTES), 16, 0, 0);
        }
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int sw = (lane >> 1) & 7, hi = lane >> 5;
    const int a_off = (wm * WTM + (lane & 31)) * ROW_BYTES;
    const int b_off = A_BYTES + (wn * WTN + (lane & 31)) * ROW_BYTES;

    const int nk = g.kdim / BK;
#ifdef EXP_DEPTH
    for (int d = 0; d < EXP_DEPTH; ++d) issue(d & 1, d * BK);
#else
    issue(0, 0);
    if (nk > 1) issue(1, BK);
#endif
    for (int kt = 0; kt < nk; ++kt) {
        // k-tile kt has landed once at most the next tile's loads are still in flight
#ifdef EXP_DEPTH
        if (kt + EXP_DEPTH <= nk) WAIT_VM((EXP_DEPTH - 1) * (LA + LB));
        else WAIT_VM(0);
#elif !defined(EXP_NO_DMA)
        if (kt + 1 < nk) WAIT_VM(LA + LB);
        else WAIT_VM(0);
#endif
#ifndef EXP_NO_BARRIER
        __builtin_amdgcn_s_barrier();
#endif
        asm volatile("" ::: "memory");
        const unsigned char* st = smem + (kt & 1) * STAGE;
        bf16x8 af[2][FM], bq[2][FN];
        auto lfrag = [&](int buf, int ks) {
            const int co = (((ks << 1) | hi) ^ sw) << 4;
#pragma unroll
            for (int i = 0; i < FM; ++i) af[buf][i] = *(const bf16x8*)(st + a_off + i * 32 * ROW_BYTES + co);
#pragma unroll
            for (int j = 0; j < FN; ++j) bq[buf][j] = *(const bf16x8*)(st + b_off + j * 32 * ROW_BYTES + co);
        };
        lfrag(0, 0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            // the LDS reads of the next k-step go out before this k-step's MFMAs start, so
            // their latency hides behind FM*FN MFMAs; the fences keep the scheduler from
            // sinking them back next to their uses
#ifndef EXP_NO_LDS
            if (ks + 1 < KS) lfrag((ks + 1) & 1, ks + 1);
#endif
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#ifndef EXP_NO_MFMA
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bq[ks & 1][j], acc[i][j], 0, 0, 0);
#else
                    acc[i][j][0] += (float)af[ks & 1][i][0] * (float)bq[ks & 1][j][0];
#endif
            __builtin_amdgcn_sched_barrier(0);
        }
        if (kt + 2 < nk) {
            // every wave must be done reading this stage before new data may land in it
            WAIT_LGKM0();
            asm volatile("" ::: "memory");
#ifndef EXP_NO_BARRIER
            __builtin_amdgcn_s_barrier();
#endif
#ifdef EXP_DEPTH
            if (kt + EXP_DEPTH < nk) issue((kt + EXP_DEPTH) & 1, (kt + EXP_DEPTH) * BK);
#elif !defined(EXP_NO_DMA)
            issue(kt & 1, (kt + 2) * BK);
#endif
        }
    }
#ifdef EXP_NO_EPI
    float ssum = 0.f;
    for (int i = 0; i < FM; ++i) for (int j = 0; j < FN; ++j) for (int r = 0; r < 16; ++r) ssum += acc[i][j][r];
    if (ssum == 123.456f) g.C[threadIdx.x] = f2bf(ssum);
#elif defined(EXP_DIRECT_EPI)
    epilogue<BM, BN, WGM, WGN, EPI>(g, tc, acc);
#else
    EPILOGUE<BM, BN, WGM, WGN, EPI>(g, tc, acc, smem);
#endif
}

// ---- variant 3: direct global -> LDS feed, software pipelined, one barrier per k-tile -----
// Per k-tile a wave issues FM*FN*4 MFMAs, (FM+FN)*4 LDS fragment reads and LA+LB 1 KB loads.
// Every non-MFMA instruction is placed between two MFMAs so that it issues in their shadow:
//   k-steps 0..2 : MFMAs of step s interleaved with the fragment reads of step s+1;
//   k-step 3     : the wave has now read everything it needs from this stage, so it waits
//                  for its own loads of the next k-tile, crosses the one barrier, and then
//                  interleaves the last MFMAs with the loads of k-tile t+2 (into the stage just
//                  released) and with the fragment reads of step 0 of k-tile t+1.
// The fences (sched_barrier) pin that order; without them the scheduler sinks every LDS read
// next to its first use and the MFMA pipe idles for an LDS round trip per k-step.
template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_pipe_kernel(const GemmArgs g) {
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
    constexpr int KS = BK / 16;
    constexpr int NMF = FM * FN, NRD = FM + FN, NLD = LA + LB;
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "dma split");
    static_assert(EPI == EPI_BX || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
#ifdef EXP_SAME_TILE
    const bf16_t* Pb = g.P;
    const bf16_t* Qb = g.Q;
#else
    const bf16_t* Pb = g.P + tc.bidx * g.strideP + m0 * g.ldp;
    const bf16_t* Qb = g.Q + tc.bidx * g.strideQ + n0 * g.ldq;
#endif

    const int drow = lane >> 3;
    const bf16_t* pa = Pb + (long)(wave * 8 * LA + drow) * g.ldp;
    const bf16_t* pb = Qb + (long)(wave * 8 * LB + drow) * g.ldq;
    const int lds_a = wave * 8 * LA * ROW_BYTES;
    const int lds_b = A_BYTES + wave * 8 * LB * ROW_BYTES;
    const int ch_even = ((lane & 7) ^ (drow >> 1)) * 8, ch_odd = ((lane & 7) ^ (4 | (drow >> 1))) * 8;

    // load instruction n (0..NLD-1) of a k-tile: A rows first, then B rows
    auto issue_one = [&](int n, int stage, int k0) {
        unsigned char* s = smem + stage * STAGE;
        if (n < LA) {
            const int ch = ((wave * LA + n) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pa + (long)n * 8 * g.ldp + k0 + ch),
                                             (lds_void_ptr)(s + lds_a + n * 8 * ROW_BYTES), 16, 0, 0);
        } else {
            const int i = n - LA;
            const int ch = ((wave * LB + i) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pb + (long)i * 8 * g.ldq + k0 + ch),
                                             (lds_void_ptr)(s + lds_b + i * 8 * ROW_BYTES), 16, 0, 0);
        }
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int sw = (lane >> 1) & 7, hi = lane >> 5;
    const int a_off = (wm * WTM + (lane & 31)) * ROW_BYTES;
    const int b_off = A_BYTES + (wn * WTN + (lane & 31)) * ROW_BYTES;

    bf16x8 fr[2][NRD];  // fragment double buffer: [0..FM) rows of P, [FM..NRD) rows of Q
    auto read_one = [&](int buf, int n, const unsigned char* st, int ks) {
        const int co = (((ks << 1) | hi) ^ sw) << 4;
        if (n < FM) fr[buf][n] = *(const bf16x8*)(st + a_off + n * 32 * ROW_BYTES + co);
        else fr[buf][n] = *(const bf16x8*)(st + b_off + (n - FM) * 32 * ROW_BYTES + co);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / FN, j = idx % FN;
#ifdef EXP_NO_MFMA
        acc[i][j][0] += (float)fr[buf][i][0] * (float)fr[buf][FM + j][0];
#else
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[buf][i], fr[buf][FM + j], acc[i][j], 0, 0, 0);
#endif
    };

    const int nk = g.kdim / BK;
#pragma unroll
    for (int n = 0; n < NLD; ++n) issue_one(n, 0, 0);
    if (nk > 1) {
#pragma unroll
        for (int n = 0; n < NLD; ++n) issue_one(n, 1, BK);
        WAIT_VM(NLD);
    } else {
        WAIT_VM(0);
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < NRD; ++n) read_one(0, n, smem, 0);

#ifdef EXP_TRACE
    long long* trace = (long long*)g.Ct + (long)blockIdx.x * 8192 + (threadIdx.x >> 6) * 1024;
    int tn = 0;
#define TRACE_POINT() do { if (lane == 0 && tn < 1000) trace[tn] = clock64(); ++tn; } while (0)
#else
#define TRACE_POINT() do {} while (0)
#endif
    for (int kt = 0; kt < nk; ++kt) {
        const unsigned char* st = smem + (kt & 1) * STAGE;
        const unsigned char* stn = smem + ((kt + 1) & 1) * STAGE;
        TRACE_POINT();
#pragma unroll
        for (int ks = 0; ks < KS - 1; ++ks) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int idx = 0; idx < NMF; ++idx) {
                mfma_one(ks & 1, idx);
                if (idx < NRD) {
                    __builtin_amdgcn_sched_barrier(0);
                    read_one((ks + 1) & 1, idx, st, ks + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // Fragments of the last k-step are in: this wave is done with stage kt&1.  The tail is
        // branch free: past the end it re-loads the last k-tile into a stage nobody reads and
        // pre-reads fragments nobody uses, which costs 2 of nk loads and keeps the MFMAs in
        // one basic block.
        TRACE_POINT();
        WAIT_LGKM0();
        WAIT_VM(0);  // its loads of k-tile kt+1 (the only ones in flight) have landed
        TRACE_POINT();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        TRACE_POINT();
        const int k2 = (kt + 2 < nk ? kt + 2 : nk - 1) * BK;
        constexpr int PER = (NLD + NRD + NMF - 1) / NMF;  // loads and reads per MFMA slot
#pragma unroll
        for (int idx = 0; idx < NMF; ++idx) {
            mfma_one((KS - 1) & 1, idx);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < PER; ++u) {
                const int o = idx * PER + u;
                if (o < NRD) read_one(KS & 1, o, stn, 0);
                else if (o < NRD + NLD) issue_one(o - NRD, kt & 1, k2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    WAIT_VM(0);  // the dummy loads of the last two tails must not land in the epilogue's tile
#ifdef EXP_NO_EPI
    float ssum = 0.f;
    for (int i = 0; i < FM; ++i) for (int j = 0; j < FN; ++j) for (int r = 0; r < 16; ++r) ssum += acc[i][j][r];
    if (ssum == 123.456f) g.C[threadIdx.x] = f2bf(ssum);
#else
    EPILOGUE<BM, BN, WGM, WGN, EPI>(g, tc, acc, smem);
#endif
}

// ---- variant 4: 32-wide k-tiles in four LDS stages ----------------------------------------
// The L1 -> LDS path moves 64 B/clk per CU, so feeding a 256x256 tile keeps it busy half of
// the time; when the loads of a k-tile are issued in one burst (variant 3, two stages) every
// wave of the CU queues on the one address path and its MFMAs starve behind the blocked
// load.  Four stages of 32 columns leave a stage free for a whole k-tile, so the loads are
// spread evenly: 4 per 16 MFMAs.  Timeline of wave w for k-tile t (stage t&3, two k-steps):
//   phase A: MFMAs of k-step 0 | fragment reads of k-step 1 | B-half loads of k-tile t+3
//   wait own reads; wait own loads of k-tile t+1; barrier   (stage t&3 is now free)
//   phase B: MFMAs of k-step 1 | fragment reads of k-tile t+1 step 0 | A-half loads of k-tile t+4
// LDS rows are 64 B (4 chunks); chunk c of row r sits at position c ^ ((r>>2)&3).
template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_pipe4_kernel(const GemmArgs g) {
    constexpr int NW = WGM * WGN;
    constexpr int BK4 = 32, ROWB = 64, NST = 4;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 16 / NW, LB = BN / 16 / NW;  // 1 KB loads (16 rows) per wave per k-tile
    constexpr int NMF = FM * FN, NRD = FM + FN;
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "dma split");
    // Slot plan of one phase (NMF MFMAs, NRD fragment reads, L loads): the loads sit behind every
    // (NMF/L)-th MFMA so that the four waves of the CU, which run in lockstep, hand the one L1
    // address path 4 loads (64 cycles of work) per NMF/L MFMAs instead of 16 back to back; the
    // reads fill the other slots from the front.
    constexpr int LSP_A = NMF / LB > 0 ? NMF / LB : 1, LSP_B = NMF / LA > 0 ? NMF / LA : 1;
    constexpr int RPS_A = (NRD + (NMF - NMF / LSP_A) - 1) / (NMF - NMF / LSP_A > 0 ? NMF - NMF / LSP_A : 1);
    constexpr int RPS_B = (NRD + (NMF - NMF / LSP_B) - 1) / (NMF - NMF / LSP_B > 0 ? NMF - NMF / LSP_B : 1);
    static_assert(EPI == EPI_BX || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
    const bf16_t* Pb = g.P + tc.bidx * g.strideP + m0 * g.ldp;
    const bf16_t* Qb = g.Q + tc.bidx * g.strideQ + n0 * g.ldq;

    // lane L of a load lands on row L>>2, position L&3 and so fetches chunk (L&3)^((L>>4)&3)
    const int drow = lane >> 2;
    const int dch = ((lane & 3) ^ ((lane >> 4) & 3)) * 8;
    const bf16_t* pa = Pb + (long)(wave * 16 * LA + drow) * g.ldp + dch;
    const bf16_t* pb = Qb + (long)(wave * 16 * LB + drow) * g.ldq + dch;
    const int lds_a = wave * 16 * LA * ROWB;
    const int lds_b = A_BYTES + wave * 16 * LB * ROWB;
    const int nk = g.kdim / BK4;

    auto issue_a = [&](int n, int kt) {  // kt may run past the end: re-load the last k-tile
        const int kk = (kt < nk ? kt : nk - 1) * BK4;
        __builtin_amdgcn_global_load_lds((glb_void_ptr)(pa + (long)n * 16 * g.ldp + kk),
                                         (lds_void_ptr)(smem + (kt & 3) * STAGE + lds_a + n * 16 * ROWB), 16, 0, 0);
    };
    auto issue_b = [&](int n, int kt) {
        const int kk = (kt < nk ? kt : nk - 1) * BK4;
        __builtin_amdgcn_global_load_lds((glb_void_ptr)(pb + (long)n * 16 * g.ldq + kk),
                                         (lds_void_ptr)(smem + (kt & 3) * STAGE + lds_b + n * 16 * ROWB), 16, 0, 0);
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int sw = (lane >> 2) & 3, hi = lane >> 5;
    const int a_off = (wm * WTM + (lane & 31)) * ROWB;
    const int b_off = A_BYTES + (wn * WTN + (lane & 31)) * ROWB;

    bf16x8 fr[2][NRD];
    auto read_one = [&](int buf, int n, const unsigned char* st, int ks) {
        const int co = (((ks << 1) | hi) ^ sw) << 4;
        if (n < FM) fr[buf][n] = *(const bf16x8*)(st + a_off + n * 32 * ROWB + co);
        else fr[buf][n] = *(const bf16x8*)(st + b_off + (n - FM) * 32 * ROWB + co);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / FN, j = idx % FN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[buf][i], fr[buf][FM + j], acc[i][j], 0, 0, 0);
    };

    // prologue: k-tiles 0..2 and the A half of k-tile 3
#pragma unroll
    for (int t = 0; t < 3; ++t) {
#pragma unroll
        for (int n = 0; n < LA; ++n) issue_a(n, t);
#pragma unroll
        for (int n = 0; n < LB; ++n) issue_b(n, t);
    }
#pragma unroll
    for (int n = 0; n < LA; ++n) issue_a(n, 3);
    WAIT_VM(2 * (LA + LB) + LA);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < NRD; ++n) read_one(0, n, smem, 0);

#ifdef EXP_TRACE
    long long* trace = (long long*)g.Ct + (long)blockIdx.x * 8192 + (threadIdx.x >> 6) * 1024;
    int tn = 0;
#endif
    for (int kt = 0; kt < nk; ++kt) {
        const unsigned char* st = smem + (kt & 3) * STAGE;
        const unsigned char* stn = smem + ((kt + 1) & 3) * STAGE;
        TRACE_POINT();
        // phase A
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int idx = 0; idx < NMF; ++idx) {
            mfma_one(0, idx);
            __builtin_amdgcn_sched_barrier(0);
            if ((idx + 1) % LSP_A == 0) {
#ifndef EXP4_NO_DMA
                if (idx / LSP_A < LB) issue_b(idx / LSP_A, kt + 3);
#endif
            } else {
#ifndef EXP4_NO_RD
                const int r0 = (idx - idx / LSP_A) * RPS_A;
#pragma unroll
                for (int u = 0; u < RPS_A; ++u)
                    if (r0 + u < NRD) read_one(1, r0 + u, st, 1);
#endif
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // own reads of this stage are complete, own loads of k-tile kt+1 have landed
        TRACE_POINT();
        WAIT_LGKM0();
#ifndef EXP4_NO_DMA
        WAIT_VM(2 * (LA + LB));
#endif
        TRACE_POINT();
        asm volatile("" ::: "memory");
#ifndef EXP4_NO_BAR
        __builtin_amdgcn_s_barrier();
#endif
        asm volatile("" ::: "memory");
        TRACE_POINT();
        // phase B
#pragma unroll
        for (int idx = 0; idx < NMF; ++idx) {
            mfma_one(1, idx);
            __builtin_amdgcn_sched_barrier(0);
            if ((idx + 1) % LSP_B == 0) {
#ifndef EXP4_NO_DMA
                if (idx / LSP_B < LA) issue_a(idx / LSP_B, kt + 4);
#endif
            } else {
#ifndef EXP4_NO_RD
                const int r0 = (idx - idx / LSP_B) * RPS_B;
#pragma unroll
                for (int u = 0; u < RPS_B; ++u)
                    if (r0 + u < NRD) read_one(0, r0 + u, stn, 0);
#endif
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    WAIT_VM(0);  // the loads issued past the end must not land in the epilogue's tile
#ifdef EXP_NO_EPI
    float ssum = 0.f;
    for (int i = 0; i < FM; ++i) for (int j = 0; j < FN; ++j) for (int r = 0; r < 16; ++r) ssum += acc[i][j][r];
    if (ssum == 123.456f) g.C[threadIdx.x] = f2bf(ssum);
#else
    EPILOGUE<BM, BN, WGM, WGN, EPI>(g, tc, acc, smem);
#endif
}

// ---- variant 5: eight waves in two groups that alternate between memory and MFMA phases ----
// Every wave runs the same loop  { M(t): read its fragments of k-tile t from LDS, issue its
// share of the loads of k-tile t+3, wait;  barrier;  C(t): FM*FN*2 MFMAs;  barrier }  over
// 32-column k-tiles in four LDS stages, but waves 4..7 enter it one barrier later than waves
// 0..3.  Wave w and wave w+4 share a SIMD, so at any time one of them is issuing nothing but
// MFMAs from registers while the other does all the LDS and address-path work and absorbs the
// waits; the barrier is crossed when the MFMA wave has issued its last MFMA.
// Timeline (phase p between two barriers): group 0 runs M(t) in p=2t and C(t) in p=2t+1,
// group 1 runs M(t) in p=2t+1 and C(t) in p=2t+2.  Stage t&3 is last read in p=2t+1, the
// loads of k-tile t+4 into it are issued in p=2t+2 / 2t+3, each wave waits for its own at the
// end of its M phase two k-tiles later (p=2t+6 / 2t+7), and k-tile t+4 is first read in p=2t+8.
template <int BM, int BN, int WGM, int WGN, int EPI, int NST>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_pp_kernel(const GemmArgs g) {
    constexpr int NW = WGM * WGN;
    constexpr int BK4 = 32, ROWB = 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 16 / NW, LB = BN / 16 / NW;
    constexpr int NLD = LA + LB;
    static_assert(NW == 8, "two groups of four waves, one of each per SIMD");
    static_assert(NST == 4 || NST == 5, "four or five LDS stages");
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "dma split");
    static_assert(EPI == EPI_BX || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    const long m0 = (long)tc.ti * BM, n0 = (long)tc.tj * BN;
#ifdef EXPP_SAME_TILE
    const bf16_t* Pb = uniform_ptr(g.P);
    const bf16_t* Qb = uniform_ptr(g.Q);
#else
    const bf16_t* Pb = uniform_ptr(g.P + tc.bidx * g.strideP + m0 * g.ldp);
    const bf16_t* Qb = uniform_ptr(g.Q + tc.bidx * g.strideQ + n0 * g.ldq);
#endif

    // Loads: a wave-uniform base pointer (advanced along k with scalar adds) plus a 32-bit byte
    // offset per lane, so that no vector ALU instruction is needed per load: in the memory phase
    // every VALU instruction would queue behind the sibling wave's MFMAs.
    const int drow = lane >> 2;
    const int dch = ((lane & 3) ^ ((lane >> 4) & 3)) * 8;
    unsigned offa[LA], offb[LB];
#pragma unroll
    for (int n = 0; n < LA; ++n) offa[n] = (unsigned)(((wave * 16 * LA + n * 16 + drow) * (long)g.ldp + dch) * 2);
#pragma unroll
    for (int n = 0; n < LB; ++n) offb[n] = (unsigned)(((wave * 16 * LB + n * 16 + drow) * (long)g.ldq + dch) * 2);
    const int lds_a = wave * 16 * LA * ROWB;
    const int lds_b = A_BYTES + wave * 16 * LB * ROWB;
    const int nk = g.kdim / BK4;

    // global_load_lds_dwordx4 with a scalar base and a 32-bit vector offset; the LDS destination
    // of lane 0 goes through M0 (the wave's 64 lanes fill 1 KB from there in lane order).
#ifdef EXPP_TO_VGPR
    f32x4 sink[4] = {};
    int sink_i = 0;
    auto dma = [&](const char* base, unsigned voff, unsigned lds_byte) {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sink[0]) : "v"(voff), "s"(base) : "memory");
    };
#else
#ifdef EXPP_DWORD
    auto dma = [&](const char* base, unsigned voff, unsigned lds_byte) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                     :
                     : "s"(lds_byte), "v"(voff), "s"(base)
                     : "memory");
    };
#else
    auto dma = [&](const char* base, unsigned voff, unsigned lds_byte) {
#ifdef EXPP_L1_HIT
        voff = lane * 16; base = (const char*)Pb;
#endif
#ifndef EXPP_CACHE_BITS
#define EXPP_CACHE_BITS ""
#endif
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" EXPP_CACHE_BITS
                     :
                     : "s"(lds_byte), "v"(voff), "s"(base)
                     : "memory");
    };
#endif
#endif
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_void_ptr)smem;
    // load n (0..NLD-1) of k-tile kt into LDS stage `stage`; kt may run past the end: re-load the last k-tile
    auto issue_one = [&](int kt, int stage, int n) {
#ifdef EXPP_KWRAP
        const int kk = ((kt < nk ? kt : nk - 1) & (EXPP_KWRAP - 1)) * BK4;
#else
        const int kk = (kt < nk ? kt : nk - 1) * BK4;
#endif
        const unsigned st = lds_base + stage * STAGE;
        if (n < LA)
            dma((const char*)(Pb + kk), offa[n], st + lds_a + n * 16 * ROWB);
        else
            dma((const char*)(Qb + kk), offb[n - LA], st + lds_b + (n - LA) * 16 * ROWB);
    };
    auto issue_tile = [&](int kt, int stage) {
#pragma unroll
        for (int n = 0; n < NLD; ++n) issue_one(kt, stage, n);
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int sw = (lane >> 2) & 3, hi = lane >> 5;
    const int a_off = (wm * WTM + (lane & 31)) * ROWB;
    const int b_off = A_BYTES + (wn * WTN + (lane & 31)) * ROWB;

#pragma unroll
    for (int t = 0; t < NST - 1; ++t) issue_tile(t, t);
    WAIT_VM((NST - 2) * NLD);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (grp) __builtin_amdgcn_s_barrier();

#ifdef EXP_TRACE
    long long* trace = (long long*)g.Ct + (long)blockIdx.x * 8192 + (threadIdx.x >> 6) * 1024;
    int tn = 0;
#endif
    // LDS read addresses: one register per operand, k-step and pair of stages; the stage inside
    // the pair and the fragment index are instruction offsets (below 64 KB) once the k loop is
    // unrolled by the four stages.
    constexpr int NPAIR = (NST + 1) / 2;
    const unsigned char* ra[2][NPAIR];
    const unsigned char* rb[2][NPAIR];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int co = (((ks << 1) | hi) ^ sw) << 4;
#pragma unroll
        for (int half = 0; half < NPAIR; ++half) {
            ra[ks][half] = smem + half * 2 * STAGE + a_off + co;
            rb[ks][half] = smem + half * 2 * STAGE + b_off + co;
        }
    }
    auto body = [&](int kt, auto stage_c, auto masked_c) {
        constexpr int SIDX = decltype(stage_c)::value;
        constexpr bool MASKED = decltype(masked_c)::value;
        TRACE_POINT();
        // ---- M(kt)
        // The loads are throttled by the 64 B/clk path into the CU and the reads by LDS bandwidth:
        // interleaved, the two queues drain side by side instead of one after the other.
        bf16x8 fa[2][FM], fb[2][FN];
        constexpr int NRD = 2 * (FM + FN), RD_PER_LD = (NRD + NLD - 1) / NLD;
#pragma unroll
        for (int r = 0; r < NRD; ++r) {
#ifndef EXPP_NO_DMA
            if (r % RD_PER_LD == 0 && r / RD_PER_LD < NLD) issue_one(kt + NST - 1, (SIDX + NST - 1) % NST, r / RD_PER_LD);
#endif
            const int ks = r / (FM + FN), o = r % (FM + FN);
            if (o < FM)
                fa[ks][o] = *(const bf16x8*)(ra[ks][SIDX >> 1] + (SIDX & 1) * STAGE + o * 32 * ROWB);
            else
                fb[ks][o - FM] = *(const bf16x8*)(rb[ks][SIDX >> 1] + (SIDX & 1) * STAGE + (o - FM) * 32 * ROWB);
        }
        TRACE_POINT();
        WAIT_LGKM0();
#ifndef EXPP_NO_DMA
        WAIT_VM((NST - 2) * NLD);  // own loads of k-tile kt+1 have landed
#endif
        if (MASKED && kt >= nk) {  // a k-tile past the end (only in the peeled last group) contributes nothing
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int i = 0; i < FM; ++i) fa[ks][i] = bf16x8{};
        }
        TRACE_POINT();
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        TRACE_POINT();
        // ---- C(kt)
#ifdef EXPP_SETPRIO
        __builtin_amdgcn_s_setprio(3);
#endif
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][i], fb[ks][j], acc[i][j], 0, 0, 0);
#ifdef EXPP_SETPRIO
        __builtin_amdgcn_s_setprio(0);
#endif
        __builtin_amdgcn_sched_barrier(0);
        TRACE_POINT();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    if constexpr (NST == 4) {  // nk is a multiple of 4 (k extents are multiples of 128)
        for (int kt = 0; kt < nk; kt += 4) {
            body(kt, integral_constant<int, 0>{}, integral_constant<bool, false>{});
            body(kt + 1, integral_constant<int, 1>{}, integral_constant<bool, false>{});
            body(kt + 2, integral_constant<int, 2>{}, integral_constant<bool, false>{});
            body(kt + 3, integral_constant<int, 3>{}, integral_constant<bool, false>{});
        }
    } else {  // groups of five k-tiles; the last group is peeled and masks the k-tiles past the end
        int kt = 0;
        for (; kt + 5 < nk; kt += 5) {
            body(kt, integral_constant<int, 0>{}, integral_constant<bool, false>{});
            body(kt + 1, integral_constant<int, 1>{}, integral_constant<bool, false>{});
            body(kt + 2, integral_constant<int, 2>{}, integral_constant<bool, false>{});
            body(kt + 3, integral_constant<int, 3>{}, integral_constant<bool, false>{});
            body(kt + 4, integral_constant<int, 4>{}, integral_constant<bool, false>{});
        }
        body(kt, integral_constant<int, 0>{}, integral_constant<bool, true>{});
        body(kt + 1, integral_constant<int, 1>{}, integral_constant<bool, true>{});
        body(kt + 2, integral_constant<int, 2>{}, integral_constant<bool, true>{});
        body(kt + 3, integral_constant<int, 3>{}, integral_constant<bool, true>{});
        body(kt + 4, integral_constant<int, 4>{}, integral_constant<bool, true>{});
    }
    if (!grp) __builtin_amdgcn_s_barrier();
    WAIT_VM(0);  // the loads issued past the end must not land in the epilogue's tile
#ifdef EXP_NO_EPI
    float ssum = 0.f;
    for (int i = 0; i < FM; ++i) for (int j = 0; j < FN; ++j) for (int r = 0; r < 16; ++r) ssum += acc[i][j][r];
#ifdef EXPP_TO_VGPR
    ssum += sink[0][0] + sink[0][1] + sink[0][2] + sink[0][3];
#endif
    if (ssum == 123.456f) g.C[threadIdx.x] = f2bf(ssum);
#else
    EPILOGUE<BM, BN, WGM, WGN, EPI>(g, tc, acc, smem);
#endif
}

template <int BM, int BN, int WGM, int WGN, int EPI, int FEED>
hipError_t launch_one(const GemmArgs& g, int nblocks, hipStream_t stream) {
    constexpr int stage2 = FEED == 5 ? 5 * (BM + BN) * 64 : 2 * (BM + BN) * ROW_BYTES, epi = EPILOGUE_BYTES<BM, BN>();
    constexpr int smem = stage2 > epi ? stage2 : epi;
    static bool configured = false;  // per instantiation; the attribute is idempotent
    auto kern = FEED == 5 ? gemm_nt_pp_kernel<BM, BN, 2, 4, EPI, 5>
              : FEED == 4 ? gemm_nt_pp_kernel<BM, BN, 2, 4, EPI, 4>
              : FEED == 3 ? gemm_nt_pipe4_kernel<BM, BN, WGM, WGN, EPI>
              : FEED == 2 ? gemm_nt_pipe_kernel<BM, BN, WGM, WGN, EPI>
              : FEED == 1 ? gemm_nt_dlds_kernel<BM, BN, WGM, WGN, EPI>
                          : gemm_nt_kernel<BM, BN, WGM, WGN, EPI>;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(nblocks), dim3(WGM * WGN * 64), smem, stream, g);
    return hipGetLastError();
}

template <int EPI>
hipError_t launch_cfg(int cfg, const GemmArgs& g, int nblocks, hipStream_t stream) {
    switch (cfg) {
        case GEMM_CFG_128x128_W4: return launch_one<128, 128, 2, 2, EPI, 0>(g, nblocks, stream);
        case GEMM_CFG_256x256_W4: return launch_one<256, 256, 2, 2, EPI, 0>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8: return launch_one<256, 256, 2, 4, EPI, 0>(g, nblocks, stream);
        case GEMM_CFG_128x128_W4_DLDS: return launch_one<128, 128, 2, 2, EPI, 1>(g, nblocks, stream);
        case GEMM_CFG_256x256_W4_DLDS: return launch_one<256, 256, 2, 2, EPI, 1>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8_DLDS: return launch_one<256, 256, 2, 4, EPI, 1>(g, nblocks, stream);
        case GEMM_CFG_128x128_W4_PIPE: return launch_one<128, 128, 2, 2, EPI, 2>(g, nblocks, stream);
        case GEMM_CFG_256x256_W4_PIPE: return launch_one<256, 256, 2, 2, EPI, 2>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8_PIPE: return launch_one<256, 256, 2, 4, EPI, 2>(g, nblocks, stream);
        case GEMM_CFG_128x128_W4_PIPE4: return launch_one<128, 128, 2, 2, EPI, 3>(g, nblocks, stream);
        case GEMM_CFG_256x256_W4_PIPE4: return launch_one<256, 256, 2, 2, EPI, 3>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8_PIPE4: return launch_one<256, 256, 2, 4, EPI, 3>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8_PINGPONG: return launch_one<256, 256, 2, 4, EPI, 4>(g, nblocks, stream);
        case GEMM_CFG_256x256_W8_PINGPONG5: return launch_one<256, 256, 2, 4, EPI, 5>(g, nblocks, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int gemm_cfg_tile(int cfg) {
    switch (cfg) {
        case GEMM_CFG_128x128_W4:
        case GEMM_CFG_128x128_W4_DLDS:
        case GEMM_CFG_128x128_W4_PIPE:
        case GEMM_CFG_128x128_W4_PIPE4: return 128;
        case GEMM_CFG_256x256_W4:
        case GEMM_CFG_256x256_W8:
        case GEMM_CFG_256x256_W4_DLDS:
        case GEMM_CFG_256x256_W8_DLDS:
        case GEMM_CFG_256x256_W4_PIPE:
        case GEMM_CFG_256x256_W8_PIPE:
        case GEMM_CFG_256x256_W4_PIPE4:
        case GEMM_CFG_256x256_W8_PIPE4:
        case GEMM_CFG_256x256_W8_PINGPONG:
        case GEMM_CFG_256x256_W8_PINGPONG5: return 256;
        default: return 0;
    }
}

hipError_t launch_gemm_nt(int cfg, int epi, const GemmArgs& g, hipStream_t stream) {
    const int nblocks = g.tiles_per_mat * g.batch;
    if (nblocks <= 0) return hipSuccess;
    switch (epi) {
        case EPI_SYRK: return launch_cfg<EPI_SYRK>(cfg, g, nblocks, stream);
        case EPI_SYMPOLY: return launch_cfg<EPI_SYMPOLY>(cfg, g, nblocks, stream);
        case EPI_BX: return launch_cfg<EPI_BX>(cfg, g, nblocks, stream);
        default: return hipErrorInvalidValue;
    }
}
