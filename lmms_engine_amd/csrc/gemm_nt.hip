// GEMM family for the Newton-Schulz chain on gfx950, built on v_mfma_f32_16x16x32_bf16.
//
// Why the 16x16x32 instruction: under matrix-pipe load the part lowers its clock to stay inside its power
// limit, and on operands with random mantissas a loop of nothing but MFMAs (probe.hip, a measurement library of its own) sustains about
// 1.85 PFLOP/s with 32x32x16 and about 2.09 with 16x16x32 (both reach 2.45 on constant operands): the deeper dot
// product updates each fp32 accumulator half as often per FLOP.  The same kernels built on 32x32x16 ran 4 to 8 %
// slower at a 3 to 9 % lower clock.  Operand fragment: lane l holds row l%16, eight consecutive k from 8*(l/16)
// (16 bytes).  Accumulator fragment: lane l holds column l%16, rows 4*(l/16)+0..3 (f32x4).
//
// The three products of one NS iteration:
//   SYRK     A  = bf(X Xt)                         P = Q = X   (M x K)           C[i][j] = sum_k P[i][k] Q[j][k]
//   SYMPOLY  B  = bf(bf(b A) + bf(c bf(A A)))      P = Q = A   (M x M, symmetric so A A = A At)      same
//   BX       X' = bf(bf(a X) + bf(B X))            P = B (M x M), Q = X (M x K)  C[i][j] = sum_k P[i][k] Q[k][j]
// SYRK/SYMPOLY contract rows with rows and compute only tiles on or above the diagonal, mirrored in the
// epilogue, which makes the result symmetric bit for bit.  BX contracts rows of B with columns of X: its Q
// fragments come out of LDS through the transposing read ds_read_b64_tr_b16, so X is kept in one
// orientation only.
//
// Every bf16 rounding point of the reference's torch expressions
// (/root/reference/src/lmms_engine/utils/muon_utils.py:149-152) is applied in registers.
//
// Operands and results live in the blocked layout of common.h (256 x 32 blocks), zero padded
// by the producers to whole tiles, so there is no masking here; the host launcher checks that
// the shapes it is given are whole tiles before launching.
#include <atomic>
#include <type_traits>

#include "common.h"
#include "gemm_nt.h"

namespace {

// Upper-triangle tile order in row groups of GM: inside a group, column by column, so the
// ~32 tiles an XCD works on at a time touch few distinct row panels.
template <int GM>
__device__ __forceinline__ void tri_decode(int t, int T, int& ti, int& tj) {
    int r0 = 0, gm, cnt;
    for (;;) {  // find the row group that holds tile t
        gm = (T - r0 < GM) ? (T - r0) : GM;
        cnt = gm * (T - r0) - gm * (gm - 1) / 2;
        if (t < cnt || r0 + gm >= T) break;
        t -= cnt;
        r0 += gm;
    }
    const int tri = gm * (gm + 1) / 2;
    int c = 0, u = t;  // column c of the leading gm x gm triangle holds c+1 tiles
    while (u >= c + 1 && c < gm - 1) { u -= c + 1; ++c; }
    const int rest = t - tri;
    const bool in_tri = t < tri;
    ti = r0 + (in_tri ? u : rest % gm);
    tj = r0 + (in_tri ? c : gm + rest / gm);
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

// Tile `logical` (0 .. tiles_per_mat * batch - 1) in the launch order: matrix by matrix, 4-row groups.
template <int EPI>
__device__ __forceinline__ TileCoord tile_of(const GemmArgs& g, int logical) {
    const int bidx = logical / g.tiles_per_mat;
    const int t = logical - bidx * g.tiles_per_mat;
    int ti = 0, tj = 0;  // plain locals: references into the struct kept it in scratch memory
    if (epi_is_bx(EPI)) rect_decode<4>(t, g.tiles_m, g.tiles_n, ti, tj);
    else tri_decode<4>(t, g.tiles_m, ti, tj);
    return TileCoord{bidx, ti, tj};
}

template <int EPI>
__device__ __forceinline__ TileCoord decode_tile(const GemmArgs& g) {
    return tile_of<EPI>(g, xcd_remap(blockIdx.x, gridDim.x, g.xcd_shift));
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* glb_void_ptr;

#define WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)
// s_waitcnt with only vmcnt set: vmcnt is split over bits [3:0] and [15:14] (N < 64)
#define WAIT_VM(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))

// Start of row panel `row0` (a multiple of the tile edge, so the panel lies inside one row of
// blocks) of a blocked matrix with cb column blocks: add kblock * BLK_ELEMS to reach a k-tile.
__device__ __forceinline__ long panel_offset(int row0, int cb) {
    return (long)(row0 >> 8) * cb * BLK_ELEMS + (row0 & 255) * BLK_COLS;
}

// ---- epilogue ------------------------------------------------------------------------------
// One LDS copy of the tile, both output orientations written as 16-byte vectors.  The tile
// lives in LDS as Tt[n][m] (n = local column, m = local row of the accumulator tile), the
// orientation of Ct and of the elementwise source Et.  Every lane writes its rounded accumulators
// as 8-byte pieces (4 consecutive m of one n, exactly what an accumulator lane holds: lane&15 owns
// column n, its four registers are rows 4*(lane>>4) + 0..3 of the 16x16 fragment); after one barrier rows of Tt
// leave as rows of Ct (SYMPOLY adds the b.A term there, from pieces of Et that each thread loaded
// into registers before the accumulators were written, and puts the sums back), while rows of C
// are gathered with ds_read_b64_tr_b16: in a group of 16 lanes, lane i receives element i%4 of the
// 8-byte pieces addressed by lanes i/4, 4+i/4, 8+i/4, 12+i/4.
// Diagonal tiles of the symmetric kernels: only the 32x32 fragments on or above the diagonal need to be
// computed; the Ct pass writes them as the lower half (and the diagonal fragments) of the tile, the gather
// writes the upper half.  Inside a diagonal fragment acc(i,j) and acc(j,i) are sums of the same exact products
// in the same order, so the result is symmetric bit for bit.
template <int BM, int BN>
constexpr int epilogue_bytes() { return BN * (BM * 2 + 16); }

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ s16x4 lds_read_tr16(const unsigned char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(lds_void_ptr)p);
}

template <int BM, int BN, int WGM, int WGN, int EPI, bool MASKED>
__device__ __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc,
                                         f32x4 (&acc)[BM / WGM / 16][BN / WGN / 16], unsigned char* smem) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int S = BM * 2 + 16;      // Tt row pitch (bytes): conflict-free for the 8-byte pieces
    constexpr int NLE = BN * (BM / 8) / NT;  // 16-byte chunks per thread for a whole tile
    static_assert((BN * (BM / 8)) % NT == 0 && BM % 64 == 0, "even split");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN, quad = lane >> 4;
    const int m0 = tc.ti * BM, n0 = tc.tj * BN;
    const bool diag = (!epi_is_bx(EPI)) && (tc.ti == tc.tj);
    // Et and Ct hold the tile as rows n0.. (BN of them) x columns m0.. (BM of them).  Chunk c of a
    // thread: 16 bytes j = c%8 of the 128-byte row piece of row n = (c/8)%BN in column block c/8/BN,
    // so that a wave touches 8 rows x 128 bytes = 1 KB of one block, contiguous in memory.
    // The return value says whether the chunk is a computed one: in a diagonal tile of a MASKED caller (the
    // ping-pong kernel, which skips the others) only the 32x32 fragments on or above the diagonal are, i.e. column
    // block m/32 <= row block n/32 of Tt.  A caller that computes whole diagonal tiles writes them in the Ct pass.
    auto tile_chunk = [&](int c, int cb, long& goff, int& loff) {
        constexpr int CPB = BLK_COLS / 8;  // 16-byte chunks per row of a block
        static_assert(BLK_COLS == 32, "a column block is one fragment wide");
        const int j = c % CPB, n = (c / CPB) % BN, cbk = (c / CPB) / BN;
        goff = panel_offset(n0, cb) + (long)((m0 >> BLK_SHIFT) + cbk) * BLK_ELEMS + n * BLK_COLS + j * 8;
        loff = n * S + (cbk * CPB + j) * 16;
        return !MASKED || !diag || cbk <= (n >> 5);
    };
    // SYMPOLY: this thread's 16-byte pieces of the b.A term, in the layout of the Ct pass, go to registers
    // first, so that the loads are in flight while the accumulators are rounded into LDS
    bf16x8 ev[EPI == EPI_SYMPOLY ? NLE : 1];
    if (EPI == EPI_SYMPOLY) {
        const bf16_t* Et = g.Et + tc.bidx * g.strideEt;
#pragma unroll
        for (int u = 0; u < NLE; ++u) {
            long goff;
            int loff;
            tile_chunk(tid + u * NT, g.cbEt, goff, loff);
            ev[u] = *(const bf16x8*)(Et + goff);
        }
    }
    __syncthreads();  // the operand stages are no longer read
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            bf16x4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = rbf(acc[i][j][r]);
                if (EPI == EPI_SYMPOLY) v = g.s1 * v;
                o[r] = f2bf(v);
            }
            *(bf16x4*)(smem + (wn * WTN + j * 16 + (lane & 15)) * S + (wm * WTM + i * 16 + quad * 4) * 2) = o;
        }
    __syncthreads();
    {
        // rows of Tt leave as rows of Ct; SYMPOLY adds the rounded b.A term here and, when the tile itself is
        // gathered from LDS afterwards, puts the finished pieces back
        bf16_t* Ct = g.Ct + tc.bidx * g.strideCt;
#pragma unroll
        for (int u = 0; u < NLE; ++u) {
            long goff;
            int loff;
            const bool computed = tile_chunk(tid + u * NT, g.cbCt, goff, loff);
            bf16x8 t = *(const bf16x8*)(smem + loff);
            if (EPI == EPI_SYMPOLY) {
#pragma unroll
                for (int k = 0; k < 8; ++k) t[k] = f2bf(rbf(g.s0 * bf2f(ev[u][k])) + bf2f(t[k]));
                if (MASKED ? computed : !diag) *(bf16x8*)(smem + loff) = t;
            }
            if (g.Ct && computed) *(bf16x8*)(Ct + goff) = t;
        }
        if (EPI == EPI_SYMPOLY && (MASKED || !diag)) __syncthreads();
    }
    if (g.C && (MASKED || !diag)) {
        // lane j = 4r+s of a group addresses row n + 8s + r (then + 4), pieces m = 4c..4c+3: lane i = 4s+e
        // receives Tt[n+8s .. n+8s+7][4c+e], 16 bytes of row 4c+e of C.  The four groups of a wave sit
        // side by side along n (128 columns = two column blocks): 4 rows x 128 bytes per block and store.
        const int grp = lane >> 4, i16 = lane & 15;
        const unsigned char* src = smem + ((i16 & 3) * 8 + (i16 >> 2) + grp * 32) * S;
        bf16_t* dst = g.C + tc.bidx * g.strideC + panel_offset(m0, g.cbC) +
                      (long)((n0 >> BLK_SHIFT) + ((grp * 32) >> BLK_SHIFT)) * BLK_ELEMS + (i16 & 3) * BLK_COLS +
                      ((grp * 32) & (BLK_COLS - 1)) + (i16 >> 2) * 8;
        constexpr int NSTRIP = BN / 128, NQUAD = BM / 4, NW = NT / 64;
        constexpr int NUNIT = NSTRIP * NQUAD / NW;
        static_assert(BN % 128 == 0 && (NSTRIP * NQUAD) % NW == 0, "whole 128-column strips per wave");
#pragma unroll 8
        for (int u = 0; u < NUNIT; ++u) {
            const int wu = wave + u * NW, strip = wu % NSTRIP, c = wu / NSTRIP;
            const unsigned char* q = src + strip * 128 * S + c * 8;
            const s16x4 lo = lds_read_tr16(q), hi4 = lds_read_tr16(q + 4 * S);
            const s16x8 o = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            // a diagonal tile: the pieces strictly above the diagonal fragments (row block c/8 < column block);
            // the Ct pass has written the rest
            if (!diag || (c >> 3) < strip * 4 + grp)
                *(s16x8*)(dst + (long)strip * (128 / BLK_COLS) * BLK_ELEMS + c * 4 * BLK_COLS) = o;
        }
    }
}

// Epilogue of BX.  The accumulators were built with the MFMA operands swapped, so a lane holds 4
// consecutive columns n of one row m (lane&15 owns row m of its P fragment, its four registers are columns
// 4*(lane>>4) + 0..3 of its Q fragment): 8-byte pieces of rows of X'.  Every thread first issues the
// loads of its share of the a.X tile (16-byte pieces of rows, the layout of the output pass) into registers,
// then the rounded accumulators go to LDS as T[m][n] while those loads are in flight; after one barrier each
// thread reads its pieces of T, adds the rounded a.X term and stores rows of X' (1 KB contiguous per wave
// instruction).
template <int BM, int BN>
constexpr int epilogue_nn_bytes() { return BM * (BN * 2 + 16); }

// Folded parameter update: eight consecutive elements of one parameter row, o = bf16(X' * scale);
// p <- rnd(p * decay); p <- rnd(p + alpha * o), the arithmetic of the stand-alone update kernel (elementwise.hip).
// The parameter piece is fetched into registers early (fold_load) and applied after the tile has been through LDS.
struct FoldPiece {
    f32x4 lo;  // bf16 parameter: the eight values; fp32 parameter: the first four (the other four are fetched
               // when the piece is applied, from the cache line that this fetch brought in)
};
template <typename PT>
__device__ __forceinline__ FoldPiece fold_load(const PT* p, bool vec, int left) {
    FoldPiece f;
    f.lo = f32x4{0.f, 0.f, 0.f, 0.f};
    if (vec && left >= 8) f.lo = __builtin_nontemporal_load((const f32x4*)p);
    return f;
}
template <typename PT>
__device__ __forceinline__ void fold_apply(PT* p, const FoldPiece& f, const bf16x8& x, bool vec, int left, const GemmArgs& g) {
    constexpr bool PBF = std::is_same<PT, bf16_t>::value;
    auto one = [&](float pv, bf16_t xv) {
        const float os = rbf(bf2f(xv) * g.upd_scale);
        const float pd = PBF ? rbf(pv * g.upd_decay) : pv * g.upd_decay;
        return fmaf(g.upd_alpha, os, pd);
    };
    if (vec && left >= 8) {
        if constexpr (PBF) {
            bf16x8 pv = *(const bf16x8*)&f.lo;
#pragma unroll
            for (int k = 0; k < 8; ++k) pv[k] = f2bf(one(bf2f(pv[k]), x[k]));
            __builtin_nontemporal_store(pv, (bf16x8*)p);
        } else {
            f32x4 a = f.lo, b = __builtin_nontemporal_load((const f32x4*)(p + 4));
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a[k] = one(a[k], x[k]);
                b[k] = one(b[k], x[4 + k]);
            }
            __builtin_nontemporal_store(a, (f32x4*)p);
            __builtin_nontemporal_store(b, (f32x4*)(p + 4));
        }
    } else {  // ragged row end or unaligned parameter: element by element
        for (int k = 0; k < 8 && k < left; ++k) {
            if constexpr (PBF) p[k] = f2bf(one(bf2f(p[k]), x[k]));
            else p[k] = one(p[k], x[k]);
        }
    }
}

template <int BM, int BN, int WGM, int WGN, int FOLD>
__device__ __forceinline__ void epilogue_nn(const GemmArgs& g, const TileCoord& tc,
                                            f32x4 (&acc)[BM / WGM / 16][BN / WGN / 16], unsigned char* smem) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int S = BN * 2 + 16;           // T row pitch (bytes)
    constexpr int CPB = BLK_COLS / 8;        // 16-byte chunks per row of a block
    constexpr int NLE = BM * (BN / 8) / NT;  // 16-byte chunks per thread for a whole tile
    static_assert((BM * (BN / 8)) % NT == 0 && BN % BLK_COLS == 0, "even split");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN, quad = lane >> 4;
    const int m0 = tc.ti * BM, n0 = tc.tj * BN;
    // Last iteration of a step, parameter in the orientation of X: the scaled update goes straight into the
    // parameter (apply_scaling and the decay / update lines, muon_utils.py:167-175, :324-325) and X' is not written.
    constexpr bool fold = FOLD == 1;
    // chunk c: 16 bytes j of the row piece of row m in column block cbk of the tile.  Writing X' a wave covers
    // 16 rows of one block = 1 KB contiguous in the blocked layout; writing the parameter (row-major) it covers
    // whole tile rows instead, 2 x 512 B of bf16, and reads E in 64-byte pieces.
    auto decode = [&](int c, int& j, int& m, int& cbk) {
        if constexpr (fold) {
            const int piece = c % (BN / 8);
            m = c / (BN / 8);
            cbk = piece / CPB;
            j = piece % CPB;
        } else {
            j = c % CPB;
            m = (c / CPB) % BM;
            cbk = (c / CPB) / BM;
        }
    };
    auto tile_chunk = [&](int c, int cb, long& goff, int& loff) {
        int j, m, cbk;
        decode(c, j, m, cbk);
        goff = panel_offset(m0, cb) + (long)((n0 >> BLK_SHIFT) + cbk) * BLK_ELEMS + m * BLK_COLS + j * 8;
        loff = m * S + (cbk * CPB + j) * 16;
    };
    const bf16_t* Et = g.Et + tc.bidx * g.strideEt;
    bf16x8 ev[NLE];
#pragma unroll
    for (int u = 0; u < NLE; ++u) {
        long goff;
        int loff;
        tile_chunk(tid + u * NT, g.cbEt, goff, loff);
        ev[u] = *(const bf16x8*)(Et + goff);
    }
    __syncthreads();  // the operand stages are no longer read
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            bf16x4 t;
#pragma unroll
            for (int r = 0; r < 4; ++r) t[r] = f2bf(acc[i][j][r]);
            *(bf16x4*)(smem + (wm * WTM + i * 16 + (lane & 15)) * S + (wn * WTN + j * 16 + quad * 4) * 2) = t;
        }
    bf16_t* C = g.C + tc.bidx * g.strideC;
    if constexpr (FOLD == 0) {
        __syncthreads();
#pragma unroll
        for (int u = 0; u < NLE; ++u) {
            long goff;
            int loff;
            tile_chunk(tid + u * NT, g.cbC, goff, loff);
            const bf16x8 t = *(const bf16x8*)(smem + loff);
            bf16x8 o;
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = f2bf(rbf(g.s0 * bf2f(ev[u][k])) + bf2f(t[k]));
            *(bf16x8*)(C + goff) = o;
        }
        return;
    }
    if constexpr (FOLD == 2) {
        // The parameter is the transpose of X (rows > cols): row n0 + n of the parameter is column n of the tile.  The
        // finished X' values go back into T in place, and after a barrier a wave gathers them the other way round with
        // ds_read_b64_tr_b16 (the gather of the symmetric epilogue): lane i16 of a group of 16 receives
        // T[m .. m+7][4c + i16 % 4] with m = strip * 128 + grp * 32 + (i16 / 4) * 8, i.e. 16 bytes of row 4c + i16 % 4
        // of the parameter tile; a wave instruction covers 4 parameter rows x 128 columns.
        constexpr int NSTRIP = BM / 128, NQUAD = BN / 4, NWV = NT / 64;
        constexpr int NUNIT = NSTRIP * NQUAD / NWV;
        static_assert(BM % 128 == 0 && (NSTRIP * NQUAD) % NWV == 0, "whole 128-row strips per wave");
        void* pbase = const_cast<void*>(g.upd_ptrs[tc.bidx]);
        const bool pvec = (g.upd_cols % 8 == 0) && ((((uintptr_t)pbase) & 15) == 0);
        const bool pbf = g.upd_dtype == MUON_HIP_BF16;
        const int grp = lane >> 4, i16 = lane & 15;
        auto piece = [&](int u, long& poff, int& left) {
            const int wu = wave + u * NWV, strip = wu % NSTRIP, c = wu / NSTRIP;
            const int row = n0 + c * 4 + (i16 & 3), col = m0 + strip * 128 + grp * 32 + (i16 >> 2) * 8;
            poff = (long)row * g.upd_cols + col;
            left = g.upd_cols - col;
            return row < g.upd_rows && left > 0;
        };
        FoldPiece pv[NUNIT];
#pragma unroll
        for (int u = 0; u < NUNIT; ++u) {
            long poff;
            int left;
            if (piece(u, poff, left))
                pv[u] = pbf ? fold_load<bf16_t>((const bf16_t*)pbase + poff, pvec, left) : fold_load<float>((const float*)pbase + poff, pvec, left);
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < NLE; ++u) {
            long goff;
            int loff;
            tile_chunk(tid + u * NT, g.cbC, goff, loff);
            const bf16x8 t = *(const bf16x8*)(smem + loff);
            bf16x8 o;
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = f2bf(rbf(g.s0 * bf2f(ev[u][k])) + bf2f(t[k]));
            *(bf16x8*)(smem + loff) = o;
        }
        __syncthreads();
        // lane j = 4r+s of a group addresses row m + 8s + r of T (then + 4), columns 4c..4c+3
        const unsigned char* src = smem + ((i16 & 3) * 8 + (i16 >> 2) + grp * 32) * S;
#pragma unroll  // fully: the parameter pieces are indexed by u and must stay in registers
        for (int u = 0; u < NUNIT; ++u) {
            const int wu = wave + u * NWV, strip = wu % NSTRIP, c = wu / NSTRIP;
            const unsigned char* q = src + strip * 128 * S + c * 8;
            const s16x4 lo = lds_read_tr16(q), hi4 = lds_read_tr16(q + 4 * S);
            const s16x8 t8 = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            long poff;
            int left;
            if (piece(u, poff, left)) {
                const bf16x8 o = *(const bf16x8*)&t8;
                if (pbf) fold_apply<bf16_t>((bf16_t*)pbase + poff, pv[u], o, pvec, left, g);
                else fold_apply<float>((float*)pbase + poff, pv[u], o, pvec, left, g);
            }
        }
        return;
    }
    void* pbase = const_cast<void*>(g.upd_ptrs[tc.bidx]);
    const bool pvec = (g.upd_cols % 8 == 0) && ((((uintptr_t)pbase) & 15) == 0);
    const bool pbf = g.upd_dtype == MUON_HIP_BF16;
    // The parameter pieces are fetched here, with the accumulators already in LDS, so that their latency passes
    // behind the barrier.
    auto piece = [&](int c, long& poff, int& left) {
        int j, m, cbk;
        decode(c, j, m, cbk);
        const int row = m0 + m, col = n0 + cbk * BLK_COLS + j * 8;
        poff = (long)row * g.upd_cols + col;
        left = g.upd_cols - col;
        return row < g.upd_rows && left > 0;
    };
    FoldPiece pv[NLE];
#pragma unroll
    for (int u = 0; u < NLE; ++u) {
        long poff;
        int left;
        if (piece(tid + u * NT, poff, left))
            pv[u] = pbf ? fold_load<bf16_t>((const bf16_t*)pbase + poff, pvec, left) : fold_load<float>((const float*)pbase + poff, pvec, left);
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NLE; ++u) {
        long goff, poff;
        int loff, left;
        const int c = tid + u * NT;
        tile_chunk(c, g.cbC, goff, loff);
        const bf16x8 t = *(const bf16x8*)(smem + loff);
        bf16x8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o[k] = f2bf(rbf(g.s0 * bf2f(ev[u][k])) + bf2f(t[k]));
        if (piece(c, poff, left)) {
            if (pbf) fold_apply<bf16_t>((bf16_t*)pbase + poff, pv[u], o, pvec, left, g);
            else fold_apply<float>((float*)pbase + poff, pv[u], o, pvec, left, g);
        }
    }
}

// The same result for EPI_BX without LDS and without a barrier.  A lane holds, of fragment (i, j), columns 4q..4q+3
// (q = lane / 16) of row lane % 16 as two packed registers.  v_permlane16_swap_b32 exchanges the odd 16-lane rows of
// its first operand with the even rows of its second: applied to the registers of fragments j = 2t and 2t+1 it leaves
// a lane of row 0 / 2 with columns 0..7 / 8..15 of fragment 2t and a lane of row 1 / 3 with those of fragment 2t+1,
// i.e. 16 consecutive bytes of a row of X', and the 64 lanes of a wave with 16 rows x 64 bytes = one contiguous KB of
// the blocked layout, the same store the LDS version issues.  The a.X pieces are loaded in the same pattern.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) {
    const bf16x2 p = {f2bf(a), f2bf(b)};
    return *(const unsigned*)&p;
}
template <int BM, int BN, int WGM, int WGN>
__device__ __forceinline__ void epilogue_nn_reg(const GemmArgs& g, const TileCoord& tc,
                                                f32x4 (&acc)[BM / WGM / 16][BN / WGN / 16]) {
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    static_assert(FN % 2 == 0 && BLK_COLS == 32, "a pair of fragments is one column block");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN, row = lane >> 4;
    const int m0 = tc.ti * BM, n0 = tc.tj * BN;
    // piece (i, t): row m0 + wm*WTM + 16 i + lane%16, columns n0 + wn*WTN + 32 t + 16 (row & 1) + 8 (row >> 1) .. + 7
    const long lane_off = (long)((n0 >> BLK_SHIFT) + wn * (WTN / 32)) * BLK_ELEMS + (wm * WTM + (lane & 15)) * BLK_COLS +
                          (row & 1) * 16 + (row >> 1) * 8;
    const bf16_t* Et = g.Et + tc.bidx * g.strideEt + panel_offset(m0, g.cbEt) + lane_off;
    bf16_t* C = g.C + tc.bidx * g.strideC + panel_offset(m0, g.cbC) + lane_off;
    bf16x8 ev[FM][FN / 2];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int t = 0; t < FN / 2; ++t) ev[i][t] = *(const bf16x8*)(Et + i * 16 * BLK_COLS + (long)t * BLK_ELEMS);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int t = 0; t < FN / 2; ++t) {
            const f32x4 a = acc[i][2 * t], b = acc[i][2 * t + 1];
            const u32x2v lo = __builtin_amdgcn_permlane16_swap(pack_bf16x2(a[0], a[1]), pack_bf16x2(b[0], b[1]), false, false);
            const u32x2v hi = __builtin_amdgcn_permlane16_swap(pack_bf16x2(a[2], a[3]), pack_bf16x2(b[2], b[3]), false, false);
            const u32x4 tw = {lo[0], hi[0], lo[1], hi[1]};
            const bf16x8 tv = *(const bf16x8*)&tw;
            bf16x8 o;
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = f2bf(rbf(g.s0 * bf2f(ev[i][t][k])) + bf2f(tv[k]));
            *(bf16x8*)(C + i * 16 * BLK_COLS + (long)t * BLK_ELEMS) = o;
        }
}

// Symmetric products without LDS and without a barrier.  A lane holds, of fragment (i, j), rows 4q..4q+3 (q = lane / 16)
// of column lane % 16: 8-byte pieces of rows of the mirror image Ct, which leave exactly as the rows of X' above, with
// fragments i = 2t and 2t+1 paired by v_permlane16_swap_b32 (SYMPOLY adds the b.A term to the paired pieces, read from
// the mirror tile of A in the same pattern).  For the tile itself the finished values return to the fragment layout
// (the swap is its own inverse) and every group of four lanes transposes its 4 x 4 elements in two exchanges:
//   with the lane one away (DPP quad_perm [1,0,3,2]) the 16-bit halves of each register,
//   with the lane two away (quad_perm [2,3,0,1]) one of the two registers,
// after which lane 4a+s of row q holds columns 4a..4a+3 of row 4q+s of the fragment: 8-byte pieces of rows of C, a wave
// store covering 16 rows x 32 bytes.  In a diagonal tile only the 32x32 blocks on or above the diagonal hold computed
// values: they go out as Ct pieces (the lower half and the diagonal blocks) and, strictly above it, as C pieces.
__device__ __forceinline__ void quad_transpose_b16(unsigned& p0, unsigned& p1, unsigned sel, bool upper) {
    const unsigned t0 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)p0, 0xB1, 0xF, 0xF, false);
    const unsigned t1 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)p1, 0xB1, 0xF, 0xF, false);
    p0 = __builtin_amdgcn_perm(t0, p0, sel);
    p1 = __builtin_amdgcn_perm(t1, p1, sel);
    const unsigned send = upper ? p0 : p1;
    const unsigned recv = (unsigned)__builtin_amdgcn_update_dpp(0, (int)send, 0x4E, 0xF, 0xF, false);
    p0 = upper ? recv : p0;
    p1 = upper ? p1 : recv;
}
template <int BM, int BN, int WGM, int WGN, int EPI, unsigned MASK = 0>
__device__ __forceinline__ void epilogue_sym_reg(const GemmArgs& g, const TileCoord& tc,
                                                 f32x4 (&acc)[BM / WGM / 16][BN / WGN / 16]) {
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    static_assert(FM % 2 == 0 && FN % 2 == 0 && BLK_COLS == 32, "a pair of fragments is one column block");
    static_assert(EPI == EPI_SYRK || EPI == EPI_SYMPOLY, "symmetric products");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WGN, wn = wave % WGN, row = lane >> 4;
    const int m0 = tc.ti * BM, n0 = tc.tj * BN;
    const bool diag = tc.ti == tc.tj;
    // Ct piece (t, j): row n0 + wn*WTN + 16 j + lane%16, columns m0 + wm*WTM + 32 t + 16 (row & 1) + 8 (row >> 1) .. + 7
    const long ct_off = (long)((m0 >> BLK_SHIFT) + wm * (WTM / 32)) * BLK_ELEMS + (wn * WTN + (lane & 15)) * BLK_COLS +
                        (row & 1) * 16 + (row >> 1) * 8;
    bf16_t* Ct = g.Ct + tc.bidx * g.strideCt + panel_offset(n0, g.cbCt) + ct_off;
    // C piece of fragment (i, j): row m0 + wm*WTM + 16 i + 4 row + lane%4, columns n0 + wn*WTN + 16 j + 4 (lane/4 % 4) .. + 3
    bf16_t* C = g.C + tc.bidx * g.strideC + panel_offset(m0, g.cbC) + (long)((n0 >> BLK_SHIFT) + wn * (WTN / 32)) * BLK_ELEMS +
                (wm * WTM + 4 * row + (lane & 3)) * BLK_COLS + ((lane >> 2) & 3) * 4;
    const unsigned sel = (lane & 1) ? 0x03020706u : 0x05040100u;
    const bool upper = (lane & 2) != 0;
    // SYMPOLY: the b.A pieces of EV_AHEAD rows of pairs are in flight at a time; those of row t + EV_AHEAD are fetched
    // when row t starts (all of them at once do not fit beside the accumulators in the persistent kernel)
    bf16x8 ev[EPI == EPI_SYMPOLY ? FM / 2 : 1][EPI == EPI_SYMPOLY ? FN : 1];
    const bf16_t* Et = g.Et + tc.bidx * g.strideEt + panel_offset(n0, g.cbEt) + ct_off;
    constexpr int EV_AHEAD = 2 < FM / 2 ? 2 : FM / 2;  // measured: 3 no faster, 4 spills an accumulator fragment
    auto load_ev = [&](int t) {
#pragma unroll
        for (int j = 0; j < FN; ++j) ev[t][j] = *(const bf16x8*)(Et + j * 16 * BLK_COLS + (long)t * BLK_ELEMS);
    };
    if constexpr (EPI == EPI_SYMPOLY) {
#pragma unroll
        for (int t = 0; t < EV_AHEAD; ++t) load_ev(t);
    }
    auto rounded = [&](float v) {
        v = rbf(v);
        if (EPI == EPI_SYMPOLY) v = g.s1 * v;
        return v;
    };
#pragma unroll
    for (int t = 0; t < FM / 2; ++t) {
        if constexpr (EPI == EPI_SYMPOLY) {
            if (t + EV_AHEAD < FM / 2) load_ev(t + EV_AHEAD);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            // MASK: the fragments that this copy of a diagonal tile's loop has not computed (pp_skip_mask), known when
            // the caller has one copy of the epilogue per mask; the test on the block indices covers the other callers
            if ((MASK >> (2 * t * FN + j)) & 1) continue;
            const int mblk = wm * (WTM / 32) + t, nblk = wn * (WTN / 32) + (j >> 1);
            if (diag && mblk > nblk) continue;  // not computed: the mirror image of a block another wave holds
            const f32x4 a = acc[2 * t][j], b = acc[2 * t + 1][j];
            unsigned a01 = pack_bf16x2(rounded(a[0]), rounded(a[1])), a23 = pack_bf16x2(rounded(a[2]), rounded(a[3]));
            unsigned b01 = pack_bf16x2(rounded(b[0]), rounded(b[1])), b23 = pack_bf16x2(rounded(b[2]), rounded(b[3]));
            u32x2v lo = __builtin_amdgcn_permlane16_swap(a01, b01, false, false);
            u32x2v hi = __builtin_amdgcn_permlane16_swap(a23, b23, false, false);
            if constexpr (EPI == EPI_SYMPOLY) {
                const u32x4 tw = {lo[0], hi[0], lo[1], hi[1]};
                const bf16x8 tv = *(const bf16x8*)&tw;
                bf16x8 o;
#pragma unroll
                for (int k = 0; k < 8; ++k) o[k] = f2bf(rbf(g.s0 * bf2f(ev[t][j][k])) + bf2f(tv[k]));
                *(bf16x8*)(Ct + j * 16 * BLK_COLS + (long)t * BLK_ELEMS) = o;
                if (diag && mblk == nblk) continue;
                const u32x4 ow = *(const u32x4*)&o;
                lo = __builtin_amdgcn_permlane16_swap(ow[0], ow[2], false, false);
                hi = __builtin_amdgcn_permlane16_swap(ow[1], ow[3], false, false);
                a01 = lo[0], b01 = lo[1], a23 = hi[0], b23 = hi[1];
            } else {
                const u32x4 tw = {lo[0], hi[0], lo[1], hi[1]};
                *(u32x4*)(Ct + j * 16 * BLK_COLS + (long)t * BLK_ELEMS) = tw;
                if (diag && mblk == nblk) continue;
            }
            quad_transpose_b16(a01, a23, sel, upper);
            quad_transpose_b16(b01, b23, sel, upper);
            bf16_t* cp = C + (2 * t) * 16 * BLK_COLS + (long)(j >> 1) * BLK_ELEMS + (j & 1) * 16;
            *(u32x2v*)cp = u32x2v{a01, a23};
            *(u32x2v*)(cp + 16 * BLK_COLS) = u32x2v{b01, b23};
        }
    }
}

// Transposing LDS read of a Q fragment of BX: the stage holds the k-tile of X as pieces of 32 columns,
// [piece][k][32 columns] with 64-byte rows, and a fragment is 16 columns x 32 k.  ds_read_b64_tr_b16 works in
// groups of 16 lanes: lane j = 4r+s addresses row k+r, columns 4s..4s+3 of the group's 16 columns, and lane
// i = 4s+e receives rows k..k+3 of column 4s+e; a second read takes rows k+4..k+7.  Group g = lane/16 starts at
// k = 8g, which gives the MFMA operand layout (lane l: column l%16, eight consecutive k from 8*(l/16)).
// Two groups that are served together (g and g^1) would read the same 32-byte window of rows 64*8 bytes = two
// bank rounds apart, so the two 32-byte halves of a row are stored swapped in rows whose k has bit 3 set (the
// global side of the load applies the swap): fragment half h of group g sits at byte (h ^ (g & 1)) * 32.
// qt_lane_offset(lane, h): byte offset of this lane's first read inside the piece, k-step 0.
__device__ __forceinline__ int qt_lane_offset(int lane, int h) {
    const int grp = lane >> 4, i16 = lane & 15;
    return (grp * 8 + (i16 >> 2)) * 64 + ((h ^ (grp & 1)) * 32) + (i16 & 3) * 8;
}
__device__ __forceinline__ bf16x8 lds_read_qt(const unsigned char* q) {
    const s16x4 lo = lds_read_tr16(q), hi4 = lds_read_tr16(q + 4 * 64);
    const s16x8 t = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
    return *(const bf16x8*)&t;
}

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// ---- kernel 1: 64-column k-tiles in two LDS stages, one barrier per k-tile -------------------
// Operand panels go from global memory straight into LDS (global_load_lds_dwordx4): one wave
// instruction fills 1 KB of LDS in lane order, i.e. 8 rows of 128 bytes, so the XOR swizzle
// that keeps the fragment reads conflict free (16-byte chunk c of row r sits at c ^ ((r>>1)&7))
// is applied on the global side: lane L fetches the chunk whose swizzled position is L&7.
// Per k-tile (two 32-column MFMA steps) a wave issues FM*FN*2 MFMAs, (FM+FN)*2 LDS fragment reads and
// LA+LB loads.  Every non-MFMA instruction is placed between two MFMAs so that it issues in their shadow:
//   k-step 0 : MFMAs of step 0 interleaved with the fragment reads of step 1;
//   k-step 1 : the wave has now read everything it needs from this stage, so it waits
//              for its own loads of the next k-tile, crosses the one barrier, and then
//              interleaves the last MFMAs with the loads of k-tile t+2 (into the stage just
//              released) and with the fragment reads of step 0 of k-tile t+1.
// The fences (sched_barrier) pin that order; without them the scheduler sinks every LDS read
// next to its first use and the MFMA pipe idles for an LDS round trip per k-step.  Barriers are
// raw s_barrier with explicit s_waitcnt: __syncthreads() would wait for the loads in flight.
constexpr int ROW_BYTES = 128;

template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_pipe_kernel(const GemmArgs g) {
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
    constexpr int KS = 2;  // 32-column MFMA steps per k-tile
    constexpr int NMF = FM * FN, NRD = FM + FN, NLD = LA + LB;
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "dma split");
    static_assert(epi_is_bx(EPI) || BM == BN, "triangular tiles are square");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const TileCoord tc = decode_tile<EPI>(g);
    constexpr bool QT = epi_is_bx(EPI);  // Q is X itself, rows = reduction index
    const int kb = g.kdim / BLK_COLS;
    const bf16_t* Pb = g.P + tc.bidx * g.strideP + panel_offset(tc.ti * BM, kb);
    const bf16_t* Qb = g.Q + tc.bidx * g.strideQ +
                       (QT ? (long)(tc.tj * BN >> BLK_SHIFT) * BLK_ELEMS : panel_offset(tc.tj * BN, kb));

    const int drow = lane >> 3;
    const bf16_t* pa = Pb + (wave * 8 * LA + drow) * BLK_COLS;
    // BX: a k-tile of Q is BN/32 pieces of 64 rows x 32 columns, each a contiguous 4 KB run of one block;
    // load instruction t of the tile (1 KB) is the quarter t%4 of piece t/4, in lane order, with the two halves
    // of a row swapped in rows whose k has bit 3 set (see qt_lane_offset)
    const bf16_t* pb = QT ? Qb + (lane >> 2) * BLK_COLS + ((lane & 3) ^ (((lane >> 5) & 1) << 1)) * 8
                          : Qb + (wave * 8 * LB + drow) * BLK_COLS;
    const int lds_a = wave * 8 * LA * ROW_BYTES;
    const int lds_b = A_BYTES + wave * 8 * LB * ROW_BYTES;
    // element offset of the 16-byte chunk this lane fetches inside a row of the 64-column k-tile, as an offset
    // in the blocked layout (a k-tile is 64 / BLK_COLS column blocks)
    auto chunk_off = [](int e) { return (long)(e >> BLK_SHIFT) * BLK_ELEMS + (e & (BLK_COLS - 1)); };
    const long ch_even = chunk_off(((lane & 7) ^ (drow >> 1)) * 8), ch_odd = chunk_off(((lane & 7) ^ (4 | (drow >> 1))) * 8);
    constexpr int KT_BLOCKS = 64 / BLK_COLS;

    // load instruction n (0..NLD-1) of k-tile kt: A rows first, then B rows
    auto issue_one = [&](int n, int stage, int kt) {
        unsigned char* s = smem + stage * STAGE;
        if (n < LA) {
            const long ch = ((wave * LA + n) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pa + (long)kt * KT_BLOCKS * BLK_ELEMS + n * 8 * BLK_COLS + ch),
                                             (lds_void_ptr)(s + lds_a + n * 8 * ROW_BYTES), 16, 0, 0);
        } else if (QT) {
            const int i = n - LA, t = wave * LB + i, k0 = kt * 64;
            const long off = ((long)(k0 >> 8) * g.cbQ + (t >> 2)) * BLK_ELEMS + ((k0 & 255) + (t & 3) * 16) * BLK_COLS;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pb + off), (lds_void_ptr)(s + lds_b + i * 8 * ROW_BYTES), 16, 0, 0);
        } else {
            const int i = n - LA;
            const long ch = ((wave * LB + i) & 1) ? ch_odd : ch_even;
            __builtin_amdgcn_global_load_lds((glb_void_ptr)(pb + (long)kt * KT_BLOCKS * BLK_ELEMS + i * 8 * BLK_COLS + ch),
                                             (lds_void_ptr)(s + lds_b + i * 8 * ROW_BYTES), 16, 0, 0);
        }
    };

    f32x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // fragment reads: lane l takes row l%16 of the fragment, 16-byte chunk 4*ks + l/16 of the 128-byte row
    const int sw = (lane >> 1) & 7, kq = lane >> 4;
    const int a_off = (wm * WTM + (lane & 15)) * ROW_BYTES;
    const int b_off = A_BYTES + (wn * WTN + (lane & 15)) * ROW_BYTES;
    const int q_off[2] = {A_BYTES + (wn * WTN / 32) * 4096 + qt_lane_offset(lane, 0),
                          A_BYTES + (wn * WTN / 32) * 4096 + qt_lane_offset(lane, 1)};

    bf16x8 fr[2][NRD];  // fragment double buffer: [0..FM) rows of P, [FM..NRD) rows (BX: columns) of Q
    auto read_one = [&](int buf, int n, const unsigned char* st, int ks) {
        const int co = (((ks << 2) | kq) ^ sw) << 4;
        if (n < FM) fr[buf][n] = *(const bf16x8*)(st + a_off + n * 16 * ROW_BYTES + co);
        else if (QT) fr[buf][n] = lds_read_qt(st + q_off[(n - FM) & 1] + ((n - FM) >> 1) * 4096 + ks * 32 * 64);
        else fr[buf][n] = *(const bf16x8*)(st + b_off + (n - FM) * 16 * ROW_BYTES + co);
    };
    auto mfma_one = [&](int buf, int idx) {
        const int i = idx / FN, j = idx % FN;
        if (QT)  // operands swapped: a lane then holds 4 consecutive columns of one row of the tile
            acc[i][j] = mfma16(fr[buf][FM + j], fr[buf][i], acc[i][j]);
        else
            acc[i][j] = mfma16(fr[buf][i], fr[buf][FM + j], acc[i][j]);
    };

    const int nk = g.kdim / 64;
#pragma unroll
    for (int n = 0; n < NLD; ++n) issue_one(n, 0, 0);
#pragma unroll
    for (int n = 0; n < NLD; ++n) issue_one(n, 1, 1);  // kdim >= 128: there are at least two k-tiles
    WAIT_VM(NLD);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < NRD; ++n) read_one(0, n, smem, 0);

    for (int kt = 0; kt < nk; ++kt) {
        const unsigned char* st = smem + (kt & 1) * STAGE;
        const unsigned char* stn = smem + ((kt + 1) & 1) * STAGE;
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
        // one basic block (a branch here makes the register allocator spill the accumulators).
        WAIT_LGKM0();
        WAIT_VM(0);  // its loads of k-tile kt+1 (the only ones in flight) have landed
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int k2 = kt + 2 < nk ? kt + 2 : nk - 1;
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
    if constexpr (QT) epilogue_nn<BM, BN, WGM, WGN, epi_fold_mode(EPI)>(g, tc, acc, smem);
    else epilogue<BM, BN, WGM, WGN, EPI, false>(g, tc, acc, smem);
}

// 16x16 fragments (i, j) of wave `wave` of a WGM x WGN wave grid whose enclosing 32x32 block lies entirely below
// the diagonal of a diagonal tile (the epilogue masks at that granularity).
template <int WTM, int WTN, int FM, int FN, int WGN>
constexpr unsigned pp_skip_mask(int wave) {
    const int wm = wave / WGN, wn = wave % WGN;
    unsigned m = 0;
    for (int i = 0; i < FM; ++i)
        for (int j = 0; j < FN; ++j)
            if ((wm * WTM + i * 16) / 32 > (wn * WTN + j * 16) / 32) m |= 1u << (i * FN + j);
    return m;
}
template <int WTM, int WTN, int FM, int FN, int WGN>
constexpr bool pp_first_with_mask(int wave) {
    for (int w = 0; w < wave; ++w)
        if (pp_skip_mask<WTM, WTN, FM, FN, WGN>(w) == pp_skip_mask<WTM, WTN, FM, FN, WGN>(wave)) return false;
    return true;
}

// Where the 16-byte chunks of a 64-byte LDS row go: chunk c of a row in row group rg = (row / 4) % 4 sits at
// c ^ pp_swizzle(rg) = c ^ [0, 2, 3, 1][rg].  ds_read_b128 serves a wave in four passes of 16 lanes, and the
// passes are not lanes 0-15, 16-31, ...: the first takes lanes 0-3, 12-15, 20-23, 24-27, the second 4-7, 8-11,
// 16-19, 28-31, the other two the same plus 32.  With fragment lane l on row l%16, chunk l/16, this table is the
// one that gives every pass sixteen different 16-byte bank groups: 256 bytes per clock measured, against 144
// with the plain c ^ rg, which collides two ways in every pass.
__device__ __forceinline__ int pp_swizzle(int rg) { return (0x78 >> (2 * rg)) & 3; }

// ---- kernel 2: eight waves in two groups that alternate between memory and MFMA phases --------
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
template <int BM, int BN, int WGM, int WGN, int EPI>
__device__ __forceinline__ void pp_tile(const GemmArgs& g, const TileCoord& tc, unsigned char* smem) {
    constexpr int NW = WGM * WGN;
    constexpr int BK4 = 32, ROWB = 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 16 / NW, LB = BN / 16 / NW;
    constexpr int NLD = LA + LB;
    static_assert(FM * FN <= 32, "one mask bit per fragment");
    static_assert(NW == 8, "two groups of four waves, one of each per SIMD");
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "dma split");
    static_assert(epi_is_bx(EPI) || BM == BN, "triangular tiles are square");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int wm = wave / WGN, wn = wave % WGN;
    constexpr bool QT = epi_is_bx(EPI);  // Q is X itself, rows = reduction index
    const int kb = g.kdim / BLK_COLS;
    const bf16_t* Pb = uniform_ptr(g.P + tc.bidx * g.strideP + panel_offset(tc.ti * BM, kb));
    const bf16_t* Qb = uniform_ptr(g.Q + tc.bidx * g.strideQ +
                                   (QT ? (long)(tc.tj * BN >> BLK_SHIFT) * BLK_ELEMS : panel_offset(tc.tj * BN, kb)));

    // Loads: a wave-uniform base pointer (advanced along k with scalar adds) plus a 32-bit byte
    // offset per lane, so that no vector ALU instruction is needed per load: in the memory phase
    // every VALU instruction would queue behind the sibling wave's MFMAs.
    const int drow = lane >> 2;
    const int dch = ((lane & 3) ^ pp_swizzle((lane >> 4) & 3)) * 8;
    unsigned offa[LA], offb[LB];
#pragma unroll
    for (int n = 0; n < LA; ++n) offa[n] = (unsigned)(((wave * 16 * LA + n * 16 + drow) * BLK_COLS + dch) * 2);
    // BX: a k-tile of Q is BN/32 pieces of 32 rows x 32 columns, each a contiguous 2 KB run of one block; load
    // instruction t of the tile (1 KB) is the half t%2 of piece t/2, in lane order, with the two 32-byte halves
    // of a row swapped in rows whose k has bit 3 set (see qt_lane_offset)
    const int qch = ((lane & 3) ^ (((drow >> 3) & 1) << 1)) * 8;
#pragma unroll
    for (int n = 0; n < LB; ++n) {
        const int t = wave * LB + n;
        offb[n] = QT ? (unsigned)(((t >> 1) * BLK_ELEMS + ((t & 1) * 16 + drow) * BLK_COLS + qch) * 2)
                     : (unsigned)(((wave * 16 * LB + n * 16 + drow) * BLK_COLS + dch) * 2);
    }
    const int lds_a = wave * 16 * LA * ROWB;
    const int lds_b = A_BYTES + wave * 16 * LB * ROWB;
    const int nk = g.kdim / BK4;

    // global_load_lds_dwordx4 with a scalar base and a 32-bit vector offset; the LDS destination
    // of lane 0 goes through M0 (the wave's 64 lanes fill 1 KB from there in lane order).
    auto dma = [&](const char* base, unsigned voff, unsigned lds_byte) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_byte), "v"(voff), "s"(base)
                     : "memory");
    };
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_void_ptr)smem;
    auto issue_tile = [&](int kt) {  // kt may run past the end: re-load the last k-tile
        const int k0 = (kt < nk ? kt : nk - 1) * BK4;
        const long koff = (long)(k0 >> BLK_SHIFT) * BLK_ELEMS + (k0 & (BLK_COLS - 1));
        const char* ba = (const char*)(Pb + koff);
        const char* bb = (const char*)(Qb + (QT ? (long)(k0 >> 8) * g.cbQ * BLK_ELEMS + (k0 & 255) * BLK_COLS : koff));
        const unsigned st = lds_base + (kt & 3) * STAGE;
#pragma unroll
        for (int n = 0; n < LA; ++n) dma(ba, offa[n], st + lds_a + n * 16 * ROWB);
#pragma unroll
        for (int n = 0; n < LB; ++n) dma(bb, offb[n], st + lds_b + n * 16 * ROWB);
    };

    f32x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    // Diagonal tile of a symmetric product: a fragment of a wave that lies entirely below the diagonal is the
    // mirror image of one another wave computes, and the epilogue does not read it.  Bit i*FN+j of a wave's mask:
    // skip that fragment's MFMAs (and the fragment reads nobody needs).
    const bool diag = !epi_is_bx(EPI) && tc.ti == tc.tj;
    // fragment reads: lane l takes row l%16 of the fragment and the 16-byte chunk l/16 of its 64-byte row
    // (chunk c of row r sits at c ^ pp_swizzle((r>>2)&3))
    const int sw = pp_swizzle((lane >> 2) & 3), kq = lane >> 4;
    const int co = (kq ^ sw) << 4;
    const int a_off = (wm * WTM + (lane & 15)) * ROWB + co;
    const int b_off = A_BYTES + (wn * WTN + (lane & 15)) * ROWB + co;

    issue_tile(0);
    issue_tile(1);
    issue_tile(2);
    WAIT_VM(2 * NLD);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (grp) __builtin_amdgcn_s_barrier();

    // LDS read addresses: one register per operand (BX: per half of a piece) and pair of stages; the stage
    // inside the pair and the fragment index are instruction offsets (below 64 KB) once the k loop is unrolled
    // by the four stages.
    const unsigned char* ra[2];
    const unsigned char* rb[2][2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        ra[half] = smem + half * 2 * STAGE + a_off;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            rb[half][h] = QT ? smem + half * 2 * STAGE + A_BYTES + (wn * WTN / 32) * 2048 + qt_lane_offset(lane, h)
                             : smem + half * 2 * STAGE + b_off;
    }
    auto body = [&](int kt, auto stage_c, auto mask_c) {
        constexpr int SIDX = decltype(stage_c)::value;
        constexpr unsigned MASK = decltype(mask_c)::value;
        auto kept = [](int i, int j) { return !((MASK >> (i * FN + j)) & 1); };
        // ---- M(kt)
        bf16x8 fa[FM], fb[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            bool used = false;
#pragma unroll
            for (int j = 0; j < FN; ++j) used |= kept(i, j);
            if (used) fa[i] = *(const bf16x8*)(ra[SIDX >> 1] + (SIDX & 1) * STAGE + i * 16 * ROWB);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            bool used = false;
#pragma unroll
            for (int i = 0; i < FM; ++i) used |= kept(i, j);
            if (!used) continue;
            if (QT) fb[j] = lds_read_qt(rb[SIDX >> 1][j & 1] + (SIDX & 1) * STAGE + (j >> 1) * 2048);
            else fb[j] = *(const bf16x8*)(rb[SIDX >> 1][0] + (SIDX & 1) * STAGE + j * 16 * ROWB);
        }
        issue_tile(kt + 3);
        WAIT_LGKM0();
        WAIT_VM(2 * NLD);  // own loads of k-tile kt+1 have landed
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // ---- C(kt): column fragment outermost, so that consecutive MFMAs share the Q fragment (measured +1 to 2 %
        // for B.X against rows outermost)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int ii = 0; ii < FM; ++ii) {
                const int i = (j & 1) ? FM - 1 - ii : ii;
                if (QT)  // operands swapped: a lane then holds 4 consecutive columns of one row of the tile
                    acc[i][j] = mfma16(fb[j], fa[i], acc[i][j]);
                else if (kept(i, j))
                    acc[i][j] = mfma16(fa[i], fb[j], acc[i][j]);
            }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    // nk is a multiple of 4 (k extents are multiples of 128)
    auto k_loop = [&](auto mask_c) {
        for (int kt = 0; kt < nk; kt += 4) {
            body(kt, std::integral_constant<int, 0>{}, mask_c);
            body(kt + 1, std::integral_constant<int, 1>{}, mask_c);
            body(kt + 2, std::integral_constant<int, 2>{}, mask_c);
            body(kt + 3, std::integral_constant<int, 3>{}, mask_c);
        }
    };
    // One copy of the loop per distinct mask (the masks are compile-time facts of the wave grid), chosen once per
    // tile: no test inside the loop.  Tiles off the diagonal, nearly all, take the first.
    if (!diag) {
        k_loop(std::integral_constant<unsigned, 0>{});
    } else {
        auto run_if_mine = [&](auto wave_c) {
            constexpr int W = decltype(wave_c)::value;
            constexpr unsigned M = pp_skip_mask<WTM, WTN, FM, FN, WGN>(W);
            if constexpr (pp_first_with_mask<WTM, WTN, FM, FN, WGN>(W)) {
                if (pp_skip_mask<WTM, WTN, FM, FN, WGN>(wave) == M) k_loop(std::integral_constant<unsigned, M>{});
            }
        };
        run_if_mine(std::integral_constant<int, 0>{});
        run_if_mine(std::integral_constant<int, 1>{});
        run_if_mine(std::integral_constant<int, 2>{});
        run_if_mine(std::integral_constant<int, 3>{});
        run_if_mine(std::integral_constant<int, 4>{});
        run_if_mine(std::integral_constant<int, 5>{});
        run_if_mine(std::integral_constant<int, 6>{});
        run_if_mine(std::integral_constant<int, 7>{});
    }
    if (!grp) __builtin_amdgcn_s_barrier();
    if constexpr (EPI == EPI_BX) {
        // no LDS in this epilogue: the loads issued past the end may land while it runs (its own loads are behind
        // them in the queue, so they have landed before the wave ends)
        epilogue_nn_reg<BM, BN, WGM, WGN>(g, tc, acc);
        return;
    }
    if constexpr (EPI == EPI_SYMPOLY && BM == 256) {
        // measured: without LDS b.A + c.A.A is 0.5 % faster on whole 256-tiles, X.Xt 0.6 % slower
        epilogue_sym_reg<BM, BN, WGM, WGN, EPI>(g, tc, acc);
        return;
    }
    WAIT_VM(0);  // the loads issued past the end must not land in the epilogue's tile
    if constexpr (QT) epilogue_nn<BM, BN, WGM, WGN, epi_fold_mode(EPI)>(g, tc, acc, smem);
    else epilogue<BM, BN, WGM, WGN, EPI, true>(g, tc, acc, smem);
}

template <int BM, int BN, int WGM, int WGN, int EPI>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_nt_pp_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) unsigned char smem[];
    pp_tile<BM, BN, WGM, WGN, EPI>(g, decode_tile<EPI>(g), smem);
}

// The same with a split tail: when the tile count leaves the last round of the compute units mostly empty,
// the first g.big_blocks workgroups compute 256x256 tiles as above and every remaining tile is cut
// into four 128x128 tiles, one workgroup each, which fill the CUs that would otherwise idle for a
// whole tile time.  The lower-left quarter of a diagonal tile of the symmetric kernels is the mirror
// of the upper-right one and is skipped.
template <int EPI>
__global__ void __launch_bounds__(512) gemm_nt_pp_tail_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) unsigned char smem[];
    if ((int)blockIdx.x < g.big_blocks) {
        pp_tile<256, 256, 2, 4, EPI>(g, tile_of<EPI>(g, xcd_remap(blockIdx.x, g.big_blocks, g.xcd_shift)), smem);
    } else {
        const int s = blockIdx.x - g.big_blocks, quarter = s & 3;
        TileCoord tc = tile_of<EPI>(g, g.big_blocks + (s >> 2));
        if (!epi_is_bx(EPI) && tc.ti == tc.tj && quarter == 2) return;
        tc.ti = tc.ti * 2 + (quarter >> 1);
        tc.tj = tc.tj * 2 + (quarter & 1);
        pp_tile<128, 128, 2, 4, EPI>(g, tc, smem);
    }
}

// ---- kernel 3: the ping-pong loop as a persistent kernel ----------------------------------------
// With an epilogue that needs no LDS (epilogue_nn_reg, epilogue_sym_reg) nothing stands between the k loops of two tiles: one
// workgroup per compute unit walks tiles, the last three memory phases of a tile issue the first three k-tiles of the
// workgroup's NEXT tile into the stages the current one has finished with, and they land while the waves drain their
// accumulators.  What a one-tile workgroup pays around its k loop on top of the epilogue - the cold first loads (2 to
// 3 us) and the hand-over of the compute unit to the next workgroup (2 to 3 us) - is a sixth of a tile when the
// reduction is 24 k-tiles long (a 768-row expert matrix) and 4 % at 128.
//
// Tiles are handed out per XCD, in the order xcd_remap gives a one-tile-per-workgroup launch: workgroup b sits on
// XCD b % 8 and takes "virtual workgroup ids" 8 n + b % 8.  Its first two n are static (b / 8 and b / 8 + grid / 8),
// later ones come from an atomic counter of its XCD, asked for during the epilogue of the tile before the one whose
// last phases need it.  The counters are the caller's (GemmArgs::ppx, a piece of the workspace of the call): a launch
// finds them zero, and the last workgroup to leave puts them back to zero, so the library keeps no state of its own
// and calls with different workspaces do not meet.
struct PpxCounters {
    unsigned next[GEMM_MAX_XCDS][16];  // a cache line per XCD: tiles handed out beyond the two static rounds
    unsigned done[16];                 // workgroups that have left
};
static_assert(sizeof(PpxCounters) == GEMM_PPX_COUNTER_BYTES, "the size the header promises");

template <int EPI>
__global__ void __launch_bounds__(512) gemm_nt_ppx_kernel(const GemmArgs g) {
    static_assert(EPI == EPI_BX || EPI == EPI_SYRK || EPI == EPI_SYMPOLY, "the epilogues that need no LDS");
    constexpr bool QT = EPI == EPI_BX;  // Q is X itself, rows = reduction index
    constexpr int BM = 256, BN = 256, WGM = 2, WGN = 4, NW = 8;
    constexpr int BK4 = 32, ROWB = 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 16, FN = WTN / 16;
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int LA = BM / 16 / NW, LB = BN / 16 / NW;
    constexpr int NLD = LA + LB;
    constexpr int SLOT_OFF = 4 * STAGE;  // behind the four stages: where lane 0 leaves the next tile's id for the others

    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int wm = wave / WGN, wn = wave % WGN;
    const int kb = g.kdim / BLK_COLS;
    const int total = g.tiles_per_mat * g.batch;
    const int grid = gridDim.x, xcds = 1 << g.xcd_shift, xcd = blockIdx.x & (xcds - 1);
    PpxCounters& ctr = *(PpxCounters*)g.ppx;

    auto panel_p = [&](const TileCoord& t) { return uniform_ptr(g.P + t.bidx * g.strideP + panel_offset(t.ti * BM, kb)); };
    auto panel_q = [&](const TileCoord& t) {
        return uniform_ptr(g.Q + t.bidx * g.strideQ +
                           (QT ? (long)(t.tj * BN >> BLK_SHIFT) * BLK_ELEMS : panel_offset(t.tj * BN, kb)));
    };

    // per-lane load offsets and LDS addresses: as in pp_tile
    const int drow = lane >> 2;
    const int dch = ((lane & 3) ^ pp_swizzle((lane >> 4) & 3)) * 8;
    unsigned offa[LA], offb[LB];
#pragma unroll
    for (int n = 0; n < LA; ++n) offa[n] = (unsigned)(((wave * 16 * LA + n * 16 + drow) * BLK_COLS + dch) * 2);
    const int qch = ((lane & 3) ^ (((drow >> 3) & 1) << 1)) * 8;
#pragma unroll
    for (int n = 0; n < LB; ++n) {
        const int t = wave * LB + n;
        offb[n] = QT ? (unsigned)(((t >> 1) * BLK_ELEMS + ((t & 1) * 16 + drow) * BLK_COLS + qch) * 2)
                     : (unsigned)(((wave * 16 * LB + n * 16 + drow) * BLK_COLS + dch) * 2);
    }
    const int lds_a = wave * 16 * LA * ROWB;
    const int lds_b = A_BYTES + wave * 16 * LB * ROWB;
    const int nk = g.kdim / BK4;  // a multiple of 4, at least 8 (the launcher checks)

    auto dma = [&](const char* base, unsigned voff, unsigned lds_byte) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_byte), "v"(voff), "s"(base)
                     : "memory");
    };
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_void_ptr)smem;
    // k-tile kt of the tile whose panels are (P, Q), into stage kt & 3
    auto issue_tile = [&](const bf16_t* P, const bf16_t* Q, int kt) {
        const int k0 = kt * BK4;
        const long koff = (long)(k0 >> BLK_SHIFT) * BLK_ELEMS + (k0 & (BLK_COLS - 1));
        const char* ba = (const char*)(P + koff);
        const char* bb = (const char*)(Q + (QT ? (long)(k0 >> 8) * g.cbQ * BLK_ELEMS + (k0 & 255) * BLK_COLS : koff));
        const unsigned st = lds_base + (kt & 3) * STAGE;
#pragma unroll
        for (int n = 0; n < LA; ++n) dma(ba, offa[n], st + lds_a + n * 16 * ROWB);
#pragma unroll
        for (int n = 0; n < LB; ++n) dma(bb, offb[n], st + lds_b + n * 16 * ROWB);
    };

    const int sw = pp_swizzle((lane >> 2) & 3), kq = lane >> 4;
    const int co = (kq ^ sw) << 4;
    const int a_off = (wm * WTM + (lane & 15)) * ROWB + co;
    const int b_off = A_BYTES + (wn * WTN + (lane & 15)) * ROWB + co;
    const unsigned char* ra[2];
    const unsigned char* rb[2][2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        ra[half] = smem + half * 2 * STAGE + a_off;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            rb[half][h] = QT ? smem + half * 2 * STAGE + A_BYTES + (wn * WTN / 32) * 2048 + qt_lane_offset(lane, h)
                             : smem + half * 2 * STAGE + b_off;
    }

    // this workgroup's tiles: the current one, the one after it (virtual ids; >= total means none)
    int pid_cur = blockIdx.x, pid_nxt = blockIdx.x + grid;
    TileCoord tc = tile_of<EPI>(g, xcd_remap(pid_cur, total, g.xcd_shift));
    const bf16_t* Pb = panel_p(tc);
    const bf16_t* Qb = panel_q(tc);

    issue_tile(Pb, Qb, 0);
    issue_tile(Pb, Qb, 1);
    issue_tile(Pb, Qb, 2);
    WAIT_VM(0);  // a tile starts with its k-tiles 0, 1 and 2 in LDS
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (grp) __builtin_amdgcn_s_barrier();

    for (;;) {
        const bool has_next = pid_nxt < total;
        // without a next tile the last phases load this tile's first k-tiles again, into stages nobody reads any more
        const TileCoord ntc = has_next ? tile_of<EPI>(g, xcd_remap(pid_nxt, total, g.xcd_shift)) : tc;
        const bf16_t* Pn = panel_p(ntc);
        const bf16_t* Qn = panel_q(ntc);

        const bool diag = !QT && tc.ti == tc.tj;
        unsigned fetched = 0;
        // One tile, k loop and epilogue, for the waves whose skip mask in a diagonal tile is `mask_c` (pp_tile): a copy of
        // its own per mask, each with its own accumulators from the first MFMA to the last store.
        auto run_tile = [&](auto mask_c) {
            f32x4 acc[FM][FN];  // defined by the MFMAs of the tile's first k-tile, which add to zero

            // NEXT: the memory phase issues k-tile kt+3-nk of the next tile instead of k-tile kt+3 of this one.
            // NOWAIT: the first two phases of a tile wait for no load: its k-tiles 0, 1 and 2 are in LDS when it starts
            // (a count would make them wait for the stores of the epilogue before).
            constexpr unsigned MASK = decltype(mask_c)::value;  // fragments a wave skips in a diagonal tile
            auto body = [&](int kt, auto stage_c, auto next_c, auto nowait_c, auto first_c) {
                constexpr int SIDX = decltype(stage_c)::value;
                constexpr bool NEXT = decltype(next_c)::value;
                constexpr bool NOWAIT = decltype(nowait_c)::value;
                constexpr bool FIRST = decltype(first_c)::value;
                auto kept = [](int i, int j) { return !((MASK >> (i * FN + j)) & 1); };
                bf16x8 fa[FM], fb[FN];
    #pragma unroll
                for (int i = 0; i < FM; ++i) {
                    bool used = false;
    #pragma unroll
                    for (int j = 0; j < FN; ++j) used |= kept(i, j);
                    if (used) fa[i] = *(const bf16x8*)(ra[SIDX >> 1] + (SIDX & 1) * STAGE + i * 16 * ROWB);
                }
    #pragma unroll
                for (int j = 0; j < FN; ++j) {
                    bool used = false;
    #pragma unroll
                    for (int i = 0; i < FM; ++i) used |= kept(i, j);
                    if (!used) continue;
                    if (QT) fb[j] = lds_read_qt(rb[SIDX >> 1][j & 1] + (SIDX & 1) * STAGE + (j >> 1) * 2048);
                    else fb[j] = *(const bf16x8*)(rb[SIDX >> 1][0] + (SIDX & 1) * STAGE + j * 16 * ROWB);
                }
                if constexpr (NEXT) issue_tile(Pn, Qn, kt + 3 - nk);
                else issue_tile(Pb, Qb, kt + 3);
                WAIT_LGKM0();
                if constexpr (!NOWAIT) WAIT_VM(2 * NLD);  // own loads of k-tile kt+1 have landed
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
                for (int j = 0; j < FN; ++j)
    #pragma unroll
                    for (int ii = 0; ii < FM; ++ii) {
                        const int i = (j & 1) ? FM - 1 - ii : ii;  // back and forth: consecutive MFMAs share an operand
                        const f32x4 c = FIRST ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[i][j];
                        if (QT) acc[i][j] = mfma16(fb[j], fa[i], c);
                        else if (kept(i, j)) acc[i][j] = mfma16(fa[i], fb[j], c);
                    }
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            using I3 = std::integral_constant<int, 3>;
            using No = std::false_type;
            using Yes = std::true_type;
            body(0, I0{}, No{}, Yes{}, Yes{});
            body(1, I1{}, No{}, Yes{}, No{});
            body(2, I2{}, No{}, No{}, No{});
            body(3, I3{}, No{}, No{}, No{});
            for (int kt = 4; kt < nk - 4; kt += 4) {
                body(kt, I0{}, No{}, No{}, No{});
                body(kt + 1, I1{}, No{}, No{}, No{});
                body(kt + 2, I2{}, No{}, No{}, No{});
                body(kt + 3, I3{}, No{}, No{}, No{});
            }
            body(nk - 4, I0{}, No{}, No{}, No{});
            body(nk - 3, I1{}, Yes{}, No{}, No{});
            body(nk - 2, I2{}, Yes{}, No{}, No{});
            body(nk - 1, I3{}, Yes{}, No{}, No{});
            if (!grp) __builtin_amdgcn_s_barrier();  // the two groups leave the k loop together

            // Every wave drains its accumulators on its own.  One lane asks for the id of the tile after the next (an
            // increment with wrap-around at 2^32 - 1: a plain atomicAdd of a uniform value is turned into a wave-wide
            // reduction by the compiler, which then waits for the answer on the spot); the answer is needed at the end.
            if (has_next && tid == 0) fetched = atomicInc(&ctr.next[xcd][0], 0xffffffffu);
            if constexpr (QT) {
                epilogue_nn_reg<BM, BN, WGM, WGN>(g, tc, acc);
            } else {
                epilogue_sym_reg<BM, BN, WGM, WGN, EPI, MASK>(g, tc, acc);
                // What says that this wave's share of the next tile's first k-tiles has landed: B.X and b.A + c.A.A consume
                // loads that were issued after them (the queue returns in order).  X.Xt loads nothing, and in a diagonal
                // tile a wave may have nothing to finish at all: there the count is explicit (48 stores went out after the
                // loads off the diagonal, an unknown number on it).
                asm volatile("" ::: "memory");
                if (diag) WAIT_VM(0);
                else if (EPI == EPI_SYRK) WAIT_VM(FM * FN / 2 * 3);
                asm volatile("" ::: "memory");
            }
        };  // run_tile
        if (!diag) {
            run_tile(std::integral_constant<unsigned, 0>{});
        } else {
            auto run_if_mine = [&](auto wave_c) {
                constexpr int W = decltype(wave_c)::value;
                constexpr unsigned M = pp_skip_mask<WTM, WTN, FM, FN, WGN>(W);
                if constexpr (pp_first_with_mask<WTM, WTN, FM, FN, WGN>(W)) {
                    if (pp_skip_mask<WTM, WTN, FM, FN, WGN>(wave) == M) run_tile(std::integral_constant<unsigned, M>{});
                }
            };
            run_if_mine(std::integral_constant<int, 0>{});
            run_if_mine(std::integral_constant<int, 1>{});
            run_if_mine(std::integral_constant<int, 2>{});
            run_if_mine(std::integral_constant<int, 3>{});
            run_if_mine(std::integral_constant<int, 4>{});
            run_if_mine(std::integral_constant<int, 5>{});
            run_if_mine(std::integral_constant<int, 6>{});
            run_if_mine(std::integral_constant<int, 7>{});
        }
        // (the answer stays untouched until here: any arithmetic on it would be scheduled next to the atomic, with a
        // wait for it)
        asm volatile("" : "+v"(fetched));
        if (tid == 0) *(int*)(smem + SLOT_OFF) = has_next ? (((2 * (grid >> g.xcd_shift) + (int)fetched)) << g.xcd_shift) + xcd : total;
        // The loads of the epilogue are behind those of the next tile's first k-tiles in the queue and have been
        // consumed, so every wave's share of those k-tiles has landed: publish them, and the id.
        __syncthreads();
        if (!has_next) break;
        pid_cur = pid_nxt;
        pid_nxt = __builtin_amdgcn_readfirstlane(*(const int*)(smem + SLOT_OFF));
        tc = ntc;
        Pb = Pn;
        Qb = Qn;
        if (grp) __builtin_amdgcn_s_barrier();  // and enter the next tile a phase apart again
    }
    if (tid == 0) {
        // every workgroup has its last answer from `next` before it counts itself out, so the last one out may reset
        if (atomicAdd(&ctr.done[0], 1u) == (unsigned)grid - 1) {
            for (int x = 0; x < xcds; ++x) atomicExch(&ctr.next[x][0], 0u);
            atomicExch(&ctr.done[0], 0u);
        }
    }
}

// Dynamic LDS beyond 64 KB has to be allowed per kernel, and the attribute belongs to the device that is current when
// it is set: once per (kernel instantiation, device), remembered as one bit per device in the instantiation's mask.
hipError_t allow_dynamic_lds(const void* kern, int bytes, std::atomic<unsigned long long>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return e;
    done.fetch_or(bit, std::memory_order_release);
    return hipSuccess;
}

template <int EPI>
hipError_t launch_ppx(const GemmArgs& g, int nblocks, int cus, hipStream_t stream) {
    constexpr int smem = 4 * (256 + 256) * 64 + 64;
    static std::atomic<unsigned long long> configured{0};  // per instantiation
    if (hipError_t e = allow_dynamic_lds((const void*)gemm_nt_ppx_kernel<EPI>, smem, configured); e != hipSuccess) return e;
    const int grid = nblocks < cus ? nblocks : cus;  // a whole number of XCDs: the caller launches more tiles than CUs
    hipLaunchKernelGGL(gemm_nt_ppx_kernel<EPI>, dim3(grid), dim3(512), smem, stream, g);
    return hipGetLastError();
}

template <int BM, int BN, int WGM, int WGN, int EPI, int FEED>
hipError_t launch_one(const GemmArgs& g, int nblocks, hipStream_t stream) {
    constexpr int stages = 2 * (BM + BN) * ROW_BYTES;
    constexpr int epi = epi_is_bx(EPI) ? epilogue_nn_bytes<BM, BN>() : epilogue_bytes<BM, BN>();
    constexpr int smem = stages > epi ? stages : epi;
    static std::atomic<unsigned long long> configured{0};  // per instantiation; setting the attribute twice is harmless
    void (*kern)(const GemmArgs);
    if constexpr (FEED == 1) kern = gemm_nt_pp_kernel<BM, BN, WGM, WGN, EPI>;
    else kern = gemm_nt_pipe_kernel<BM, BN, WGM, WGN, EPI>;
    if (hipError_t e = allow_dynamic_lds((const void*)kern, smem, configured); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(nblocks), dim3(WGM * WGN * 64), smem, stream, g);
    return hipGetLastError();
}

template <int EPI>
hipError_t launch_cfg(int cfg, const GemmArgs& g, int nblocks, hipStream_t stream) {
    switch (cfg) {
        case GEMM_CFG_128_PIPE: return launch_one<128, 128, 2, 2, EPI, 0>(g, nblocks, stream);
        case GEMM_CFG_256_PIPE: return launch_one<256, 256, 2, 4, EPI, 0>(g, nblocks, stream);
        case GEMM_CFG_256_PINGPONG: return launch_one<256, 256, 2, 4, EPI, 1>(g, nblocks, stream);
        case GEMM_CFG_128_PINGPONG: return launch_one<128, 128, 2, 4, EPI, 1>(g, nblocks, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int gemm_cfg_tile(int cfg) {
    switch (cfg) {
        case GEMM_CFG_128_PIPE:
        case GEMM_CFG_128_PINGPONG: return 128;
        case GEMM_CFG_256_PIPE:
        case GEMM_CFG_256_PINGPONG:
        case GEMM_CFG_256_PERSIST: return 256;
        default: return 0;
    }
}

template <int EPI>
hipError_t launch_pp_tail(GemmArgs g, int nblocks, int rest, hipStream_t stream) {
    constexpr int stages = 2 * (256 + 256) * ROW_BYTES;
    constexpr int epi = epi_is_bx(EPI) ? epilogue_nn_bytes<256, 256>() : epilogue_bytes<256, 256>();
    constexpr int smem = stages > epi ? stages : epi;  // the 128-tiles need less of both
    static std::atomic<unsigned long long> configured{0};
    auto kern = gemm_nt_pp_tail_kernel<EPI>;
    if (hipError_t e = allow_dynamic_lds((const void*)kern, smem, configured); e != hipSuccess) return e;
    g.big_blocks = nblocks - rest;
    hipLaunchKernelGGL(kern, dim3(g.big_blocks + 4 * rest), dim3(512), smem, stream, g);
    return hipGetLastError();
}

#ifndef PPX_SYRK_MAXK
#define PPX_SYRK_MAXK 2048
#endif
#ifndef PPX_SYMPOLY_MAXK
#define PPX_SYMPOLY_MAXK 2048
#endif
hipError_t machine_shape(MachineShape& ms) {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];  // compute units per device ordinal, 0 = not read yet
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    int cus = (dev >= 0 && dev < kMaxDevices) ? cached[dev].load(std::memory_order_relaxed) : 0;
    if (cus == 0) {
        if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev); e != hipSuccess) return e;
        if (cus <= 0) return hipErrorInvalidDevice;
        if (dev >= 0 && dev < kMaxDevices) cached[dev].store(cus, std::memory_order_relaxed);
    }
    ms.cus = cus;
    int xcds = cus / 32;  // 32 active compute units per XCD on gfx950
    ms.xcd_shift = 0;
    while ((2 << ms.xcd_shift) <= xcds && (2 << ms.xcd_shift) <= GEMM_MAX_XCDS && cus % (2 << ms.xcd_shift) == 0) ++ms.xcd_shift;
    return hipSuccess;
}

hipError_t launch_gemm_nt(int cfg, int epi, const GemmArgs& args, hipStream_t stream) {
    GemmArgs g = args;
    MachineShape ms;
    if (hipError_t e = machine_shape(ms); e != hipSuccess) return e;
    g.xcd_shift = ms.xcd_shift;
    const int cus = ms.cus;
    const int nblocks = g.tiles_per_mat * g.batch;
    if (nblocks <= 0) return hipSuccess;
    // Ping-pong kernel: split the tiles of a last round that would fill at most a quarter of the CUs (a 128x128
    // tile takes about 0.6 of the time of a 256x256 one, so one round of quarters beats a round of whole tiles).
    const int rest = nblocks % cus;
    if (cfg == GEMM_CFG_256_PERSIST) {
        // at least 8 k-tiles, more tiles than compute units and a counter buffer; everything else takes the one-tile kernel
        if (g.kdim >= 256 && nblocks > cus && g.ppx) {
            if (epi == EPI_BX) return launch_ppx<EPI_BX>(g, nblocks, cus, stream);
            if (epi == EPI_SYRK && g.kdim <= PPX_SYRK_MAXK) return launch_ppx<EPI_SYRK>(g, nblocks, cus, stream);
            if (epi == EPI_SYMPOLY && g.kdim <= PPX_SYMPOLY_MAXK) return launch_ppx<EPI_SYMPOLY>(g, nblocks, cus, stream);
        }
        cfg = GEMM_CFG_256_PINGPONG;
    }
    if (cfg == GEMM_CFG_256_PINGPONG && nblocks > cus && rest > 0 && rest <= cus / 4) {
        switch (epi) {
            case EPI_SYRK: return launch_pp_tail<EPI_SYRK>(g, nblocks, rest, stream);
            case EPI_SYMPOLY: return launch_pp_tail<EPI_SYMPOLY>(g, nblocks, rest, stream);
            case EPI_BX: return launch_pp_tail<EPI_BX>(g, nblocks, rest, stream);
            case EPI_BX_UPD: return launch_pp_tail<EPI_BX_UPD>(g, nblocks, rest, stream);
            case EPI_BX_UPD_T: return launch_pp_tail<EPI_BX_UPD_T>(g, nblocks, rest, stream);
            default: return hipErrorInvalidValue;
        }
    }
    switch (epi) {
        case EPI_SYRK: return launch_cfg<EPI_SYRK>(cfg, g, nblocks, stream);
        case EPI_SYMPOLY: return launch_cfg<EPI_SYMPOLY>(cfg, g, nblocks, stream);
        case EPI_BX: return launch_cfg<EPI_BX>(cfg, g, nblocks, stream);
        case EPI_BX_UPD: return launch_cfg<EPI_BX_UPD>(cfg, g, nblocks, stream);
        case EPI_BX_UPD_T: return launch_cfg<EPI_BX_UPD_T>(cfg, g, nblocks, stream);
        default: return hipErrorInvalidValue;
    }
}
