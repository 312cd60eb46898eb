// Multi-token unpack-dequantise-matmul with the de-quantised weights staged in LDS (2-, 3- and 4-bit codes).
//
// A block of four waves owns a tile of output rows that share their scale / zero rows and a batch tile of BMT
// columns, and walks its K range in steps of 64 columns.  Per step
//   * the table entries of the tile (8 or 10 table rows x 64 columns, 8-bit with their meta values or fp16) are
//     de-quantised once into LDS, fp16(fp16(q - mz) * ms) as the reference does (src/custom_layers.py:63-66);
//   * every thread rebuilds 32 or 40 weights bit-exactly, w = fp16(fp16(q - z) * s) (src/custom_layers.py:111):
//     the code field is inserted into the mantissa of a power of two (one v_bfi per pair), the power is subtracted,
//     then zero and scale are applied on pairs; the weights go to LDS as a plain [row][k] fp16 tile;
//   * the x tile is copied to LDS as it is, [batch row][k];
//   * the waves run v_mfma_f32_16x16x32_f16 over the two tiles: 64 x 64 outputs per wave at the widest batch tile,
//     one 128-bit LDS read per operand of four MFMAs.
// Every weight is rebuilt once per block, whatever the width of the batch tile, which is what the register-built
// tile kernel (gemm_tile.hip) cannot do: there each wave rebuilds the weights of its own 16 batch columns.
//
// Rows of a tile.  2- and 4-bit: the packed table rows jt*JPB .. +JPB-1 (F*JPB = 8 consecutive table rows) by 16
// packed rows r = 16*rb .. 16*rb+15 by F fields, 128 output rows n = F*(jp + r*GP) + i.  3-bit: the word rows
// w0 + P*(16*rb + t), t = 0..15, of one window w0 (they share ten table rows, P = G / gcd(10, G)), ten fields each,
// 160 row slots.  Steps are double-buffered in LDS with one barrier per step; codes and tables are requested four
// steps ahead into registers, the x tile (which comes from L2) two steps ahead.  Loads are unconditional (a step
// past the end re-reads the last one, a batch row past M the last row) so that the compiler's wait counts are
// exact.  K may be split over blocks: fp32 partial sums [K block][M][N] and a finishing kernel.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"

namespace hqq {
using namespace gemv;
namespace {

constexpr int kLK = 64;          // columns per step
constexpr int kLPitch = kLK + 8; // halves per LDS row: 144 bytes, so that sixteen rows fall into sixteen bank groups
constexpr int kLThreads = 256;

struct LdsParams {
    const uint8_t *codes;
    const uint8_t *sq, *zq; // table data, 8-bit or fp16
    const f16 *s_ms, *s_mz; // per-column meta of the scale table
    const f16 *z_ms, *z_mz; // whole-tensor meta of the zero table
    uint32_t s_cols, s_inv;
    const f16 *x;
    f16 *y;
    const f16 *bias;
    float *part; // [KSP][M][N] when K is split over blocks, else null
    const f16 *row_scale;
    int accumulate;
    int M, N, K, G, GP;
    int KSP, KTS; // blocks along K, steps per block
    int P, NW;    // 3-bit: window period, word rows
};

template <int NBITS> struct LdsGeo {
    static constexpr int F = 8 / NBITS;
    static constexpr int JPB = 8 / F; // packed table rows per tile: eight table rows
    static constexpr int BN = 128, TROWS = 8, NRB = 8;
    static constexpr int CODE_BYTES = NBITS == 2 ? 8 : 16; // per thread and step
};
template <> struct LdsGeo<3> {
    static constexpr int F = 10;
    static constexpr int BN = 160, TROWS = 10, NRB = 10;
};

// position of a field inside the 16-bit half that holds it, the mask that selects it there, the exponent bits of the
// power of two 2^(10 - pos) whose mantissa it is inserted into (the sum then reads 2^(10 - pos) + q), and that power
__host__ __device__ constexpr uint32_t lds_mask(int nbits, int pos) { return (((1u << nbits) - 1u) * 0x00010001u) << pos; }
__host__ __device__ constexpr uint32_t lds_expo(int pos) { return (uint32_t)((10 - pos + 15) << 10) * 0x00010001u; }
__host__ __device__ constexpr float lds_power(int pos) { return (float)(1 << (10 - pos)); }
__host__ __device__ constexpr int w3pos(int i) { return (3 * (9 - i)) & 7; }
// byte selector that brings, for two words (k even in the second operand, k odd in the first), the two bytes holding
// field i into the low and the high half
__host__ __device__ constexpr uint32_t w3sel(int i)
{
    const uint32_t B = (uint32_t)(3 * (9 - i)) >> 3;
    const uint32_t lo0 = B, hi0 = B < 3 ? B + 1 : 0x0cu, lo1 = 4 + B, hi1 = B < 3 ? 4 + B + 1 : 0x0cu;
    return (hi1 << 24) | (lo1 << 16) | (hi0 << 8) | lo0;
}

__device__ __forceinline__ f16x2 h2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }
__device__ __forceinline__ uint32_t u32(f16x2 v) { return __builtin_bit_cast(uint32_t, v); }

// one pair of weights: codes in the low bytes of the two halves of `src` at bit `pos`
template <int NBITS> __device__ __forceinline__ uint32_t rebuild_pair(uint32_t src, int pos_c, uint32_t z, uint32_t s)
{
    const uint32_t mk = lds_mask(NBITS, pos_c), ex = lds_expo(pos_c);
    const f16 offv = (f16)lds_power(pos_c);
    const f16x2 off = {offv, offv};
    const f16x2 q = h2((mk & src) | (~mk & ex)) - off; // the exact code (one v_bfi_b32)
    return u32((q - h2(z)) * h2(s));                   // two fp16 roundings, as the reference
}

struct LdsWeightRegs {
    u32x4 cw; // 8 or 16 code bytes (2 / 4 bit), four words (3 bit)
};
struct LdsTableRegs {
    u32x2 d[2];  // four table bytes in .x (8-bit) or four halves (fp16), per item
    u32x2 ms[2]; // scale items only: four halves of meta scale / meta zero
    u32x2 mz[2];
};

// Q8: scale 8-bit with per-column meta and zero 8-bit with whole-tensor meta (what HQQ writes), else fp16 tables
template <int NBITS, int BMT, bool Q8>
__global__ __launch_bounds__(kLThreads, 2) void gemm_lds_kernel(LdsParams p)
{
    using Geo = LdsGeo<NBITS>;
    constexpr int F = Geo::F, BN = Geo::BN, TROWS = Geo::TROWS, NRB = Geo::NRB;
    constexpr int NCB = BMT / 16;                 // column blocks of the batch tile
    constexpr int WC = BMT >= 128 ? 2 : 1;        // waves across the batch tile
    constexpr int WR = 4 / WC;                    // waves down the rows
    constexpr int RBW = (NRB + WR - 1) / WR;      // row blocks per wave (the last wave of a 3-bit tile has fewer)
    constexpr int CBW = NCB / WC;                 // column blocks per wave
    constexpr int XCH = (BMT * 8 + kLThreads - 1) / kLThreads; // 16-byte chunks of the x tile per thread
    constexpr int TITEMS = 2 * TROWS * 16;        // four-entry pieces of the two table tiles
    constexpr int TPER = (TITEMS + kLThreads - 1) / kLThreads;

    __shared__ __attribute__((aligned(16))) f16 a_lds[2][BN][kLPitch];
    __shared__ __attribute__((aligned(16))) f16 b_lds[2][BMT][kLPitch];
    __shared__ __attribute__((aligned(16))) f16 t_lds[2][2][TROWS][kLPitch]; // [buffer][scale, zero]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = blockIdx.x / p.KSP, ks = blockIdx.x - tile * p.KSP;
    const int rb = blockIdx.y;
    const int m0 = blockIdx.z * BMT;
    const int K = p.K;
    const int s_begin = ks * p.KTS;
    const int nsteps = p.KTS;

    // ---------------------------------------------------------------- who loads what
    // codes
    const uint8_t *cptr;
    int a_row0, a_col; // first LDS row of this thread's weights (its fields follow, one row each) and their column
    int t_row0;        // table row of field 0 inside the tile
    if constexpr (NBITS == 3) {
        const int t = tid >> 4, cg = tid & 15;
        int wr = tile + p.P * (16 * rb + t);
        wr = wr < p.NW ? wr : tile; // a word row past the end repeats the window's first one; its outputs are not stored
        cptr = p.codes + ((size_t)wr * K + 4 * cg) * 4;
        a_row0 = t, a_col = 4 * cg, t_row0 = 0;
    } else {
        constexpr int CH = kLK / Geo::CODE_BYTES; // threads per packed row
        const int prl = tid / CH, ch = tid % CH;
        const int jl = prl >> 4, rr = prl & 15;
        const uint32_t prow = (uint32_t)(tile * Geo::JPB + jl) + (uint32_t)(16 * rb + rr) * (uint32_t)p.GP;
        cptr = p.codes + (size_t)prow * K + Geo::CODE_BYTES * ch;
        a_row0 = prl * F, a_col = Geo::CODE_BYTES * ch, t_row0 = jl * F;
    }
    // table items: item it = (table, row, four columns)
    uint32_t t_at[TPER];  // flat index of the item's first entry at step 0 of the block
    int t_dst[TPER];      // where it goes in a table tile: (table * TROWS + row) * kLPitch + column
    bool t_scale[TPER], t_on[TPER];
#pragma unroll
    for (int q = 0; q < TPER; ++q) {
        const int it = tid + q * kLThreads;
        t_on[q] = it < TITEMS;
        const int itc = t_on[q] ? it : 0;
        const int tab = itc / (TROWS * 16), rem = itc - tab * TROWS * 16, tr = rem >> 4, tc = rem & 15;
        uint32_t j;
        if constexpr (NBITS == 3) {
            j = ((uint32_t)(10 * tile) % (uint32_t)p.G) + (uint32_t)tr;
            j -= j >= (uint32_t)p.G ? (uint32_t)p.G : 0u;
        } else {
            j = (uint32_t)(8 * tile + tr);
        }
        t_at[q] = j * (uint32_t)K + (uint32_t)(4 * tc) + (uint32_t)(s_begin * kLK);
        t_dst[q] = (tab * TROWS + tr) * kLPitch + 4 * tc;
        t_scale[q] = tab == 0;
    }
    f16x2 zms = {(f16)0, (f16)0}, zmz = zms;
    if constexpr (Q8) {
        const f16 a = gload<f16>(p.z_ms), b = gload<f16>(p.z_mz);
        zms = (f16x2){a, a}, zmz = (f16x2){b, b};
    }
    // x tile: chunk c of the thread = eight consecutive halves of one batch row
    const f16 *xsrc[XCH];
    int xdst[XCH];
    bool x_on[XCH];
#pragma unroll
    for (int c = 0; c < XCH; ++c) {
        const int chk = tid + c * kLThreads;
        x_on[c] = chk < BMT * 8;
        const int cc = x_on[c] ? chk : 0;
        int m = m0 + (cc >> 3);
        m = m < p.M ? m : p.M - 1;
        xsrc[c] = p.x + (size_t)m * K + 8 * (cc & 7) + (size_t)s_begin * kLK;
        xdst[c] = (cc >> 3) * kLPitch + 8 * (cc & 7);
    }

    const int last = nsteps - 1;
    auto load_w = [&](LdsWeightRegs &r, int ls) __attribute__((always_inline)) {
        ls = ls < last ? ls : last;
        const size_t k0 = (size_t)(s_begin + ls) * kLK * (NBITS == 3 ? 4 : 1);
        if constexpr (NBITS == 2) {
            const u32x2 v = gload<u32x2>(cptr + k0);
            r.cw = (u32x4){v.x, v.y, 0u, 0u};
        } else {
            r.cw = gload<u32x4>(cptr + k0);
        }
    };
    auto load_t = [&](LdsTableRegs &r, int ls) __attribute__((always_inline)) {
        ls = ls < last ? ls : last;
#pragma unroll
        for (int q = 0; q < TPER; ++q) {
            const uint32_t c = t_at[q] + (uint32_t)(ls * kLK);
            const uint8_t *tab = t_scale[q] ? p.sq : p.zq;
            if constexpr (Q8) {
                r.d[q] = (u32x2){gload<uint32_t>(tab + c), 0u};
                // the meta values of the scale table; zero-table items repeat the load and ignore it (a load under a
                // branch would turn every later wait into a wait for all loads)
                uint32_t cm = c - __umulhi(c, p.s_inv) * p.s_cols; // c mod cols; the quotient estimate is at most 2 short
                cm -= cm >= p.s_cols ? p.s_cols : 0;
                cm -= cm >= p.s_cols ? p.s_cols : 0;
                r.ms[q] = gload<u32x2>(p.s_ms + cm);
                r.mz[q] = gload<u32x2>(p.s_mz + cm);
            } else {
                r.d[q] = gload<u32x2>(reinterpret_cast<const f16 *>(tab) + c);
            }
        }
    };
    auto load_x = [&](u32x4(&r)[XCH], int ls) __attribute__((always_inline)) {
        ls = ls < last ? ls : last;
#pragma unroll
        for (int c = 0; c < XCH; ++c)
            r[c] = gload<u32x4>(xsrc[c] + (size_t)ls * kLK);
    };

    // ---------------------------------------------------------------- staging
    auto stage_t = [&](const LdsTableRegs &r, int buf) __attribute__((always_inline)) {
        f16 *base = &t_lds[buf][0][0][0];
#pragma unroll
        for (int q = 0; q < TPER; ++q) {
            u32x2 o;
            if constexpr (Q8) {
                // bytes -> fp16 exactly: 0x6400 | b is 1024 + b, then subtract 1024
                const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
                const f16x2 q01 = h2(__builtin_amdgcn_perm(0x64646464u, r.d[q].x, 0x04010400u)) - k1024;
                const f16x2 q23 = h2(__builtin_amdgcn_perm(0x64646464u, r.d[q].x, 0x04030402u)) - k1024;
                const f16x2 mz01 = t_scale[q] ? h2(r.mz[q].x) : zmz, mz23 = t_scale[q] ? h2(r.mz[q].y) : zmz;
                const f16x2 ms01 = t_scale[q] ? h2(r.ms[q].x) : zms, ms23 = t_scale[q] ? h2(r.ms[q].y) : zms;
                o = (u32x2){u32((q01 - mz01) * ms01), u32((q23 - mz23) * ms23)};
            } else {
                o = r.d[q];
            }
            if (TITEMS % kLThreads == 0 || t_on[q])
                *reinterpret_cast<u32x2 *>(base + t_dst[q]) = o;
        }
    };
    auto stage_x = [&](const u32x4(&r)[XCH], int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < XCH; ++c)
            if ((BMT * 8) % kLThreads == 0 || x_on[c])
                *reinterpret_cast<u32x4 *>(&b_lds[buf][0][0] + xdst[c]) = r[c];
    };
    // weights of one step: tables from t_lds[tb], result into a_lds[ab]
    auto stage_w = [&](const LdsWeightRegs &r, int tb, int ab) __attribute__((always_inline)) {
        if constexpr (NBITS == 3) {
#pragma unroll
            for (int i = 0; i < 10; ++i) {
                const uint32_t pa = __builtin_amdgcn_perm(r.cw.y, r.cw.x, w3sel(i));
                const uint32_t pb = __builtin_amdgcn_perm(r.cw.w, r.cw.z, w3sel(i));
                const u32x2 S = *reinterpret_cast<const u32x2 *>(&t_lds[tb][0][i][a_col]);
                const u32x2 Z = *reinterpret_cast<const u32x2 *>(&t_lds[tb][1][i][a_col]);
                const u32x2 o = {rebuild_pair<3>(pa, w3pos(i), Z.x, S.x), rebuild_pair<3>(pb, w3pos(i), Z.y, S.y)};
                *reinterpret_cast<u32x2 *>(&a_lds[ab][i * 16 + a_row0][a_col]) = o;
            }
        } else {
            constexpr int NW = Geo::CODE_BYTES / 4; // code words of the thread
            uint32_t pw[2 * NW];                     // pairs of code bytes, in column order
            const uint32_t d[4] = {r.cw.x, r.cw.y, r.cw.z, r.cw.w};
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                pw[2 * w] = __builtin_amdgcn_perm(0u, d[w], 0x0c010c00u);
                pw[2 * w + 1] = __builtin_amdgcn_perm(0u, d[w], 0x0c030c02u);
            }
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const int pos = NBITS * (F - 1 - i);
#pragma unroll
                for (int v = 0; v < NW / 2; ++v) { // eight columns = one 128-bit piece
                    const u32x4 S = *reinterpret_cast<const u32x4 *>(&t_lds[tb][0][t_row0 + i][a_col + 8 * v]);
                    const u32x4 Z = *reinterpret_cast<const u32x4 *>(&t_lds[tb][1][t_row0 + i][a_col + 8 * v]);
                    u32x4 o;
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        o[t] = rebuild_pair<NBITS>(pw[4 * v + t], pos, Z[t], S[t]);
                    *reinterpret_cast<u32x4 *>(&a_lds[ab][a_row0 + i][a_col + 8 * v]) = o;
                }
            }
        }
    };

    // ---------------------------------------------------------------- matrix cores
    const int wr_i = wave / WC, wc_i = wave - wr_i * WC;
    const int rb0 = wr_i * RBW; // first row block of the wave
    f32x4 acc[RBW][CBW];
#pragma unroll
    for (int a = 0; a < RBW; ++a)
#pragma unroll
        for (int b = 0; b < CBW; ++b)
            acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int frag_off = (lane & 15) * kLPitch + 8 * (lane >> 4);
    auto mma = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            f16x8 B[CBW];
#pragma unroll
            for (int b = 0; b < CBW; ++b)
                B[b] = *reinterpret_cast<const f16x8 *>(&b_lds[buf][0][0] + (wc_i * CBW + b) * 16 * kLPitch + frag_off + 32 * kk);
#pragma unroll
            for (int a = 0; a < RBW; ++a) {
                if (NRB % WR == 0 || rb0 + a < NRB) {
                    const f16x8 A = *reinterpret_cast<const f16x8 *>(&a_lds[buf][0][0] + (rb0 + a) * 16 * kLPitch + frag_off + 32 * kk);
#pragma unroll
                    for (int b = 0; b < CBW; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[b], acc[a][b], 0, 0, 0);
                }
            }
        }
    };

    // ---------------------------------------------------------------- pipeline
    LdsWeightRegs W0, W1, W2, W3;
    LdsTableRegs T0, T1, T2, T3;
    u32x4 X0[XCH], X1[XCH];
    load_t(T0, 0);
    load_x(X0, 0);
    load_w(W0, 0);
    load_t(T1, 1);
    load_x(X1, 1);
    load_w(W1, 1);
    load_t(T2, 2);
    load_w(W2, 2);
    load_t(T3, 3);
    load_w(W3, 3);
    stage_t(T0, 0);
    load_t(T0, 4);
    stage_t(T1, 1);
    load_t(T1, 5);
    __syncthreads();
    stage_w(W0, 0, 0);
    load_w(W0, 4);
    stage_x(X0, 0);
    load_x(X0, 2);
    __syncthreads();
    // iteration ls: weights and x of step ls + 1 and the tables of step ls + 2 are staged while step ls is multiplied
    auto iter = [&](LdsWeightRegs &Wn, u32x4(&Xn)[XCH], LdsTableRegs &Tn, int ls) __attribute__((always_inline)) {
        stage_w(Wn, (ls + 1) & 1, (ls + 1) & 1);
        load_w(Wn, ls + 5);
        stage_x(Xn, (ls + 1) & 1);
        load_x(Xn, ls + 3);
        mma(ls & 1); // (steps come in fours, so every iteration of the loop below has a step to multiply)
        stage_t(Tn, ls & 1);
        load_t(Tn, ls + 6);
        if constexpr (BMT >= 64) {
            // Ask the scheduler to thread the rebuilding of the next step's weights (VALU, LDS) through this step's
            // MFMAs: left to itself it runs the phases one after the other, and a block of four waves has nothing else
            // to overlap them with (128 columns, 512 rows of 14336x4096: 144 us without, 97 us with).
#pragma unroll
            for (int i = 0; i < RBW * CBW * 2; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 8, 0); // up to eight VALU
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // one LDS write
            }
        }
        __syncthreads();
    };
    for (int ls = 0; ls < nsteps; ls += 4) {
        iter(W1, X1, T2, ls);
        iter(W2, X0, T3, ls + 1);
        iter(W3, X1, T0, ls + 2);
        iter(W0, X0, T1, ls + 3);
    }

    // ---------------------------------------------------------------- results: D column = batch column lane & 15,
    // rows 4 * (lane >> 4) + v of the row block.  Plain stores only (bias, routing weight and accumulation are the
    // finishing kernel's: a launch that needs them goes through the partial sums even with one block along K).
#pragma unroll
    for (int a = 0; a < RBW; ++a) {
        if (!(NRB % WR == 0 || rb0 + a < NRB))
            continue;
#pragma unroll
        for (int b = 0; b < CBW; ++b) {
            const int m = m0 + (wc_i * CBW + b) * 16 + (lane & 15);
            if (m >= p.M)
                continue;
            const int lr0 = (rb0 + a) * 16 + 4 * (lane >> 4);
            const f32x4 o = acc[a][b];
            float *const prow = p.part ? p.part + ((int64_t)ks * p.M + m) * p.N : nullptr;
            f16 *const yrow = p.y + (int64_t)m * p.N;
            if constexpr (NBITS == 3) {
                const int i = lr0 >> 4;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int wr = tile + p.P * (16 * rb + (lr0 & 15) + v);
                    const int64_t n = (int64_t)10 * wr + i;
                    if (wr >= p.NW || n >= p.N)
                        continue;
                    if (prow)
                        prow[n] = o[v];
                    else
                        yrow[n] = (f16)o[v];
                }
            } else if constexpr (NBITS == 2) {
                // the four rows are the four fields of one packed row: four consecutive outputs
                const int prl = lr0 >> 2;
                const int64_t n = (int64_t)4 * ((tile * Geo::JPB + (prl >> 4)) + (int64_t)(16 * rb + (prl & 15)) * p.GP);
                if (prow)
                    *reinterpret_cast<f32x4 *>(prow + n) = o;
                else
                    *reinterpret_cast<f16x4 *>(yrow + n) = (f16x4){(f16)o[0], (f16)o[1], (f16)o[2], (f16)o[3]};
            } else {
                // two packed rows of two fields each
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int prl = (lr0 >> 1) + h;
                    const int64_t n = (int64_t)2 * ((tile * Geo::JPB + (prl >> 4)) + (int64_t)(16 * rb + (prl & 15)) * p.GP);
                    if (prow)
                        *reinterpret_cast<float2 *>(prow + n) = make_float2(o[2 * h], o[2 * h + 1]);
                    else
                        *reinterpret_cast<f16x2 *>(yrow + n) = (f16x2){(f16)o[2 * h], (f16)o[2 * h + 1]};
                }
            }
        }
    }
}

// y = cast(sum over the K blocks) (+ bias) (* row_scale) (+ y), four outputs per thread
__global__ __launch_bounds__(256) void lds_finish_kernel(const float *__restrict__ part, int KSP, int64_t M, int64_t N,
                                                          const f16 *__restrict__ bias, const f16 *__restrict__ row_scale,
                                                          int accumulate, f16 *__restrict__ y)
{
    const int64_t quads = M * N / 4;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < quads; idx += (int64_t)gridDim.x * 256) {
        const int64_t e = idx * 4, m = e / N, n = e - m * N;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < KSP; ++s)
            sum += *reinterpret_cast<const f32x4 *>(part + (int64_t)s * M * N + e);
        f16 o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f16 v = (f16)sum[i];
            if (bias)
                v = v + bias[n + i];
            if (row_scale)
                v = v * row_scale[m];
            if (accumulate)
                v = y[e + i] + v;
            o[i] = v;
        }
        *reinterpret_cast<f16x4 *>(y + e) = (f16x4){o[0], o[1], o[2], o[3]};
    }
}

struct LdsPlan {
    int BMT, KSP, KTS, tiles, RB, P, NW, GP;
    bool q8;
};

bool make_lds_plan(const hqq_linear *l, int64_t M, LdsPlan &pl)
{
    if (M < 1 || l->K % kLK != 0 || l->N % 4 != 0 || l->N % l->group_size != 0)
        return false;
    const int64_t G = l->N / l->group_size;
    if (G * l->K >= (1ll << 32) || !aligned16(l->codes))
        return false;
    const int sk = table_kind(l->scale), zk = table_kind(l->zero);
    if (sk == TK_U8_COLS && zk == TK_U8_SCALAR) {
        pl.q8 = true;
        if (l->scale.meta_cols % 4 != 0 || (reinterpret_cast<uintptr_t>(l->scale.meta_scale) & 7u) ||
            (reinterpret_cast<uintptr_t>(l->scale.meta_zero) & 7u) || (reinterpret_cast<uintptr_t>(l->scale.data) & 3u) ||
            (reinterpret_cast<uintptr_t>(l->zero.data) & 3u))
            return false;
    } else if (sk == TK_F16 && zk == TK_F16) {
        pl.q8 = false;
        if ((reinterpret_cast<uintptr_t>(l->scale.data) & 7u) || (reinterpret_cast<uintptr_t>(l->zero.data) & 7u))
            return false;
    } else {
        return false;
    }
    pl.P = 0, pl.NW = 0, pl.GP = 0;
    if (l->nbits == 3) {
        if (G < 10)
            return false;
        int64_t g = G, t = 10; // gcd(10, G)
        while (t) {
            const int64_t r = g % t;
            g = t, t = r;
        }
        pl.P = (int)(G / g);
        pl.NW = (int)((l->N + 9) / 10);
        const int64_t per_window = (pl.NW + pl.P - 1) / pl.P; // word rows of a window
        pl.tiles = pl.P < pl.NW ? pl.P : pl.NW;
        pl.RB = (int)((per_window + 15) / 16);
    } else {
        const int F = 8 / l->nbits, JPB = 8 / F;
        if (l->group_size % 16 != 0 || G % 8 != 0)
            return false;
        pl.GP = (int)(G / F);
        pl.tiles = pl.GP / JPB;
        pl.RB = l->group_size / 16;
    }
    if (pl.RB > 65535)
        return false;
    pl.BMT = M <= 16 ? 16 : (M <= 32 ? 32 : (M <= 64 ? 64 : 128));
    pl.BMT = tuning_int("HQQ_LDS_BMT", pl.BMT);
    if (pl.BMT != 16 && pl.BMT != 32 && pl.BMT != 64 && pl.BMT != 128)
        return false;
    const int64_t mtiles = (M + pl.BMT - 1) / pl.BMT;
    if (mtiles > 65535)
        return false;
    // K over blocks, in whole groups of four steps, until every compute unit has a block; the narrowest batch tile
    // leaves room for two blocks on a unit and its partial sums are small, so it is split until every unit has two
    const int KT = (int)(l->K / kLK);
    const int64_t blocks = (int64_t)pl.tiles * pl.RB * mtiles;
    const int max_split = pl.BMT == 16 ? 16 : 8;
    const int64_t want = pl.BMT == 16 ? 448 : 256;
    int ksp = 1;
    for (int c = 1; c <= max_split; ++c) {
        if (KT % c != 0 || (KT / c) % 4 != 0 || KT / c < 8)
            continue;
        ksp = c;
        if (blocks * c >= want)
            break;
    }
    if (KT % 4 != 0)
        return false;
    ksp = tuning_int("HQQ_LDS_KSP", ksp);
    if (ksp < 1 || KT % ksp != 0 || (KT / ksp) % 4 != 0)
        return false;
    pl.KSP = ksp, pl.KTS = KT / ksp;
    return (int64_t)pl.tiles * pl.KSP <= 0x7fffffff;
}

template <int NBITS, int BMT> void launch_lds_kinds(const LdsParams &p, bool q8, dim3 grid, hipStream_t s)
{
    if (q8)
        gemm_lds_kernel<NBITS, BMT, true><<<grid, dim3(kLThreads), 0, s>>>(p);
    else
        gemm_lds_kernel<NBITS, BMT, false><<<grid, dim3(kLThreads), 0, s>>>(p);
}

template <int NBITS> void launch_lds_bmt(const LdsParams &p, const LdsPlan &pl, dim3 grid, hipStream_t s)
{
    switch (pl.BMT) {
    case 16: launch_lds_kinds<NBITS, 16>(p, pl.q8, grid, s); break;
    case 32: launch_lds_kinds<NBITS, 32>(p, pl.q8, grid, s); break;
    case 64: launch_lds_kinds<NBITS, 64>(p, pl.q8, grid, s); break;
    default: launch_lds_kinds<NBITS, 128>(p, pl.q8, grid, s); break;
    }
}

} // namespace

bool ldsgemm_supported(const hqq_linear *l, int64_t M)
{
    LdsPlan pl;
    return make_lds_plan(l, M, pl);
}

size_t ldsgemm_workspace_bytes(const hqq_linear *l, int64_t M)
{
    LdsPlan pl;
    if (!make_lds_plan(l, M, pl))
        return 0;
    // partial sums of the planned split (one set even without a split: an epilogue with bias, routing weight or
    // accumulation goes through them)
    return kHeadBytes + (size_t)pl.KSP * (size_t)M * (size_t)l->N * sizeof(float);
}

int launch_ldsgemm_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                          const SmallBatchEpilogue *ep)
{
    LdsPlan pl;
    if (!make_lds_plan(l, M, pl))
        return HQQ_E_UNSUPPORTED;
    // bias, routing weight and accumulation are applied by the finishing kernel
    const bool fancy = l->bias || (ep && (ep->row_scale || ep->accumulate));
    const size_t part_bytes = pl.KSP > 1 || fancy ? (size_t)pl.KSP * (size_t)M * (size_t)l->N * sizeof(float) : 0;
    if (part_bytes && (!ws || ws_bytes < kHeadBytes + part_bytes))
        return HQQ_E_WORKSPACE;
    LdsParams p = {};
    p.codes = static_cast<const uint8_t *>(l->codes);
    p.sq = static_cast<const uint8_t *>(l->scale.data), p.zq = static_cast<const uint8_t *>(l->zero.data);
    p.s_ms = static_cast<const f16 *>(l->scale.meta_scale), p.s_mz = static_cast<const f16 *>(l->scale.meta_zero);
    p.z_ms = static_cast<const f16 *>(l->zero.meta_scale), p.z_mz = static_cast<const f16 *>(l->zero.meta_zero);
    p.s_cols = pl.q8 ? (uint32_t)l->scale.meta_cols : 1u;
    p.s_inv = (uint32_t)(0xFFFFFFFFull / p.s_cols);
    p.x = x, p.y = y, p.bias = static_cast<const f16 *>(l->bias);
    p.part = part_bytes ? reinterpret_cast<float *>(static_cast<char *>(ws) + kHeadBytes) : nullptr;
    p.row_scale = ep ? ep->row_scale : nullptr, p.accumulate = ep ? ep->accumulate : 0;
    p.M = (int)M, p.N = (int)l->N, p.K = (int)l->K, p.G = (int)(l->N / l->group_size), p.GP = pl.GP;
    p.KSP = pl.KSP, p.KTS = pl.KTS, p.P = pl.P, p.NW = pl.NW;
    const dim3 grid((unsigned)(pl.tiles * pl.KSP), (unsigned)pl.RB, (unsigned)((M + pl.BMT - 1) / pl.BMT));
    if (l->nbits == 2)
        launch_lds_bmt<2>(p, pl, grid, s);
    else if (l->nbits == 4)
        launch_lds_bmt<4>(p, pl, grid, s);
    else
        launch_lds_bmt<3>(p, pl, grid, s);
    int rc = launch_status();
    if (rc != HQQ_OK || !p.part)
        return rc;
    const int64_t quads = M * l->N / 4;
    const unsigned blocks = (unsigned)((quads + 255) / 256 < 4096 ? (quads + 255) / 256 : 4096);
    lds_finish_kernel<<<dim3(blocks), dim3(256), 0, s>>>(p.part, pl.KSP, M, l->N, p.bias, p.row_scale, p.accumulate, y);
    return launch_status();
}

} // namespace hqq
