// Multi-token (prefill) unpack-dequantise-matmul for 2- and 4-bit codes on the matrix cores.
//
// Above ~16 batch rows folding the scale into the activations costs more than it saves, so here the weights
// themselves are rebuilt, bit-exactly as the reference does (w = fp16(fp16(q - z) * s)), and fed to
// v_mfma_f32_16x16x32_f16 with fp32 accumulation.
//
// A block is four wavefronts; wave w owns the 16 x F output rows of one packed table row jp = 4*blockIdx.x + w
// (rows n = F*(jp + r*GP) + i, r = 16*rb .. 16*rb+15: they share scale and zero), for BM batch columns, and
// walks all of K in 64-column steps.  Per step
//   * the block copies the x tile (BM x 64 fp16) to LDS once, in B-operand order, for all four waves;
//   * each wave de-quantises its 8-bit (or fp16) scale / zero entries once (F x 64 of each) into LDS;
//   * each lane builds its A operands in registers: 16 code bytes -> for every field i and each half of the
//     step, eight exact fp16 weights (mask-and-insert into 2^e, subtract, subtract z, multiply s);
//   * 2 * F * BM/16 MFMAs per wave.
// Weight bytes come from HBM once; the x tile is re-read by N / (64*F) blocks, from L2.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"
#include "table_reader.hpp"

#include <cstdlib>
#include <type_traits>

namespace hqq {
using gemv::gload;
using gemv::TK_F16;
using gemv::TK_U8_COLS;
using gemv::TK_U8_SCALAR;
namespace {

constexpr int kStepK = 64;
constexpr int kWaves = 4;

struct TileParams {
    const uint8_t *codes;
    Table sc, zr;
    uint32_t sc_inv, zr_inv;
    const f16 *x;
    const f16 *bias;
    f16 *y;
    float *part; // [KSP][N/F][M][F] fp32 partial sums when K is split over several blocks, else null: the sixteen
                 // batch rows a lane group holds for one row group are then 256 consecutive bytes
    int M, N, K, GP, KT;
    int KSP; // blocks along K
    int KTS; // steps per block
    // second layer of a fused gate launch (pipelined kernel only): blocks JB * KSP and up work on it and write
    // their partial sums part_lstride floats further; JB = row blocks per layer
    const uint8_t *codes_b;
    Table sc_b, zr_b;
    uint32_t sc_b_inv;
    int JB;
    int64_t part_lstride;
    // pipelined kernel and its finishing pass only: y = o (+ bias) (* row_scale[m]) (+ y), each step rounded to fp16
    const f16 *row_scale;
    int accumulate;
};

template <int NBITS> struct WField {
    static constexpr int F = 8 / NBITS;
    static constexpr int pos(int i) { return NBITS * (F - 1 - i); }
    static constexpr uint32_t mask(int i) { return (((1u << NBITS) - 1u) * 0x00010001u) << pos(i); }
    // the masked field OR-ed into the mantissa of 2^e (e = 10 - pos) reads as 2^e + q
    static constexpr uint32_t expo(int i) { return (uint32_t)((10 - pos(i) + 15) << 10) * 0x00010001u; }
    static constexpr float offset(int i) { return (float)(1 << (10 - pos(i))); }
};

template <int NBITS, int BM>
__global__ __launch_bounds__(kWaves * 64) void gemm_tile_kernel(TileParams p)
{
    constexpr int F = 8 / NBITS;
    constexpr int MB = BM / 16;
    // x tile: [k block of 8 (8 per step)][batch column][8 halves in B-operand order]
    __shared__ __attribute__((aligned(16))) f16 x_lds[8 * BM * 8];
    // per wave: scale and zero of the step, entry ((i*2 + h)*4 + kg) of 8 halves, same order
    __shared__ __attribute__((aligned(16))) f16 s_lds[kWaves][F * 2 * 4 * 8];
    __shared__ __attribute__((aligned(16))) f16 z_lds[kWaves][F * 2 * 4 * 8];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int jblk = blockIdx.x / p.KSP, ks = blockIdx.x - jblk * p.KSP;
    const int jp = jblk * kWaves + wave;
    const int s_begin = ks * p.KTS;
    const int s_end = s_begin + p.KTS < p.KT ? s_begin + p.KTS : p.KT;
    const int rb = blockIdx.y;
    const int m0 = blockIdx.z * BM;
    const int K = p.K;
    const int rr = lane & 15, kg = lane >> 4;
    const int ti = lane >> 4, kq = lane & 15;
    const bool tlane = ti < F;

    const uint32_t prow = (uint32_t)jp + (uint32_t)(16 * rb + rr) * (uint32_t)p.GP;
    const uint8_t *cptr = p.codes + (size_t)prow * K + 16 * kg;
    TableCursor<0> sc, zr;
    {
        const uint32_t c0 = (uint32_t)(F * jp + (tlane ? ti : 0)) * (uint32_t)K + (uint32_t)(4 * kq) + (uint32_t)(s_begin * kStepK);
        sc.init(p.sc, c0, p.sc_inv);
        zr.init(p.zr, c0, p.zr_inv);
    }
    // x tile copy: thread t moves chunks (column m, k block kb) = (c / 8, c % 8) for c = t, t + 256, ...
    constexpr int XCHUNKS = (BM * 8 + kWaves * 64 - 1) / (kWaves * 64);

    f32x4 acc[F][MB];
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int b = 0; b < MB; ++b)
            acc[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    u32x4 cw_n = {0, 0, 0, 0};
    TableRaw sraw_n, zraw_n;
    u32x4 xr_n[XCHUNKS];
    auto issue = [&](int s) {
        const int k0 = s * kStepK;
        cw_n = *reinterpret_cast<const u32x4 *>(cptr + k0);
        if (tlane) {
            sraw_n = table_load(sc);
            zraw_n = table_load(zr);
        }
        sc.advance(kStepK);
        zr.advance(kStepK);
#pragma unroll
        for (int c = 0; c < XCHUNKS; ++c) {
            const int ch = threadIdx.x + c * kWaves * 64;
            const int m = m0 + ch / 8, kb = ch % 8;
            xr_n[c] = (u32x4){0, 0, 0, 0};
            // k block kb = h*4 + kg holds the columns half h of lane group kg works on: 16*kg + 8*h .. +7
            if (m < p.M && ch < BM * 8)
                xr_n[c] = *reinterpret_cast<const u32x4 *>(p.x + (size_t)m * K + k0 + 16 * (kb & 3) + 8 * (kb >> 2));
        }
    };
    issue(s_begin);

    f16 *s_w = &s_lds[wave][(((ti * 2 + ((kq >> 1) & 1)) * 4 + (kq >> 2)) * 8) + 4 * (kq & 1)];
    f16 *z_w = &z_lds[wave][(((ti * 2 + ((kq >> 1) & 1)) * 4 + (kq >> 2)) * 8) + 4 * (kq & 1)];

    for (int s = s_begin; s < s_end; ++s) {
        const u32x4 cw = cw_n;
        const TableRaw sraw = sraw_n, zraw = zraw_n;
        u32x4 xr[XCHUNKS];
#pragma unroll
        for (int c = 0; c < XCHUNKS; ++c)
            xr[c] = xr_n[c];
        if (s + 1 < s_end)
            issue(s + 1);

        __syncthreads(); // everyone is done reading the previous step's tiles
#pragma unroll
        for (int c = 0; c < XCHUNKS; ++c) {
            const int ch = threadIdx.x + c * kWaves * 64;
            const int m = ch / 8, kb = ch % 8;
            // eight columns (0..7) stored in B-operand order (0,2,1,3,4,6,5,7)
            const f16x8 v = __builtin_bit_cast(f16x8, xr[c]);
            const f16x8 o = {v[0], v[2], v[1], v[3], v[4], v[6], v[5], v[7]};
            if (ch < BM * 8)
                *reinterpret_cast<f16x8 *>(&x_lds[(kb * BM + m) * 8]) = o;
        }
        if (tlane) {
            f16x2 s01, s23, z01, z23;
            table_decode(sc, sraw, s01, s23);
            table_decode(zr, zraw, z01, z23);
            *reinterpret_cast<f16x4 *>(s_w) = (f16x4){s01.x, s23.x, s01.y, s23.y};
            *reinterpret_cast<f16x4 *>(z_w) = (f16x4){z01.x, z23.x, z01.y, z23.y};
        }
        __syncthreads();

        const uint32_t d[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
            const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
            f16x8 B[MB];
#pragma unroll
            for (int b = 0; b < MB; ++b)
                B[b] = *reinterpret_cast<const f16x8 *>(&x_lds[(((h * 4 + kg) * BM) + b * 16 + (lane & 15)) * 8]);
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const u32x4 S = *reinterpret_cast<const u32x4 *>(&s_lds[wave][((i * 2 + h) * 4 + kg) * 8]);
                const u32x4 Z = *reinterpret_cast<const u32x4 *>(&z_lds[wave][((i * 2 + h) * 4 + kg) * 8]);
                const uint32_t mk = WField<NBITS>::mask(i), ex = WField<NBITS>::expo(i);
                const f16 offv = (f16)WField<NBITS>::offset(i);
                const f16x2 off = {offv, offv};
                const uint32_t src[4] = {d0, d0s, d1, d1s};
                u32x4 Au; // whole 32-bit words throughout: a pair of weights per register, no element inserts
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const f16x2 q = as_f16x2((src[t] & mk) | ex) - off;          // exact code
                    const f16x2 w = (q - as_f16x2(Z[t])) * as_f16x2(S[t]);        // two fp16 roundings, as the reference
                    Au[t] = __builtin_bit_cast(uint32_t, w);
                }
                const f16x8 A = __builtin_bit_cast(f16x8, Au);
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[b], acc[i][b], 0, 0, 0);
            }
        }
    }

    // D layout: column = batch column (lane & 15) of block b, rows r = 4*(lane>>4) + v
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = m0 + b * 16 + (lane & 15);
        if (m >= p.M)
            continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 16 * rb + 4 * kg + v;
            const int64_t n = (int64_t)F * (jp + (int64_t)r * p.GP);
            if (p.part) { // K is split over blocks: fp32 partial sums, added by the finishing kernel
                float *dst = p.part + (((int64_t)ks * (p.N / F) + n / F) * p.M + m) * F; // [K block][row group][batch row][F]
                if constexpr (F == 4)
                    *reinterpret_cast<f32x4 *>(dst) = (f32x4){acc[0][b][v], acc[1][b][v], acc[2][b][v], acc[3][b][v]};
                else
                    *reinterpret_cast<float2 *>(dst) = make_float2(acc[0][b][v], acc[1][b][v]);
                continue;
            }
            f16 o[F];
#pragma unroll
            for (int i = 0; i < F; ++i) {
                o[i] = (f16)acc[i][b][v];
                if (p.bias)
                    o[i] = o[i] + p.bias[n + i];
            }
            f16 *dst = p.y + (int64_t)m * p.N + n;
            if constexpr (F == 4)
                *reinterpret_cast<f16x4 *>(dst) = (f16x4){o[0], o[1], o[2], o[3]};
            else
                *reinterpret_cast<f16x2 *>(dst) = (f16x2){o[0], o[1]};
        }
    }
}


// ---------------------------------------------------------------------------------------------------------------
// The kernel for the two table layouts HQQ produces (8-bit tables with per-column meta for the scale and whole-tensor
// meta for the zero; or fp16 tables).  Same tiling as above, organised around memory latency: codes and tables, which
// come from HBM, are requested four steps ahead into one of four register sets; the x tile, which every block
// re-reads from L2, two steps ahead into one of two; the x tile and the de-quantised tables of the next step are
// written to the other half of a double-buffered LDS while this step is worked on, and there is one barrier per
// step.  Every load is unconditional (a step past the end re-reads the last one; batch rows past M re-read row
// M - 1, whose results are never stored), so the compiler's wait counts are exact; within a step the x loads are
// issued before the weight loads, because loads retire in issue order and the x tile is needed first.  The x tile
// is padded by two entries per k block: the sixteen lanes of an LDS write then fall into sixteen different groups
// of banks.
struct TileWeightRegs {
    u32x4 cw;             // 16 code bytes: four columns per word, rows by field
    uint32_t sq, zq;      // four table bytes (8-bit kinds)
    u32x2 sm_s, sm_z;     // per-column meta of the scale: four halves each
    u32x2 sf, zf;         // four table halves (fp16 kind)
};

// NFW: waves that share a packed table row, each taking F / NFW of its fields (1: a wave owns all fields; 2: the block
// is eight waves, every weight is still rebuilt once, and a wave holds half the accumulators -- what lets two waves
// share a SIMD at the 128-column batch tile).
// JW packed table rows per block, KW parts of the block's K range worked on by different waves: at the narrowest
// batch tile a block is one packed row and eight K parts, which meet in LDS, so that a projection with K = 4096
// needs neither partial sums in memory nor a finishing launch.  G2 (with JW = 2): the two "rows" of the block are the
// two projections of a gate for the same packed row; they share the x tile, and when the block holds all of K the
// first projection's wave applies silu(a) * b itself.
template <int NBITS, int BM, int SKIND, int ZKIND, int NFW, int JW = kWaves, int KW = 1, bool G2 = false>
__global__ __launch_bounds__(JW * NFW * KW * 64) void gemm_tile2_kernel(TileParams p)
{
    static_assert(!G2 || (JW == 2 && NFW == 1 && KW > 1), "the gate form is two projections by several K parts");
    constexpr int F = 8 / NBITS;
    constexpr int FW = F / NFW;       // fields per wave
    constexpr int NWK = JW * NFW;     // waves per K part
    constexpr int NW = NWK * KW;      // waves per block
    constexpr int MB = BM / 16;
    constexpr int XP = BM + 2;
    // the widest batch tile runs its loop as a software pipeline (compute_pipelined below)
    constexpr bool PIPE = KW == 1 && BM >= 128;
    // With K parts every wave stages an x tile of its own and the steps of the loop need no block barrier: the
    // waves of a block share nothing until their sums meet at the end.
    constexpr bool PRIV = KW > 1;
    constexpr int XT = PRIV ? 64 : NWK * 64; // threads that stage one x tile
    constexpr int XCH = (BM * 8 + XT - 1) / XT;
    constexpr int TAB = FW * 2 * 4 * 8; // halves per wave and table: entry ((i*2 + h)*4 + kg) of 8 halves
    __shared__ __attribute__((aligned(16))) f16 x_lds[2][PRIV ? NW : 1][8 * XP * 8];
    __shared__ __attribute__((aligned(16))) f16 s_lds[2][NW][TAB];
    __shared__ __attribute__((aligned(16))) f16 z_lds[2][NW][TAB];
    // where the K parts' sums meet after the loop: the memory of the x tiles, which are no longer needed then
    constexpr int RED_ROWS = FW * MB * 4;
    static_assert(!PRIV || sizeof(float) * (KW - 1) * NWK * RED_ROWS * 64 <= sizeof(x_lds), "the sums fit the x tiles");
    float(*red_lds)[RED_ROWS][64] = reinterpret_cast<float(*)[RED_ROWS][64]>(&x_lds[0][0][0]);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kpart = wave / NWK, wl = wave - kpart * NWK; // K part of the block, wave inside the part
    const int tk = PRIV ? lane : (int)threadIdx.x;         // thread among those that stage its x tile
    const int xi = PRIV ? wave : 0;                        // which x tile
    const int jall = blockIdx.x / p.KSP, ks = blockIdx.x - jall * p.KSP;
    // second projection of a gate: a block of its own (block-uniform), or with G2 the block's odd waves
    const bool second = G2 ? (wl & 1) != 0 : jall >= p.JB;
    const int jblk = jall - (!G2 && second ? p.JB : 0);
    const int jp = G2 ? jblk : jblk * JW + wl / NFW;
    const int f0 = (wl % NFW) * FW; // first field of this wave
    const Table &sc_t = second ? p.sc_b : p.sc, &zr_t = second ? p.zr_b : p.zr;
    const uint32_t sc_inv = second ? p.sc_b_inv : p.sc_inv;
    const int s_begin = (ks * KW + kpart) * p.KTS; // KTS: steps per K part
    const int s_stop = s_begin + p.KTS;            // the same trip count for every wave of the block
    const int s_end = s_stop < p.KT ? s_stop : p.KT;
    const int s_last = s_end > 0 ? s_end - 1 : 0;
    const int rb = blockIdx.y;
    const int m0 = blockIdx.z * BM;
    const int K = p.K;
    const int rr = lane & 15, kg = lane >> 4;
    const int ti = lane >> 4, kq = lane & 15;
    const bool tlane = ti < FW;
    const int ti_l = ti & (FW - 1); // lanes past the table rows repeat a table lane's loads: issuing loads never diverges

    const uint8_t *codes = (second ? p.codes_b : p.codes) + ((size_t)((uint32_t)jp + (uint32_t)(16 * rb + rr) * (uint32_t)p.GP) * K + 16 * kg);
    const uint32_t c_row = (uint32_t)(F * jp + f0 + ti_l) * (uint32_t)K + (uint32_t)(4 * kq);
    const uint8_t *s_tab = static_cast<const uint8_t *>(sc_t.data), *z_tab = static_cast<const uint8_t *>(zr_t.data);
    const f16 *s_ms = sc_t.ms, *s_mz = sc_t.mz;
    const uint32_t s_cols = (uint32_t)sc_t.meta_cols;
    // whole-tensor meta of the zero table, splat
    f16x2 zms = {(f16)0, (f16)0}, zmz = zms;
    if constexpr (ZKIND == TK_U8_SCALAR) {
        const f16 a = gload<f16>(zr_t.ms), b = gload<f16>(zr_t.mz);
        zms = (f16x2){a, a}, zmz = (f16x2){b, b};
    }
    // x tile: thread t moves chunks (column m, k block kb) = (ch / 8, ch % 8), ch = t, t + 256, ...; k block kb = h*4 + kg
    // holds the columns half h of lane group kg works on: 16*kg + 8*h .. +7
    const f16 *xsrc[XCH];
    int xdst[XCH];
#pragma unroll
    for (int c = 0; c < XCH; ++c) {
        const int ch = tk + c * XT;
        const int chc = ch < BM * 8 ? ch : BM * 8 - 1;
        int m = m0 + chc / 8;
        m = m < p.M ? m : p.M - 1;
        const int kb = chc % 8;
        xsrc[c] = p.x + (size_t)m * K + 16 * (kb & 3) + 8 * (kb >> 2);
        xdst[c] = (kb * XP + chc / 8) * 8;
    }

    typedef TileWeightRegs Regs;
    struct XRegs {
        u32x4 xr[XCH];
    };
    auto issue = [&](Regs &r, int s) __attribute__((always_inline)) {
        s = s < s_last ? s : s_last;
        const uint32_t k0 = (uint32_t)s * kStepK;
        r.cw = gload<u32x4>(codes + k0);
        const uint32_t c = c_row + k0;
        if constexpr (SKIND == TK_F16) {
            r.sf = gload<u32x2>(reinterpret_cast<const f16 *>(s_tab) + c);
            r.zf = gload<u32x2>(reinterpret_cast<const f16 *>(z_tab) + c);
        } else {
            r.sq = gload<uint32_t>(s_tab + c);
            r.zq = gload<uint32_t>(z_tab + c);
            uint32_t cm = c - __umulhi(c, sc_inv) * s_cols; // c mod cols; the quotient estimate is at most 2 short
            cm -= cm >= s_cols ? s_cols : 0;
            cm -= cm >= s_cols ? s_cols : 0;
            r.sm_s = gload<u32x2>(s_ms + cm);
            r.sm_z = gload<u32x2>(s_mz + cm);
        }
    };
    auto issue_x = [&](XRegs &r, int s) __attribute__((always_inline)) {
        s = s < s_last ? s : s_last;
        const uint32_t k0 = (uint32_t)s * kStepK;
#pragma unroll
        for (int c2 = 0; c2 < XCH; ++c2)
            r.xr[c2] = gload<u32x4>(xsrc[c2] + k0);
    };

    // x tile and de-quantised tables of one step into LDS half `buf`
    const int tab_w = (((ti_l * 2 + ((kq >> 1) & 1)) * 4 + (kq >> 2)) * 8) + 4 * (kq & 1);
    auto stage = [&](const Regs &r, const XRegs &xr, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < XCH; ++c) {
            // eight columns (0..7) stored in B-operand order (0,2,1,3,4,6,5,7)
            const u32x4 v = xr.xr[c];
            u32x4 o;
            o.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
            o.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
            o.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
            o.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
            if (XCH * XT == BM * 8 || tk + c * XT < BM * 8)
                *reinterpret_cast<u32x4 *>(&x_lds[buf][xi][xdst[c]]) = o;
        }
        // (at the widest tile the lanes past the table rows store their twin's values a second time: no branch, so
        // that the step stays one scheduling region)
        if (tlane || PIPE) {
            f16x2 s01, s23, z01, z23;
            if constexpr (SKIND == TK_F16) {
                s01 = as_f16x2(r.sf.x), s23 = as_f16x2(r.sf.y);
                z01 = as_f16x2(r.zf.x), z23 = as_f16x2(r.zf.y);
            } else {
                // bytes -> fp16 exactly: 0x6400 | b is 1024 + b, then subtract 1024
                const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
                const f16x2 a01 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, r.sq, 0x04010400u)) - k1024;
                const f16x2 a23 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, r.sq, 0x04030402u)) - k1024;
                const f16x2 b01 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, r.zq, 0x04010400u)) - k1024;
                const f16x2 b23 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, r.zq, 0x04030402u)) - k1024;
                s01 = (a01 - as_f16x2(r.sm_z.x)) * as_f16x2(r.sm_s.x);
                s23 = (a23 - as_f16x2(r.sm_z.y)) * as_f16x2(r.sm_s.y);
                z01 = (b01 - zmz) * zms;
                z23 = (b23 - zmz) * zms;
            }
            *reinterpret_cast<f16x4 *>(&s_lds[buf][wave][tab_w]) = (f16x4){s01.x, s23.x, s01.y, s23.y};
            *reinterpret_cast<f16x4 *>(&z_lds[buf][wave][tab_w]) = (f16x4){z01.x, z23.x, z01.y, z23.y};
        }
    };

    f32x4 acc[FW][MB];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int b = 0; b < MB; ++b)
            acc[i][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // The constants of this wave's fields for the pipelined loop (f0 is uniform over the wave, so the selects are
    // scalar).  The exponent pattern is kept in a vector register: with mask and pattern both scalar operands the
    // field merge would take two instructions (and, or) instead of one.
    uint32_t f_mask[FW], f_expo[FW];
    f16x2 f_off[FW];
#pragma unroll
    for (int i = 0; i < FW; ++i) {
        f_mask[i] = f0 ? WField<NBITS>::mask(i + (NFW - 1) * FW) : WField<NBITS>::mask(i);
        f_expo[i] = f0 ? WField<NBITS>::expo(i + (NFW - 1) * FW) : WField<NBITS>::expo(i);
        const f16 offv = (f16)(f0 ? WField<NBITS>::offset(i + (NFW - 1) * FW) : WField<NBITS>::offset(i));
        f_off[i] = (f16x2){offv, offv};
        if constexpr (PIPE)
            asm volatile("" : "+v"(f_expo[i]));
    }

    // the narrower tiles: groups one after the other
    auto compute_simple = [&](const u32x4 cw, int buf) __attribute__((always_inline)) {
        const uint32_t d[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
            const uint32_t src[4] = {d0, d0 >> 8, d1, d1 >> 8};
            f16x8 B[MB];
#pragma unroll
            for (int b = 0; b < MB; ++b)
                B[b] = *reinterpret_cast<const f16x8 *>(&x_lds[buf][xi][(((h * 4 + kg) * XP) + b * 16 + rr) * 8]);
#pragma unroll
            for (int i = 0; i < FW; ++i) {
                const u32x4 S = *reinterpret_cast<const u32x4 *>(&s_lds[buf][wave][((i * 2 + h) * 4 + kg) * 8]);
                const u32x4 Z = *reinterpret_cast<const u32x4 *>(&z_lds[buf][wave][((i * 2 + h) * 4 + kg) * 8]);
                // the field's constants: f0 is uniform over the wave, so these are scalar selects
                const uint32_t mk = f0 ? WField<NBITS>::mask(i + (NFW - 1) * FW) : WField<NBITS>::mask(i);
                const uint32_t ex = f0 ? WField<NBITS>::expo(i + (NFW - 1) * FW) : WField<NBITS>::expo(i);
                const f16 offv = (f16)(f0 ? WField<NBITS>::offset(i + (NFW - 1) * FW) : WField<NBITS>::offset(i));
                const f16x2 off = {offv, offv};
                u32x4 Au;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const f16x2 q = as_f16x2((mk & src[t]) | (~mk & ex)) - off; // exact code (one v_bfi_b32)
                    const f16x2 w = (q - as_f16x2(Z[t])) * as_f16x2(S[t]); // two fp16 roundings, as the reference
                    Au[t] = __builtin_bit_cast(uint32_t, w);
                }
                const f16x8 A = __builtin_bit_cast(f16x8, Au);
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[i][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[b], acc[i][b], 0, 0, 0);
            }
        }
    };

    // One step: 2 * FW groups (column half h, field i) of MB MFMAs that share an A operand.  Written as a pipeline
    // -- the weights of group g + 1 are rebuilt and the tables of group g + 2 read while the MFMAs of group g run --
    // because a wave has at most one other wave on its SIMD to hide latencies behind.
    auto compute_pipelined = [&](const u32x4 cw, int buf) __attribute__((always_inline)) {
        constexpr int NG = 2 * FW;
        const uint32_t d[4] = {cw.x, cw.y, cw.z, cw.w};
        u32x4 S[2], Z[2];
        f16x8 A[2];
        f16x8 B[2][MB];
        auto read_tables = [&](int g) __attribute__((always_inline)) {
            const int h = g / FW, i = g % FW;
            S[g & 1] = *reinterpret_cast<const u32x4 *>(&s_lds[buf][wave][((i * 2 + h) * 4 + kg) * 8]);
            Z[g & 1] = *reinterpret_cast<const u32x4 *>(&z_lds[buf][wave][((i * 2 + h) * 4 + kg) * 8]);
        };
        auto read_x = [&](int h) __attribute__((always_inline)) {
#pragma unroll
            for (int b = 0; b < MB; ++b)
                B[h][b] = *reinterpret_cast<const f16x8 *>(&x_lds[buf][xi][(((h * 4 + kg) * XP) + b * 16 + rr) * 8]);
        };
        auto build = [&](int g) __attribute__((always_inline)) {
            const int h = g / FW, i = g % FW;
            const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
            const uint32_t src[4] = {d0, d0 >> 8, d1, d1 >> 8};
            u32x4 Au;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const f16x2 q = as_f16x2((f_mask[i] & src[t]) | (~f_mask[i] & f_expo[i])) - f_off[i]; // exact code
                const f16x2 w = (q - as_f16x2(Z[g & 1][t])) * as_f16x2(S[g & 1][t]); // two fp16 roundings, as the reference
                Au[t] = __builtin_bit_cast(uint32_t, w);
            }
            A[g & 1] = __builtin_bit_cast(f16x8, Au);
        };
        read_tables(0);
        read_x(0);
        if constexpr (NG > 1)
            read_tables(1);
        build(0);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (g + 1 < NG)
                build(g + 1);
            if (g + 2 < NG)
                read_tables(g + 2);
            if (g == 0)
                read_x(1);
#pragma unroll
            for (int b = 0; b < MB; ++b)
                acc[g % FW][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[g & 1], B[g / FW][b], acc[g % FW][b], 0, 0, 0);
        }
    };

    // Step s is worked on from LDS half (s - s_begin) & 1 while step s + 1 is staged into the other half; the
    // register sets that step s + 1 leaves are refilled with the x tile of step s + 3 and the weights of step s + 5.
    Regs T0, T1, T2, T3;
    XRegs X0, X1;
    issue_x(X0, s_begin);
    issue(T0, s_begin);
    issue_x(X1, s_begin + 1);
    issue(T1, s_begin + 1);
    issue(T2, s_begin + 2);
    issue(T3, s_begin + 3);
    stage(T0, X0, 0);
    u32x4 cw = T0.cw;
    issue_x(X0, s_begin + 2);
    issue(T0, s_begin + 4);
    auto staged = [&]() __attribute__((always_inline)) { // what was staged is visible to those who read it
        if constexpr (PRIV) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        } else {
            __syncthreads();
        }
    };
    staged();
    // guard: whether the step may lie past the end of the block's K range (then it only moves data).  Without the
    // branch a step is one scheduling region, which the hints below shape: after every MFMA a few of the VALU
    // instructions that rebuild the next group's weights, stage the next step and form the addresses of later ones.
    auto step = [&](auto guard, Regs &Tn, XRegs &Xn, int buf, int s) __attribute__((always_inline)) {
        if constexpr (PIPE) {
            if (!decltype(guard)::value || s < s_end)
                compute_pipelined(cw, buf);
        } else {
            if (s < s_end)
                compute_simple(cw, buf);
        }
        stage(Tn, Xn, buf ^ 1);
        cw = Tn.cw;
        issue_x(Xn, s + 3);
        issue(Tn, s + 5);
        if constexpr (PIPE && !decltype(guard)::value) {
#pragma unroll
            for (int n = 0; n < 2 * FW * MB; ++n) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 5, 0); // up to five VALU
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // one LDS write
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); // one global load
            }
        }
        staged();
    };
    constexpr std::true_type guarded{};
    constexpr std::false_type whole{};
    int s = s_begin;
    if constexpr (PIPE) {
        for (; s + 4 <= s_end; s += 4) {
            step(whole, T1, X1, 0, s);
            step(whole, T2, X0, 1, s + 1);
            step(whole, T3, X1, 0, s + 2);
            step(whole, T0, X0, 1, s + 3);
        }
    }
    for (; s < (KW > 1 ? s_stop : s_end); s += 4) {
        step(guarded, T1, X1, 0, s);
        step(guarded, T2, X0, 1, s + 1);
        step(guarded, T3, X1, 0, s + 2);
        step(guarded, T0, X0, 1, s + 3);
    }

    if constexpr (KW > 1) {
        // the K parts of the block meet in LDS: part 0 adds the others' sums in a fixed order and goes on alone
        __syncthreads(); // every wave is through with its x tiles
        if (kpart > 0) {
#pragma unroll
            for (int i = 0; i < FW; ++i)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        red_lds[(kpart - 1) * NWK + wl][(i * MB + b) * 4 + v][lane] = acc[i][b][v];
        }
        __syncthreads();
        if (kpart > 0)
            return;
        for (int q = 0; q < KW - 1; ++q)
#pragma unroll
            for (int i = 0; i < FW; ++i)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        acc[i][b][v] += red_lds[q * NWK + wl][(i * MB + b) * 4 + v][lane];
        if constexpr (G2) {
            if (!p.part) {
                // Both projections are complete in this block.  The second one's wave hands its sums over through
                // the LDS rows only it has read; the first one's wave rounds both to fp16, applies SiLU in fp32
                // rounded once and multiplies in fp16 (the reference's three ops, src/custom_layers.py:253-256).
                if (second) {
#pragma unroll
                    for (int i = 0; i < FW; ++i)
#pragma unroll
                        for (int b = 0; b < MB; ++b)
#pragma unroll
                            for (int v = 0; v < 4; ++v)
                                red_lds[1][(i * MB + b) * 4 + v][lane] = acc[i][b][v];
                }
                __syncthreads(); // the two waves that are left
                if (second)
                    return;
#pragma unroll
                for (int i = 0; i < FW; ++i)
#pragma unroll
                    for (int b = 0; b < MB; ++b)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const float u = (float)(f16)acc[i][b][v];
                            const f16 h = (f16)(u / (1.0f + __expf(-u))) * (f16)red_lds[1][(i * MB + b) * 4 + v][lane];
                            acc[i][b][v] = (float)h; // exact: the store below rounds an fp16 value to fp16
                        }
            }
        }
    }

    // D layout: column = batch column (lane & 15) of block b, rows r = 4*(lane>>4) + v
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = m0 + b * 16 + (lane & 15);
        if (m >= p.M)
            continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 16 * rb + 4 * kg + v;
            const int64_t ng = (int64_t)F * (jp + (int64_t)r * p.GP); // first output row of the group of F
            const int64_t n = ng + f0;                                // first output row of this wave's fields
            if (p.part) { // K is split over blocks: fp32 partial sums, added by the finishing kernel
                float *dst = p.part + (second ? p.part_lstride : 0) +
                             (((int64_t)ks * (p.N / F) + ng / F) * p.M + m) * F + f0; // [K block][row group][batch row][F]
                if constexpr (FW == 4)
                    *reinterpret_cast<f32x4 *>(dst) = (f32x4){acc[0][b][v], acc[1][b][v], acc[2][b][v], acc[3][b][v]};
                else if constexpr (FW == 2)
                    *reinterpret_cast<float2 *>(dst) = make_float2(acc[0][b][v], acc[1][b][v]);
                else
                    *dst = acc[0][b][v];
                continue;
            }
            f16 o[FW];
            f16 *dst = p.y + (int64_t)m * p.N + n;
#pragma unroll
            for (int i = 0; i < FW; ++i) {
                o[i] = (f16)acc[i][b][v];
                if (p.bias)
                    o[i] = o[i] + p.bias[n + i];
                if (p.row_scale)
                    o[i] = o[i] * p.row_scale[m];
                if (p.accumulate)
                    o[i] = dst[i] + o[i];
            }
            if constexpr (FW == 4)
                *reinterpret_cast<f16x4 *>(dst) = (f16x4){o[0], o[1], o[2], o[3]};
            else if constexpr (FW == 2)
                *reinterpret_cast<f16x2 *>(dst) = (f16x2){o[0], o[1]};
            else
                *dst = o[0];
        }
    }
}

// y = cast(sum over the K blocks) (+ bias).  A block adds a tile of 16 row groups x 16 batch rows: read along the
// batch rows (the order the partial sums are stored in), written along the output row (the order y is stored in).
// GATE: two sets of partial sums, lstride floats apart; y = silu(a) * b with both projections rounded to fp16, SiLU
// in fp32 rounded once, product in fp16 (the reference's three ops, src/custom_layers.py:253-256).
template <int F, bool GATE>
__device__ __forceinline__ void tile_finish_block(const float *__restrict__ part, int KSP, int M, int N,
                                                  const f16 *__restrict__ bias, f16 *__restrict__ y, int64_t lstride,
                                                  const f16 *__restrict__ row_scale, int accumulate)
{
    __shared__ f16 t_lds[16][16][F];
    const int NG = N / F;
    const int g0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
    {
        const int m = m0 + (threadIdx.x & 15), gl = threadIdx.x >> 4, g = g0 + gl;
        if (m < M && g < NG) {
            float a[F], b[F];
#pragma unroll
            for (int i = 0; i < F; ++i)
                a[i] = b[i] = 0.f;
            for (int s = 0; s < KSP; ++s) {
                const float *src = part + (((int64_t)s * NG + g) * M + m) * F;
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    a[i] += src[i];
                    if constexpr (GATE)
                        b[i] += src[lstride + i];
                }
            }
#pragma unroll
            for (int i = 0; i < F; ++i) {
                f16 v = (f16)a[i];
                if constexpr (GATE) {
                    const float u = (float)v;
                    v = (f16)(u / (1.0f + __expf(-u))) * (f16)b[i];
                } else if (bias) {
                    v = v + bias[F * g + i];
                }
                if (row_scale)
                    v = v * row_scale[m];
                t_lds[threadIdx.x & 15][gl][i] = v;
            }
        }
    }
    __syncthreads();
    {
        const int gl = threadIdx.x & 15, m = m0 + (threadIdx.x >> 4), g = g0 + gl;
        if (m < M && g < NG) {
            f16 *dst = y + (int64_t)m * N + F * g;
#pragma unroll
            for (int i = 0; i < F; ++i)
                dst[i] = accumulate ? (f16)(dst[i] + t_lds[threadIdx.x >> 4][gl][i]) : t_lds[threadIdx.x >> 4][gl][i];
        }
    }
}

template <int F, bool GATE>
__global__ __launch_bounds__(256) void tile_finish_kernel(const float *__restrict__ part, int KSP, int M, int N,
                                                           const f16 *__restrict__ bias, f16 *__restrict__ y,
                                                           int64_t lstride, const f16 *__restrict__ row_scale,
                                                           int accumulate)
{
    tile_finish_block<F, GATE>(part, KSP, M, N, bias, y, lstride, row_scale, accumulate);
}

// The finishing passes of several launches as one: blockIdx.z names the launch, whose own grid may be smaller than
// this one's.
struct TileFinishGroup {
    TileFinish f[kTileFinishGroupMax];
};
template <int F> __global__ __launch_bounds__(256) void tile_finish_group_kernel(TileFinishGroup g)
{
    const TileFinish &d = g.f[blockIdx.z];
    if ((int)blockIdx.x * 16 >= d.N / F || (int)blockIdx.y * 16 >= d.M)
        return;
    tile_finish_block<F, false>(d.part, d.KSP, d.M, d.N, d.bias, d.y, 0, d.row_scale, d.accumulate);

}

// 3-bit codes (ten per 32-bit word, rows 10p .. 10p+9) rewritten as 4-bit codes (rows 2q, 2q+1 per byte, the even
// row in the high nibble): a 3-bit code is a 4-bit code with the same value, so the tile kernel then runs unchanged
// on the same tables.  Rows 2q and 2q+1 always share a word.  One thread: one word row, four columns.
__global__ __launch_bounds__(256) void repack3_as4_kernel(const uint32_t *__restrict__ in, int64_t N, int64_t K,
                                                          uint8_t *__restrict__ out)
{
    const int64_t words = (N + 9) / 10, chunks = K / 4;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < words * chunks; idx += (int64_t)gridDim.x * 256) {
        const int64_t p = idx / chunks, c = (idx - p * chunks) * 4;
        const u32x4 w = *reinterpret_cast<const u32x4 *>(in + p * K + c);
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const int64_t q = 5 * p + i;
            if (2 * q >= N)
                break;
            const int sh = 3 * (8 - 2 * i); // fields 2i (upper three bits of the six) and 2i+1
            uint32_t b = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t v = (w[t] >> sh) & 0x3Fu;
                b |= (((v >> 3) << 4) | (v & 7u)) << (8 * t);
            }
            *reinterpret_cast<uint32_t *>(out + q * K + c) = b;
        }
    }
}

// the layer as the tile kernel sees it: 3-bit layers are run through their 4-bit rewrite
hqq_linear tile_view(const hqq_linear *l)
{
    hqq_linear v = *l;
    if (l->nbits == 3)
        v.nbits = 4;
    return v;
}

size_t rewrite_bytes(const hqq_linear *l)
{
    return l->nbits == 3 ? (((size_t)(l->N / 2) * (size_t)l->K + 255) & ~(size_t)255) : 0;
}

struct TilePlan {
    int F, GP, RB, KT, BM, KSP, KTS;
    int JW, KW; // packed table rows per block, K parts per block
    int kinds; // 1: 8-bit tables as HQQ writes them, 3: fp16 tables (both run the pipelined kernel), 0: anything else
};

// nl: layers of the launch (2 for the fused gate, whose blocks count twice towards filling the chip)
bool make_plan(const hqq_linear *l, int64_t M, TilePlan &pl, int nl = 1)
{
    if ((l->nbits != 2 && l->nbits != 4) || M < 1)
        return false;
    const int F = 8 / l->nbits;
    const int64_t G = l->N / l->group_size;
    if (l->group_size % 16 != 0 || G % F != 0 || l->K % kStepK != 0 || l->N % 4 != 0 || (G / F) % kWaves != 0)
        return false;
    if (l->N * l->K / l->group_size >= (1ll << 31) || G / F > 65535 * (int64_t)kWaves || l->group_size / 16 > 65535)
        return false;
    if (!aligned16(l->codes))
        return false;
    for (const hqq_table *t : {&l->scale, &l->zero}) {
        if (t->kind == HQQ_TABLE_U8) {
            if (reinterpret_cast<uintptr_t>(t->data) & 3u)
                return false;
            if (t->meta_cols != 1 && (t->meta_cols % 4 != 0 || t->meta_cols < kStepK ||
                                      (reinterpret_cast<uintptr_t>(t->meta_scale) & 7u) ||
                                      (reinterpret_cast<uintptr_t>(t->meta_zero) & 7u)))
                return false;
        } else if (reinterpret_cast<uintptr_t>(t->data) & 7u) {
            return false;
        }
    }
    pl.F = F;
    pl.GP = (int)(G / F);
    pl.RB = l->group_size / 16;
    pl.KT = (int)(l->K / kStepK);
    const int sk = gemv::table_kind(l->scale), zk = gemv::table_kind(l->zero);
    pl.kinds = sk == TK_U8_COLS && zk == TK_U8_SCALAR ? 1 : (sk == TK_F16 && zk == TK_F16 ? 3 : 0);
    // batch tile: as wide as the batch, so that every weight is rebuilt as few times as possible; past 64 columns
    // the width (64 or 128, the latter in the pipelined kernel only) that costs less over all tiles, a tile costing
    // about 760 cycles of rebuilding and 8 cycles of MFMA per column and step
    pl.BM = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
    if (M > 128 && pl.kinds != 0 && ((M + 127) / 128) * (760 + 8 * 128) <= ((M + 63) / 64) * (760 + 8 * 64))
        pl.BM = 128;
    pl.BM = tuning_int("HQQ_TILE_BM", pl.BM);
    const int64_t mtiles = (M + pl.BM - 1) / pl.BM;
    if (mtiles > 65535)
        return false;
    pl.JW = kWaves, pl.KW = 1;
    if (pl.BM <= 32 && pl.kinds != 0 && !tuning_flag("HQQ_TILE_KW1")) {
        // the narrowest batch tile: a block is one packed row, its eight waves split the block's K range.  Blocks
        // along K only until the chip is covered, with at least four steps (256 columns) per wave.
        pl.JW = nl == 2 ? 2 : 1, pl.KW = 8; // a gate: both projections of a packed row in one block of sixteen waves
        if (nl == 2 && pl.BM == 32)
            pl.KW = 4; // the wider tile needs more registers than sixteen waves leave each
        const int64_t rows = (int64_t)pl.GP * pl.RB * mtiles;
        int64_t kb = (224 + rows - 1) / rows;
        if (kb > pl.KT / (4 * pl.KW))
            kb = pl.KT / (4 * pl.KW);
        if (kb < 1)
            kb = 1;
        kb = tuning_int("HQQ_TILE_KSP", (int)kb);
        pl.KTS = (int)((pl.KT + kb * pl.KW - 1) / (kb * pl.KW));
        pl.KSP = (pl.KT + pl.KTS * pl.KW - 1) / (pl.KTS * pl.KW);
        return (int64_t)pl.GP * pl.KSP <= 0x7fffffff;
    }
    // K is split over blocks until every SIMD has a wave (two for batches up to 128 rows, whose partial sums are
    // small), with at least eight steps per block.  Measured at Mixtral shapes: a split beyond that, which leaves
    // waves over for a partly filled round, costs 20-40 %.
    const int64_t blocks = (int64_t)(pl.GP / kWaves) * pl.RB * mtiles * nl;
    const int64_t waves = blocks * kWaves;
    int64_t ksp = (M <= 128 ? 2048 : 1024) / waves;
    if (ksp > 16)
        ksp = 16;
    if (ksp > pl.KT / 8)
        ksp = pl.KT / 8;
    if (ksp < 1)
        ksp = 1;
    ksp = tuning_int("HQQ_TILE_KSP", (int)ksp);
    pl.KTS = (int)((pl.KT + ksp - 1) / ksp);
    pl.KSP = (pl.KT + pl.KTS - 1) / pl.KTS;
    if ((int64_t)(pl.GP / kWaves) * pl.KSP * nl > 0x7fffffff)
        return false;
    return true;
}

template <int NBITS, int BM> void launch_tile2_kinds(const TileParams &p, const TilePlan &pl, dim3 grid, hipStream_t s)
{
    // the widest batch tile runs with two waves per packed table row (half the accumulators each)
    constexpr int NFW = BM == 128 ? 2 : 1;
    if constexpr (BM <= 32) {
        if constexpr (BM == 16) {
            if (pl.KW == 8 && pl.JW == 2) {
                if (pl.kinds == 1)
                    gemm_tile2_kernel<NBITS, BM, TK_U8_COLS, TK_U8_SCALAR, 1, 2, 8, true><<<grid, 16 * 64, 0, s>>>(p);
                else
                    gemm_tile2_kernel<NBITS, BM, TK_F16, TK_F16, 1, 2, 8, true><<<grid, 16 * 64, 0, s>>>(p);
                return;
            }
        }
        if (pl.KW == 8) {
            if (pl.kinds == 1)
                gemm_tile2_kernel<NBITS, BM, TK_U8_COLS, TK_U8_SCALAR, 1, 1, 8><<<grid, 8 * 64, 0, s>>>(p);
            else
                gemm_tile2_kernel<NBITS, BM, TK_F16, TK_F16, 1, 1, 8><<<grid, 8 * 64, 0, s>>>(p);
            return;
        }
        if (pl.KW == 4) {
            if (pl.kinds == 1)
                gemm_tile2_kernel<NBITS, BM, TK_U8_COLS, TK_U8_SCALAR, 1, 2, 4, true><<<grid, 8 * 64, 0, s>>>(p);
            else
                gemm_tile2_kernel<NBITS, BM, TK_F16, TK_F16, 1, 2, 4, true><<<grid, 8 * 64, 0, s>>>(p);
            return;
        }
    }
    if (pl.kinds == 1)
        gemm_tile2_kernel<NBITS, BM, TK_U8_COLS, TK_U8_SCALAR, NFW><<<grid, kWaves * NFW * 64, 0, s>>>(p);
    else
        gemm_tile2_kernel<NBITS, BM, TK_F16, TK_F16, NFW><<<grid, kWaves * NFW * 64, 0, s>>>(p);
}

template <int NBITS> void launch_tile2_bm(const TileParams &p, const TilePlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.BM == 16)
        launch_tile2_kinds<NBITS, 16>(p, pl, grid, s);
    else if (pl.BM == 32)
        launch_tile2_kinds<NBITS, 32>(p, pl, grid, s);
    else if (pl.BM == 64)
        launch_tile2_kinds<NBITS, 64>(p, pl, grid, s);
    else
        launch_tile2_kinds<NBITS, 128>(p, pl, grid, s);
}

void launch_tile2(const TileParams &p, const TilePlan &pl, int nbits, dim3 grid, hipStream_t s)
{
    if (nbits == 2)
        launch_tile2_bm<2>(p, pl, grid, s);
    else
        launch_tile2_bm<4>(p, pl, grid, s);
}

} // namespace

bool tile_supported(const hqq_linear *l, int64_t M)
{
    TilePlan pl;
    if (l->nbits == 3) { // up to four rows the 3-bit row kernel, run in passes of two rows, is faster than the rewrite
        const hqq_linear v = tile_view(l);
        return M > 4 && l->N % 2 == 0 && l->K % 4 == 0 && aligned16(l->codes) && make_plan(&v, M, pl);
    }
    return M > 4 && make_plan(l, M, pl);
}

// [arrival counters of the decode kernels][fp32 partial sums per layer][4-bit rewrite of 3-bit codes per layer]
static size_t tile_job_bytes(const hqq_linear *l, int64_t M, int nl)
{
    TilePlan pl;
    const hqq_linear v = tile_view(l);
    if (!make_plan(&v, M, pl, nl))
        return 0;
    const bool partial = pl.KSP > 1 || (nl == 2 && pl.KW == 1);
    const size_t one = partial ? (((size_t)pl.KSP * (size_t)M * (size_t)l->N * sizeof(float) + 255) & ~(size_t)255) : 0;
    const size_t body = nl * (one + rewrite_bytes(l));
    return body ? workspace_head_bytes() + body : 0;
}

// one layer (lb == nullptr) or the two projections of a gate: y = x W^T (+ bias), or y = silu(x Wa^T) * (x Wb^T)
// part_at / defer (one layer only): the partial sums of a K split go to part_at instead of the workspace, and the
// finishing pass is described in *defer instead of launched (defer->part is null when there is nothing to finish)
static int tile_job(const hqq_linear *la, const hqq_linear *lb, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                    hipStream_t s, const SmallBatchEpilogue *ep = nullptr, void *part_at = nullptr, TileFinish *defer = nullptr)
{
    if (defer) {
        *defer = TileFinish{};
        if (lb || !part_at || (reinterpret_cast<uintptr_t>(part_at) & 255u))
            return HQQ_E_UNSUPPORTED;
    }
    const int nl = lb ? 2 : 1;
    TilePlan pl;
    hqq_linear view[2] = {tile_view(la), tile_view(lb ? lb : la)};
    if (!make_plan(&view[0], M, pl, nl) || (reinterpret_cast<uintptr_t>(x) & 15u))
        return HQQ_E_UNSUPPORTED;
    if (nl == 2 && pl.kinds == 0)
        return HQQ_E_UNSUPPORTED;
    const bool scaled = ep && (ep->row_scale || ep->accumulate);
    if (scaled && (pl.kinds == 0 || nl == 2))
        return HQQ_E_UNSUPPORTED;
    const size_t need = tile_job_bytes(la, M, nl);
    if (need > 0 && (!ws || ws_bytes < need))
        return HQQ_E_WORKSPACE;
    const bool partial = pl.KSP > 1 || (nl == 2 && pl.KW == 1);
    const size_t one = partial ? (((size_t)pl.KSP * (size_t)M * (size_t)la->N * sizeof(float) + 255) & ~(size_t)255) : 0;
    char *body = static_cast<char *>(ws) + workspace_head_bytes();
    if (la->nbits == 3) {
        const hqq_linear *src[2] = {la, lb};
        for (int i = 0; i < nl; ++i) {
            uint8_t *codes4 = reinterpret_cast<uint8_t *>(body + nl * one + i * rewrite_bytes(la));
            const int64_t work = ((la->N + 9) / 10) * (la->K / 4);
            const int grid = (int)(work / 256 < 1 ? 1 : (work / 256 > 8192 ? 8192 : work / 256));
            repack3_as4_kernel<<<grid, 256, 0, s>>>(static_cast<const uint32_t *>(src[i]->codes), la->N, la->K, codes4);
            view[i].codes = codes4;
        }
    }
    const hqq_linear *l = &view[0];
    TileParams p = {};
    p.codes = static_cast<const uint8_t *>(l->codes);
    p.sc = make_table(l->scale), p.zr = make_table(l->zero);
    p.sc_inv = l->scale.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->scale.meta_cols) : 0;
    p.zr_inv = l->zero.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->zero.meta_cols) : 0;
    p.codes_b = static_cast<const uint8_t *>(view[1].codes);
    p.sc_b = make_table(view[1].scale), p.zr_b = make_table(view[1].zero);
    p.sc_b_inv = view[1].scale.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)view[1].scale.meta_cols) : 0;
    p.JB = pl.GP / pl.JW;
    p.part_lstride = (int64_t)(one / sizeof(float));
    p.x = x, p.bias = nl == 1 ? static_cast<const f16 *>(l->bias) : nullptr, p.y = y;
    p.M = (int)M, p.N = (int)l->N, p.K = (int)l->K, p.GP = pl.GP, p.KT = pl.KT;
    p.KSP = pl.KSP, p.KTS = pl.KTS;
    p.row_scale = scaled ? ep->row_scale : nullptr, p.accumulate = scaled ? ep->accumulate : 0;
    p.part = partial ? reinterpret_cast<float *>(defer ? static_cast<char *>(part_at) : body) : nullptr;
    // blocks along x: packed rows (per projection, unless a block holds both) by K blocks
    const int jrows = pl.JW == 2 ? pl.GP : pl.GP / pl.JW * nl;
    const dim3 grid((unsigned)(jrows * pl.KSP), (unsigned)pl.RB, (unsigned)((M + pl.BM - 1) / pl.BM));
    if (pl.kinds != 0) {
        launch_tile2(p, pl, l->nbits, grid, s);
    } else if (l->nbits == 2) {
        if (pl.BM == 16)
            gemm_tile_kernel<2, 16><<<grid, kWaves * 64, 0, s>>>(p);
        else if (pl.BM == 32)
            gemm_tile_kernel<2, 32><<<grid, kWaves * 64, 0, s>>>(p);
        else
            gemm_tile_kernel<2, 64><<<grid, kWaves * 64, 0, s>>>(p);
    } else {
        if (pl.BM == 16)
            gemm_tile_kernel<4, 16><<<grid, kWaves * 64, 0, s>>>(p);
        else if (pl.BM == 32)
            gemm_tile_kernel<4, 32><<<grid, kWaves * 64, 0, s>>>(p);
        else
            gemm_tile_kernel<4, 64><<<grid, kWaves * 64, 0, s>>>(p);
    }
    int rc = launch_status();
    if (rc != HQQ_OK || !partial)
        return rc;
    if (defer) {
        defer->part = p.part, defer->KSP = pl.KSP, defer->M = (int)M, defer->N = (int)l->N, defer->F = pl.F;
        defer->bias = p.bias, defer->y = y, defer->row_scale = p.row_scale, defer->accumulate = p.accumulate;
        return HQQ_OK;
    }
    const dim3 fgrid((unsigned)((l->N / pl.F + 15) / 16), (unsigned)((M + 15) / 16));
    if (nl == 2) {
        if (pl.F == 4)
            tile_finish_kernel<4, true><<<fgrid, 256, 0, s>>>(p.part, pl.KSP, (int)M, (int)l->N, nullptr, y, p.part_lstride, nullptr, 0);
        else
            tile_finish_kernel<2, true><<<fgrid, 256, 0, s>>>(p.part, pl.KSP, (int)M, (int)l->N, nullptr, y, p.part_lstride, nullptr, 0);
    } else if (pl.F == 4) {
        tile_finish_kernel<4, false><<<fgrid, 256, 0, s>>>(p.part, pl.KSP, (int)M, (int)l->N, p.bias, y, 0, p.row_scale, p.accumulate);
    } else {
        tile_finish_kernel<2, false><<<fgrid, 256, 0, s>>>(p.part, pl.KSP, (int)M, (int)l->N, p.bias, y, 0, p.row_scale, p.accumulate);
    }
    return launch_status();
}

size_t tile_workspace_bytes(const hqq_linear *l, int64_t M) { return tile_job_bytes(l, M, 1); }

// bytes of partial sums a one-layer launch writes (0: K is not split, nothing to finish)
size_t tile_partial_bytes(const hqq_linear *l, int64_t M)
{
    TilePlan pl;
    const hqq_linear v = tile_view(l);
    if (!make_plan(&v, M, pl, 1) || pl.KSP <= 1)
        return 0;
    return ((size_t)pl.KSP * (size_t)M * (size_t)l->N * sizeof(float) + 255) & ~(size_t)255;
}

int launch_tile_matmul_deferred(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                                const SmallBatchEpilogue *ep, void *part_at, TileFinish *finish)
{
    return tile_job(l, nullptr, x, M, y, ws, ws_bytes, s, ep, part_at, finish);
}

// the finishing passes of up to kTileFinishGroupMax deferred launches in one launch per code width
int launch_tile_finish_group(const TileFinish *f, int n, hipStream_t s)
{
    for (int F = 2; F <= 4; F += 2) {
        TileFinishGroup g = {};
        int cnt = 0, gx = 0, gy = 0;
        for (int i = 0; i < n; ++i) {
            if (!f[i].part || f[i].F != F)
                continue;
            if (cnt == kTileFinishGroupMax)
                return HQQ_E_UNSUPPORTED;
            g.f[cnt++] = f[i];
            const int x = (f[i].N / F + 15) / 16, y = (f[i].M + 15) / 16;
            gx = x > gx ? x : gx, gy = y > gy ? y : gy;
        }
        if (!cnt)
            continue;
        const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)cnt);
        if (F == 4)
            tile_finish_group_kernel<4><<<grid, 256, 0, s>>>(g);
        else
            tile_finish_group_kernel<2><<<grid, 256, 0, s>>>(g);
        const int rc = launch_status();
        if (rc != HQQ_OK)
            return rc;
    }
    return HQQ_OK;
}

int launch_tile_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                       const SmallBatchEpilogue *ep)
{
    return tile_job(l, nullptr, x, M, y, ws, ws_bytes, s, ep);
}

// whether the routing weight and the accumulation can ride in the matmul's own epilogue
bool tile_epilogue_supported(const hqq_linear *l, int64_t M)
{
    TilePlan pl;
    const hqq_linear v = tile_view(l);
    return tile_supported(l, M) && make_plan(&v, M, pl) && pl.kinds != 0;
}

// the two projections of an expert's gate in one launch, silu(a) * b applied by the finishing kernel
bool tile_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    TilePlan a, b;
    const hqq_linear va = tile_view(w1), vb = tile_view(w3);
    return tile_supported(w1, M) && tile_supported(w3, M) && w1->N == w3->N && w1->K == w3->K && w1->nbits == w3->nbits &&
           w1->group_size == w3->group_size && !w1->bias && !w3->bias && make_plan(&va, M, a, 2) && make_plan(&vb, M, b, 2) &&
           a.kinds != 0 && a.kinds == b.kinds && w1->scale.meta_cols == w3->scale.meta_cols;
}

size_t tile_gate_workspace_bytes(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    return tile_gate_supported(w1, w3, M) ? tile_job_bytes(w1, M, 2) : 0;
}

int launch_tile_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                        size_t ws_bytes, hipStream_t s)
{
    if (!tile_gate_supported(w1, w3, M))
        return HQQ_E_UNSUPPORTED;
    return tile_job(w1, w3, x, M, h, ws, ws_bytes, s);
}

} // namespace hqq
