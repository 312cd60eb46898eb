// Small-batch (M <= 16) unpack-dequantise-matmul for 2- and 4-bit codes: the
// decode-time GEMV family.  Bounded by HBM: every code byte and every scale /
// zero byte is read once, as 128-bit and 32-bit coalesced loads.
//
// Geometry.  HQQ groups run down the output dimension: weight (n, k) uses table
// row j = n % G, so the `gs` rows n = j + r*G (r = 0..gs-1) share one scale and
// one zero per column k.  Packed row p holds F = 8/nbits adjacent output rows,
// hence F adjacent table rows; "jp" = p % (G/F) names them and r = p / (G/F).
//
// A wavefront owns one tile (jp, 16 values of r) and a K slab.  Because its 16
// rows share scale and zero, the scale is folded into the activations instead of
// the weights:
//      y[n, m] = sum_k q[n,k] * xs[j,k,m]  -  sum_k z[j,k] * xs[j,k,m],     xs = s[j,k] * x[m,k]
// so the per-weight work is only "extract the code as an fp16 number".  The
// sum over k runs on the matrix cores (v_mfma_f32_16x16x32_f16: A = 16 rows r x
// 32 k of codes, B = 32 k x 16 batch columns of xs), which also removes every
// cross-lane reduction.  A code becomes an fp16 operand with one AND: masked in
// place it is the subnormal q * 2^(pos-24), which the matrix cores take exactly.
//
// Per 64-column step a wave does
//   table phase : each lane de-quantises F*64/64 table entries x 4 columns (8-bit
//                 codes with their fp16 meta pair, or fp16 tables), multiplies by
//                 x for every batch row, adds z*xs to its bias sum and writes xs
//                 to LDS in B-operand order;
//   code phase  : one 128-bit load per lane (16 columns of one packed row), 2*F
//                 MFMAs fed from registers (A) and LDS (B).
// Split-K partial sums of the slabs are combined by a second, tiny kernel that
// also applies the epilogue (bias, fp16 cast, SiLU-gate product, routing scale).
#include "hqq_common.hpp"
#include "table_reader.hpp"

#include <cstdlib>

namespace hqq {
namespace {

constexpr int kStepK = 64;       // columns per wave step
// xs = s * x is held in fp16; scales are ~1e-3..1e-1, so the scale is raised by 2^5 first to keep small
// activations out of the fp16 subnormal range (|s*x| would have to exceed 2047 to overflow).  Undone in fp32.
constexpr float kXsScale = 32.0f;

struct SBLayer {
    const uint8_t *codes;
    Table sc, zr;
    uint32_t sc_inv, zr_inv; // floor((2^32-1) / meta_cols): the kernel reduces indices mod meta_cols without dividing
    float *part;             // [NSG][M][N]
};

struct SBParams {
    SBLayer layer[2];
    const f16 *x;
    int M, N, K;
    int GP;     // G / F: packed table rows
    int RB;     // gs / 16: row blocks per jp
    int RBG;    // RB / WR: r-block groups per jp
    int WR, WS; // waves of a block along r-blocks / along K slabs
    int WR_log2;
    int force_partial; // always leave fp32 partial sums (the fused gate pass)
    int probe;         // tuning aid: 1 = wait for the loads but skip the arithmetic (memory-only time)
    int KT;     // K / 64
    int NSG;    // slab groups (= partial-sum copies)
};

// Field i of a packed byte sits at bit `pos` of the byte.  Masked in place, the low byte of a 16-bit half reads as
// the fp16 SUBNORMAL number q * 2^(pos - 24): no shift, no convert.  The matrix cores take fp16 subnormals
// exactly (checked on gfx950 by the parity tests: a flush to zero would zero every output), so the code goes to
// the MFMA as it is and the factor 2^(24 - pos) is applied once to the fp32 result.
template <int NBITS> struct Field {
    static constexpr int F = 8 / NBITS;
    static constexpr int pos(int i) { return NBITS * (F - 1 - i); }
    static constexpr uint32_t mask(int i) { return (((1u << NBITS) - 1u) * 0x00010001u) << pos(i); }
    static constexpr float unscale(int i) { return (float)(1u << (24 - pos(i))); }
};

// sum over the 16 lanes of a DPP row; every lane of the row gets the total
__device__ __forceinline__ float row16_sum(float v)
{
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)); // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)); // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)); // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)); // row_mirror
    return v;
}

// What the block does with its finished tile.
struct SBEpilogue {
    f16 *y;               // direct store target (NSG == 1)
    const f16 *bias;      // fp16[N] or null
    const f16 *row_scale; // fp16[M] or null
    int accumulate;
};

template <int NBITS, int MT, int WAVES, int SK, int TMODE>
__global__ __launch_bounds__(WAVES * 64) void smallbatch_kernel(SBParams p, SBEpilogue ep)
{
    constexpr int F = 8 / NBITS;
    constexpr int XS_HALVES = F * 2 * 4 * MT * 8; // per wave, one step
    constexpr int SCALE_KIND = TMODE == TM_HQQ8 ? 1 : (TMODE == TM_F16 ? 3 : 0);
    constexpr int ZERO_KIND = TMODE == TM_HQQ8 ? 2 : (TMODE == TM_F16 ? 3 : 0);
    __shared__ __attribute__((aligned(16))) f16 xs_lds[WAVES + 1][XS_HALVES]; // [WAVES] stays zero
    __shared__ float bias_lds[WAVES][F][MT];
    __shared__ __attribute__((aligned(16))) float red_lds[WAVES][16][MT][F]; // [wave][row r][batch m][i]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wr = wave & (p.WR - 1), ws = wave >> p.WR_log2;
    // grid: x = K slab group, y = (layer, r-block group), z = jp
    const int sg = blockIdx.x;
    const int layer = (int)blockIdx.y >= p.RBG ? 1 : 0;
    const int rbg = (int)blockIdx.y - layer * p.RBG;
    const SBLayer &L = p.layer[layer];
    const int jp = blockIdx.z;
    const int rb = rbg * p.WR + wr;
    const int step_begin = (sg * p.WS + ws) * SK;
    const bool active = step_begin < p.KT; // KT is a multiple of SK; idle waves only join the reduction

    const int K = p.K;
    const int M = MT == 1 ? 1 : p.M;
    // code lane role: packed row of (jp, r), 16 columns at 16*kg
    const int rr = lane & 15, kg = lane >> 4;
    const uint32_t prow = (uint32_t)jp + (uint32_t)(16 * rb + rr) * (uint32_t)p.GP;
    const uint32_t coff = prow * (uint32_t)K + (uint32_t)(step_begin * kStepK + 16 * kg); // codes are < 4 GiB
    // table lane role: table row F*jp + ti, columns 4*kq .. 4*kq+3
    const int ti = lane >> 4, kq = lane & 15;
    const bool tlane = ti < F;
    const uint32_t c0 = (uint32_t)(F * jp + (tlane ? ti : 0)) * (uint32_t)K + (uint32_t)(step_begin * kStepK + 4 * kq);
    const uint32_t xoff = (uint32_t)(step_begin * kStepK + 4 * kq);

    // ---- issue every load of the wave's slab up front; the whole matrix is in flight at once
    u32x4 cw[SK];
    TableRaw sraw[SK], zraw[SK];
    u32x2 xv[SK][MT];
    TableCursor<SCALE_KIND> sc;
    TableCursor<ZERO_KIND> zr;
    sc.init(L.sc, c0, L.sc_inv);
    zr.init(L.zr, c0, L.zr_inv);
    if (active) {
#pragma unroll
        for (int s = 0; s < SK; ++s) {
            cw[s] = *reinterpret_cast<const u32x4 *>(L.codes + (coff + s * kStepK));
            if (tlane) {
                sraw[s] = table_load(sc);
                zraw[s] = table_load(zr);
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    if (m < M)
                        xv[s][m] = *reinterpret_cast<const u32x2 *>(p.x + (xoff + (uint32_t)(m * K + s * kStepK)));
            }
            sc.advance(kStepK);
            zr.advance(kStepK);
        }
    }

    // where this lane's xs go: entry ((ti*2 + h)*4 + kgt)*MT + m, 16 B each, second half when kq is odd
    f16 *xs_w = &xs_lds[wave][((((ti * 2 + ((kq >> 1) & 1)) * 4 + (kq >> 2)) * MT) * 8) + 4 * (kq & 1)];
    // B operand: column = batch row lane&15; lanes past MT read the block's all-zero copy
    const int mcol = lane & 15;
    const f16 *xs_r = mcol < MT ? &xs_lds[wave][(kg * MT + mcol) * 8] : &xs_lds[WAVES][0];
    // LDS rows of batch entries m >= M are never written by the table phase: clear once
    if (M < MT)
        for (int i = lane; i < XS_HALVES / 8; i += 64)
            *reinterpret_cast<u32x4 *>(&xs_lds[wave][i * 8]) = (u32x4){0, 0, 0, 0};
    if constexpr (MT < 16) {
        if (wave == 0)
            for (int i = lane; i < XS_HALVES / 8; i += 64)
                *reinterpret_cast<u32x4 *>(&xs_lds[WAVES][i * 8]) = (u32x4){0, 0, 0, 0};
        __syncthreads();
    }

    f32x4 acc[F];
#pragma unroll
    for (int i = 0; i < F; ++i)
        acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float bias_acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        bias_acc[m] = 0.f;

    if (p.probe == 1 && active) { // keep every load alive, do no arithmetic
        uint32_t x = 0;
#pragma unroll
        for (int s = 0; s < SK; ++s) {
            x ^= cw[s].x ^ cw[s].y ^ cw[s].z ^ cw[s].w;
            if (tlane)
                x ^= sraw[s].data.x ^ zraw[s].data.x ^ sraw[s].ms.x ^ sraw[s].mz.y ^ xv[s][0].x;
        }
        acc[0][0] = (float)(x & 1u);
    } else if (active) {
#pragma unroll
        for (int s = 0; s < SK; ++s) {
            // ---- table phase
            if (tlane) {
                f16x2 s01, s23, z01, z23;
                table_decode(sc, sraw[s], s01, s23);
                table_decode(zr, zraw[s], z01, z23);
                s01 = s01 * (f16x2){(f16)kXsScale, (f16)kXsScale};
                s23 = s23 * (f16x2){(f16)kXsScale, (f16)kXsScale};
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    if (m < M) {
                        const f16x2 a01 = s01 * as_f16x2(xv[s][m].x);
                        const f16x2 a23 = s23 * as_f16x2(xv[s][m].y);
                        bias_acc[m] = __builtin_amdgcn_fdot2(z01, a01, bias_acc[m], false);
                        bias_acc[m] = __builtin_amdgcn_fdot2(z23, a23, bias_acc[m], false);
                        // B-operand order inside an 8-column block: columns (0,2,1,3)
                        const f16x4 o = {a01.x, a23.x, a01.y, a23.y};
                        *reinterpret_cast<f16x4 *>(xs_w + m * 8) = o;
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

            // ---- code phase: all B operands first, then extract-and-multiply
            f16x8 B[2][F];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < F; ++i)
                    B[h][i] = *reinterpret_cast<const f16x8 *>(xs_r + ((i * 2 + h) * 4 * MT) * 8);
            const uint32_t d[4] = {cw[s].x, cw[s].y, cw[s].z, cw[s].w};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
                const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const uint32_t mk = Field<NBITS>::mask(i);
                    const u32x4 Au = {d0 & mk, d0s & mk, d1 & mk, d1s & mk};
                    const f16x8 A = __builtin_bit_cast(f16x8, Au);
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[h][i], acc[i], 0, 0, 0);
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }

    // ---- bias: sum the 16 table lanes of each table row, hand it to the lanes that hold D
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float v = row16_sum(bias_acc[m]);
        if (tlane && kq == 0)
            bias_lds[wave][ti][m] = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // D layout: column = batch row (lane & 15), rows 4*(lane>>4)+v.  Every wave leaves its tile, bias removed and
    // still scaled, in LDS as [row r][batch m][i]; then one thread per (r-block, r, m) adds the block's K slabs.
    if (mcol < MT) {
        float bz[F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            bz[i] = bias_lds[wave][i][mcol];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float o[F];
#pragma unroll
            for (int i = 0; i < F; ++i)
                o[i] = __builtin_fmaf(acc[i][v], Field<NBITS>::unscale(i), -bz[i]);
            float *dst = &red_lds[wave][4 * kg + v][mcol][0];
            if constexpr (F == 4)
                *reinterpret_cast<f32x4 *>(dst) = (f32x4){o[0], o[1], o[2], o[3]};
            else
                *reinterpret_cast<float2 *>(dst) = make_float2(o[0], o[1]);
        }
    }
    __syncthreads();
    // a DPP row of 16 lanes per output (wr, r, m): lane w of the row brings slab w (WS <= 16)
    for (int t = threadIdx.x; t < p.WR * 16 * MT * 16; t += WAVES * 64) {
        const int w = t & 15, u = t >> 4;
        const int wr_t = u / (16 * MT), r_t = (u / MT) & 15, m_t = u % MT;
        float o[F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            o[i] = 0.f;
        if (w < p.WS) {
            const float *src = &red_lds[w * p.WR + wr_t][r_t][m_t][0];
#pragma unroll
            for (int i = 0; i < F; ++i)
                o[i] = src[i];
        }
#pragma unroll
        for (int i = 0; i < F; ++i)
            o[i] = row16_sum(o[i]) * (1.0f / kXsScale);
        if (w != 0 || m_t >= M)
            continue;

        // ---- row r = 16*rb + r_t of the tile holds outputs n = F*(jp + r*GP) + i
        const int r = 16 * (rbg * p.WR + wr_t) + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * p.GP);
        if (p.NSG > 1 || p.force_partial) { // split over several blocks: fp32 partial sums for the finish kernel
            float *dst = L.part + ((int64_t)sg * M + m_t) * p.N + n;
            if constexpr (F == 4)
                *reinterpret_cast<f32x4 *>(dst) = (f32x4){o[0], o[1], o[2], o[3]};
            else
                *reinterpret_cast<float2 *>(dst) = make_float2(o[0], o[1]);
            continue;
        }
        f16 *dst = ep.y + (int64_t)m_t * p.N + n;
        f16 h[F];
#pragma unroll
        for (int i = 0; i < F; ++i) {
            f16 val = (f16)o[i];
            if (ep.bias)
                val = val + ep.bias[n + i];
            if (ep.row_scale)
                val = val * ep.row_scale[m_t];
            if (ep.accumulate)
                val = dst[i] + val;
            h[i] = val;
        }
        if constexpr (F == 4)
            *reinterpret_cast<f16x4 *>(dst) = (f16x4){h[0], h[1], h[2], h[3]};
        else
            *reinterpret_cast<f16x2 *>(dst) = (f16x2){h[0], h[1]};
    }
}

// Sum the slab partials and apply the epilogue.  MODE 0: y = cast(sum) (+bias) (*row_scale) (+= y);
// MODE 1: h = silu(sum of layer 0) * (sum of layer 1), the expert FFN's gate.
template <int MODE>
__global__ __launch_bounds__(64) void smallbatch_finish_kernel(const float *__restrict__ part0,
                                                                const float *__restrict__ part1, int NSG, int M,
                                                                int N, const f16 *__restrict__ bias,
                                                                const f16 *__restrict__ row_scale, int accumulate,
                                                                f16 *__restrict__ y)
{
    const int64_t total = (int64_t)M * N / 4;
    const int64_t stride = (int64_t)M * N;
    for (int64_t idx = blockIdx.x * 64ll + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 64) {
        const int64_t e = idx * 4;
        f32x4 a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
        for (int s = 0; s < NSG; ++s) {
            a += *reinterpret_cast<const f32x4 *>(part0 + s * stride + e);
            if constexpr (MODE == 1)
                b += *reinterpret_cast<const f32x4 *>(part1 + s * stride + e);
        }
        f16x4 out;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if constexpr (MODE == 1) {
                // the reference rounds both projections to fp16, applies SiLU in fp32, rounds, multiplies in fp16
                const float g = (float)(f16)a[t];
                const f16 act = (f16)(g / (1.0f + __expf(-g)));
                out[t] = act * (f16)b[t];
            } else {
                f16 v = (f16)a[t];
                if (bias)
                    v = v + bias[(e + t) % N];
                if (row_scale)
                    v = v * row_scale[(e + t) / N];
                if (accumulate)
                    v = y[e + t] + v;
                out[t] = v;
            }
        }
        *reinterpret_cast<f16x4 *>(y + e) = out;
    }
}

struct SBPlan {
    int F, GP, RB, WR, WS, KT, NS, NSG, MT, WAVES, SK, TMODE;
};

int table_kind(const hqq_table &t) { return t.kind == HQQ_TABLE_F16 ? 3 : (t.meta_cols == 1 ? 2 : 1); }

bool make_plan(const hqq_linear *l, int64_t M, SBPlan &pl)
{
    if (l->nbits != 2 && l->nbits != 4)
        return false;
    if (M < 1 || M > 16)
        return false;
    const int F = 8 / l->nbits;
    const int64_t G = l->N / l->group_size;
    if (l->group_size % 16 != 0 || G % F != 0 || l->K % kStepK != 0 || l->N % 4 != 0)
        return false;
    if (l->N * l->K / l->group_size >= (1ll << 31) || l->N * l->K / F >= (1ll << 32) || 16 * l->K >= (1ll << 31))
        return false; // 32-bit offsets inside the kernel
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
    pl.MT = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)));
    pl.WAVES = pl.MT <= 4 ? 16 : (pl.MT == 8 ? 8 : 4);
    {
        const int forced = tuning_int("HQQ_SB_BLOCK_WAVES", 0);
        if ((forced == 4 || forced == 8 || forced == 16) && forced <= pl.WAVES)
            pl.WAVES = forced;
    }
    pl.WR = pl.RB >= 4 ? 4 : (pl.RB >= 2 ? 2 : 1);
    if (pl.RB % pl.WR != 0)
        pl.WR = 1;
    pl.KT = (int)(l->K / kStepK);
    pl.SK = pl.KT % 4 == 0 ? 4 : (pl.KT % 2 == 0 ? 2 : 1); // steps per wave; their loads are all issued up front
    pl.NS = pl.KT / pl.SK;
    const int ks = table_kind(l->scale), kz = table_kind(l->zero);
    pl.TMODE = (ks == 1 && kz == 2) ? TM_HQQ8 : ((ks == 3 && kz == 3) ? TM_F16 : TM_GENERIC);
    // a block need not be wider than the slabs there are
    while (pl.WAVES > 4 && pl.WAVES / pl.WR >= 2 * pl.NS)
        pl.WAVES /= 2;
    pl.WS = pl.WAVES / pl.WR;
    pl.NSG = (pl.NS + pl.WS - 1) / pl.WS;
    return true;
}

template <int NBITS, int MT, int WAVES, int SK>
void launch_tm(const SBParams &p, const SBEpilogue &ep, int tmode, dim3 grid, hipStream_t s)
{
    const dim3 block(WAVES * 64);
    if (tmode == TM_HQQ8)
        smallbatch_kernel<NBITS, MT, WAVES, SK, TM_HQQ8><<<grid, block, 0, s>>>(p, ep);
    else if (tmode == TM_F16)
        smallbatch_kernel<NBITS, MT, WAVES, SK, TM_F16><<<grid, block, 0, s>>>(p, ep);
    else
        smallbatch_kernel<NBITS, MT, WAVES, SK, TM_GENERIC><<<grid, block, 0, s>>>(p, ep);
}

template <int NBITS, int MT, int WAVES>
void launch_sk(const SBParams &p, const SBEpilogue &ep, const SBPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.SK == 4)
        launch_tm<NBITS, MT, WAVES, 4>(p, ep, pl.TMODE, grid, s);
    else if (pl.SK == 2)
        launch_tm<NBITS, MT, WAVES, 2>(p, ep, pl.TMODE, grid, s);
    else
        launch_tm<NBITS, MT, WAVES, 1>(p, ep, pl.TMODE, grid, s);
}

template <int NBITS, int MT>
void launch_mt(const SBParams &p, const SBEpilogue &ep, const SBPlan &pl, dim3 grid, hipStream_t s)
{
    // wide blocks only where their LDS (xs staging grows with MT) fits
    if constexpr (MT <= 4) {
        if (pl.WAVES == 16)
            return launch_sk<NBITS, MT, 16>(p, ep, pl, grid, s);
    }
    if constexpr (MT <= 8) {
        if (pl.WAVES >= 8)
            return launch_sk<NBITS, MT, 8>(p, ep, pl, grid, s);
    }
    launch_sk<NBITS, MT, 4>(p, ep, pl, grid, s);
}

template <int NBITS>
void launch_main(const SBParams &p, const SBEpilogue &ep, const SBPlan &pl, dim3 grid, hipStream_t s)
{
    switch (pl.MT) {
    case 1: launch_mt<NBITS, 1>(p, ep, pl, grid, s); break;
    case 2: launch_mt<NBITS, 2>(p, ep, pl, grid, s); break;
    case 4: launch_mt<NBITS, 4>(p, ep, pl, grid, s); break;
    case 8: launch_mt<NBITS, 8>(p, ep, pl, grid, s); break;
    default: launch_mt<NBITS, 16>(p, ep, pl, grid, s); break;
    }
}

int finish_grid(int64_t M, int64_t N)
{
    int64_t b = (M * N / 4 + 63) / 64;
    return (int)(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

} // namespace

bool smallbatch_supported(const hqq_linear *l, int64_t M)
{
    SBPlan pl;
    return strip_supported(l, M) || make_plan(l, M, pl);
}

// the first workspace_head_bytes() of a workspace belong to the slab kernel's arrival counters
size_t smallbatch_workspace_bytes(const hqq_linear *l, int64_t M)
{
    if (strip_supported(l, M))
        return strip_workspace_bytes(l, M);
    SBPlan pl;
    if (!make_plan(l, M, pl))
        return 0;
    return workspace_head_bytes() + (size_t)pl.NSG * (size_t)M * (size_t)l->N * sizeof(float);
}

static void fill_params(SBParams &p, const SBPlan &pl, const hqq_linear *l, int which, float *part)
{
    p.layer[which].codes = static_cast<const uint8_t *>(l->codes);
    p.layer[which].sc = make_table(l->scale);
    p.layer[which].zr = make_table(l->zero);
    p.layer[which].part = part;
    p.layer[which].sc_inv = l->scale.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->scale.meta_cols) : 0;
    p.layer[which].zr_inv = l->zero.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->zero.meta_cols) : 0;
    p.N = (int)l->N, p.K = (int)l->K;
    p.GP = pl.GP, p.RB = pl.RB, p.RBG = pl.RB / pl.WR, p.WR = pl.WR, p.WR_log2 = pl.WR == 4 ? 2 : (pl.WR == 2 ? 1 : 0), p.WS = pl.WS, p.KT = pl.KT, p.NSG = pl.NSG;
}

int launch_smallbatch_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                             const SmallBatchEpilogue &ep, hipStream_t s)
{
    if (strip_supported(l, M))
        return launch_strip_matmul(l, x, M, y, ws, ws_bytes, ep, s);
    SBPlan pl;
    if (!make_plan(l, M, pl))
        return HQQ_E_UNSUPPORTED;
    if (pl.NSG > 1 && ws_bytes < smallbatch_workspace_bytes(l, M))
        return HQQ_E_WORKSPACE;
    SBParams p = {};
    fill_params(p, pl, l, 0, reinterpret_cast<float *>(static_cast<char *>(ws) + workspace_head_bytes()));
    p.layer[1] = p.layer[0];
    p.x = x, p.M = (int)M;
    p.probe = tuning_int("HQQ_SB_PROBE", 0);
    SBEpilogue e = {y, static_cast<const f16 *>(l->bias), ep.row_scale, ep.accumulate};
    const dim3 grid((unsigned)pl.NSG, (unsigned)(pl.RB / pl.WR), (unsigned)pl.GP);
    if (l->nbits == 2)
        launch_main<2>(p, e, pl, grid, s);
    else
        launch_main<4>(p, e, pl, grid, s);
    int rc = launch_status();
    if (rc != HQQ_OK || pl.NSG == 1)
        return rc;
    smallbatch_finish_kernel<0><<<finish_grid(M, l->N), 64, 0, s>>>(
        p.layer[0].part, nullptr, pl.NSG, (int)M, (int)l->N, static_cast<const f16 *>(l->bias), ep.row_scale,
        ep.accumulate, y);
    return launch_status();
}

int launch_smallbatch_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                              size_t ws_bytes, hipStream_t s)
{
    if (strip_gate_supported(w1, w3, M))
        return launch_strip_gate_up(w1, w3, x, M, h, ws, ws_bytes, s);
    SBPlan pl, pl3;
    if (!make_plan(w1, M, pl) || !make_plan(w3, M, pl3) || w1->N != w3->N || w1->K != w3->K ||
        w1->nbits != w3->nbits || w1->group_size != w3->group_size)
        return HQQ_E_UNSUPPORTED;
    // the gate needs both projections of an output, which different blocks compute: always via partial sums
    const size_t one = (size_t)pl.NSG * (size_t)M * (size_t)w1->N * sizeof(float);
    const size_t head = workspace_head_bytes();
    if (ws_bytes < head + 2 * one)
        return HQQ_E_WORKSPACE;
    SBParams p = {};
    fill_params(p, pl, w1, 0, reinterpret_cast<float *>(static_cast<char *>(ws) + head));
    fill_params(p, pl, w3, 1, reinterpret_cast<float *>(static_cast<char *>(ws) + head + one));
    p.x = x, p.M = (int)M;
    p.NSG = pl.NSG;
    p.force_partial = 1;
    SBEpilogue e = {nullptr, nullptr, nullptr, 0};
    const dim3 grid((unsigned)pl.NSG, (unsigned)(2 * (pl.RB / pl.WR)), (unsigned)pl.GP);
    if (w1->nbits == 2)
        launch_main<2>(p, e, pl, grid, s);
    else
        launch_main<4>(p, e, pl, grid, s);
    int rc = launch_status();
    if (rc != HQQ_OK)
        return rc;
    smallbatch_finish_kernel<1><<<finish_grid(M, w1->N), 64, 0, s>>>(p.layer[0].part, p.layer[1].part, pl.NSG, (int)M,
                                                                      (int)w1->N, nullptr, nullptr, 0, h);
    return launch_status();
}

} // namespace hqq
