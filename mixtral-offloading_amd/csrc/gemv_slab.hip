// Decode-time GEMV (batch M <= 4) for 2- and 4-bit codes: one launch per matmul, or per fused w1/w3 gate.
//
// Same algebra as the per-step small-batch kernel (scale folded into the activations, codes fed to the matrix
// cores as fp16 subnormals, zero handled as a bias), reorganised so that a wavefront treats a whole slab of 256
// columns at once:
//   * every load of the slab is 128 bits wide and issued before any arithmetic: four code loads per lane, and for
//     the table lanes one load each of 16 scale bytes, 16 zero bytes, their fp16 meta values and x;
//   * the table phase runs once per slab (16 table entries per lane) and leaves xs for all four 64-column MFMA
//     steps in LDS, so there is one LDS hand-over per wave instead of one per step;
//   * the K slabs of a block are summed through LDS, and when a tile is split over several blocks (or is one of
//     the two projections of the gate) the block that arrives last at the tile's counter adds the partial sums in
//     a fixed order and applies the epilogue -- no second kernel.
//
// Lane roles.  Code lanes: (rr = lane & 15, kg = lane >> 4) own packed row jp + (16*rb + rr)*GP, bytes
// 64*s + 16*kg .. +15 of the slab for step s.  Table lanes: (ti = lane >> 4 < F, kq = lane & 15) own table row
// F*jp + ti, columns 16*kq .. 16*kq+15 of the slab, i.e. step kq >> 2, MFMA lane group kq & 3.
#include "hqq_common.hpp"

#include <cstdlib>

namespace hqq {
namespace {

constexpr int kSlab = 256;           // columns per wave
constexpr float kXsScale = 32.0f;    // xs = 32 * s * x keeps small activations out of the fp16 subnormal range
constexpr size_t kCounterBytes = 64 * 1024; // head of the workspace: one arrival counter per tile

struct SlabLayer {
    const uint8_t *codes;
    const uint8_t *sq, *zq; // 8-bit tables, or fp16 tables when !u8
    const f16 *s_ms, *s_mz; // meta of the scale table
    const f16 *z_ms, *z_mz; // meta of the zero table
    uint32_t s_cols, z_cols, s_inv, z_inv;
    float *part; // [NSG][M][N]
};

struct SlabParams {
    SlabLayer layer[2];
    const f16 *x;
    int M, N, K;
    int GP, RBG, WR, WR_log2, WS;
    int NS;      // K / 256
    int NSG;     // slab groups = blocks per (layer, tile)
    int NL;      // layers in this launch (2 = fused gate)
    int *counter; // one per tile, zero between launches
    // epilogue
    f16 *y;
    const f16 *bias, *row_scale;
    int accumulate;
    int probe;
};

enum { TK_U8_COLS = 1, TK_U8_SCALAR = 2, TK_F16 = 3 };

__device__ __forceinline__ f16x2 as_h2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }
__device__ __forceinline__ uint32_t as_u32(f16x2 v) { return __builtin_bit_cast(uint32_t, v); }

__device__ __forceinline__ float row16_sum(float v)
{
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

// 16 table entries of a lane, raw
template <int KIND> struct Raw16 {
    u32x4 q;       // 16 bytes (u8 kinds) / first 8 halves (fp16)
    u32x4 q_hi;    // fp16 only: last 8 halves
    u32x4 ms[2], mz[2]; // per-column meta, 16 halves each
};

template <int KIND>
__device__ __forceinline__ void load16(Raw16<KIND> &r, const uint8_t *tab, const f16 *ms, const f16 *mz, uint32_t c,
                                       uint32_t cm)
{
    if constexpr (KIND == TK_F16) {
        const u32x4 *p = reinterpret_cast<const u32x4 *>(reinterpret_cast<const f16 *>(tab) + c);
        r.q = p[0];
        r.q_hi = p[1];
    } else {
        r.q = *reinterpret_cast<const u32x4 *>(tab + c);
        if constexpr (KIND == TK_U8_COLS) {
            const u32x4 *a = reinterpret_cast<const u32x4 *>(ms + cm);
            const u32x4 *b = reinterpret_cast<const u32x4 *>(mz + cm);
            r.ms[0] = a[0], r.ms[1] = a[1];
            r.mz[0] = b[0], r.mz[1] = b[1];
        }
    }
}

// decode to 8 fp16 pairs: pair t holds columns (2t, 2t+1) of the lane's 16
template <int KIND>
__device__ __forceinline__ void decode16(const Raw16<KIND> &r, f16x2 ms_s, f16x2 mz_s, f16x2 (&out)[8])
{
    if constexpr (KIND == TK_F16) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            out[t] = as_h2(r.q[t]);
            out[4 + t] = as_h2(r.q_hi[t]);
        }
    } else {
        const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            // bytes -> fp16 exactly: 0x6400 | b is 1024 + b
            const f16x2 lo = as_h2(__builtin_amdgcn_perm(0x64646464u, r.q[w], 0x04010400u)) - k1024;
            const f16x2 hi = as_h2(__builtin_amdgcn_perm(0x64646464u, r.q[w], 0x04030402u)) - k1024;
            if constexpr (KIND == TK_U8_COLS) {
                out[2 * w] = (lo - as_h2(r.mz[w >> 1][2 * (w & 1)])) * as_h2(r.ms[w >> 1][2 * (w & 1)]);
                out[2 * w + 1] = (hi - as_h2(r.mz[w >> 1][2 * (w & 1) + 1])) * as_h2(r.ms[w >> 1][2 * (w & 1) + 1]);
            } else {
                out[2 * w] = (lo - mz_s) * ms_s;
                out[2 * w + 1] = (hi - mz_s) * ms_s;
            }
        }
    }
}

template <int NBITS> struct Field {
    static constexpr int F = 8 / NBITS;
    static constexpr int pos(int i) { return NBITS * (F - 1 - i); }
    // field i of the byte in the low half of each 16-bit word; masked in place it is the fp16 subnormal
    // q * 2^(pos - 24), which the matrix cores multiply exactly
    static constexpr uint32_t mask(int i) { return (((1u << NBITS) - 1u) * 0x00010001u) << pos(i); }
    static constexpr float unscale(int i) { return (float)(1u << (24 - pos(i))) / kXsScale; }
};

template <int NBITS, int MT, int WAVES, int SKIND, int ZKIND, int EPI>
__global__ __launch_bounds__(WAVES * 64) void gemv_slab_kernel(SlabParams p)
{
    constexpr int F = 8 / NBITS;
    constexpr int ENTRY = 8;                        // halves per B-operand entry (16 bytes)
    constexpr int STEP_HALVES = F * 2 * 4 * MT * ENTRY;
    constexpr int XS_HALVES = 4 * STEP_HALVES;      // four steps
    __shared__ __attribute__((aligned(16))) f16 xs_lds[WAVES][XS_HALVES];
    __shared__ float bias_lds[WAVES][F][MT];
    __shared__ __attribute__((aligned(16))) float red_lds[WAVES][16][MT][F];
    __shared__ int ticket_lds;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wr = wave & (p.WR - 1), ws = wave >> p.WR_log2;
    const int sg = blockIdx.x;
    const int layer = (int)blockIdx.y >= p.RBG ? 1 : 0;
    const int rbg = (int)blockIdx.y - layer * p.RBG;
    const int jp = blockIdx.z;
    // both layer records are read from the kernel arguments in one go and selected in registers: no dependent loads
    SlabLayer L;
    {
        const SlabLayer &A = p.layer[0], &B = p.layer[1];
        L.codes = layer ? B.codes : A.codes;
        L.sq = layer ? B.sq : A.sq;
        L.zq = layer ? B.zq : A.zq;
        L.s_ms = layer ? B.s_ms : A.s_ms;
        L.s_mz = layer ? B.s_mz : A.s_mz;
        L.z_ms = layer ? B.z_ms : A.z_ms;
        L.z_mz = layer ? B.z_mz : A.z_mz;
        L.s_cols = layer ? B.s_cols : A.s_cols;
        L.z_cols = layer ? B.z_cols : A.z_cols;
        L.s_inv = layer ? B.s_inv : A.s_inv;
        L.z_inv = layer ? B.z_inv : A.z_inv;
        L.part = layer ? B.part : A.part;
    }
    const int rb = rbg * p.WR + wr;
    const int slab = sg * p.WS + ws;
    const bool active = slab < p.NS;
    const int K = p.K;
    const int M = MT == 1 ? 1 : p.M;

    const int rr = lane & 15, kg = lane >> 4;
    const int ti = lane >> 4, kq = lane & 15;
    const bool tlane = ti < F;  // lanes that own table entries (all of them for 2-bit codes)
    const int ti_l = ti & (F - 1); // the other lanes repeat a table lane's loads, so that issuing loads never diverges

    // ---------------------------------------------------------------- loads, all up front, tables first
    Raw16<SKIND> sraw;
    Raw16<ZKIND> zraw;
    u32x4 xv[MT][2];
    u32x4 cw[4];
    f16 zms_r = 0, zmz_r = 0, sms_r = 0, smz_r = 0; // whole-tensor meta, splat only when the table phase needs it
    if (active) {
        {
            const uint32_t c = (uint32_t)(F * jp + ti_l) * (uint32_t)K + (uint32_t)(slab * kSlab + 16 * kq);
            uint32_t scm = 0, zcm = 0;
            if constexpr (SKIND == TK_U8_COLS) {
                scm = c - __umulhi(c, L.s_inv) * L.s_cols; // c mod cols; the quotient estimate is at most 2 short
                scm -= scm >= L.s_cols ? L.s_cols : 0;
                scm -= scm >= L.s_cols ? L.s_cols : 0;
            }
            if constexpr (ZKIND == TK_U8_COLS) {
                zcm = c - __umulhi(c, L.z_inv) * L.z_cols;
                zcm -= zcm >= L.z_cols ? L.z_cols : 0;
                zcm -= zcm >= L.z_cols ? L.z_cols : 0;
            }
            load16<SKIND>(sraw, L.sq, L.s_ms, L.s_mz, c, scm);
            load16<ZKIND>(zraw, L.zq, L.z_ms, L.z_mz, c, zcm);
            if constexpr (SKIND == TK_U8_SCALAR) {
                sms_r = L.s_ms[0];
                smz_r = L.s_mz[0];
            }
            if constexpr (ZKIND == TK_U8_SCALAR) {
                zms_r = L.z_ms[0];
                zmz_r = L.z_mz[0];
            }
            const uint32_t xo = (uint32_t)(slab * kSlab + 16 * kq);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    const u32x4 *xp = reinterpret_cast<const u32x4 *>(p.x + (xo + (uint32_t)(m * K)));
                    xv[m][0] = xp[0];
                    xv[m][1] = xp[1];
                }
            }
        }
        const uint32_t prow = (uint32_t)jp + (uint32_t)(16 * rb + rr) * (uint32_t)p.GP;
        const uint32_t coff = prow * (uint32_t)K + (uint32_t)(slab * kSlab + 16 * kg);
#pragma unroll
        for (int s = 0; s < 4; ++s)
            cw[s] = *reinterpret_cast<const u32x4 *>(L.codes + (coff + 64 * s));
    }

    // B operand of lane (mcol, kg) for (step s, field i, half h): entry ((s*F + i)*2 + h)*4 + kg, batch column mcol.
    // Column m of the MFMA result depends on column m of B only, and columns m >= M are never read back, so lanes
    // past the batch simply re-read a valid column instead of needing zeros.
    const int mcol = lane & 15;
    const f16 *xs_r = &xs_lds[wave][(kg * MT + (mcol < M ? mcol : 0)) * ENTRY];

    f32x4 acc[F];
#pragma unroll
    for (int i = 0; i < F; ++i)
        acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float bias_acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        bias_acc[m] = 0.f;

    if (p.probe >= 1 && active) { // tuning aid: wait for every load, no arithmetic
        uint32_t t = 0;
#pragma unroll
        for (int s = 0; s < 4; ++s)
            t ^= cw[s].x ^ cw[s].y ^ cw[s].z ^ cw[s].w;
        if (tlane)
            t ^= sraw.q.x ^ zraw.q.w ^ sraw.ms[0].x ^ sraw.mz[1].y ^ xv[0][0].x ^ xv[0][1].w;
        acc[0][0] = (float)(t & 1u);
    } else if (active) {
        // ------------------------------------------------------------ table phase, once per slab
        if (tlane) {
            f16x2 sv[8], zv[8];
            const f16x2 sms = {sms_r, sms_r}, smz = {smz_r, smz_r}, zms = {zms_r, zms_r}, zmz = {zmz_r, zmz_r};
            decode16<SKIND>(sraw, sms, smz, sv);
            decode16<ZKIND>(zraw, zms, zmz, zv);
            const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
#pragma unroll
            for (int t = 0; t < 8; ++t)
                sv[t] = sv[t] * k32;
            // lane's 16 columns are step kq>>2, lane group kq&3, halves h = 0 (cols 0-7) and 1 (cols 8-15)
            f16 *dst = &xs_lds[wave][(kq >> 2) * STEP_HALVES + ((ti * 2) * 4 + (kq & 3)) * MT * ENTRY];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    f16x2 a[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        a[t] = sv[t] * as_h2(xv[m][t >> 2][t & 3]);
                        bias_acc[m] = __builtin_amdgcn_fdot2(zv[t], a[t], bias_acc[m], false);
                    }
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        // B-operand order inside an 8-column block: columns (0,2,1,3,4,6,5,7)
                        const f16x2 *q = &a[4 * h];
                        const f16x8 o = {q[0].x, q[1].x, q[0].y, q[1].y, q[2].x, q[3].x, q[2].y, q[3].y};
                        *reinterpret_cast<f16x8 *>(dst + (h * 4 * MT + m) * ENTRY) = o;
                    }
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ------------------------------------------------------------ code phase: 4 steps x 2F MFMAs
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            f16x8 B[2][F];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < F; ++i)
                    B[h][i] = *reinterpret_cast<const f16x8 *>(xs_r + s * STEP_HALVES + ((i * 2 + h) * 4 * MT) * ENTRY);
            const uint32_t d[4] = {cw[s].x, cw[s].y, cw[s].z, cw[s].w};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
                const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const uint32_t mk = Field<NBITS>::mask(i);
                    const u32x4 Au = {d0 & mk, d0s & mk, d1 & mk, d1s & mk};
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, Au), B[h][i], acc[i], 0, 0, 0);
                }
            }
        }
    }

    // ---------------------------------------------------------------- wave tile -> LDS (bias removed, unscaled)
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float v = row16_sum(bias_acc[m]);
        if (tlane && kq == 0)
            bias_lds[wave][ti][m] = v * (1.0f / kXsScale);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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

    // ---------------------------------------------------------------- block tile: 16 lanes per output row bring the slabs
    const bool alone = p.NSG == 1 && p.NL == 1; // no other block contributes to this tile
    const int tile = jp * p.RBG + rbg;
    const int tile_rows = p.WR * 16 * MT;
    for (int t = threadIdx.x; t < tile_rows * 16; t += WAVES * 64) {
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
            o[i] = row16_sum(o[i]);
        if (w != 0 || m_t >= M)
            continue;
        const int r = 16 * (rbg * p.WR + wr_t) + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * p.GP); // outputs n .. n+F-1
        if (!alone) {
            // device-scope stores: written through the (per-XCD, mutually non-coherent) L2 so that the finishing
            // block, which may run on another XCD, can read them without any cache-wide flush
            float *dst = L.part + ((int64_t)sg * M + m_t) * p.N + n;
#pragma unroll
            for (int i = 0; i < F; ++i)
                __hip_atomic_store(dst + i, o[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        f16 *dst = p.y + (int64_t)m_t * p.N + n;
        f16 hv[F];
#pragma unroll
        for (int i = 0; i < F; ++i) {
            f16 val = (f16)o[i];
            if (p.bias)
                val = val + p.bias[n + i];
            if (p.row_scale)
                val = val * p.row_scale[m_t];
            if (p.accumulate)
                val = dst[i] + val;
            hv[i] = val;
        }
        if constexpr (F == 4)
            *reinterpret_cast<f16x4 *>(dst) = (f16x4){hv[0], hv[1], hv[2], hv[3]};
        else
            *reinterpret_cast<f16x2 *>(dst) = (f16x2){hv[0], hv[1]};
    }
    if (alone)
        return;

    // ---------------------------------------------------------------- the block that arrives last finishes the tile
    // The partial sums were stored at device scope; once those stores are acknowledged the arrival is counted
    // with a device-scope atomic.  No cache-wide write-back or invalidate is involved (a __threadfence here
    // flushes the whole L2 of the XCD and costs more than the matmul).
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0) expcnt(0) lgkmcnt(0): every store of this thread is acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const int total = p.NSG * p.NL;
        const int prev = __hip_atomic_fetch_add(&p.counter[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == total - 1) // every contributor has arrived: leave the counter ready for the next launch
            __hip_atomic_store(&p.counter[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket_lds = prev;
    }
    __syncthreads();
    if (ticket_lds != p.NSG * p.NL - 1)
        return;
    for (int u = threadIdx.x; u < tile_rows; u += WAVES * 64) {
        const int wr_t = u / (16 * MT), r_t = (u / MT) & 15, m_t = u % MT;
        if (m_t >= M)
            continue;
        const int r = 16 * (rbg * p.WR + wr_t) + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * p.GP);
        float a[F], b[F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            a[i] = b[i] = 0.f;
        for (int s = 0; s < p.NSG; ++s) { // fixed order: results do not depend on which block came last
            const int64_t off = ((int64_t)s * M + m_t) * p.N + n;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                a[i] += __hip_atomic_load(p.layer[0].part + off + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if constexpr (EPI == 1)
                    b[i] += __hip_atomic_load(p.layer[1].part + off + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        f16 *dst = p.y + (int64_t)m_t * p.N + n;
        f16 hv[F];
#pragma unroll
        for (int i = 0; i < F; ++i) {
            if constexpr (EPI == 1) {
                // both projections rounded to fp16, SiLU in fp32 rounded once, product in fp16: as the reference's ops do
                const float g = (float)(f16)a[i];
                const f16 act = (f16)(g / (1.0f + __expf(-g)));
                hv[i] = act * (f16)b[i];
            } else {
                f16 val = (f16)a[i];
                if (p.bias)
                    val = val + p.bias[n + i];
                if (p.row_scale)
                    val = val * p.row_scale[m_t];
                if (p.accumulate)
                    val = dst[i] + val;
                hv[i] = val;
            }
        }
        if constexpr (F == 4)
            *reinterpret_cast<f16x4 *>(dst) = (f16x4){hv[0], hv[1], hv[2], hv[3]};
        else
            *reinterpret_cast<f16x2 *>(dst) = (f16x2){hv[0], hv[1]};
    }
}

__global__ void zero_words_kernel(uint32_t *p, size_t n)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        p[i] = 0;
}

int env_int(const char *name, int dflt)
{
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : dflt;
}

int table_kind(const hqq_table &t) { return t.kind == HQQ_TABLE_F16 ? TK_F16 : (t.meta_cols == 1 ? TK_U8_SCALAR : TK_U8_COLS); }

int block_waves_for(int MT, int waves);

struct SlabPlan {
    int F, GP, RB, RBG, WR, WS, NS, NSG, MT, WAVES, SKIND, ZKIND;
};

bool make_plan(const hqq_linear *l, int64_t M, SlabPlan &pl)
{
    if (env_int("HQQ_NO_SLAB", 0))
        return false;
    if ((l->nbits != 2 && l->nbits != 4) || M < 1 || M > 4)
        return false;
    const int F = 8 / l->nbits;
    const int64_t G = l->N / l->group_size;
    if (l->group_size % 16 != 0 || G % F != 0 || l->K % kSlab != 0 || l->N % 4 != 0)
        return false;
    if (l->N * l->K / l->group_size >= (1ll << 31) || l->N * l->K / F >= (1ll << 32) || 16 * l->K >= (1ll << 31))
        return false; // 32-bit offsets inside the kernel
    if (!aligned16(l->codes) || !aligned16(l->scale.data) || !aligned16(l->zero.data))
        return false;
    pl.SKIND = table_kind(l->scale);
    pl.ZKIND = table_kind(l->zero);
    // instantiated table combinations: HQQ default (scale u8 per-column meta, zero u8 scalar meta) and fp16 tables
    if (!((pl.SKIND == TK_U8_COLS && pl.ZKIND == TK_U8_SCALAR) || (pl.SKIND == TK_F16 && pl.ZKIND == TK_F16)))
        return false;
    if (pl.SKIND == TK_U8_COLS && (l->scale.meta_cols % 16 != 0 || !aligned16(l->scale.meta_scale) ||
                                   !aligned16(l->scale.meta_zero)))
        return false;
    pl.F = F;
    pl.GP = (int)(G / F);
    pl.RB = l->group_size / 16;
    pl.MT = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
    pl.WAVES = pl.MT == 1 ? 16 : (pl.MT == 2 ? 8 : 4);
    const int forced = env_int("HQQ_SLAB_WAVES", 0);
    if ((forced == 4 || forced == 8 || forced == 16) && forced <= pl.WAVES)
        pl.WAVES = forced;
    // Waves of a block go along K first: a block that holds every slab of its tile finishes it alone, with no
    // partial sums and no arrival counter.  Only what is left over goes to further row blocks of the same jp.
    pl.NS = (int)(l->K / kSlab);
    pl.WS = pl.WAVES;
    while (pl.WS / 2 >= pl.NS)
        pl.WS /= 2;
    pl.WR = pl.WAVES / pl.WS;
    while (pl.WR > 1 && (pl.WR > pl.RB || pl.RB % pl.WR != 0))
        pl.WR /= 2;
    // narrow blocks are launched at the next instantiated width; the extra waves get slab indices past K and idle
    if (pl.WR * pl.WS < 4)
        pl.WS = 4 / pl.WR;
    pl.WAVES = block_waves_for(pl.MT, pl.WR * pl.WS);
    pl.WS = pl.WAVES / pl.WR;
    pl.RBG = pl.RB / pl.WR;
    pl.NSG = (pl.NS + pl.WS - 1) / pl.WS;
    if ((int64_t)pl.GP * pl.RBG * sizeof(int) > kCounterBytes || pl.GP > 65535 || 2 * pl.RBG > 65535)
        return false;
    return true;
}

void fill_layer(SlabLayer &L, const hqq_linear *l, float *part)
{
    L.codes = static_cast<const uint8_t *>(l->codes);
    L.sq = static_cast<const uint8_t *>(l->scale.data);
    L.zq = static_cast<const uint8_t *>(l->zero.data);
    L.s_ms = static_cast<const f16 *>(l->scale.meta_scale);
    L.s_mz = static_cast<const f16 *>(l->scale.meta_zero);
    L.z_ms = static_cast<const f16 *>(l->zero.meta_scale);
    L.z_mz = static_cast<const f16 *>(l->zero.meta_zero);
    L.s_cols = (uint32_t)l->scale.meta_cols;
    L.z_cols = (uint32_t)l->zero.meta_cols;
    L.s_inv = L.s_cols ? (uint32_t)(0xFFFFFFFFull / L.s_cols) : 0;
    L.z_inv = L.z_cols ? (uint32_t)(0xFFFFFFFFull / L.z_cols) : 0;
    L.part = part;
}

template <int NBITS, int MT, int WAVES, int EPI>
void launch_kinds(const SlabParams &p, const SlabPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.SKIND == TK_F16)
        gemv_slab_kernel<NBITS, MT, WAVES, TK_F16, TK_F16, EPI><<<grid, dim3(WAVES * 64), 0, s>>>(p);
    else
        gemv_slab_kernel<NBITS, MT, WAVES, TK_U8_COLS, TK_U8_SCALAR, EPI><<<grid, dim3(WAVES * 64), 0, s>>>(p);
}

// instantiated block widths: MT 1 -> 16, 8, 4 waves; MT 2 -> 8, 4; MT 4 -> 4 (LDS staging grows with MT)
int block_waves_for(int MT, int waves)
{
    if (MT == 1)
        return waves > 8 ? 16 : (waves > 4 ? 8 : 4);
    if (MT == 2)
        return waves > 4 ? 8 : 4;
    return 4;
}

template <int NBITS, int EPI> void launch_shape(const SlabParams &p, const SlabPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.MT == 1) {
        if (pl.WAVES == 16)
            launch_kinds<NBITS, 1, 16, EPI>(p, pl, grid, s);
        else if (pl.WAVES == 8)
            launch_kinds<NBITS, 1, 8, EPI>(p, pl, grid, s);
        else
            launch_kinds<NBITS, 1, 4, EPI>(p, pl, grid, s);
    } else if (pl.MT == 2) {
        if (pl.WAVES == 8)
            launch_kinds<NBITS, 2, 8, EPI>(p, pl, grid, s);
        else
            launch_kinds<NBITS, 2, 4, EPI>(p, pl, grid, s);
    } else {
        launch_kinds<NBITS, 4, 4, EPI>(p, pl, grid, s);
    }
}

int run(const hqq_linear *l0, const hqq_linear *l1, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
        const SmallBatchEpilogue &ep, hipStream_t s)
{
    SlabPlan pl;
    if (!make_plan(l0, M, pl))
        return HQQ_E_UNSUPPORTED;
    const int NL = l1 ? 2 : 1;
    const size_t one = (size_t)pl.NSG * (size_t)M * (size_t)l0->N * sizeof(float);
    const bool alone = pl.NSG == 1 && NL == 1;
    if (!alone && (!ws || ws_bytes < kCounterBytes + NL * one))
        return HQQ_E_WORKSPACE;
    SlabParams p = {};
    char *base = static_cast<char *>(ws);
    fill_layer(p.layer[0], l0, alone ? nullptr : reinterpret_cast<float *>(base + kCounterBytes));
    if (l1)
        fill_layer(p.layer[1], l1, reinterpret_cast<float *>(base + kCounterBytes + one));
    else
        p.layer[1] = p.layer[0];
    p.x = x, p.M = (int)M, p.N = (int)l0->N, p.K = (int)l0->K;
    p.GP = pl.GP, p.RBG = pl.RBG, p.WR = pl.WR, p.WR_log2 = pl.WR == 4 ? 2 : (pl.WR == 2 ? 1 : 0), p.WS = pl.WS;
    p.NS = pl.NS, p.NSG = pl.NSG, p.NL = NL;
    p.counter = reinterpret_cast<int *>(base);
    p.y = y, p.bias = static_cast<const f16 *>(l0->bias), p.row_scale = ep.row_scale, p.accumulate = ep.accumulate;
    p.probe = env_int("HQQ_SB_PROBE", 0);
    const dim3 grid((unsigned)pl.NSG, (unsigned)(NL * pl.RBG), (unsigned)pl.GP);
    if (l1) {
        if (l0->nbits == 2)
            launch_shape<2, 1>(p, pl, grid, s);
        else
            launch_shape<4, 1>(p, pl, grid, s);
    } else {
        if (l0->nbits == 2)
            launch_shape<2, 0>(p, pl, grid, s);
        else
            launch_shape<4, 0>(p, pl, grid, s);
    }
    return launch_status();
}

} // namespace

bool slab_supported(const hqq_linear *l, int64_t M)
{
    SlabPlan pl;
    return make_plan(l, M, pl);
}

size_t slab_workspace_bytes(const hqq_linear *l, int64_t M)
{
    SlabPlan pl;
    if (!make_plan(l, M, pl))
        return 0;
    return kCounterBytes + (size_t)pl.NSG * (size_t)M * (size_t)l->N * sizeof(float);
}

int launch_slab_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                       const SmallBatchEpilogue &ep, hipStream_t s)
{
    return run(l, nullptr, x, M, y, ws, ws_bytes, ep, s);
}

int launch_slab_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                        size_t ws_bytes, hipStream_t s)
{
    SlabPlan a, b;
    if (!make_plan(w1, M, a) || !make_plan(w3, M, b) || w1->N != w3->N || w1->K != w3->K || w1->nbits != w3->nbits ||
        w1->group_size != w3->group_size || a.SKIND != b.SKIND || a.ZKIND != b.ZKIND)
        return HQQ_E_UNSUPPORTED;
    return run(w1, w3, x, M, h, ws, ws_bytes, SmallBatchEpilogue{}, s);
}

int launch_zero_workspace_head(void *ws, size_t ws_bytes, hipStream_t s)
{
    const size_t n = (ws_bytes < kCounterBytes ? ws_bytes : kCounterBytes) / 4;
    if (n == 0)
        return HQQ_OK;
    zero_words_kernel<<<16, 256, 0, s>>>(static_cast<uint32_t *>(ws), n);
    return launch_status();
}

size_t workspace_head_bytes() { return kCounterBytes; }

} // namespace hqq
