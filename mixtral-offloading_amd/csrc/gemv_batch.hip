// Decode batches of 3 to 16 rows for 2- and 4-bit codes: the single-row kernel's structure (a block per tile, waves
// split K, every load 128 bits wide and issued before any arithmetic, the block's own epilogue) with the batch rows
// in the MFMA's B columns.
//
// Algebra as in gemv_strip.hip: y[n, m] = sum_k q[n, k] * xs[i, k, m] - sum_k zs[i, k] * x[m, k], with
// xs = 32 * s[i, k] * x[m, k] and zs = 32 * s[i, k] * z[i, k] in fp16 and the codes masked in place (fp16 subnormals).
//
// Layout of v_mfma_f32_16x16x32_f16.  PH column phases (4 for up to 4 batch rows, else 2):
//   A rows    a = (rho, phi):  16 / PH tile rows, each at PH column phases.  A code load covers those rows over
//             64 * PH columns; lane (a, g) reads 16 bytes at chunk g * PH + phi, so PH neighbouring lanes read
//             16 * PH consecutive bytes of one row and the lane's bytes are its A operands as they arrive.
//   B columns c = (m, phi):    16 / PH batch rows at PH phases; lane (c, g) holds xs of batch row m for the 16
//             columns of chunk g * PH + phi.  Output (row (rho, phi), column (m, phi')) is kept where phi == phi';
//             the phases of a row are added once per wave, at the end.
// The tables are loaded and decoded as in the single-row kernel (lane = table row x 16 columns, four lanes to 64
// consecutive bytes) and reach the B lanes through LDS in B-operand order; x is read straight into the B lanes.
// The zero term is one more MFMA per column half: A = zs (rows (field, phase)), B = x.
// Sixteen batch rows are two sets of eight that share every A operand.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"

namespace hqq {
using namespace gemv;
namespace {

struct BatchParams {
    LayerRecord layer[2];
    const f16 *x;
    f16 *y;
    const f16 *bias;
    const f16 *row_scale;
    int accumulate;
    int M, K, N, GP, RB, NS;
    int KS;  // waves per layer
    int SPW; // slabs per wave
    int BK;  // blocks along K
    int NL;  // layers per block (2: gate)
    unsigned long long *slots;
    // indexed launch (table != null): the layer records are read from a device table instead, record
    // table[sel[0] * table_stride + table_first + layer], so that which expert runs is decided on the device
    const LayerRecord *table;
    const int *sel;
    int table_stride, table_first;
};

__device__ __forceinline__ float quad_xor1(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float quad_xor2(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
}
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// eight halves in column order -> B-operand order (0,2,1,3,4,6,5,7), the order in which the masked code bytes sit in
// the A operand
__device__ __forceinline__ u32x4 to_b_order(u32x4 v)
{
    u32x4 o;
    o.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u); // (k0, k2)
    o.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u); // (k1, k3)
    o.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u); // (k4, k6)
    o.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u); // (k5, k7)
    return o;
}

// EPI: 0 y = o (+ bias) (* row_scale) (+ y);  1 y = silu(o0) * o1 (two layers)
// WAVES: 16 for up to eight batch rows (the kernel then stays within the 128 registers that four waves to a SIMD
// leave each), so that a block's whole share of K is requested at once; 8 for sixteen rows
template <int NBITS, int PH, int MS, int SKIND, int ZKIND, int EPI, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv_batch_kernel(BatchParams p)
{
    constexpr int kBatchWaves = WAVES;
    constexpr int F = 8 / NBITS;
    constexpr int LP = PH == 4 ? 2 : 1;
    constexpr int MB = 16 / PH;  // batch rows per set
    constexpr int MT = MB * MS;  // batch rows of the kernel
    constexpr int KP = 4 / PH;   // column parts of a slab (a code load covers 64 * PH columns)
    constexpr int RG = PH;       // row groups of a tile (a code load covers 16 / PH rows)
    constexpr int CH = 4 * PH;   // 16-column chunks per column part
    // per wave: the folded tables of a slab in B-operand order, [field][half][chunk][8]
    __shared__ __attribute__((aligned(16))) f16 s_lds[kBatchWaves][F][2][16][8];
    __shared__ __attribute__((aligned(16))) f16 zs_lds[kBatchWaves][F][2][16][8];
    __shared__ float bias_lds[kBatchWaves][F][MT];
    __shared__ __attribute__((aligned(16))) float red_lds[kBatchWaves][16][MT][F];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kb = blockIdx.x, rb = blockIdx.y, jp = blockIdx.z;
    const int layer = wave >= p.KS ? 1 : 0;
    const int ks = wave - layer * p.KS;
    const bool wave_on = wave < p.KS * p.NL;
    const LayerRecord &A0 = p.layer[0], &A1 = p.layer[1];
    LayerRecord L;
    if (p.table) {
        // one word of the record per lane, then broadcast
        const int e = __builtin_amdgcn_readfirstlane(p.sel[0]);
        const uint32_t *src = reinterpret_cast<const uint32_t *>(p.table + (e * p.table_stride + p.table_first + layer));
        const uint32_t word = src[lane < 18 ? lane : 0];
        uint32_t rec[18];
#pragma unroll
        for (int i = 0; i < 18; ++i)
            rec[i] = __builtin_amdgcn_readlane(word, i);
        __builtin_memcpy(&L, rec, sizeof(L));
    } else {
        L.codes = layer ? A1.codes : A0.codes;
        L.sq = layer ? A1.sq : A0.sq;
        L.zq = layer ? A1.zq : A0.zq;
        L.s_ms = layer ? A1.s_ms : A0.s_ms;
        L.s_mz = layer ? A1.s_mz : A0.s_mz;
        L.z_ms = layer ? A1.z_ms : A0.z_ms;
        L.z_mz = layer ? A1.z_mz : A0.z_mz;
        L.s_cols = layer ? A1.s_cols : A0.s_cols;
        L.z_cols = layer ? A1.z_cols : A0.z_cols;
        L.s_inv = layer ? A1.s_inv : A0.s_inv;
        L.z_inv = layer ? A1.z_inv : A0.z_inv;
    }
    const int K = p.K, M = p.M, GP = p.GP, N = p.N;

    // table role: table row ti of the tile, chunk qT (16 columns) of the slab
    const int g = lane >> 4;
    const int ti = (lane >> 2) & 3, qT = 4 * g + (lane & 3);
    const bool tlane = ti < F;
    const int ti_l = ti & (F - 1);
    const uint32_t trow = (uint32_t)(F * jp + ti_l) * (uint32_t)K + (uint32_t)(16 * qT);
    // code and B roles: phase, and tile row / batch row within the group
    const int phi = lane & (PH - 1), hi = (lane & 15) >> LP;
    const int qc = g * PH + phi; // chunk within a column part
    // code load (rg, kp): tile row rg * (16 / PH) + hi, columns kp * 64 * PH + 16 * qc
    const uint32_t crow = ((uint32_t)jp + (uint32_t)(16 * rb + hi) * (uint32_t)GP) * (uint32_t)K + (uint32_t)(16 * qc);
    const uint32_t crow_step = (uint32_t)MB * (uint32_t)GP * (uint32_t)K;
    // x of the lane's batch rows (rows past the batch re-read row 0: their columns are never written)
    uint32_t xrow[MS];
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
        const int m = ms * MB + hi;
        xrow[ms] = (uint32_t)(m < M ? m : 0) * (uint32_t)K + (uint32_t)(16 * qc);
    }

    f32x4 acc[MS][RG][F];
    f32x4 accb[MS][KP];
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
            for (int i = 0; i < F; ++i)
                acc[ms][r][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kp = 0; kp < KP; ++kp)
            accb[ms][kp] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    const int slab_begin = (kb * p.KS + ks) * p.SPW;
    if (wave_on) {
        for (int si = 0; si < p.SPW; ++si) {
            const int slab = slab_begin + si;
            if (slab >= p.NS)
                break;
            // ------------------------------------------------------------ every load of the slab
            const uint32_t k0 = (uint32_t)slab * kSlab;
            const uint32_t c = trow + k0;
            uint32_t scm = 0, zcm = 0;
            if constexpr (SKIND == TK_U8_COLS) {
                scm = c - __umulhi(c, L.s_inv) * L.s_cols;
                scm -= scm >= L.s_cols ? L.s_cols : 0;
                scm -= scm >= L.s_cols ? L.s_cols : 0;
            }
            if constexpr (ZKIND == TK_U8_COLS) {
                zcm = c - __umulhi(c, L.z_inv) * L.z_cols;
                zcm -= zcm >= L.z_cols ? L.z_cols : 0;
                zcm -= zcm >= L.z_cols ? L.z_cols : 0;
            }
            Raw16<SKIND> rs;
            Raw16<ZKIND> rz;
            load16<SKIND>(rs, L.sq, L.s_ms, L.s_mz, c, scm);
            load16<ZKIND>(rz, L.zq, L.z_ms, L.z_mz, c, zcm);
            u32x4 xw[MS][KP][2];
#pragma unroll
            for (int ms = 0; ms < MS; ++ms)
#pragma unroll
                for (int kp = 0; kp < KP; ++kp) {
                    const u32x4 *xp = reinterpret_cast<const u32x4 *>(p.x + (xrow[ms] + k0 + (uint32_t)(kp * 64 * PH)));
                    xw[ms][kp][0] = gload<u32x4>(xp);
                    xw[ms][kp][1] = gload<u32x4>(xp + 1);
                }
            u32x4 cw[RG][KP];
#pragma unroll
            for (int r = 0; r < RG; ++r)
#pragma unroll
                for (int kp = 0; kp < KP; ++kp)
                    cw[r][kp] = gload<u32x4>(L.codes + (crow + k0 + (uint32_t)r * crow_step + (uint32_t)(kp * 64 * PH)));
            const int zero_off = lane >> 6; // (not known to be zero: keeps these loads in vector registers, see gemv_strip.hip)
            uint32_t sms_r = 0, smz_r = 0, zms_r = 0, zmz_r = 0;
            if constexpr (SKIND == TK_U8_SCALAR) {
                sms_r = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.s_ms) + zero_off);
                smz_r = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.s_mz) + zero_off);
            }
            if constexpr (ZKIND == TK_U8_SCALAR) {
                zms_r = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.z_ms) + zero_off);
                zmz_r = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.z_mz) + zero_off);
            }

            // ------------------------------------------------------------ table phase: 32 * s and 32 * s * z to LDS
            if (tlane) {
                f16x2 sv[8], zv[8];
                decode16<SKIND>(rs, as_h2(sms_r * 0x10001u), as_h2(smz_r * 0x10001u), sv);
                decode16<ZKIND>(rz, as_h2(zms_r * 0x10001u), as_h2(zmz_r * 0x10001u), zv);
                const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
                u32x4 so[2], zo[2];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    sv[t] = sv[t] * k32;
                    zv[t] = zv[t] * sv[t];
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    so[h] = to_b_order((u32x4){as_u32(sv[4 * h]), as_u32(sv[4 * h + 1]), as_u32(sv[4 * h + 2]), as_u32(sv[4 * h + 3])});
                    zo[h] = to_b_order((u32x4){as_u32(zv[4 * h]), as_u32(zv[4 * h + 1]), as_u32(zv[4 * h + 2]), as_u32(zv[4 * h + 3])});
                    *reinterpret_cast<u32x4 *>(&s_lds[wave][ti][h][qT][0]) = so[h];
                    *reinterpret_cast<u32x4 *>(&zs_lds[wave][ti][h][qT][0]) = zo[h];
                }
            }
            wave_sync();

            // ------------------------------------------------------------ per column part: B operands, then the MFMAs
#pragma unroll
            for (int kp = 0; kp < KP; ++kp) {
                const int qB = kp * CH + qc; // the lane's chunk of the slab in this part
                // zero term: A rows (field, [part,] phase)
                int fz, qz;
                if constexpr (PH == 4) {
                    fz = (lane >> 2) & 3, qz = qB;
                } else {
                    fz = (lane >> 2) & 3, qz = ((lane >> 1) & 1) * CH + g * PH + (lane & 1);
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    f16x8 xb[MS];
#pragma unroll
                    for (int ms = 0; ms < MS; ++ms)
                        xb[ms] = __builtin_bit_cast(f16x8, to_b_order(xw[ms][kp][h]));
                    {
                        const f16x8 az = *reinterpret_cast<const f16x8 *>(&zs_lds[wave][fz & (F - 1)][h][qz][0]);
#pragma unroll
                        for (int ms = 0; ms < MS; ++ms)
                            accb[ms][kp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(az, xb[ms], accb[ms][kp], 0, 0, 0);
                    }
                    f16x8 B[F][MS];
#pragma unroll
                    for (int i = 0; i < F; ++i) {
                        const f16x8 sB = *reinterpret_cast<const f16x8 *>(&s_lds[wave][i][h][qB][0]);
#pragma unroll
                        for (int ms = 0; ms < MS; ++ms)
                            B[i][ms] = sB * xb[ms];
                    }
#pragma unroll
                    for (int r = 0; r < RG; ++r) {
                        const u32x4 cws = cw[r][kp];
                        const uint32_t d0 = h ? cws.z : cws.x, d1 = h ? cws.w : cws.y;
                        const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
#pragma unroll
                        for (int i = 0; i < F; ++i) {
                            const uint32_t mk = Field<NBITS>::mask(i);
                            const u32x4 Au = {d0 & mk, d0s & mk, d1 & mk, d1s & mk};
#pragma unroll
                            for (int ms = 0; ms < MS; ++ms)
                                acc[ms][r][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, Au), B[i][ms],
                                                                                       acc[ms][r][i], 0, 0, 0);
                        }
                    }
                }
            }
            wave_sync(); // the next slab's table phase overwrites the LDS tables
        }
    }

    // ---------------------------------------------------------------- wave tile -> LDS
    // Lane (column c = (m, phi), group gq) holds rows 4 * gq + v of column c in element v.
    const int gq = lane >> 4, mB = hi;
    // zero term of (field gq, batch row m): rows (field, [part,] phase) whose phase (and part) are the column's
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
        float bz;
        if constexpr (PH == 4) {
            const f32x4 t = accb[ms][0];
            bz = phi == 0 ? t[0] : (phi == 1 ? t[1] : (phi == 2 ? t[2] : t[3]));
            bz += quad_xor1(bz);
            bz += quad_xor2(bz);
        } else {
            const f32x4 t0 = accb[ms][0], t1 = accb[ms][KP - 1];
            bz = (phi == 0 ? t0[0] : t0[1]) + (phi == 0 ? t1[2] : t1[3]);
            bz += quad_xor1(bz);
        }
        if (phi == 0 && gq < F)
            bias_lds[wave][gq][ms * MB + mB] = bz * (1.0f / kXsScale);
    }
    wave_sync();
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) {
        const int m = ms * MB + mB;
#pragma unroll
        for (int r = 0; r < RG; ++r) {
            if constexpr (PH == 4) {
                float o[F];
#pragma unroll
                for (int i = 0; i < F; ++i) {
                    const f32x4 t = acc[ms][r][i];
                    float e = phi == 0 ? t[0] : (phi == 1 ? t[1] : (phi == 2 ? t[2] : t[3]));
                    e += quad_xor1(e);
                    e += quad_xor2(e);
                    o[i] = __builtin_fmaf(e, Field<NBITS>::unscale(i), -bias_lds[wave][i][m]);
                }
                if (phi == 0) {
                    float *dst = &red_lds[wave][4 * r + gq][m][0];
#pragma unroll
                    for (int i = 0; i < F; ++i)
                        dst[i] = o[i];
                }
            } else {
#pragma unroll
                for (int u = 0; u < 2; ++u) { // tile rows 8 * r + 2 * gq + u
                    float o[F];
#pragma unroll
                    for (int i = 0; i < F; ++i) {
                        const f32x4 t = acc[ms][r][i];
                        float e = phi == 0 ? t[2 * u] : t[2 * u + 1];
                        e += quad_xor1(e);
                        o[i] = __builtin_fmaf(e, Field<NBITS>::unscale(i), -bias_lds[wave][i][m]);
                    }
                    if (phi == 0) {
                        float *dst = &red_lds[wave][8 * r + 2 * gq + u][m][0];
#pragma unroll
                        for (int i = 0; i < F; ++i)
                            dst[i] = o[i];
                    }
                }
            }
        }
    }
    __syncthreads();

    // ---------------------------------------------------------------- block tile: a thread per (tile row, batch row)
    auto gate = [](float a, float b) __attribute__((always_inline)) -> f16 {
        const float u = (float)(f16)a;
        const f16 act = (f16)(u / (1.0f + __expf(-u)));
        return act * (f16)b;
    };
    for (int u = threadIdx.x; u < 16 * MT; u += kBatchWaves * 64) {
        const int r_t = u / MT, m_t = u % MT;
        if (m_t >= M)
            continue;
        float o[2][F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            o[0][i] = o[1][i] = 0.f;
        for (int w = 0; w < p.KS; ++w) {
#pragma unroll
            for (int l = 0; l < (EPI == 1 ? 2 : 1); ++l) {
                const float *src = &red_lds[l * p.KS + w][r_t][m_t][0];
#pragma unroll
                for (int i = 0; i < F; ++i)
                    o[l][i] += src[i];
            }
        }
        const int r = 16 * rb + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * GP); // outputs n .. n+F-1
        f16 *dst = p.y + (int64_t)m_t * N + n;
        if (EPI == 0 && p.BK > 1) {
            // K over several blocks: the blocks' results meet in one 64-bit fixed-point slot per output (gemv_parts.hpp)
#pragma unroll
            for (int i = 0; i < F; ++i) {
                unsigned long long *slot = p.slots + ((n + i) * MT + m_t);
                const unsigned long long mine = slot_term(o[0][i]);
                const unsigned long long before = __hip_atomic_fetch_add(slot, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (slot_count(before) != p.BK - 1)
                    continue;
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                f16 val = (f16)slot_total(before + mine, p.BK);
                if (p.bias)
                    val = val + p.bias[n + i];
                if (p.row_scale)
                    val = val * p.row_scale[m_t];
                dst[i] = p.accumulate ? (f16)(dst[i] + val) : val;
            }
            continue;
        }
        f16 hv[F];
#pragma unroll
        for (int i = 0; i < F; ++i) {
            if constexpr (EPI == 1) {
                hv[i] = gate(o[0][i], o[1][i]);
            } else {
                f16 val = (f16)o[0][i];
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

struct BatchPlan {
    int F, GP, RB, NS, PH, MS, WAVES, KS, SPW, BK, SKIND, ZKIND;
};

bool make_batch_plan(const hqq_linear *l, int64_t M, int NL, BatchPlan &pl)
{
    if ((l->nbits != 2 && l->nbits != 4) || M < 3 || M > 16)
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
    if (!((pl.SKIND == TK_U8_COLS && pl.ZKIND == TK_U8_SCALAR) || (pl.SKIND == TK_F16 && pl.ZKIND == TK_F16)))
        return false;
    if (pl.SKIND == TK_U8_COLS && (l->scale.meta_cols % 16 != 0 || !aligned16(l->scale.meta_scale) || !aligned16(l->scale.meta_zero)))
        return false;
    pl.F = F;
    pl.GP = (int)(G / F);
    pl.RB = l->group_size / 16;
    pl.NS = (int)(l->K / kSlab);
    if (pl.GP > 65535 || pl.RB > 65535)
        return false;
    pl.PH = M <= 4 ? 4 : 2;
    pl.MS = M <= 8 ? 1 : 2;
    const int64_t tiles = (int64_t)pl.GP * pl.RB;
    // K over as many blocks as it takes to cover the chip about once, a block holding at least a slab per wave of eight
    int BK = 1;
    while (tiles * BK < 200 && (pl.NS + BK) / (BK + 1) >= 8 / NL && BK < 8)
        ++BK;
    // Sixteen waves where they were measured ahead of eight: five to eight rows in blocks that hold all of K (the gate
    // 17.7 -> 15.6 us, 14336x4096 10.2 -> 9.3 us; with K over four blocks the down projection loses, 10.8 -> 13.3 us,
    // and so do batches of up to four rows)
    pl.WAVES = pl.MS == 1 && pl.PH == 2 && BK == 1 ? tuning_int("HQQ_BATCH_WAVES", 16) : 8;
    pl.KS = pl.WAVES / NL;
    if (NL == 2 && BK > 1)
        return false; // the gate's epilogue needs both projections whole
    pl.BK = BK;
    const int per_block = (pl.NS + BK - 1) / BK;
    pl.SPW = (per_block + pl.KS - 1) / pl.KS;
    if (BK > 1 && (int64_t)l->N * (pl.PH == 4 ? 4 : 8 * pl.MS) * (int64_t)sizeof(unsigned long long) > (int64_t)kSlotBytes)
        return false;
    return true;
}

template <int NBITS, int PH, int MS, int EPI, int WAVES>
void launch_batch_kinds(const BatchParams &p, const BatchPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.SKIND == TK_F16)
        gemv_batch_kernel<NBITS, PH, MS, TK_F16, TK_F16, EPI, WAVES><<<grid, dim3(WAVES * 64), 0, s>>>(p);
    else
        gemv_batch_kernel<NBITS, PH, MS, TK_U8_COLS, TK_U8_SCALAR, EPI, WAVES><<<grid, dim3(WAVES * 64), 0, s>>>(p);
}

template <int NBITS, int EPI> void launch_batch_shape(const BatchParams &p, const BatchPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.MS == 2)
        launch_batch_kinds<NBITS, 2, 2, EPI, 8>(p, pl, grid, s);
    else if (pl.PH == 4)
        launch_batch_kinds<NBITS, 4, 1, EPI, 8>(p, pl, grid, s);
    else
        pl.WAVES == 16 ? launch_batch_kinds<NBITS, 2, 1, EPI, 16>(p, pl, grid, s) : launch_batch_kinds<NBITS, 2, 1, EPI, 8>(p, pl, grid, s);
}

int run_batch(const hqq_linear *l0, const hqq_linear *l1, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
              const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix)
{
    const int NL = l1 ? 2 : 1;
    BatchPlan pl;
    if (!make_batch_plan(l0, M, NL, pl))
        return HQQ_E_UNSUPPORTED;
    BatchParams p = {};
    fill_layer_record(p.layer[0], l0);
    fill_layer_record(p.layer[1], l1 ? l1 : l0);
    p.x = x, p.y = y, p.bias = l1 ? nullptr : static_cast<const f16 *>(l0->bias);
    p.row_scale = ep.row_scale, p.accumulate = ep.accumulate;
    p.M = (int)M, p.K = (int)l0->K, p.N = (int)l0->N, p.GP = pl.GP, p.RB = pl.RB, p.NS = pl.NS;
    p.KS = pl.KS, p.SPW = pl.SPW, p.BK = pl.BK, p.NL = NL;
    if (ix) {
        p.table = static_cast<const LayerRecord *>(ix->table);
        p.sel = ix->sel, p.table_stride = ix->stride, p.table_first = ix->first;
    }
    if (!aligned16(x))
        return HQQ_E_ALIGN;
    if (pl.BK > 1) {
        if (!ws || ws_bytes < kHeadBytes)
            return HQQ_E_WORKSPACE;
        p.slots = reinterpret_cast<unsigned long long *>(static_cast<char *>(ws) + kCounterBytes);
    }
    const dim3 grid((unsigned)pl.BK, (unsigned)pl.RB, (unsigned)pl.GP);
    if (l1) {
        l0->nbits == 2 ? launch_batch_shape<2, 1>(p, pl, grid, s) : launch_batch_shape<4, 1>(p, pl, grid, s);
    } else {
        l0->nbits == 2 ? launch_batch_shape<2, 0>(p, pl, grid, s) : launch_batch_shape<4, 0>(p, pl, grid, s);
    }
    return launch_status();
}

} // namespace

bool batch_supported(const hqq_linear *l, int64_t M)
{
    BatchPlan pl;
    return make_batch_plan(l, M, 1, pl);
}

bool batch_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    BatchPlan a, b;
    return make_batch_plan(w1, M, 2, a) && make_batch_plan(w3, M, 2, b) && w1->N == w3->N && w1->K == w3->K &&
           w1->nbits == w3->nbits && w1->group_size == w3->group_size && a.SKIND == b.SKIND && a.ZKIND == b.ZKIND;
}

size_t batch_workspace_bytes(const hqq_linear *l, int64_t M)
{
    BatchPlan pl;
    if (!make_batch_plan(l, M, 1, pl))
        return 0;
    return kHeadBytes;
}

int launch_batch_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                        const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix)
{
    return run_batch(l, nullptr, x, M, y, ws, ws_bytes, ep, s, ix);
}

int launch_batch_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                         size_t ws_bytes, hipStream_t s, const StripIndex *ix)
{
    if (!batch_gate_supported(w1, w3, M))
        return HQQ_E_UNSUPPORTED;
    return run_batch(w1, w3, x, M, h, ws, ws_bytes, SmallBatchEpilogue{}, s, ix);
}

} // namespace hqq
