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
// cross-lane reduction.  Codes become fp16 with one AND-OR (the field lands in
// the mantissa of 2^e, giving 2^e + q) and one packed subtract.
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

#include <cstdlib>

namespace hqq {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kStepK = 64; // columns per wave step
// xs = s * x is held in fp16; scales are ~1e-3..1e-1, so the scale is raised by 2^5 first to keep small
// activations out of the fp16 subnormal range (|s*x| would have to exceed 2047 to overflow).  Undone in fp32.
constexpr float kXsScale = 32.0f;

struct SBLayer {
    const uint8_t *codes;
    Table sc, zr;
    float *part; // [NSG][M][N]
};

struct SBParams {
    SBLayer layer[2];
    const f16 *x;
    int M, N, K;
    int GP;     // G / F: packed table rows
    int RB;     // gs / 16: row blocks per jp
    int WR, WS; // waves of a block along r-blocks / along K slabs
    int SK;     // steps per wave
    int KT;     // K / 64
    int NSG;    // slab groups (= partial-sum copies)
};

// Running reader of one (G, K) table for the four columns a lane owns.
struct TableCursor {
    const uint8_t *u8;
    const f16 *f;
    const f16 *ms, *mz;
    int64_t c;    // flat index j*K + k of the lane's first column
    int64_t cm;   // c % meta_cols
    int64_t cols; // meta_cols
    bool is_u8, scalar;
    f16x2 ms_s, mz_s; // scalar meta, splat

    __device__ void init(const Table &t, int64_t c0)
    {
        is_u8 = t.kind == HQQ_TABLE_U8;
        u8 = static_cast<const uint8_t *>(t.data);
        f = static_cast<const f16 *>(t.data);
        ms = t.ms, mz = t.mz;
        cols = t.meta_cols;
        scalar = is_u8 && cols == 1;
        c = c0;
        cm = (is_u8 && !scalar) ? c0 % cols : 0;
        if (scalar) {
            ms_s = (f16x2){ms[0], ms[0]};
            mz_s = (f16x2){mz[0], mz[0]};
        }
    }
    __device__ void advance(int64_t d)
    {
        c += d;
        if (is_u8 && !scalar) {
            cm += d;
            while (cm >= cols)
                cm -= cols;
        }
    }
};

struct TableRaw {
    u32x2 data;  // 4 bytes (u8 table) or 4 halves (fp16 table)
    u32x2 ms, mz; // 4 halves each (u8 table with per-column meta)
};

__device__ __forceinline__ TableRaw table_load(const TableCursor &t)
{
    TableRaw r;
    r.data = (u32x2){0, 0};
    r.ms = r.data;
    r.mz = r.data;
    if (t.is_u8) {
        r.data.x = *reinterpret_cast<const uint32_t *>(t.u8 + t.c);
        if (!t.scalar) {
            r.ms = *reinterpret_cast<const u32x2 *>(t.ms + t.cm);
            r.mz = *reinterpret_cast<const u32x2 *>(t.mz + t.cm);
        }
    } else {
        r.data = *reinterpret_cast<const u32x2 *>(t.f + t.c);
    }
    return r;
}

__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }

// four table entries as fp16: stored values, or fp16(fp16(q - mz) * ms)
__device__ __forceinline__ void table_decode(const TableCursor &t, const TableRaw &r, f16x2 &lo, f16x2 &hi)
{
    if (t.is_u8) {
        // bytes -> fp16 exactly: 0x6400 | b is 1024 + b, then subtract 1024
        const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
        const uint32_t w = r.data.x;
        f16x2 q01 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, w, 0x04010400u)) - k1024;
        f16x2 q23 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, w, 0x04030402u)) - k1024;
        if (t.scalar) {
            lo = (q01 - t.mz_s) * t.ms_s;
            hi = (q23 - t.mz_s) * t.ms_s;
        } else {
            lo = (q01 - as_f16x2(r.mz.x)) * as_f16x2(r.ms.x);
            hi = (q23 - as_f16x2(r.mz.y)) * as_f16x2(r.ms.y);
        }
    } else {
        lo = as_f16x2(r.data.x);
        hi = as_f16x2(r.data.y);
    }
}

// codes of field i of the two bytes that sit in the low byte of each 16-bit half
// of d, as the fp16 pair (q, q'): AND-OR drops the field into the mantissa of 2^e.
template <int NBITS> __device__ __forceinline__ f16x2 extract_pair(uint32_t d, int i)
{
    constexpr int F = 8 / NBITS;
    const int pos = NBITS * (F - 1 - i);
    const int e = 10 - pos;
    const uint32_t mask = (((1u << NBITS) - 1u) * 0x00010001u) << pos;
    const uint32_t expo = (uint32_t)((e + 15) << 10) * 0x00010001u;
    const f16 off = (f16)(float)(1 << e);
    return as_f16x2((d & mask) | expo) - (f16x2){off, off};
}

template <int NBITS, int MT>
__global__ __launch_bounds__(kWavesPerBlock * 64) void smallbatch_kernel(SBParams p)
{
    constexpr int F = 8 / NBITS;
    constexpr int XS_HALVES = F * 2 * 4 * MT * 8; // per wave, one step
    __shared__ __attribute__((aligned(16))) f16 xs_lds[kWavesPerBlock][XS_HALVES];
    __shared__ float bias_lds[kWavesPerBlock][F][MT];
    __shared__ __attribute__((aligned(16))) float red_lds[kWavesPerBlock][F][64][4];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wr = wave % p.WR, ws = wave / p.WR;
    const SBLayer &L = p.layer[blockIdx.y];

    int b = blockIdx.x;
    const int sg = b % p.NSG;
    b /= p.NSG;
    const int RBG = p.RB / p.WR;
    const int rbg = b % RBG;
    const int jp = b / RBG;
    const int rb = rbg * p.WR + wr;
    const int slab = sg * p.WS + ws;
    const int step_begin = slab * p.SK;
    int step_end = step_begin + p.SK;
    if (step_end > p.KT)
        step_end = p.KT;

    const int64_t K = p.K;
    // code lane role: packed row of (jp, r), 16 columns at 16*kg
    const int rr = lane & 15, kg = lane >> 4;
    const int64_t prow = (int64_t)jp + (int64_t)(16 * rb + rr) * p.GP;
    const uint8_t *cptr = L.codes + prow * K + 16 * kg;
    // table lane role: table row F*jp + ti, columns 4*kq .. 4*kq+3
    const int ti = lane >> 4, kq = lane & 15;
    const bool tlane = ti < F;
    TableCursor sc, zr;
    {
        const int64_t c0 = ((int64_t)F * jp + (tlane ? ti : 0)) * K + (int64_t)step_begin * kStepK + 4 * kq;
        sc.init(L.sc, c0);
        zr.init(L.zr, c0);
    }
    const f16 *xptr = p.x + 4 * kq;
    // where this lane's xs go: entry ((ti*2 + h)*4 + kgt)*MT + m, 16 B each, second half when kq is odd
    f16 *xs_w = &xs_lds[wave][((((ti * 2 + ((kq >> 1) & 1)) * 4 + (kq >> 2)) * MT) * 8) + 4 * (kq & 1)];
    const f16 *xs_r = &xs_lds[wave][(kg * MT + (lane & 15)) * 8];

    // LDS rows of batch entries m >= M are never written by the table phase: clear once
    for (int i = lane; i < XS_HALVES / 8; i += 64)
        *reinterpret_cast<u32x4 *>(&xs_lds[wave][i * 8]) = (u32x4){0, 0, 0, 0};

    f32x4 acc[F];
#pragma unroll
    for (int i = 0; i < F; ++i)
        acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float bias_acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        bias_acc[m] = 0.f;

    // software pipeline: loads of step s+1 are issued before the arithmetic of step s
    u32x4 cw_n = {0, 0, 0, 0};
    TableRaw sraw_n, zraw_n;
    u32x2 x_n[MT];
    auto issue = [&](int s) {
        const int64_t k0 = (int64_t)s * kStepK;
        cw_n = *reinterpret_cast<const u32x4 *>(cptr + k0);
        if (tlane) {
            sraw_n = table_load(sc);
            zraw_n = table_load(zr);
#pragma unroll
            for (int m = 0; m < MT; ++m)
                if (m < p.M)
                    x_n[m] = *reinterpret_cast<const u32x2 *>(xptr + (int64_t)m * K + k0);
        }
        sc.advance(kStepK);
        zr.advance(kStepK);
    };
    if (step_begin < step_end)
        issue(step_begin);

    for (int s = step_begin; s < step_end; ++s) {
        const u32x4 cw = cw_n;
        const TableRaw sraw = sraw_n, zraw = zraw_n;
        u32x2 xv[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            xv[m] = x_n[m];
        if (s + 1 < step_end)
            issue(s + 1);

        // ---- table phase
        if (tlane) {
            f16x2 s01, s23, z01, z23;
            table_decode(sc, sraw, s01, s23);
            table_decode(zr, zraw, z01, z23);
            s01 = s01 * (f16x2){(f16)kXsScale, (f16)kXsScale};
            s23 = s23 * (f16x2){(f16)kXsScale, (f16)kXsScale};
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < p.M) {
                    const f16x2 a01 = s01 * as_f16x2(xv[m].x);
                    const f16x2 a23 = s23 * as_f16x2(xv[m].y);
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

        // ---- code phase
        const uint32_t d[4] = {cw.x, cw.y, cw.z, cw.w};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
            const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                const f16x2 a0 = extract_pair<NBITS>(d0, i), a1 = extract_pair<NBITS>(d0s, i);
                const f16x2 a2 = extract_pair<NBITS>(d1, i), a3 = extract_pair<NBITS>(d1s, i);
                const f16x8 A = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
                f16x8 B = {0, 0, 0, 0, 0, 0, 0, 0};
                if ((lane & 15) < MT)
                    B = *reinterpret_cast<const f16x8 *>(xs_r + ((i * 2 + h) * 4 * MT) * 8);
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, acc[i], 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // ---- bias: sum the 16 table lanes of each table row, hand it to the lanes that hold D
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float v = bias_acc[m];
#pragma unroll
        for (int off = 8; off > 0; off >>= 1)
            v += __shfl_xor(v, off, 64);
        if (tlane && kq == 0)
            bias_lds[wave][ti][m] = v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int mcol = lane & 15; // D layout: column = batch row, rows 4*(lane>>4)+v
    if (mcol < MT) {
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const float bz = bias_lds[wave][i][mcol];
            acc[i] = (acc[i] - (f32x4){bz, bz, bz, bz}) * (1.0f / kXsScale);
        }
    }

    // ---- sum the K slabs of this block (waves ws > 0 hand their tile to ws == 0)
    if (p.WS > 1) {
        if (ws > 0) {
#pragma unroll
            for (int i = 0; i < F; ++i)
                *reinterpret_cast<f32x4 *>(&red_lds[wave][i][lane][0]) = acc[i];
        }
        __syncthreads();
        if (ws == 0) {
            for (int o = 1; o < p.WS; ++o)
#pragma unroll
                for (int i = 0; i < F; ++i)
                    acc[i] += *reinterpret_cast<const f32x4 *>(&red_lds[o * p.WR + wr][i][lane][0]);
        }
    }
    if (ws != 0 || mcol >= p.M)
        return;

    // ---- store the partial sums: rows r = 16*rb + 4*(lane>>4) + v, outputs n = F*(jp + r*GP) + i
    float *dst = L.part + ((int64_t)sg * p.M + mcol) * p.N;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int r = 16 * rb + 4 * (lane >> 4) + v;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * p.GP);
        if constexpr (F == 4)
            *reinterpret_cast<f32x4 *>(dst + n) = (f32x4){acc[0][v], acc[1][v], acc[2][v], acc[3][v]};
        else
            *reinterpret_cast<float2 *>(dst + n) = make_float2(acc[0][v], acc[1][v]);
    }
}

// Sum the slab partials and apply the epilogue.  MODE 0: y = cast(sum) (+bias) (*row_scale) (+= y);
// MODE 1: h = silu(sum of layer 0) * (sum of layer 1), the expert FFN's gate.
template <int MODE>
__global__ __launch_bounds__(256) void smallbatch_finish_kernel(const float *__restrict__ part0,
                                                                const float *__restrict__ part1, int NSG, int M,
                                                                int N, const f16 *__restrict__ bias,
                                                                const f16 *__restrict__ row_scale, int accumulate,
                                                                f16 *__restrict__ y)
{
    const int64_t total = (int64_t)M * N / 4;
    const int64_t stride = (int64_t)M * N;
    for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
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

int env_int(const char *name, int dflt)
{
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : dflt;
}

struct SBPlan {
    int F, GP, RB, WR, WS, SK, KT, NS, NSG, MT;
};

bool make_plan(const hqq_linear *l, int64_t M, SBPlan &pl)
{
    if (l->nbits != 2 && l->nbits != 4)
        return false;
    if (M < 1 || M > 16)
        return false;
    const int F = 8 / l->nbits;
    const int64_t G = l->N / l->group_size;
    if (l->group_size % 16 != 0 || G % F != 0 || l->K % kStepK != 0)
        return false;
    if (l->N * l->K / l->group_size >= (1ll << 31) || l->N >= (1ll << 31) || l->K >= (1ll << 31))
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
    pl.WR = pl.RB >= 4 ? 4 : (pl.RB >= 2 ? 2 : 1);
    if (pl.RB % pl.WR != 0)
        pl.WR = 1;
    pl.WS = kWavesPerBlock / pl.WR;
    pl.KT = (int)(l->K / kStepK);
    const int64_t tiles = (int64_t)pl.GP * pl.RB;
    const int target = env_int("HQQ_SB_WAVES", 4096);
    int64_t ns = (target + tiles - 1) / tiles;
    if (ns < 1)
        ns = 1;
    if (ns > pl.KT)
        ns = pl.KT;
    int sk = (int)((pl.KT + ns - 1) / ns);
    const int sk_env = env_int("HQQ_SB_STEPS", 0);
    if (sk_env > 0)
        sk = sk_env;
    pl.SK = sk;
    pl.NS = (pl.KT + sk - 1) / sk;
    pl.NSG = (pl.NS + pl.WS - 1) / pl.WS;
    pl.MT = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : (M <= 8 ? 8 : 16)));
    return true;
}

template <int NBITS> void launch_main(const SBParams &p, int MT, dim3 grid, hipStream_t s)
{
    const dim3 block(kWavesPerBlock * 64);
    switch (MT) {
    case 1: smallbatch_kernel<NBITS, 1><<<grid, block, 0, s>>>(p); break;
    case 2: smallbatch_kernel<NBITS, 2><<<grid, block, 0, s>>>(p); break;
    case 4: smallbatch_kernel<NBITS, 4><<<grid, block, 0, s>>>(p); break;
    case 8: smallbatch_kernel<NBITS, 8><<<grid, block, 0, s>>>(p); break;
    default: smallbatch_kernel<NBITS, 16><<<grid, block, 0, s>>>(p); break;
    }
}

int finish_grid(int64_t M, int64_t N)
{
    int64_t b = (M * N / 4 + 255) / 256;
    return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

} // namespace

bool smallbatch_supported(const hqq_linear *l, int64_t M)
{
    SBPlan pl;
    return make_plan(l, M, pl) && l->N % 4 == 0;
}

size_t smallbatch_workspace_bytes(const hqq_linear *l, int64_t M)
{
    SBPlan pl;
    if (!make_plan(l, M, pl))
        return 0;
    return (size_t)pl.NSG * (size_t)M * (size_t)l->N * sizeof(float);
}

static void fill_params(SBParams &p, const SBPlan &pl, const hqq_linear *l, int which, float *part)
{
    p.layer[which].codes = static_cast<const uint8_t *>(l->codes);
    p.layer[which].sc = make_table(l->scale);
    p.layer[which].zr = make_table(l->zero);
    p.layer[which].part = part;
    p.N = (int)l->N, p.K = (int)l->K;
    p.GP = pl.GP, p.RB = pl.RB, p.WR = pl.WR, p.WS = pl.WS, p.SK = pl.SK, p.KT = pl.KT, p.NSG = pl.NSG;
}

int launch_smallbatch_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                             const SmallBatchEpilogue &ep, hipStream_t s)
{
    SBPlan pl;
    if (!make_plan(l, M, pl))
        return HQQ_E_UNSUPPORTED;
    if (ws_bytes < smallbatch_workspace_bytes(l, M))
        return HQQ_E_WORKSPACE;
    SBParams p = {};
    fill_params(p, pl, l, 0, static_cast<float *>(ws));
    p.layer[1] = p.layer[0];
    p.x = x, p.M = (int)M;
    const dim3 grid((unsigned)(pl.GP * (pl.RB / pl.WR) * pl.NSG), 1);
    if (l->nbits == 2)
        launch_main<2>(p, pl.MT, grid, s);
    else
        launch_main<4>(p, pl.MT, grid, s);
    int rc = launch_status();
    if (rc != HQQ_OK)
        return rc;
    smallbatch_finish_kernel<0><<<finish_grid(M, l->N), 256, 0, s>>>(
        p.layer[0].part, nullptr, pl.NSG, (int)M, (int)l->N, static_cast<const f16 *>(l->bias), ep.row_scale,
        ep.accumulate, y);
    return launch_status();
}

int launch_smallbatch_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                              size_t ws_bytes, hipStream_t s)
{
    SBPlan pl, pl3;
    if (!make_plan(w1, M, pl) || !make_plan(w3, M, pl3) || w1->N != w3->N || w1->K != w3->K ||
        w1->nbits != w3->nbits || w1->group_size != w3->group_size)
        return HQQ_E_UNSUPPORTED;
    const size_t one = smallbatch_workspace_bytes(w1, M);
    if (ws_bytes < 2 * one)
        return HQQ_E_WORKSPACE;
    SBParams p = {};
    fill_params(p, pl, w1, 0, static_cast<float *>(ws));
    fill_params(p, pl, w3, 1, reinterpret_cast<float *>(static_cast<char *>(ws) + one));
    p.x = x, p.M = (int)M;
    const dim3 grid((unsigned)(pl.GP * (pl.RB / pl.WR) * pl.NSG), 2);
    if (w1->nbits == 2)
        launch_main<2>(p, pl.MT, grid, s);
    else
        launch_main<4>(p, pl.MT, grid, s);
    int rc = launch_status();
    if (rc != HQQ_OK)
        return rc;
    smallbatch_finish_kernel<1><<<finish_grid(M, w1->N), 256, 0, s>>>(p.layer[0].part, p.layer[1].part, pl.NSG,
                                                                       (int)M, (int)w1->N, nullptr, nullptr, 0, h);
    return launch_status();
}

} // namespace hqq
