// Decode-time GEMV for 3-bit codes, ten per int32 word (reference src/packing.py:62-81: code i of a word at bit
// 3*(9-i); kernel src/triton_kernels.py:414-509).
//
// A word row w holds output rows n = 10w .. 10w+9, which use table rows j = (10w + i) mod G.  Word rows P apart,
// P = G / gcd(10, G), use the SAME ten table rows (10P is a multiple of G), so a tile is the word rows
// w0 + P*t, t = 0..15, of one window w0: they share ten scale rows and ten zero rows, and as in the 2- and 4-bit
// kernels the scale is folded into the activations once per tile,
//     y[10w+i, m] = sum_k q_i[w, k] * xs[i, k, m]  -  sum_k z[i, k] * xs[i, k, m],     xs = 32 * s[i, k] * x[m, k]  (fp16).
//
// A wave takes one slab of 256 columns of a tile at a time.  Lane (t = lane >> 2, c = lane & 3) owns word row t,
// columns 16m + 4c .. +3 for m = 0..15: four consecutive lanes read 64 consecutive bytes, sixteen 128-bit loads per
// lane, all in flight at once.  A pair of words gives, per field, one v_perm (the two bytes that hold the field, of
// both words) and one v_and: the field masked in place is the fp16 subnormal q * 2^(rel - 24), which v_dot2_f32_f16
// multiplies exactly and accumulates in fp32.  The table phase (lane l owns columns 4l .. 4l+3 of all ten rows)
// leaves xs in LDS; the zero term is a dot product per table row, summed over the wave at the end.
//
// The waves of a block split K (two slabs each); when K needs several blocks (or the window count alone would leave
// most of the chip idle) the blocks of a tile store fp32 partial sums with device-scope stores and the block that
// arrives last at the tile's counter adds them in a fixed order.  Batches above two rows run as passes of two.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"

namespace hqq {
using namespace gemv;
namespace {

constexpr int kW3Waves = 8;
constexpr int kW3S = 2; // slabs per wave

struct W3Params {
    const uint8_t *codes; // int32 [NW][K]
    const uint8_t *sq, *zq;
    const f16 *s_ms, *s_mz, *z_ms, *z_mz;
    uint32_t s_cols, s_inv;
    const f16 *x;
    f16 *y;
    const f16 *bias;
    float *part; // [BK][M][N]
    int *counter;
    int M, N, K, G, P, NW, RB;
    int NS; // K / 256
    int KS; // waves of a block that have slabs
    int SB; // slabs per block
    int BK; // blocks along K per tile
};

// field i of a word: bit offset 3*(9-i); the two bytes B, B+1 that hold it, its offset inside them
__host__ __device__ constexpr int w3_bit(int i) { return 3 * (9 - i); }
__host__ __device__ constexpr uint32_t w3_sel(int i)
{
    const uint32_t B = (uint32_t)w3_bit(i) >> 3;
    const uint32_t lo0 = B, hi0 = B < 3 ? B + 1 : 0x0cu, lo1 = 4 + B, hi1 = B < 3 ? 4 + B + 1 : 0x0cu;
    return (hi1 << 24) | (lo1 << 16) | (hi0 << 8) | lo0;
}
__host__ __device__ constexpr uint32_t w3_mask(int i) { return (7u << (w3_bit(i) & 7)) * 0x00010001u; }
__host__ __device__ constexpr float w3_unscale(int i) { return (float)(1u << (24 - (w3_bit(i) & 7))) / kXsScale; }

__device__ __forceinline__ float quad_sum(float v)
{
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

template <int MT, bool Q8> // Q8: scale u8 + per-column meta, zero u8 + whole-tensor meta; else fp16 tables
__global__ __launch_bounds__(kW3Waves * 64) void gemv_w3_kernel(W3Params p)
{
    constexpr int NT = kW3Waves * 64;
    // xs of the slab: [4-column group q][batch row][field][4 halves]
    __shared__ __attribute__((aligned(16))) f16 xs_lds[kW3Waves][64][MT][10][4];
    __shared__ float red_lds[kW3Waves][16][10][MT];
    __shared__ int ticket_lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kb = blockIdx.x, rb = blockIdx.y, w0 = blockIdx.z;
    const int M = MT == 1 ? 1 : p.M;
    const int K = p.K;
    const int t = lane >> 2, c = lane & 3;
    const int wr = w0 + p.P * (16 * rb + t); // this lane's word row
    const bool row_ok = wr < p.NW;
    const uint32_t j0 = (uint32_t)(10 * w0) % (uint32_t)p.G;
    const uint32_t code_base = (uint32_t)(row_ok ? wr : w0) * (uint32_t)K * 4u + (uint32_t)(16 * c);

    float acc[10][MT], zacc[10][MT];
#pragma unroll
    for (int i = 0; i < 10; ++i)
#pragma unroll
        for (int m = 0; m < MT; ++m)
            acc[i][m] = zacc[i][m] = 0.f;

    const int slab_lo = kb * p.SB + wave * kW3S;
    int slab_hi = (kb + 1) * p.SB;
    if (slab_hi > p.NS)
        slab_hi = p.NS;
    // whole-tensor meta of the zero table; the address is the same in every lane but written so that the compiler
    // does not see it (lane >> 6 is zero): a load it knows to be uniform is moved to scalar registers at once,
    // which waits for it before any weight load has been issued
    uint32_t zms_raw = 0, zmz_raw = 0;
    if constexpr (Q8) {
        zms_raw = reinterpret_cast<const uint16_t *>(p.z_ms)[lane >> 6];
        zmz_raw = reinterpret_cast<const uint16_t *>(p.z_mz)[lane >> 6];
    }

    for (int sl = 0; sl < kW3S; ++sl) {
        const int slab = slab_lo + sl;
        if (wave >= p.KS || slab >= slab_hi)
            break;
        const uint32_t k0 = (uint32_t)slab * kSlab;
        // ------------------------------------------------------------ loads: tables and x (lane l: columns 4l..4l+3), codes
        uint32_t sraw[10][2], zraw[10][2];
        u32x2 msr[10], mzr[10];
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            uint32_t j = j0 + (uint32_t)i; // (10*w0 + i) mod G; G >= 10
            j -= j >= (uint32_t)p.G ? (uint32_t)p.G : 0u;
            const uint32_t ce = j * (uint32_t)K + k0 + (uint32_t)(4 * lane);
            if constexpr (Q8) {
                sraw[i][0] = *reinterpret_cast<const uint32_t *>(p.sq + ce);
                zraw[i][0] = *reinterpret_cast<const uint32_t *>(p.zq + ce);
                uint32_t cm = ce - __umulhi(ce, p.s_inv) * p.s_cols; // ce mod cols; the quotient estimate is at most 2 short
                cm -= cm >= p.s_cols ? p.s_cols : 0;
                cm -= cm >= p.s_cols ? p.s_cols : 0;
                msr[i] = *reinterpret_cast<const u32x2 *>(p.s_ms + cm);
                mzr[i] = *reinterpret_cast<const u32x2 *>(p.s_mz + cm);
            } else {
                const u32x2 a = *reinterpret_cast<const u32x2 *>(reinterpret_cast<const f16 *>(p.sq) + ce);
                const u32x2 b = *reinterpret_cast<const u32x2 *>(reinterpret_cast<const f16 *>(p.zq) + ce);
                sraw[i][0] = a.x, sraw[i][1] = a.y, zraw[i][0] = b.x, zraw[i][1] = b.y;
            }
        }
        u32x2 xr[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            xr[m] = *reinterpret_cast<const u32x2 *>(p.x + ((uint32_t)((m < M ? m : 0) * K) + k0 + (uint32_t)(4 * lane)));
        u32x4 cw[16];
#pragma unroll
        for (int m = 0; m < 16; ++m)
            cw[m] = *reinterpret_cast<const u32x4 *>(p.codes + (code_base + 4u * k0 + (uint32_t)(64 * m)));

        // ------------------------------------------------------------ table phase: xs into LDS, zero term accumulated
        {
            const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
            const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
            const f16x2 zms = as_h2(zms_raw * 0x10001u), zmz = as_h2(zmz_raw * 0x10001u);
#pragma unroll
            for (int i = 0; i < 10; ++i) {
                f16x2 s01, s23, z01, z23;
                if constexpr (Q8) {
                    // bytes -> fp16 exactly (0x6400 | b is 1024 + b), then fp16(fp16(q - mz) * ms) as the reference does
                    const f16x2 q01 = as_h2(__builtin_amdgcn_perm(0x64646464u, sraw[i][0], 0x04010400u)) - k1024;
                    const f16x2 q23 = as_h2(__builtin_amdgcn_perm(0x64646464u, sraw[i][0], 0x04030402u)) - k1024;
                    s01 = (q01 - as_h2(mzr[i].x)) * as_h2(msr[i].x);
                    s23 = (q23 - as_h2(mzr[i].y)) * as_h2(msr[i].y);
                    const f16x2 y01 = as_h2(__builtin_amdgcn_perm(0x64646464u, zraw[i][0], 0x04010400u)) - k1024;
                    const f16x2 y23 = as_h2(__builtin_amdgcn_perm(0x64646464u, zraw[i][0], 0x04030402u)) - k1024;
                    z01 = (y01 - zmz) * zms;
                    z23 = (y23 - zmz) * zms;
                } else {
                    s01 = as_h2(sraw[i][0]), s23 = as_h2(sraw[i][1]);
                    z01 = as_h2(zraw[i][0]), z23 = as_h2(zraw[i][1]);
                }
                s01 = s01 * k32, s23 = s23 * k32;
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const f16x2 a01 = s01 * as_h2(xr[m].x), a23 = s23 * as_h2(xr[m].y);
                    zacc[i][m] = __builtin_amdgcn_fdot2(z01, a01, zacc[i][m], false);
                    zacc[i][m] = __builtin_amdgcn_fdot2(z23, a23, zacc[i][m], false);
                    *reinterpret_cast<f16x4 *>(&xs_lds[wave][lane][m][i][0]) = (f16x4){a01.x, a01.y, a23.x, a23.y};
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ------------------------------------------------------------ codes: per pair of words and field, perm + and + dot2
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            const int q = 4 * m + c;
            u32x2 X[MT][10];
#pragma unroll
            for (int mm = 0; mm < MT; ++mm) {
                const u32x4 *src = reinterpret_cast<const u32x4 *>(&xs_lds[wave][q][mm][0][0]);
#pragma unroll
                for (int v = 0; v < 5; ++v) {
                    const u32x4 d = src[v];
                    X[mm][2 * v] = (u32x2){d.x, d.y};
                    X[mm][2 * v + 1] = (u32x2){d.z, d.w};
                }
            }
#pragma unroll
            for (int i = 0; i < 10; ++i) {
                const uint32_t pa = __builtin_amdgcn_perm(cw[m].y, cw[m].x, w3_sel(i)) & w3_mask(i);
                const uint32_t pb = __builtin_amdgcn_perm(cw[m].w, cw[m].z, w3_sel(i)) & w3_mask(i);
#pragma unroll
                for (int mm = 0; mm < MT; ++mm) {
                    acc[i][mm] = __builtin_amdgcn_fdot2(as_h2(pa), as_h2(X[mm][i].x), acc[i][mm], false);
                    acc[i][mm] = __builtin_amdgcn_fdot2(as_h2(pb), as_h2(X[mm][i].y), acc[i][mm], false);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    // ---------------------------------------------------------------- wave result: sum over the column lanes, zero term removed
#pragma unroll
    for (int i = 0; i < 10; ++i) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float a = quad_sum(acc[i][m]) * w3_unscale(i);
            const float z = wave_sum(zacc[i][m]) * (1.0f / kXsScale);
            if (c == 0)
                red_lds[wave][t][i][m] = a - z;
        }
    }
    __syncthreads();

    // ---------------------------------------------------------------- block result
    const bool alone = p.BK == 1;
    const int tile = w0 * p.RB + rb;
    for (int u = threadIdx.x; u < 16 * 10 * MT; u += NT) {
        const int m_t = u % MT, i_t = (u / MT) % 10, t_t = u / (10 * MT);
        float v = 0.f;
        for (int w = 0; w < p.KS; ++w) // fixed order
            v += red_lds[w][t_t][i_t][m_t];
        const int64_t wr_t = (int64_t)w0 + (int64_t)p.P * (16 * rb + t_t);
        const int64_t n = 10 * wr_t + i_t;
        if (m_t >= M || wr_t >= p.NW || n >= p.N)
            continue;
        if (alone) {
            f16 val = (f16)v;
            if (p.bias)
                val = val + p.bias[n];
            p.y[(int64_t)m_t * p.N + n] = val;
        } else {
            __hip_atomic_store(p.part + ((int64_t)kb * M + m_t) * p.N + n, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (alone)
        return;

    // the block that arrives last at the tile's counter adds the partial sums in a fixed order
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(&p.counter[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == p.BK - 1)
            __hip_atomic_store(&p.counter[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket_lds = prev;
    }
    __syncthreads();
    if (ticket_lds != p.BK - 1)
        return;
    for (int u = threadIdx.x; u < 16 * 10 * MT; u += NT) {
        const int m_t = u % MT, i_t = (u / MT) % 10, t_t = u / (10 * MT);
        const int64_t wr_t = (int64_t)w0 + (int64_t)p.P * (16 * rb + t_t);
        const int64_t n = 10 * wr_t + i_t;
        if (m_t >= M || wr_t >= p.NW || n >= p.N)
            continue;
        float v = 0.f;
        for (int s = 0; s < p.BK; ++s)
            v += __hip_atomic_load(p.part + ((int64_t)s * M + m_t) * p.N + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        f16 val = (f16)v;
        if (p.bias)
            val = val + p.bias[n];
        p.y[(int64_t)m_t * p.N + n] = val;
    }
}

struct W3Plan {
    int G, P, NW, RB, NS, KS, SB, BK;
    bool q8;
};

int gcd_int(int a, int b)
{
    while (b) {
        const int r = a % b;
        a = b, b = r;
    }
    return a;
}

bool make_plan(const hqq_linear *l, int64_t M, W3Plan &pl)
{
    if (l->nbits != 3 || M < 1)
        return false;
    const int64_t G = l->N / l->group_size;
    if (l->K % kSlab != 0 || G < 10 || G > (1 << 20))
        return false;
    const int64_t NW = (l->N + 9) / 10;
    if (G * l->K >= (1ll << 31) || NW * l->K * 4 >= (1ll << 32))
        return false; // 32-bit offsets inside the kernel
    const int sk = table_kind(l->scale), zk = table_kind(l->zero);
    pl.q8 = sk == TK_U8_COLS && zk == TK_U8_SCALAR;
    if (!pl.q8 && !(sk == TK_F16 && zk == TK_F16))
        return false;
    if (!aligned16(l->codes) || (reinterpret_cast<uintptr_t>(l->scale.data) & 7u) || (reinterpret_cast<uintptr_t>(l->zero.data) & 7u))
        return false;
    if (pl.q8 && (l->scale.meta_cols % 4 != 0 || (reinterpret_cast<uintptr_t>(l->scale.meta_scale) & 7u) ||
                  (reinterpret_cast<uintptr_t>(l->scale.meta_zero) & 7u)))
        return false;
    pl.G = (int)G;
    pl.P = (int)(G / gcd_int(10, (int)G));
    pl.NW = (int)NW;
    const int rows = (int)((NW + pl.P - 1) / pl.P); // word rows per window
    pl.RB = (rows + 15) / 16;
    pl.NS = (int)(l->K / kSlab);
    // blocks along K: enough that the windows cover the chip, and at most 16 slabs (8 waves x 2) per block
    int BK = (pl.NS + kW3Waves * kW3S - 1) / (kW3Waves * kW3S);
    while ((int64_t)pl.P * pl.RB * BK < 200 && BK < pl.NS)
        ++BK;
    pl.SB = (pl.NS + BK - 1) / BK;
    pl.BK = (pl.NS + pl.SB - 1) / pl.SB;
    pl.KS = (pl.SB + kW3S - 1) / kW3S;
    if (pl.P > 65535 || pl.RB > 65535 || (int64_t)pl.P * pl.RB * sizeof(int) > kCounterBytes)
        return false;
    return true;
}

} // namespace

bool vec3_supported(const hqq_linear *l, int64_t M)
{
    W3Plan pl;
    return M <= 16 && make_plan(l, M, pl);
}

size_t vec3_workspace_bytes(const hqq_linear *l, int64_t M)
{
    W3Plan pl;
    if (!make_plan(l, M, pl))
        return 0;
    return kCounterBytes + (size_t)pl.BK * 2 * (size_t)l->N * sizeof(float);
}

int launch_vec3_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s)
{
    W3Plan pl;
    if (!make_plan(l, M, pl))
        return HQQ_E_UNSUPPORTED;
    if (pl.BK > 1 && (!ws || ws_bytes < vec3_workspace_bytes(l, M)))
        return HQQ_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(x) & 7u)
        return HQQ_E_ALIGN;
    W3Params p = {};
    p.codes = static_cast<const uint8_t *>(l->codes);
    p.sq = static_cast<const uint8_t *>(l->scale.data);
    p.zq = static_cast<const uint8_t *>(l->zero.data);
    p.s_ms = static_cast<const f16 *>(l->scale.meta_scale), p.s_mz = static_cast<const f16 *>(l->scale.meta_zero);
    p.z_ms = static_cast<const f16 *>(l->zero.meta_scale), p.z_mz = static_cast<const f16 *>(l->zero.meta_zero);
    p.s_cols = (uint32_t)l->scale.meta_cols;
    p.s_inv = p.s_cols ? (uint32_t)(0xFFFFFFFFull / p.s_cols) : 0;
    p.bias = static_cast<const f16 *>(l->bias);
    p.counter = static_cast<int *>(ws);
    p.part = pl.BK > 1 ? reinterpret_cast<float *>(static_cast<char *>(ws) + kCounterBytes) : nullptr;
    p.N = (int)l->N, p.K = (int)l->K, p.G = pl.G, p.P = pl.P, p.NW = pl.NW, p.RB = pl.RB;
    p.NS = pl.NS, p.KS = pl.KS, p.SB = pl.SB, p.BK = pl.BK;
    const dim3 grid((unsigned)pl.BK, (unsigned)pl.RB, (unsigned)pl.P), block(kW3Waves * 64);
    for (int64_t m0 = 0; m0 < M; m0 += 2) { // passes of two batch rows; later passes find the weights in the caches
        const int mb = M - m0 >= 2 ? 2 : 1;
        p.x = x + m0 * l->K, p.y = y + m0 * l->N, p.M = mb;
        if (mb == 1) {
            if (pl.q8)
                gemv_w3_kernel<1, true><<<grid, block, 0, s>>>(p);
            else
                gemv_w3_kernel<1, false><<<grid, block, 0, s>>>(p);
        } else {
            if (pl.q8)
                gemv_w3_kernel<2, true><<<grid, block, 0, s>>>(p);
            else
                gemv_w3_kernel<2, false><<<grid, block, 0, s>>>(p);
        }
        int rc = launch_status();
        if (rc != HQQ_OK)
            return rc;
    }
    return HQQ_OK;
}

} // namespace hqq
