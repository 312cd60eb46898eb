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
// The waves of a block split K (one or two slabs each; with two, the second slab's loads are in flight while the
// first slab's codes are worked on); when K needs several blocks (or the window count alone would leave
// most of the chip idle) the blocks of a tile add their results into one 64-bit fixed-point accumulation slot per
// output with a returning device-scope atomic, and the block whose addition completes a slot writes that output
// (launches with more outputs than there are slots store fp32 partial sums instead, and the block that arrives
// last at the tile's counter adds them in a fixed order).  Batches above two rows run as passes of two.
//
// A launch may hold up to four layers of one shape (blockIdx.z = layer * P + window): the two projections of an
// expert's gate, or those of two experts.  Their records come from the kernel arguments or from a device table
// (record sel[layer / lper] * stride + first + layer % lper), so that the expert can be chosen on the device.
// XMODE 1 builds the activations on the fly as silu(xa) * xb, which is how the down projection reads the two
// gate outputs without an elementwise launch in between; the epilogue can multiply by a routing weight per row
// and add into y.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"

namespace hqq {
using namespace gemv;
namespace {

constexpr int kW3Waves = 8;
constexpr int kW3S = 2; // most slabs per wave

constexpr int kW3MaxLayers = 4;

struct W3Params {
    LayerRecord layer[kW3MaxLayers];
    const LayerRecord *table; // indexed launch (table != null)
    const int *sel;
    int stride, first, lper;
    const f16 *x;       // XMODE 0: (M, K)
    const f16 *xa, *xb; // XMODE 1: x = silu(xa) * xb, both (M, K); layer l reads them x_lstride elements further
    int64_t x_lstride;
    f16 *y;             // layer l writes y + l * y_lstride
    int64_t y_lstride;
    const f16 *bias;      // single layer from the kernel arguments only
    const f16 *row_scale; // optional multiplier per batch row
    int pair; // the layers of the launch are the down projections of two experts: y (+)= sum over l of
              // row_scale[l] * o_l, formed in the outputs' accumulation slots and rounded to fp16 once
    int accumulate;       // add into y
    float *part; // layer l: part + l * part_lstride, [BK][M][N]
    int64_t part_lstride;
    int *counter;
    unsigned long long *slots; // K over several blocks: one accumulation slot per output of the launch (or null)
    int M, N, K, G, P, NW, RB;
    int NS; // K / 256
    int KS; // waves of a block that have slabs
    int S;  // slabs per wave
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

// silu in fp32 with one rounding, then the fp16 product: the two roundings of the elementwise kernel
__device__ __forceinline__ f16 silu_mul(f16 a, f16 b)
{
    const float v = (float)a;
    return (f16)(v / (1.0f + __expf(-v))) * b;
}

// Q8: scale u8 + per-column meta, zero u8 + whole-tensor meta; else fp16 tables.  XMODE 1: x = silu(xa) * xb
// S: slabs per wave (1 or 2)
template <int MT, bool Q8, int XMODE, int S>
__global__ __launch_bounds__(kW3Waves * 64) void gemv_w3_kernel(W3Params p)
{
    constexpr int NT = kW3Waves * 64;
    // xs of the slab: [4-column group q][batch row][field][4 halves]
    __shared__ __attribute__((aligned(16))) f16 xs_lds[kW3Waves][64][MT][10][4];
    __shared__ float red_lds[kW3Waves][16][10][MT];
    __shared__ int ticket_lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kb = blockIdx.x, rb = blockIdx.y;
    const int layer = (int)(blockIdx.z >= (unsigned)p.P) + (int)(blockIdx.z >= 2u * p.P) + (int)(blockIdx.z >= 3u * p.P);
    const int w0 = (int)blockIdx.z - layer * p.P;
    // The layer's record.  From a table it is read one word per lane and broadcast; every load through it below is
    // an explicit device-memory load (a pointer out of a record has lost its address space).
    LayerRecord R;
    if (p.table) {
        const int e = __builtin_amdgcn_readfirstlane(p.sel[layer / p.lper]);
        const uint32_t *src = reinterpret_cast<const uint32_t *>(p.table + (e * p.stride + p.first + layer % p.lper));
        const uint32_t word = src[lane < 18 ? lane : 0];
        uint32_t rec[18];
#pragma unroll
        for (int i = 0; i < 18; ++i)
            rec[i] = __builtin_amdgcn_readlane(word, i);
        __builtin_memcpy(&R, rec, sizeof(R));
    } else {
        R = p.layer[__builtin_amdgcn_readfirstlane(layer)];
    }
    f16 *const yl = p.y + (int64_t)(p.pair ? 0 : layer) * p.y_lstride;
    float *const partl = p.part + (int64_t)layer * p.part_lstride;
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

    const int slab_lo = kb * p.SB + wave * S;
    int slab_hi = (kb + 1) * p.SB;
    if (slab_hi > p.NS)
        slab_hi = p.NS;

    // What a slab's table phase reads: tables, their per-column meta, the zero table's whole-tensor meta, x.
    struct Tab {
        uint32_t sraw[10][2], zraw[10][2];
        u32x2 msr[10], mzr[10];
        u32x2 xr[MT], xg[XMODE ? MT : 1];
        uint32_t zms_raw, zmz_raw;
    };
    // Every load of a slab is issued in the order the arithmetic needs them (loads retire in issue order): zero meta,
    // tables, x, then the codes.  Whole-tensor meta of the zero table: the address is the same in every lane but
    // written so that the compiler does not see it (lane >> 6 is zero): a load it knows to be uniform is moved to
    // scalar registers at once, which waits for it before any weight load has been issued.
    auto load_tab = [&](Tab &T, int slab) __attribute__((always_inline)) {
        const uint32_t k0 = (uint32_t)slab * kSlab;
        T.zms_raw = T.zmz_raw = 0;
        if constexpr (Q8) {
            T.zms_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_ms) + (lane >> 6));
            T.zmz_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_mz) + (lane >> 6));
        }
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            uint32_t j = j0 + (uint32_t)i; // (10*w0 + i) mod G; G >= 10
            j -= j >= (uint32_t)p.G ? (uint32_t)p.G : 0u;
            const uint32_t ce = j * (uint32_t)K + k0 + (uint32_t)(4 * lane);
            if constexpr (Q8) {
                T.sraw[i][0] = gload<uint32_t>(R.sq + ce);
                T.zraw[i][0] = gload<uint32_t>(R.zq + ce);
                uint32_t cm = ce - __umulhi(ce, R.s_inv) * R.s_cols; // ce mod cols; the quotient estimate is at most 2 short
                cm -= cm >= R.s_cols ? R.s_cols : 0;
                cm -= cm >= R.s_cols ? R.s_cols : 0;
                T.msr[i] = gload<u32x2>(R.s_ms + cm);
                T.mzr[i] = gload<u32x2>(R.s_mz + cm);
            } else {
                const u32x2 a = gload<u32x2>(reinterpret_cast<const f16 *>(R.sq) + ce);
                const u32x2 b = gload<u32x2>(reinterpret_cast<const f16 *>(R.zq) + ce);
                T.sraw[i][0] = a.x, T.sraw[i][1] = a.y, T.zraw[i][0] = b.x, T.zraw[i][1] = b.y;
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t at = (uint32_t)((m < M ? m : 0) * K) + k0 + (uint32_t)(4 * lane);
            if constexpr (XMODE) {
                T.xg[m] = gload<u32x2>(p.xa + (int64_t)layer * p.x_lstride + at);
                T.xr[m] = gload<u32x2>(p.xb + (int64_t)layer * p.x_lstride + at);
            } else {
                T.xr[m] = gload<u32x2>(p.x + at);
            }
        }
    };
    auto load_codes = [&](u32x4(&cw)[16], int slab) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < 16; ++m)
            cw[m] = gload<u32x4>(R.codes + (code_base + 4u * ((uint32_t)slab * kSlab) + (uint32_t)(64 * m)));
    };
    auto wave_sync = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // table phase: xs into LDS, zero term accumulated
    auto table_phase = [&](Tab &T) __attribute__((always_inline)) {
        if constexpr (Q8) // the meta values become opaque here, so no use of them is hoisted above the loads
            asm volatile("" : "+v"(T.zms_raw), "+v"(T.zmz_raw));
        if constexpr (XMODE) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const f16x2 a01 = as_h2(T.xg[m].x), a23 = as_h2(T.xg[m].y), b01 = as_h2(T.xr[m].x), b23 = as_h2(T.xr[m].y);
                T.xr[m].x = as_u32((f16x2){silu_mul(a01.x, b01.x), silu_mul(a01.y, b01.y)});
                T.xr[m].y = as_u32((f16x2){silu_mul(a23.x, b23.x), silu_mul(a23.y, b23.y)});
            }
        }
        const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
        const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
        const f16x2 zms = as_h2(T.zms_raw * 0x10001u), zmz = as_h2(T.zmz_raw * 0x10001u);
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            f16x2 s01, s23, z01, z23;
            if constexpr (Q8) {
                // bytes -> fp16 exactly (0x6400 | b is 1024 + b), then fp16(fp16(q - mz) * ms) as the reference does
                const f16x2 q01 = as_h2(__builtin_amdgcn_perm(0x64646464u, T.sraw[i][0], 0x04010400u)) - k1024;
                const f16x2 q23 = as_h2(__builtin_amdgcn_perm(0x64646464u, T.sraw[i][0], 0x04030402u)) - k1024;
                s01 = (q01 - as_h2(T.mzr[i].x)) * as_h2(T.msr[i].x);
                s23 = (q23 - as_h2(T.mzr[i].y)) * as_h2(T.msr[i].y);
                const f16x2 y01 = as_h2(__builtin_amdgcn_perm(0x64646464u, T.zraw[i][0], 0x04010400u)) - k1024;
                const f16x2 y23 = as_h2(__builtin_amdgcn_perm(0x64646464u, T.zraw[i][0], 0x04030402u)) - k1024;
                z01 = (y01 - zmz) * zms;
                z23 = (y23 - zmz) * zms;
            } else {
                s01 = as_h2(T.sraw[i][0]), s23 = as_h2(T.sraw[i][1]);
                z01 = as_h2(T.zraw[i][0]), z23 = as_h2(T.zraw[i][1]);
            }
            s01 = s01 * k32, s23 = s23 * k32;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const f16x2 a01 = s01 * as_h2(T.xr[m].x), a23 = s23 * as_h2(T.xr[m].y);
                zacc[i][m] = __builtin_amdgcn_fdot2(z01, a01, zacc[i][m], false);
                zacc[i][m] = __builtin_amdgcn_fdot2(z23, a23, zacc[i][m], false);
                *reinterpret_cast<f16x4 *>(&xs_lds[wave][lane][m][i][0]) = (f16x4){a01.x, a01.y, a23.x, a23.y};
            }
        }
        wave_sync();
    };
    // codes: per pair of words and field, perm + and + dot2
    auto code_phase = [&](const u32x4(&cw)[16]) __attribute__((always_inline)) {
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
        wave_sync();
    };

    if (wave < p.KS && slab_lo < slab_hi) {
        Tab T;
        u32x4 c0[16];
        load_tab(T, slab_lo);
        load_codes(c0, slab_lo);
        __builtin_amdgcn_sched_barrier(0); // nothing below moves above the loads, no load sinks into the arithmetic
        table_phase(T);
        if constexpr (S == 2 && MT == 1) {
            // The second slab's loads go out before the first slab's codes are worked on (unconditionally: a wave
            // whose second slab lies past its range re-reads the first and skips the arithmetic), its tables into
            // the registers the first slab's table phase has just released.
            const bool two = slab_lo + 1 < slab_hi;
            const int s1 = two ? slab_lo + 1 : slab_lo;
            u32x4 c1[16];
            load_tab(T, s1);
            load_codes(c1, s1);
            __builtin_amdgcn_sched_barrier(0);
            code_phase(c0);
            if (two) {
                table_phase(T);
                code_phase(c1);
            }
        } else if constexpr (S == 2) {
            // two batch rows leave no registers for a second set of codes: one slab after the other
            code_phase(c0);
            const bool two = slab_lo + 1 < slab_hi;
            const int s1 = two ? slab_lo + 1 : slab_lo;
            load_tab(T, s1);
            load_codes(c0, s1);
            __builtin_amdgcn_sched_barrier(0);
            if (two) {
                table_phase(T);
                code_phase(c0);
            }
        } else {
            code_phase(c0);
        }
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
    const int tile = (layer * p.P + w0) * p.RB + rb;
    auto finish = [&](int m_t, int64_t n, float v) {
        f16 val = (f16)v;
        if (p.bias)
            val = val + p.bias[n];
        if (p.row_scale && !p.pair)
            val = val * p.row_scale[m_t];
        f16 *dst = yl + (int64_t)m_t * p.N + n;
        *dst = p.accumulate ? (f16)(*dst + val) : val;
    };
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
            finish(m_t, n, v);
        } else if (p.slots) {
            // the K blocks add into the output's slot; the block whose addition completes it writes the output
            // (a pair of experts shares the slots: every block's result enters with its expert's routing weight)
            const int arrivals = p.pair ? 2 * p.BK : p.BK;
            unsigned long long *slot = p.slots + (((int64_t)(p.pair ? 0 : layer) * p.N + n) * MT + m_t);
            const unsigned long long mine = slot_term(p.pair ? v * (float)p.row_scale[layer] : v);
            const unsigned long long before = __hip_atomic_fetch_add(slot, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (slot_count(before) == arrivals - 1) {
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                finish(m_t, n, slot_total(before + mine, arrivals));
            }
        } else {
            __hip_atomic_store(partl + ((int64_t)kb * M + m_t) * p.N + n, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (alone || p.slots)
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
            v += __hip_atomic_load(partl + ((int64_t)s * M + m_t) * p.N + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        finish(m_t, n, v);
    }
}

struct W3Plan {
    int G, P, NW, RB, NS, KS, S, SB, BK;
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

// NL: layers of the launch (they share the plan)
bool make_plan(const hqq_linear *l, int64_t M, int NL, W3Plan &pl)
{
    if (l->nbits != 3 || M < 1 || NL < 1 || NL > kW3MaxLayers)
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
    while ((int64_t)pl.P * pl.RB * NL * BK < 200 && BK < pl.NS)
        ++BK;
    const bool tune = tuning_int("HQQ_W3_K", (int)l->K) == (int)l->K;
    if (tune)
        BK = tuning_int("HQQ_W3_BK", BK);
    if (BK < 1 || BK > pl.NS || (pl.NS + BK - 1) / BK > kW3Waves * kW3S)
        return false;
    pl.SB = (pl.NS + BK - 1) / BK;
    pl.BK = (pl.NS + pl.SB - 1) / pl.SB;
    pl.S = pl.SB > kW3Waves ? kW3S : 1;
    if (tune)
        pl.S = tuning_int("HQQ_W3_S", pl.S) == 2 ? 2 : pl.S;
    pl.KS = (pl.SB + pl.S - 1) / pl.S;
    if ((int64_t)pl.P * NL > 65535 || pl.RB > 65535 || (int64_t)pl.P * pl.RB * NL * sizeof(int) > kTileCounterBytes)
        return false;
    return true;
}

// Layers that may share a launch: same shape, grouping and table layout (the records carry the pointers only).
bool same_layout(const hqq_linear *a, const hqq_linear *b)
{
    return a->nbits == b->nbits && a->group_size == b->group_size && a->N == b->N && a->K == b->K &&
           table_kind(a->scale) == table_kind(b->scale) && table_kind(a->zero) == table_kind(b->zero) &&
           a->scale.meta_cols == b->scale.meta_cols;
}

struct W3Job {
    const hqq_linear *layers[kW3MaxLayers]; // NL descriptors; with a table only layers[0] is read, for the shape
    int NL;
    const StripIndex *ix; // records from a device table: layer l is record sel[l / lper] * stride + first + l % lper
    int lper;
    const f16 *x, *xa, *xb; // x, or xa and xb (x = silu(xa) * xb)
    int64_t x_lstride;      // xa, xb of layer l (paired down projections)
    int pair;
    f16 *y;
    int64_t y_lstride;
    SmallBatchEpilogue ep;
};

template <int MT, bool Q8, int S> void launch_slabs(const W3Params &p, bool fused, dim3 grid, hipStream_t s)
{
    if (fused)
        gemv_w3_kernel<MT, Q8, 1, S><<<grid, dim3(kW3Waves * 64), 0, s>>>(p);
    else
        gemv_w3_kernel<MT, Q8, 0, S><<<grid, dim3(kW3Waves * 64), 0, s>>>(p);
}

template <int MT, bool Q8> void launch_xmode(const W3Params &p, bool fused, dim3 grid, hipStream_t s)
{
    if (p.S == 2)
        launch_slabs<MT, Q8, 2>(p, fused, grid, s);
    else
        launch_slabs<MT, Q8, 1>(p, fused, grid, s);
}

size_t job_workspace_bytes(const W3Plan &pl, const hqq_linear *l, int NL)
{
    return kHeadBytes + (pl.BK > 1 ? (size_t)NL * pl.BK * 2 * (size_t)l->N * sizeof(float) : 0);
}

int run_job(const W3Job &j, int64_t M, void *ws, size_t ws_bytes, hipStream_t s)
{
    const hqq_linear *l = j.layers[0];
    W3Plan pl;
    if (!make_plan(l, M, j.NL, pl))
        return HQQ_E_UNSUPPORTED;
    const bool fused = j.xa != nullptr;
    if (!j.ix) {
        for (int i = 1; i < j.NL; ++i) {
            W3Plan other;
            if (!same_layout(l, j.layers[i]) || !make_plan(j.layers[i], M, j.NL, other))
                return HQQ_E_UNSUPPORTED;
        }
    }
    for (int i = 0; i < (j.ix ? 1 : j.NL); ++i)
        if (j.layers[i]->bias && (j.NL > 1 || j.ix))
            return HQQ_E_UNSUPPORTED; // the bias is not part of a record
    if (pl.BK > 1 && (!ws || ws_bytes < job_workspace_bytes(pl, l, j.NL)))
        return HQQ_E_WORKSPACE;
    if (fused ? ((reinterpret_cast<uintptr_t>(j.xa) | reinterpret_cast<uintptr_t>(j.xb)) & 7u) != 0
              : (reinterpret_cast<uintptr_t>(j.x) & 7u) != 0)
        return HQQ_E_ALIGN;
    W3Params p = {};
    if (j.ix) {
        p.table = static_cast<const LayerRecord *>(j.ix->table);
        p.sel = j.ix->sel;
        p.stride = j.ix->stride, p.first = j.ix->first;
    } else {
        for (int i = 0; i < j.NL; ++i)
            fill_layer_record(p.layer[i], j.layers[i]);
        p.bias = static_cast<const f16 *>(l->bias);
    }
    p.lper = j.lper > 0 ? j.lper : 1;
    p.counter = static_cast<int *>(ws);
    p.part = pl.BK > 1 ? reinterpret_cast<float *>(static_cast<char *>(ws) + kHeadBytes) : nullptr;
    if (pl.BK > 1 && pl.BK * (j.pair ? 2 : 1) <= 14 &&
        (size_t)(j.pair ? 1 : j.NL) * (size_t)l->N * 2 * sizeof(unsigned long long) <= kSlotBytes)
        p.slots = reinterpret_cast<unsigned long long *>(static_cast<char *>(ws) + kCounterBytes);
    if (j.pair && (!p.slots || M != 1 || j.NL != 2 || !fused || !j.ep.row_scale))
        return HQQ_E_UNSUPPORTED; // the shared slots are what joins the two experts
    p.pair = j.pair, p.x_lstride = j.x_lstride;
    p.part_lstride = (int64_t)pl.BK * 2 * l->N;
    p.y_lstride = j.y_lstride;
    p.accumulate = j.ep.accumulate;
    p.N = (int)l->N, p.K = (int)l->K, p.G = pl.G, p.P = pl.P, p.NW = pl.NW, p.RB = pl.RB;
    p.NS = pl.NS, p.KS = pl.KS, p.S = pl.S, p.SB = pl.SB, p.BK = pl.BK;
    const dim3 grid((unsigned)pl.BK, (unsigned)pl.RB, (unsigned)(pl.P * j.NL));
    for (int64_t m0 = 0; m0 < M; m0 += 2) { // passes of two batch rows; later passes find the weights in the caches
        const int mb = M - m0 >= 2 ? 2 : 1;
        if (fused)
            p.xa = j.xa + m0 * l->K, p.xb = j.xb + m0 * l->K;
        else
            p.x = j.x + m0 * l->K;
        p.y = j.y + m0 * l->N, p.M = mb;
        p.row_scale = j.ep.row_scale ? j.ep.row_scale + m0 : nullptr;
        if (mb == 1) {
            if (pl.q8)
                launch_xmode<1, true>(p, fused, grid, s);
            else
                launch_xmode<1, false>(p, fused, grid, s);
        } else {
            if (pl.q8)
                launch_xmode<2, true>(p, fused, grid, s);
            else
                launch_xmode<2, false>(p, fused, grid, s);
        }
        int rc = launch_status();
        if (rc != HQQ_OK)
            return rc;
    }
    return HQQ_OK;
}

} // namespace

bool vec3_supported(const hqq_linear *l, int64_t M)
{
    W3Plan pl;
    return M <= 16 && make_plan(l, M, 1, pl);
}

size_t vec3_workspace_bytes(const hqq_linear *l, int64_t M)
{
    W3Plan pl;
    if (!make_plan(l, M, 1, pl))
        return 0;
    return job_workspace_bytes(pl, l, 1);
}

int launch_vec3_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s)
{
    W3Job j = {};
    j.layers[0] = l, j.NL = 1, j.x = x, j.y = y;
    return run_job(j, M, ws, ws_bytes, s);
}

// The expert FFN of 3-bit layers in two launches: both gate projections (of one expert, or of the experts sel[0] and
// sel[1] of a record table), then the down projection reading silu(a) * b.
bool vec3_ffn_supported(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, int64_t M, int n_experts)
{
    W3Plan pl;
    return M >= 1 && M <= 16 && same_layout(w1, w3) && !w1->bias && !w3->bias && make_plan(w1, M, 2 * n_experts, pl) &&
           make_plan(w3, M, 2 * n_experts, pl) && make_plan(w2, M, 1, pl) && w2->K == w1->N && w2->N == w1->K;
}

size_t vec3_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, int64_t M, int n_experts)
{
    W3Plan a, b;
    if (!make_plan(w1, M, 2 * n_experts, a) || !make_plan(w2, M, 1, b))
        return 0;
    size_t need = job_workspace_bytes(a, w1, 2 * n_experts);
    const size_t gb = job_workspace_bytes(b, w2, 1);
    need = gb > need ? gb : need;
    W3Plan c;
    if (n_experts == 2 && make_plan(w2, M, 2, c)) { // both down projections in one launch
        const size_t gc = job_workspace_bytes(c, w2, 2);
        need = gc > need ? gc : need;
    }
    return need;
}

bool vec3_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    W3Plan pl;
    return M >= 1 && M <= 16 && same_layout(w1, w3) && !w1->bias && !w3->bias && make_plan(w1, M, 2, pl) &&
           make_plan(w3, M, 2, pl);
}

size_t vec3_gate_workspace_bytes(const hqq_linear *w1, int64_t M)
{
    W3Plan pl;
    return make_plan(w1, M, 2, pl) ? job_workspace_bytes(pl, w1, 2) : 0;
}

// ab: the gate outputs, layer l (w1 then w3 of each expert) at ab + l * ab_lstride, each (M, N)
int launch_vec3_gate(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *ab, int64_t ab_lstride,
                     int n_experts, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex *ix)
{
    if (n_experts < 1 || n_experts > 2 || (n_experts == 2 && !ix) || ab_lstride < M * w1->N)
        return HQQ_E_UNSUPPORTED;
    W3Job j = {};
    j.layers[0] = w1, j.layers[1] = w3, j.layers[2] = w1, j.layers[3] = w3;
    j.NL = 2 * n_experts, j.ix = ix, j.lper = 2;
    j.x = x, j.y = ab, j.y_lstride = ab_lstride;
    return run_job(j, M, ws, ws_bytes, s);
}

int launch_vec3_down(const hqq_linear *w2, const f16 *a, const f16 *b, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                     const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix)
{
    W3Job j = {};
    j.layers[0] = w2, j.NL = 1, j.ix = ix, j.lper = 1;
    j.xa = a, j.xb = b, j.y = y, j.ep = ep;
    return run_job(j, M, ws, ws_bytes, s);
}

// Both down projections of a token's two experts (records sel[0] and sel[1]) in one launch:
// y (+)= rw[0] * w2_0(silu(a0) * b0) + rw[1] * w2_1(silu(a1) * b1), expert e reading a, b at ab + 2 * e * ab_lstride
// and ab + (2 * e + 1) * ab_lstride.  HQQ_E_UNSUPPORTED when K fits one block (the caller makes two launches).
int launch_vec3_down_pair(const hqq_linear *w2, const f16 *ab, int64_t ab_lstride, f16 *y, const f16 *row_scale,
                          int accumulate, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix)
{
    W3Job j = {};
    j.layers[0] = w2, j.layers[1] = w2, j.NL = 2, j.ix = &ix, j.lper = 1, j.pair = 1;
    j.xa = ab, j.xb = ab + ab_lstride, j.x_lstride = 2 * ab_lstride, j.y = y;
    j.ep.row_scale = row_scale, j.ep.accumulate = accumulate;
    return run_job(j, 1, ws, ws_bytes, s);
}

} // namespace hqq
