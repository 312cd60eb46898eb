// Decode-time GEMV for 3-bit codes, ten per int32 word (reference src/packing.py:62-81: code i of a word at bit
// 3*(9-i); kernel src/triton_kernels.py:414-509).
//
// A word row w holds output rows n = 10w .. 10w+9, which use table rows j = (10w + i) mod G.  Word rows P apart,
// P = G / gcd(10, G), use the SAME ten table rows (10P is a multiple of G), so a tile is the word rows
// w0 + P*t, t = 0..15, of one window w0: they share ten scale rows and ten zero rows, and as in the 2- and 4-bit
// kernels the scale is folded into the activations once per tile,
//     y[10w+i, m] = sum_k q_i[w, k] * xs[i, k, m]  -  sum_k z[i, k] * xs[i, k, m],     xs = 32 * s[i, k] * x[m, k]  (fp16).
//
// A wave takes one slab of 256 columns of a tile at a time.
//
// One batch row (the decode step): the codes go to the matrix cores.  A word's ten fields are five sets of two, one
// field in each 16-bit half of an operand register: two sets are plain masks of the word, the other three masks of
// two byte gathers that move the fields straddling a 16-bit boundary into the low ten bits of a half (seven vector
// instructions per word instead of thirty).  A field masked in place is the fp16 subnormal q * 2^(offset - 24), which
// v_mfma_f32_16x16x32_f16 multiplies exactly.  The sixteen tile rows of the instruction are eight word rows times two
// column phases: lane (word row, phase, k group) reads 16 bytes at column 32 * step + 8 * group + 4 * phase, so the
// two lanes of a word row read 32 consecutive bytes; the sixteen columns are phase x half x set, the B operand of a
// column holding xs of its own field in its own half (zeros in the other) at the columns of its own phase, and the
// result is kept where the phases agree.  The fifth set has a B operand of its own.  The table phase works in three
// rounds, a lane owning sixteen columns of one table row (coalesced 16-byte table reads), and leaves xs in LDS in
// the order the B lanes read it; the zero term is a dot product per table row (8-bit tables: of the raw bytes as
// subnormals and of xs, the zero table's own scale and zero applied to the sums).  The codes of the slab's second
// half are requested after the table phase, see there.
//
// Two to eight batch rows: the same layout with the batch rows in the instruction's columns, column = phase + 2 *
// half + 4 * (batch row within its group of four), one or two such groups.  Every set of fields then has a B operand
// of its own per group: 32 * s of the lane's field from LDS times the lane's own x[m, k] read straight from memory,
// placed in the lane's half.  The zero term is two more matrix instructions per step and group, 32 * s * z of the
// ten table rows (from LDS) against x.  One pass over the words serves all rows; the accumulators of eight rows fill
// the register file, so a wave of such a pass takes a single slab.  Wider batches run as passes of eight.
//
// The waves of a block split K (one or two slabs each; with one batch row the second slab's loads are in flight
// while the first slab's codes are worked on); when K needs several blocks (or the window count alone would leave
// most of the chip idle) the blocks of a tile add their results into one 64-bit fixed-point accumulation slot per
// output with a returning device-scope atomic, and the block whose addition completes a slot writes that output
// (launches with more outputs than there are slots: with two blocks along K the two swap their sums through a 32-bit
// word per output in the same memory; else they store fp32 partial sums, and the block that arrives last at the
// tile's counter adds them in a fixed order).
//
// A launch may hold up to four layers of one shape (a one-dimensional grid over layer, window, row block and K
// block, see the kernel): the two projections of an
// expert's gate, or those of two experts.  Their records come from the kernel arguments or from a device table
// (record sel[layer / lper] * stride + first + layer % lper), so that the expert can be chosen on the device.
// XMODE 1 (one batch row) builds the activations on the fly as silu(xa) * xb, which is how the down projection reads
// the two gate outputs without an elementwise launch in between; the epilogue can multiply by a routing weight per
// row and add into y.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"
#include <type_traits>

namespace hqq {
using namespace gemv;
namespace {

constexpr int kW3Waves = 8;
constexpr int kW3S = 2; // most slabs per wave

constexpr int kW3MaxLayers = 4;
#ifndef HQQ_W3_EARLY
#define HQQ_W3_EARLY 4
#endif
constexpr int kW3Early = HQQ_W3_EARLY; // single rows: 32-column steps of a slab whose codes are requested before the table phase

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
    uint32_t *words;           // K over exactly two blocks: one exchange word per output instead (or null)
    int M, N, K, G, P, NW, RB;
    int NS; // K / 256
    int KS; // waves of a block that have slabs
    int S;  // slabs per wave
    int SB; // slabs per block
    int BK; // blocks along K per tile
    int meta4; // the scale table's meta columns are a multiple of 4 but not of 16
    // the work list (see the kernel): blocks per XCD, XCDs with one more, magic multipliers ceil(2^32 / d) of the
    // divisions, and the window of list position n: (n * win_mul) mod P
    uint32_t per_xcd, xcd_more, bk_magic, rb_magic, p_magic, win_mul;
#ifdef HQQ_TUNING_BUILD
    int plain_order; // timing experiments: blocks take the work list in launch order
    int skip; // timing experiments: 1 leaves out the code phase, 2 the table phase (their loads are still waited for)
    unsigned long long *stamps; // per-wave time stamps, [block][16 waves][16], or null
#endif
};
#ifdef HQQ_TUNING_BUILD
#define HQQ_W3_SKIP(p, bit) (((p).skip & (bit)) != 0)
#define W3_STAMP(i) do { if (p.stamps) st[i] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define HQQ_W3_SKIP(p, bit) false
#define W3_STAMP(i)
#endif

// Field i of a word lies at bit 3 * (9 - i).
// One batch row: a word's ten fields go to the matrix cores as five sets of two, one field in each 16-bit half of an
// operand register (so a register is one column, and the B operand keeps the halves apart with zeros).  Sets 0 and 1
// are the word itself; the others are two byte gathers, which put the fields that straddle a 16-bit boundary into
// the low ten bits of a half:
//   set 0: field 9 (offset 0) | field 3 (offset 2)      the word, halves at bits 0 and 16
//   set 1: field 8 (offset 3) | field 2 (offset 5)
//   set 2: field 7 (offset 6) | field 4 (offset 7)      gather B: bytes (0,1) | (1,2)
//   set 3: field 6 (offset 1) | field 1 (offset 0)      gather A: bytes (1,2) | (3,zero)
//   set 4: field 5 (offset 4) | field 0 (offset 3)
constexpr uint32_t kW3GatherA = 0x0c030201u, kW3GatherB = 0x02010100u;
__host__ __device__ constexpr int w3_set_offset(int set, int half)
{
    return half ? (set == 0 ? 2 : set == 1 ? 5 : set == 2 ? 7 : set == 3 ? 0 : 3)
                : (set == 0 ? 0 : set == 1 ? 3 : set == 2 ? 6 : set == 3 ? 1 : 4);
}
__host__ __device__ constexpr uint32_t w3_set_mask(int set)
{
    return (7u << w3_set_offset(set, 0)) | (7u << (16 + w3_set_offset(set, 1)));
}
__device__ __forceinline__ int w3_set_field(int set, int half)
{
    return half ? (0x01423 >> (4 * set)) & 15 : 9 - set;
}
// a field masked at offset o of a half is the fp16 subnormal q * 2^(o - 24)
__device__ __forceinline__ float w3_set_unscale(int set, int half)
{
    const int o = half ? (0x30752 >> (4 * set)) & 15 : (0x41630 >> (4 * set)) & 15;
    return __builtin_bit_cast(float, (uint32_t)(127 + 24 - 5 - o) << 23); // 2^(24 - o) / 32
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
#ifdef HQQ_TUNING_BUILD
    unsigned long long st[16] = {};
#endif
    W3_STAMP(0);
#ifdef HQQ_TUNING_BUILD
    if (p.stamps)
        st[9] = __builtin_readcyclecounter();
#endif
    // xs of each wave's slab: [32-column step][4-column piece][table row][4 halves].  (A batch: 32 * s in that layout,
    // 32 * s * z beside it, and a wave's results in the place of its own tables once it has read them for the last
    // time.)
    static_assert(MT == 1 || MT == 4 || MT == 8, "one row, or one or two column groups of four rows");
    constexpr bool kBatch = MT >= 4;
    __shared__ __attribute__((aligned(16))) f16 xs_raw[kW3Waves * 64 * 10 * 4];
    __shared__ __attribute__((aligned(16))) f16 zs_raw[kBatch ? kW3Waves * 64 * 10 * 4 : 8];
    __shared__ __attribute__((aligned(16))) f16 h_lds[XMODE ? kW3Waves : 1][kSlab]; // silu(xa) * xb of the slab
    __shared__ float zt_lds[kW3Waves][10][kBatch ? MT : 1];
    __shared__ float red_raw[kBatch ? 1 : kW3Waves * 16 * 10 * MT];
    // the results of wave w: [word row 16][field 10][batch row MT]; a batch wave puts them where its own tables were
    constexpr int kRedStride = kBatch ? 64 * 10 * 4 / 2 : 16 * 10 * MT; // floats
    static_assert(kRedStride >= 16 * 10 * MT, "the results fit where the tables were");
    float *const red_base = kBatch ? reinterpret_cast<float *>(xs_raw) : red_raw;
    auto red_lds = [&](int w) __attribute__((always_inline)) { return reinterpret_cast<float(*)[10][MT]>(red_base + w * kRedStride); };
    __shared__ int ticket_lds;

    // Every kernel argument the prologue reads is fetched here, in one batch: read where they are used, they come in
    // five or six scalar loads one after the other, each waiting for the branch before it.
    asm volatile("" ::"s"(p.table), "s"(p.sel), "s"(p.stride), "s"(p.first), "s"(p.lper), "s"(p.x), "s"(p.xa), "s"(p.xb),
                 "s"(p.x_lstride), "s"(p.P), "s"(p.G), "s"(p.K), "s"(p.NW), "s"(p.KS), "s"(p.SB), "s"(p.NS), "s"(p.pair),
                 "s"(p.y), "s"(p.y_lstride), "s"(p.part), "s"(p.part_lstride));
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Which tile this block works on.  Consecutive blocks of a launch go to the eight XCDs in turn, each with an L2 of
    // its own, and a table row is needed by several windows (ten rows per window, G / gcd(10, G) windows): block b is
    // the (b / 8)-th block of XCD b % 8, every XCD takes a contiguous range of the work list, and the list runs over
    // the windows in the order of their first table row, so that windows which share table rows meet in one L2.
    uint32_t v;
    {
        const uint32_t xcd = blockIdx.x & 7u, nth = blockIdx.x >> 3;
        v = xcd * p.per_xcd + (xcd < p.xcd_more ? xcd : p.xcd_more) + nth;
#ifdef HQQ_TUNING_BUILD
        if (p.plain_order)
            v = blockIdx.x;
#endif
    }
    auto div = [](uint32_t a, uint32_t d, uint32_t magic) { return d == 1 ? a : __umulhi(a, magic); }; // a * d < 2^32
    const uint32_t v1 = div(v, (uint32_t)p.BK, p.bk_magic), v2 = div(v1, (uint32_t)p.RB, p.rb_magic);
    const int kb = (int)(v - v1 * (uint32_t)p.BK), rb = (int)(v1 - v2 * (uint32_t)p.RB);
    const int layer = (int)div(v2, (uint32_t)p.P, p.p_magic);
    const uint32_t nthw = v2 - (uint32_t)layer * (uint32_t)p.P, step = nthw * p.win_mul; // below 2^20 each way
    const int w0 = (int)(step - div(step, (uint32_t)p.P, p.p_magic) * (uint32_t)p.P);
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
        asm volatile("" ::"s"(R.codes), "s"(R.sq), "s"(R.zq), "s"(R.s_ms), "s"(R.s_mz), "s"(R.z_ms), "s"(R.z_mz), "s"(R.s_cols),
                     "s"(R.s_inv)); // the whole record in one batch as well
    }
    f16 *const yl = p.y + (int64_t)(p.pair ? 0 : layer) * p.y_lstride;
    float *const partl = p.part + (int64_t)layer * p.part_lstride;
    const int M = MT == 1 ? 1 : p.M;
    const int K = p.K;
    const uint32_t j0 = (uint32_t)(10 * w0) % (uint32_t)p.G;

    const int slab_lo = kb * p.SB + wave * S;
    int slab_hi = (kb + 1) * p.SB;
    if (slab_hi > p.NS)
        slab_hi = p.NS;
    auto wave_sync = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    if constexpr (MT == 1) {
        // ------------------------------------------------------------ one batch row: the codes on the matrix cores
        constexpr int SK = Q8 ? TK_U8_COLS : TK_F16, ZK = Q8 ? TK_U8_SCALAR : TK_F16;
        f16 *const xs_w = xs_raw + wave * (16 * 4 * 10 * 4); // [step][piece][table row][4 halves]
        // code role: tile row lane & 15 = 2 * (word row within its group of eight) + phase, k group lane >> 4; the
        // tile's sixteen word rows are two such groups
        const int rho = (lane & 15) >> 1, phi = lane & 1, gk = lane >> 4;
        uint32_t code_at[2];
#pragma unroll
        for (int g8 = 0; g8 < 2; ++g8) {
            const int wr = w0 + p.P * (16 * rb + 8 * g8 + rho);
            code_at[g8] = (uint32_t)(wr < p.NW ? wr : w0) * (uint32_t)K * 4u + (uint32_t)(32 * gk + 16 * phi);
        }
        // column role: column lane & 15 = phase + 2 * half + 4 * set for the sets 0..3; the fifth set has a B operand
        // of its own, of which the columns 0..3 are kept
        const int set = (lane & 15) >> 2, half = (lane >> 1) & 1;
        const int fcol = w3_set_field(set, half), fcol4 = w3_set_field(4, half);
        const uint32_t b_at = (uint32_t)(((2 * gk + phi) * 10 + fcol) * 8), b4_at = (uint32_t)(((2 * gk + phi) * 10 + fcol4) * 8);
        const uint32_t sel_a = half ? 0x01000c0cu : 0x0c0c0100u, sel_b = half ? 0x03020c0cu : 0x0c0c0302u;
        // table role: round r, lane (row = lane >> 4, chunk = lane & 15); the third round has two rows only
        const int qT = lane & 15;
        const bool third_ok = lane < 32;
        uint32_t trow_at[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const int f = r < 2 ? 4 * r + (lane >> 4) : 8 + ((lane >> 4) & 1);
            uint32_t j = j0 + (uint32_t)f; // (10*w0 + f) mod G; G >= 10
            j -= j >= (uint32_t)p.G ? (uint32_t)p.G : 0u;
            trow_at[r] = j * (uint32_t)K + (uint32_t)(16 * qT);
        }

        f32x4 acc[2][5];
#pragma unroll
        for (int g8 = 0; g8 < 2; ++g8)
#pragma unroll
            for (int i = 0; i < 5; ++i)
                acc[g8][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (lane < 10)
            zt_lds[wave][lane][0] = 0.f;
        // the masks in scalar registers: as literals they double the size of the instructions that use them
        uint32_t mk[5] = {w3_set_mask(0), w3_set_mask(1), w3_set_mask(2), w3_set_mask(3), w3_set_mask(4)};
        asm volatile("" : "+s"(mk[0]), "+s"(mk[1]), "+s"(mk[2]), "+s"(mk[3]), "+s"(mk[4]));

        // What a slab has in flight or in registers.
        struct Slab {
            uint32_t k0;
            uint32_t zms_raw, zmz_raw;
            Raw16<SK> rs[3];
            Raw16<ZK> rz[3];
            u32x4 xr[2];
            u32x2 xg, xh;
            u32x4 cw[8][2]; // a step is 32 columns: four words of both row groups
        };
        // The loads of a slab's tables, activations and first code steps, in the order the arithmetic needs them.  The
        // whole-tensor meta of the zero table has the same address in every lane, written so that the compiler does not
        // see it (lane >> 6 is zero): a load it knows to be uniform moves to scalar registers and is waited for at once.
        auto issue_first = [&](Slab &L, int slab) __attribute__((always_inline)) {
            const uint32_t k0 = L.k0 = (uint32_t)slab * kSlab;
            L.zms_raw = L.zmz_raw = 0;
            if constexpr (Q8) {
                L.zms_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_ms) + (lane >> 6));
                L.zmz_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_mz) + (lane >> 6));
            }
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const uint32_t ce = trow_at[r] + k0;
                uint32_t cm = 0;
                if constexpr (Q8) {
                    cm = ce - __umulhi(ce, R.s_inv) * R.s_cols; // ce mod cols; the quotient estimate is at most 2 short
                    cm -= cm >= R.s_cols ? R.s_cols : 0;
                    cm -= cm >= R.s_cols ? R.s_cols : 0;
                }
                if (Q8 && p.meta4) {
                    // the meta columns are a multiple of 4 only: the lane's sixteen entries may wrap inside, four
                    // pieces each with its own column
                    L.rs[r].q = gload<u32x4>(R.sq + ce);
#pragma unroll
                    for (int pc = 0; pc < 4; ++pc) {
                        uint32_t c4 = cm + 4u * pc;
                        c4 -= c4 >= R.s_cols ? R.s_cols : 0;
                        const u32x2 a = gload<u32x2>(R.s_ms + c4), b = gload<u32x2>(R.s_mz + c4);
                        L.rs[r].ms[pc >> 1][2 * (pc & 1)] = a.x, L.rs[r].ms[pc >> 1][2 * (pc & 1) + 1] = a.y;
                        L.rs[r].mz[pc >> 1][2 * (pc & 1)] = b.x, L.rs[r].mz[pc >> 1][2 * (pc & 1) + 1] = b.y;
                    }
                } else {
                    load16<SK>(L.rs[r], R.sq, R.s_ms, R.s_mz, ce, cm);
                }
                load16<ZK>(L.rz[r], R.zq, nullptr, nullptr, ce, 0);
            }
            L.xg = L.xh = (u32x2){0, 0};
            if constexpr (XMODE) {
                L.xg = gload<u32x2>(p.xa + (int64_t)layer * p.x_lstride + k0 + (uint32_t)(4 * lane));
                L.xh = gload<u32x2>(p.xb + (int64_t)layer * p.x_lstride + k0 + (uint32_t)(4 * lane));
            } else {
                L.xr[0] = gload<u32x4>(p.x + k0 + (uint32_t)(16 * qT));
                L.xr[1] = gload<u32x4>(p.x + k0 + (uint32_t)(16 * qT + 8));
            }
#pragma unroll
            for (int s = 0; s < kW3Early; ++s)
#pragma unroll
                for (int g8 = 0; g8 < 2; ++g8)
                    L.cw[s][g8] = gload<u32x4>(R.codes + (code_at[g8] + 4u * k0 + (uint32_t)(128 * s)));
            __builtin_amdgcn_sched_barrier(0); // nothing below moves above the loads, no load sinks into the arithmetic
        };
        // The codes of the slab's second half are requested after the table phase: a wave that has issued its loads
        // waits there, which lets the other wave of the SIMD issue its own (the older wave is served first), so that
        // both have the first half of their data early and neither is left with a whole slab of arithmetic after the
        // last byte has arrived.
        auto issue_second = [&](Slab &L) __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = kW3Early; s < 8; ++s)
#pragma unroll
                for (int g8 = 0; g8 < 2; ++g8)
                    L.cw[s][g8] = gload<u32x4>(R.codes + (code_at[g8] + 4u * L.k0 + (uint32_t)(128 * s)));
            __builtin_amdgcn_sched_barrier(0);
        };
        // table phase: xs = 32 * s * x of the ten table rows into LDS, and the zero terms
        auto table_phase = [&](Slab &L) __attribute__((always_inline)) {
            if constexpr (Q8) // the meta values become opaque here, so no use of them is hoisted above the loads
                asm volatile("" : "+v"(L.zms_raw), "+v"(L.zmz_raw));
            if constexpr (XMODE) {
                const f16x2 a01 = as_h2(L.xg.x), a23 = as_h2(L.xg.y), b01 = as_h2(L.xh.x), b23 = as_h2(L.xh.y);
                u32x2 hv;
                hv.x = as_u32((f16x2){silu_mul(a01.x, b01.x), silu_mul(a01.y, b01.y)});
                hv.y = as_u32((f16x2){silu_mul(a23.x, b23.x), silu_mul(a23.y, b23.y)});
                *reinterpret_cast<u32x2 *>(&h_lds[wave][4 * lane]) = hv;
                wave_sync();
                L.xr[0] = *reinterpret_cast<const u32x4 *>(&h_lds[wave][16 * qT]);
                L.xr[1] = *reinterpret_cast<const u32x4 *>(&h_lds[wave][16 * qT + 8]);
            }
            const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
            const f16x2 ones = {(f16)1.0f, (f16)1.0f};
            // the zero term of the lane's table row and columns: fp16 tables sum z * xs; 8-bit tables sum zq * xs (the
            // bytes as fp16 subnormals, zq * 2^-24) and xs, and z = (zq - mz) * ms is applied to the sums
            float zacc[3] = {0.f, 0.f, 0.f}, zxs[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                if (HQQ_W3_SKIP(p, 2)) {
                    asm volatile("" ::"v"(L.rs[r].q), "v"(L.rs[r].q_hi), "v"(L.rs[r].ms[0]), "v"(L.rs[r].ms[1]), "v"(L.rs[r].mz[0]),
                                 "v"(L.rs[r].mz[1]), "v"(L.rz[r].q), "v"(L.rz[r].q_hi), "v"(L.xr[0]), "v"(L.xr[1]));
                    continue;
                }
                const int f = r < 2 ? 4 * r + (lane >> 4) : 8 + ((lane >> 4) & 1);
                f16x2 sv[8], zv[8];
                decode16<SK>(L.rs[r], k32, k32, sv);
                if constexpr (!Q8)
                    decode16<ZK>(L.rz[r], k32, k32, zv);
                uint32_t a[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const f16x2 v = (sv[t] * k32) * as_h2(L.xr[t >> 2][t & 3]);
                    if constexpr (Q8) {
                        // bytes 2 * (t & 1), 2 * (t & 1) + 1 of the word into the low bytes of the two halves
                        const uint32_t zq = __builtin_amdgcn_perm(0u, L.rz[r].q[t >> 1], (t & 1) ? 0x0c030c02u : 0x0c010c00u);
                        zacc[r] = __builtin_amdgcn_fdot2(as_h2(zq), v, zacc[r], false);
                        zxs[r] = __builtin_amdgcn_fdot2(ones, v, zxs[r], false);
                    } else {
                        zacc[r] = __builtin_amdgcn_fdot2(zv[t], v, zacc[r], false);
                    }
                    a[t] = as_u32(v);
                }
                if (r < 2 || third_ok) {
#pragma unroll
                    for (int pi = 0; pi < 4; ++pi)
                        *reinterpret_cast<u32x2 *>(xs_w + ((qT * 4 + pi) * 10 + f) * 4) = (u32x2){a[2 * pi], a[2 * pi + 1]};
                }
            }
            // the zero terms of the slab: summed over the sixteen chunk lanes of a table row and added up in LDS, here
            // rather than after the last code step, where every instruction delays the block's result
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const int f = r < 2 ? 4 * r + (lane >> 4) : 8 + ((lane >> 4) & 1);
                float z = zacc[r];
                if constexpr (Q8) {
                    const float ms = (float)__builtin_bit_cast(f16, (uint16_t)L.zms_raw), mz = (float)__builtin_bit_cast(f16, (uint16_t)L.zmz_raw);
                    z = ms * (z * 16777216.0f - mz * zxs[r]);
                }
                z = row16_sum(z);
                if (qT == 0 && (r < 2 || third_ok))
                    zt_lds[wave][f][0] += z;
            }
            wave_sync();
        };
        // code phase: per word two plain masks and two byte gathers with three masks.  The B operands of a step are read
        // from LDS a step ahead.
        auto code_phase = [&](const Slab &L) __attribute__((always_inline)) {
            auto read_b = [&](u32x2 &bx, u32x2 &by, int s) __attribute__((always_inline)) {
                bx = *reinterpret_cast<const u32x2 *>(reinterpret_cast<const char *>(xs_w) + b_at + s * 640);
                by = *reinterpret_cast<const u32x2 *>(reinterpret_cast<const char *>(xs_w) + b4_at + s * 640);
            };
            u32x2 bx, by;
            read_b(bx, by, 0);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const u32x4 bu = {__builtin_amdgcn_perm(0u, bx.x, sel_a), __builtin_amdgcn_perm(0u, bx.x, sel_b),
                                  __builtin_amdgcn_perm(0u, bx.y, sel_a), __builtin_amdgcn_perm(0u, bx.y, sel_b)};
                const u32x4 bv = {__builtin_amdgcn_perm(0u, by.x, sel_a), __builtin_amdgcn_perm(0u, by.x, sel_b),
                                  __builtin_amdgcn_perm(0u, by.y, sel_a), __builtin_amdgcn_perm(0u, by.y, sel_b)};
                const f16x8 B = __builtin_bit_cast(f16x8, bu), B4 = __builtin_bit_cast(f16x8, bv);
                if (s + 1 < 8)
                    read_b(bx, by, s + 1);
#ifdef HQQ_TUNING_BUILD
                if (s == 1 || s == 2 || s == 4 || s == 6) {
                    asm volatile("" ::"v"(L.cw[s][0]));
                    W3_STAMP(s == 1 ? 4 : s == 2 ? 5 : s == 4 ? 6 : 7);
                }
#endif
#pragma unroll
                for (int g8 = 0; g8 < 2; ++g8) {
                    const u32x4 w = L.cw[s][g8];
                    if (HQQ_W3_SKIP(p, 1)) {
                        asm volatile("" ::"v"(w));
                        continue;
                    }
                    u32x4 wa, wb;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        wa[j] = __builtin_amdgcn_perm(w[j], w[j], kW3GatherA);
                        wb[j] = __builtin_amdgcn_perm(w[j], w[j], kW3GatherB);
                    }
                    acc[g8][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w & mk[0]), B, acc[g8][0], 0, 0, 0);
                    acc[g8][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w & mk[1]), B, acc[g8][1], 0, 0, 0);
                    acc[g8][2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, wb & mk[2]), B, acc[g8][2], 0, 0, 0);
                    acc[g8][3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, wa & mk[3]), B, acc[g8][3], 0, 0, 0);
                    acc[g8][4] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, wa & mk[4]), B4, acc[g8][4], 0, 0, 0);
                }
            }
            wave_sync(); // the next table phase writes where these steps have read
        };

        if (wave < p.KS && slab_lo < slab_hi) {
            Slab A;
            W3_STAMP(1);
            issue_first(A, slab_lo);
            W3_STAMP(2);
            table_phase(A);
            issue_second(A);
            W3_STAMP(3);
            if constexpr (S == 2) {
                // The second slab's tables and first code steps are requested before the first slab's codes are worked
                // on (unconditionally: a wave whose second slab lies past its range reads the first again and leaves
                // out the arithmetic).
                const bool two = slab_lo + 1 < slab_hi;
                Slab B;
                issue_first(B, two ? slab_lo + 1 : slab_lo);
                code_phase(A);
                if (two) {
                    table_phase(B);
                    issue_second(B);
                    code_phase(B);
                }
            } else {
                code_phase(A);
            }
            W3_STAMP(8);
        }

        // wave result
        wave_sync();
        const float zt = zt_lds[wave][fcol][0] * (1.0f / kXsScale), zt4 = zt_lds[wave][fcol4][0] * (1.0f / kXsScale);
        const float un = w3_set_unscale(set, half), un4 = w3_set_unscale(4, half);
        // Accumulator element v of a lane is tile row 4 * (lane >> 4) + v = 2 * word row + phase; a column keeps the
        // rows of its own phase, and the two phases of a word row are lanes one apart: the lanes of phase 0 add their
        // neighbour's odd element to their own even one (what the lanes of phase 1 compute is not used).
        auto swapped = [](float v) __attribute__((always_inline)) {
            return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
        };
        float out[2][2], out4[2][2];
#pragma unroll
        for (int g8 = 0; g8 < 2; ++g8) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                float even = acc[g8][0][2 * e], odd = acc[g8][0][2 * e + 1]; // of the lane's own set
#pragma unroll
                for (int i = 1; i < 4; ++i) {
                    even = set == i ? (float)acc[g8][i][2 * e] : even;
                    odd = set == i ? (float)acc[g8][i][2 * e + 1] : odd;
                }
                out[g8][e] = fmaf(even + swapped(odd), un, -zt);
                out4[g8][e] = fmaf(acc[g8][4][2 * e] + swapped(acc[g8][4][2 * e + 1]), un4, -zt4);
            }
        }
        if (phi == 0) {
#pragma unroll
            for (int g8 = 0; g8 < 2; ++g8) {
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int row = 8 * g8 + 2 * gk + e;
                    red_lds(wave)[row][fcol][0] = out[g8][e];
                    if (set == 0)
                        red_lds(wave)[row][fcol4][0] = out4[g8][e];
                }
            }
        }
    } else {
        // ------------------------------------------------------------ three to eight batch rows on the matrix cores
        // The single row's layout with the batch rows in the columns: column = phase + 2 * half + 4 * (batch row within
        // its group of four), so every set of fields has a B operand of its own per group, 32 * s[k] (from LDS) times
        // the lane's own x[m, k] (read straight from memory) placed in the lane's half.  The zero term is two more
        // matrix instructions per step and group: A = 32 * s * z of table rows 0..7, then 8 and 9 (rows = table row x
        // phase, two columns per register as they lie in LDS), B = x as loaded.
        static_assert(XMODE == 0, "batches take their activations as they are");
        constexpr int BG = MT / 4;
        constexpr int SK = Q8 ? TK_U8_COLS : TK_F16, ZK = Q8 ? TK_U8_SCALAR : TK_F16;
        f16 *const s_w = xs_raw + wave * (16 * 4 * 10 * 4); // [step][piece][table row][4 halves]
        f16 *const z_w = zs_raw + wave * (16 * 4 * 10 * 4);
        const int rho = (lane & 15) >> 1, phi = lane & 1, gk = lane >> 4;
        uint32_t code_at[2];
#pragma unroll
        for (int g8 = 0; g8 < 2; ++g8) {
            const int wr = w0 + p.P * (16 * rb + 8 * g8 + rho);
            code_at[g8] = (uint32_t)(wr < p.NW ? wr : w0) * (uint32_t)K * 4u + (uint32_t)(32 * gk + 16 * phi);
        }
        const int half = (lane >> 1) & 1, mrow = (lane & 15) >> 2;
        const uint32_t piece_at = (uint32_t)((2 * gk + phi) * 10 * 8);
        const uint32_t sel_a = half ? 0x01000c0cu : 0x0c0c0100u, sel_b = half ? 0x03020c0cu : 0x0c0c0302u;
        const uint32_t z_at0 = piece_at + (uint32_t)(rho * 8), z_at1 = piece_at + (uint32_t)((8 + (rho & 1)) * 8);
        uint32_t x_at[BG]; // halves
#pragma unroll
        for (int bg = 0; bg < BG; ++bg) {
            const int m = 4 * bg + mrow;
            x_at[bg] = (uint32_t)(m < M ? m : 0) * (uint32_t)K + (uint32_t)(8 * gk + 4 * phi);
        }
        const int qT = lane & 15;
        const bool third_ok = lane < 32;
        uint32_t trow_at[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const int f = r < 2 ? 4 * r + (lane >> 4) : 8 + ((lane >> 4) & 1);
            uint32_t j = j0 + (uint32_t)f;
            j -= j >= (uint32_t)p.G ? (uint32_t)p.G : 0u;
            trow_at[r] = j * (uint32_t)K + (uint32_t)(16 * qT);
        }
        f32x4 acc[2][5][BG], accz[2][BG];
#pragma unroll
        for (int bg = 0; bg < BG; ++bg) {
#pragma unroll
            for (int g8 = 0; g8 < 2; ++g8) {
                accz[g8][bg] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 5; ++i)
                    acc[g8][i][bg] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
        }
        uint32_t mk[5] = {w3_set_mask(0), w3_set_mask(1), w3_set_mask(2), w3_set_mask(3), w3_set_mask(4)};
        asm volatile("" : "+s"(mk[0]), "+s"(mk[1]), "+s"(mk[2]), "+s"(mk[3]), "+s"(mk[4]));

        if (wave < p.KS) {
#pragma clang loop unroll(disable)
            for (int slab = slab_lo; slab < slab_lo + S && slab < slab_hi; ++slab) {
                const uint32_t k0 = (uint32_t)slab * kSlab;
                W3_STAMP(1);
                // every load of the slab in the order of use: tables, activations, codes
                uint32_t zms_raw = 0, zmz_raw = 0;
                if constexpr (Q8) {
                    zms_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_ms) + (lane >> 6));
                    zmz_raw = gload<uint16_t>(reinterpret_cast<const uint16_t *>(R.z_mz) + (lane >> 6));
                }
                Raw16<SK> rs[3];
                Raw16<ZK> rz[3];
#pragma unroll
                for (int r = 0; r < 3; ++r) {
                    const uint32_t ce = trow_at[r] + k0;
                    uint32_t cm = 0;
                    if constexpr (Q8) {
                        cm = ce - __umulhi(ce, R.s_inv) * R.s_cols;
                        cm -= cm >= R.s_cols ? R.s_cols : 0;
                        cm -= cm >= R.s_cols ? R.s_cols : 0;
                    }
                    if (Q8 && p.meta4) {
                        rs[r].q = gload<u32x4>(R.sq + ce);
#pragma unroll
                        for (int pc = 0; pc < 4; ++pc) {
                            uint32_t c4 = cm + 4u * pc;
                            c4 -= c4 >= R.s_cols ? R.s_cols : 0;
                            const u32x2 a = gload<u32x2>(R.s_ms + c4), b = gload<u32x2>(R.s_mz + c4);
                            rs[r].ms[pc >> 1][2 * (pc & 1)] = a.x, rs[r].ms[pc >> 1][2 * (pc & 1) + 1] = a.y;
                            rs[r].mz[pc >> 1][2 * (pc & 1)] = b.x, rs[r].mz[pc >> 1][2 * (pc & 1) + 1] = b.y;
                        }
                    } else {
                        load16<SK>(rs[r], R.sq, R.s_ms, R.s_mz, ce, cm);
                    }
                    load16<ZK>(rz[r], R.zq, nullptr, nullptr, ce, 0);
                }
                u32x2 xw[BG][8];
#pragma unroll
                for (int bg = 0; bg < BG; ++bg)
#pragma unroll
                    for (int s = 0; s < kW3Early; ++s)
                        xw[bg][s] = gload<u32x2>(p.x + (x_at[bg] + k0 + (uint32_t)(32 * s)));
                u32x4 cw[8][2];
#pragma unroll
                for (int s = 0; s < kW3Early; ++s)
#pragma unroll
                    for (int g8 = 0; g8 < 2; ++g8)
                        cw[s][g8] = gload<u32x4>(R.codes + (code_at[g8] + 4u * k0 + (uint32_t)(128 * s)));
                __builtin_amdgcn_sched_barrier(0);
                W3_STAMP(2);

                // table phase: 32 * s and 32 * s * z of the ten table rows into LDS
                if constexpr (Q8)
                    asm volatile("" : "+v"(zms_raw), "+v"(zmz_raw));
                const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
                const f16x2 zms = as_h2(zms_raw * 0x10001u), zmz = as_h2(zmz_raw * 0x10001u);
#pragma unroll
                for (int r = 0; r < 3; ++r) {
                    const int f = r < 2 ? 4 * r + (lane >> 4) : 8 + ((lane >> 4) & 1);
                    f16x2 sv[8], zv[8];
                    decode16<SK>(rs[r], k32, k32, sv);
                    decode16<ZK>(rz[r], zms, zmz, zv);
                    uint32_t a[8], b[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const f16x2 v = sv[t] * k32;
                        a[t] = as_u32(v), b[t] = as_u32(zv[t] * v);
                    }
                    if (r < 2 || third_ok) {
#pragma unroll
                        for (int pi = 0; pi < 4; ++pi) {
                            *reinterpret_cast<u32x2 *>(s_w + ((qT * 4 + pi) * 10 + f) * 4) = (u32x2){a[2 * pi], a[2 * pi + 1]};
                            *reinterpret_cast<u32x2 *>(z_w + ((qT * 4 + pi) * 10 + f) * 4) = (u32x2){b[2 * pi], b[2 * pi + 1]};
                        }
                    }
                }
                wave_sync();
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int bg = 0; bg < BG; ++bg) // the second half of the activations and codes, into the registers the tables have left
#pragma unroll
                    for (int s = kW3Early; s < 8; ++s)
                        xw[bg][s] = gload<u32x2>(p.x + (x_at[bg] + k0 + (uint32_t)(32 * s)));
#pragma unroll
                for (int s = kW3Early; s < 8; ++s)
#pragma unroll
                    for (int g8 = 0; g8 < 2; ++g8)
                        cw[s][g8] = gload<u32x4>(R.codes + (code_at[g8] + 4u * k0 + (uint32_t)(128 * s)));
                __builtin_amdgcn_sched_barrier(0);
                W3_STAMP(3);

                // code phase, a step is 32 columns
#pragma unroll
                for (int s = 0; s < 8; ++s) {
#ifdef HQQ_TUNING_BUILD
                    if (s == 1 || s == 2 || s == 4 || s == 6) {
                        asm volatile("" ::"v"(cw[s][0]));
                        W3_STAMP(s == 1 ? 4 : s == 2 ? 5 : s == 4 ? 6 : 7);
                    }
#endif
                    const char *s_step = reinterpret_cast<const char *>(s_w) + s * 640, *z_step = reinterpret_cast<const char *>(z_w) + s * 640;
                    const u32x2 za = *reinterpret_cast<const u32x2 *>(z_step + z_at0), zb = *reinterpret_cast<const u32x2 *>(z_step + z_at1);
                    const f16x8 Az0 = __builtin_bit_cast(f16x8, (u32x4){za.x, za.y, 0u, 0u});
                    const f16x8 Az1 = __builtin_bit_cast(f16x8, (u32x4){zb.x, zb.y, 0u, 0u});
#pragma unroll
                    for (int bg = 0; bg < BG; ++bg) {
                        const f16x8 Bx = __builtin_bit_cast(f16x8, (u32x4){xw[bg][s].x, xw[bg][s].y, 0u, 0u});
                        accz[0][bg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Az0, Bx, accz[0][bg], 0, 0, 0);
                        accz[1][bg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Az1, Bx, accz[1][bg], 0, 0, 0);
                    }
                    u32x4 wa[2];
#pragma unroll
                    for (int set = 0; set < 5; ++set) {
                        const u32x2 sb = *reinterpret_cast<const u32x2 *>(s_step + piece_at + w3_set_field(set, half) * 8);
                        f16x8 B[BG];
#pragma unroll
                        for (int bg = 0; bg < BG; ++bg) {
                            const uint32_t p01 = as_u32(as_h2(sb.x) * as_h2(xw[bg][s].x)), p23 = as_u32(as_h2(sb.y) * as_h2(xw[bg][s].y));
                            B[bg] = __builtin_bit_cast(f16x8, (u32x4){__builtin_amdgcn_perm(0u, p01, sel_a), __builtin_amdgcn_perm(0u, p01, sel_b),
                                                                     __builtin_amdgcn_perm(0u, p23, sel_a), __builtin_amdgcn_perm(0u, p23, sel_b)});
                        }
#pragma unroll
                        for (int g8 = 0; g8 < 2; ++g8) {
                            const u32x4 w = cw[s][g8];
                            u32x4 src = w;
                            if (set == 2) {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    src[j] = __builtin_amdgcn_perm(w[j], w[j], kW3GatherB);
                            } else if (set == 3) {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    wa[g8][j] = __builtin_amdgcn_perm(w[j], w[j], kW3GatherA);
                                src = wa[g8];
                            } else if (set == 4) {
                                src = wa[g8];
                            }
                            const f16x8 A = __builtin_bit_cast(f16x8, src & mk[set]);
#pragma unroll
                            for (int bg = 0; bg < BG; ++bg)
                                acc[g8][set][bg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[bg], acc[g8][set][bg], 0, 0, 0);
                        }
                    }
                }
                wave_sync();
                W3_STAMP(8);
            }
        }

        // wave result.  Element v of an accumulator is tile row 4 * (lane >> 4) + v = 2 * (row of the group) + phase; a
        // column keeps the rows of its own phase, and the two phases are lanes one apart: the lanes of phase 0 add
        // their neighbour's odd element to their own even one.  First the zero terms, through LDS to the columns of
        // their table row; then the results, in the place of the wave's own tables.
        auto both = [&](const f32x4 &c, int e) __attribute__((always_inline)) {
            return c[2 * e] + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (float)c[2 * e + 1]), 0xB1, 0xF, 0xF, true));
        };
        // the lane's roles once more, from a copy of the lane number the compiler cannot see through: derived from the
        // values of the prologue they would stay live through the whole code phase, which has no register to spare
        int lt = lane;
        asm volatile("" : "+v"(lt));
        const int phi_t = lt & 1, half_t = (lt >> 1) & 1, mrow_t = (lt & 15) >> 2, gk_t = lt >> 4;
        float zv[BG][2][2];
#pragma unroll
        for (int bg = 0; bg < BG; ++bg)
#pragma unroll
            for (int e = 0; e < 2; ++e)
                zv[bg][e][0] = both(accz[0][bg], e), zv[bg][e][1] = both(accz[1][bg], e);
        if (phi_t == 0 && half_t == 0) {
#pragma unroll
            for (int bg = 0; bg < BG; ++bg)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    zt_lds[wave][2 * gk_t + e][4 * bg + mrow_t] = zv[bg][e][0] * (1.0f / kXsScale);
                    if (gk_t == 0)
                        zt_lds[wave][8 + e][4 * bg + mrow_t] = zv[bg][e][1] * (1.0f / kXsScale);
                }
        }
        wave_sync();
        float (*const red_w)[10][MT] = red_lds(wave);
#pragma unroll
        for (int set = 0; set < 5; ++set) {
            const int f = w3_set_field(set, half_t);
            const float un = w3_set_unscale(set, half_t);
            float out[BG][2][2];
#pragma unroll
            for (int bg = 0; bg < BG; ++bg) {
                const float zt = zt_lds[wave][f][4 * bg + mrow_t];
#pragma unroll
                for (int g8 = 0; g8 < 2; ++g8)
#pragma unroll
                    for (int e = 0; e < 2; ++e)
                        out[bg][g8][e] = fmaf(both(acc[g8][set][bg], e), un, -zt);
            }
            if (phi_t == 0) {
#pragma unroll
                for (int bg = 0; bg < BG; ++bg)
#pragma unroll
                    for (int g8 = 0; g8 < 2; ++g8)
#pragma unroll
                        for (int e = 0; e < 2; ++e)
                            red_w[8 * g8 + 2 * gk_t + e][f][4 * bg + mrow_t] = out[bg][g8][e];
            }
        }
    }
#ifdef HQQ_TUNING_BUILD
    if (p.stamps)
        st[10] = __builtin_readcyclecounter();
#endif
    W3_STAMP(11);
    __syncthreads();
    W3_STAMP(12);
#ifdef HQQ_TUNING_BUILD
    auto write_stamps = [&]() __attribute__((always_inline)) {
        if (p.stamps && lane == 0) {
            st[13] = __builtin_amdgcn_s_memrealtime();
            unsigned long long *d = p.stamps + ((size_t)blockIdx.x * 16 + wave) * 16;
            for (int i = 0; i < 14; ++i)
                d[i] = st[i];
            d[14] = __builtin_amdgcn_s_getreg((31 << 11) | 4);  // HW_ID
            d[15] = __builtin_amdgcn_s_getreg((31 << 11) | 20); // XCC_ID
        }
    };
#endif

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
            v += red_lds(w)[t_t][i_t][m_t];
        const int64_t wr_t = (int64_t)w0 + (int64_t)p.P * (16 * rb + t_t);
        const int64_t n = 10 * wr_t + i_t;
        if (m_t >= M || wr_t >= p.NW || n >= p.N)
            continue;
        if (alone) {
            finish(m_t, n, v);
        } else if (p.words) {
            // Two blocks per output: each swaps its sum into the output's word.  The one that finds the word empty
            // is done; the other finds its partner's sum there, adds its own (either order gives the same sum),
            // empties the word again and writes the output.  Zero marks an empty word: a sum of +0 goes in as -0.
            uint32_t *word = p.words + (((int64_t)layer * p.N + n) * MT + m_t);
            const uint32_t bits = __builtin_bit_cast(uint32_t, v);
            const uint32_t other = __hip_atomic_exchange(word, bits ? bits : 0x80000000u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (other != 0) {
                __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                finish(m_t, n, v + __builtin_bit_cast(float, other));
            }
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
#ifdef HQQ_TUNING_BUILD
    write_stamps();
#endif
    if (alone || p.slots || p.words)
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

#ifdef HQQ_TUNING_BUILD
unsigned long long *g_w3_stamps = nullptr; // device buffer the launches write their waves' time stamps to
#endif

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
    // a lane of the table phase reads sixteen consecutive entries of a table row and of its per-column meta
    if (!aligned16(l->codes) || !aligned16(l->scale.data) || !aligned16(l->zero.data))
        return false;
    if (pl.q8 && (l->scale.meta_cols % 4 != 0 || l->scale.meta_cols < 16 || !aligned16(l->scale.meta_scale) ||
                  !aligned16(l->scale.meta_zero)))
        return false;
    pl.G = (int)G;
    pl.P = (int)(G / gcd_int(10, (int)G));
    pl.NW = (int)NW;
    const int rows = (int)((NW + pl.P - 1) / pl.P); // word rows per window
    pl.RB = (rows + 15) / 16;
    pl.NS = (int)(l->K / kSlab);
    // blocks along K: enough that the windows cover the chip, and at most 16 slabs (8 waves x 2) per block
    // (five to eight batch rows in a pass: the accumulators of every row leave no registers for a second slab's tables)
    const int per_block = M >= 5 ? kW3Waves : kW3Waves * kW3S;
    int BK = (pl.NS + per_block - 1) / per_block;
    while ((int64_t)pl.P * pl.RB * NL * BK < 200 && BK < pl.NS)
        ++BK;
    const bool tune = tuning_int("HQQ_W3_K", (int)l->K) == (int)l->K;
    if (tune)
        BK = tuning_int("HQQ_W3_BK", BK);
    if (BK < 1 || BK > pl.NS || (pl.NS + BK - 1) / BK > per_block)
        return false;
    pl.SB = (pl.NS + BK - 1) / BK;
    pl.BK = (pl.NS + pl.SB - 1) / pl.SB;
    pl.S = pl.SB > kW3Waves ? kW3S : 1;
    if (tune && M < 5)
        pl.S = tuning_int("HQQ_W3_S", pl.S) == 2 ? 2 : pl.S;
    pl.KS = (pl.SB + pl.S - 1) / pl.S;
    if ((int64_t)pl.P * NL > 65535 || pl.RB > 65535 || (int64_t)pl.P * pl.RB * NL * sizeof(int) > kTileCounterBytes)
        return false;
    if ((int64_t)pl.P * NL * pl.RB * pl.BK * (pl.RB > pl.BK ? pl.RB : pl.BK) >= (1ll << 32))
        return false; // the kernel's block-to-tile divisions are exact below this
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
    if constexpr (MT == 1) {
        if (fused) {
            gemv_w3_kernel<MT, Q8, 1, S><<<grid, dim3(kW3Waves * 64), 0, s>>>(p);
            return;
        }
    }
    gemv_w3_kernel<MT, Q8, 0, S><<<grid, dim3(kW3Waves * 64), 0, s>>>(p); // (a batch is never fused)
}

template <int MT, bool Q8> void launch_xmode(const W3Params &p, bool fused, dim3 grid, hipStream_t s)
{
    if constexpr (MT <= 4) {
        if (p.S == 2) {
            launch_slabs<MT, Q8, 2>(p, fused, grid, s);
            return;
        }
    }
    launch_slabs<MT, Q8, 1>(p, fused, grid, s); // (the plan of five to eight rows has one slab per wave)
}

// batch rows of one pass over the weights
int rows_per_pass(int64_t M) { return M >= 2 ? 8 : 1; }

size_t job_workspace_bytes(const W3Plan &pl, const hqq_linear *l, int NL, int rows)
{
    return kHeadBytes + (pl.BK > 1 ? (size_t)NL * pl.BK * rows * (size_t)l->N * sizeof(float) : 0);
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
    if (fused && M != 1)
        return HQQ_E_UNSUPPORTED; // silu(xa) * xb is built in the loads of the single-row kernel only
    const int rows = rows_per_pass(M);
    if (pl.BK > 1 && (!ws || ws_bytes < job_workspace_bytes(pl, l, j.NL, rows)))
        return HQQ_E_WORKSPACE;
    if (fused ? ((reinterpret_cast<uintptr_t>(j.xa) | reinterpret_cast<uintptr_t>(j.xb)) & 7u) != 0
              : (reinterpret_cast<uintptr_t>(j.x) & 15u) != 0)
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
    const size_t per_output = (size_t)(j.pair ? 1 : j.NL) * (size_t)l->N * (M <= 4 ? (M == 1 ? 1 : 4) : rows);
    if (pl.BK > 1 && pl.BK * (j.pair ? 2 : 1) <= 14 && per_output * sizeof(unsigned long long) <= kSlotBytes)
        p.slots = reinterpret_cast<unsigned long long *>(static_cast<char *>(ws) + kCounterBytes);
    else if (pl.BK == 2 && !j.pair && per_output * sizeof(uint32_t) <= kSlotBytes) // (the same memory, zero between launches)
        p.words = reinterpret_cast<uint32_t *>(static_cast<char *>(ws) + kCounterBytes);
    if (j.pair && (!p.slots || M != 1 || j.NL != 2 || !fused || !j.ep.row_scale))
        return HQQ_E_UNSUPPORTED; // the shared slots are what joins the two experts
    p.pair = j.pair, p.x_lstride = j.x_lstride;
    p.part_lstride = (int64_t)pl.BK * rows * l->N;
    p.y_lstride = j.y_lstride;
    p.accumulate = j.ep.accumulate;
    p.meta4 = pl.q8 && l->scale.meta_cols % 16 != 0;
#ifdef HQQ_TUNING_BUILD
    p.skip = tuning_int("HQQ_W3_SKIP", 0);
    p.plain_order = tuning_int("HQQ_W3_ORDER", 0) & 1;
    p.stamps = g_w3_stamps;
#endif
    p.N = (int)l->N, p.K = (int)l->K, p.G = pl.G, p.P = pl.P, p.NW = pl.NW, p.RB = pl.RB;
    p.NS = pl.NS, p.KS = pl.KS, p.S = pl.S, p.SB = pl.SB, p.BK = pl.BK;
    const uint32_t blocks = (uint32_t)pl.BK * (uint32_t)pl.RB * (uint32_t)(pl.P * j.NL);
    const dim3 grid(blocks);
    auto magic = [](int d) { return (uint32_t)((1ull << 32) / (uint32_t)d + 1); };
    p.per_xcd = blocks / 8, p.xcd_more = blocks % 8;
    p.bk_magic = magic(pl.BK), p.rb_magic = magic(pl.RB), p.p_magic = magic(pl.P);
    // Windows in the order of their first table row: window w starts at row 10 w mod G = g * ((10 / g) w mod P) with
    // g = gcd(10, G), so list position n holds the window with (10 / g) w = n (mod P).
    p.win_mul = 1;
    if (pl.P <= 1024 && !(tuning_int("HQQ_W3_ORDER", 0) & 2)) {
        const int t = 10 / gcd_int(10, pl.G);
        for (int w = 1; w < pl.P; ++w)
            if ((int64_t)t * w % pl.P == 1) {
                p.win_mul = (uint32_t)w;
                break;
            }
    }
    // passes of eight batch rows; later passes find the weights in the caches
    for (int64_t m0 = 0; m0 < M; m0 += rows) {
        const int mb = (int)(M - m0 >= rows ? rows : M - m0);
        if (fused)
            p.xa = j.xa + m0 * l->K, p.xb = j.xb + m0 * l->K;
        else
            p.x = j.x + m0 * l->K;
        p.y = j.y + m0 * l->N, p.M = mb;
        p.row_scale = j.ep.row_scale ? j.ep.row_scale + m0 : nullptr;
        auto launch = [&](auto mt) {
            if (pl.q8)
                launch_xmode<decltype(mt)::value, true>(p, fused, grid, s);
            else
                launch_xmode<decltype(mt)::value, false>(p, fused, grid, s);
        };
        if (mb > 4)
            launch(std::integral_constant<int, 8>());
        else if (mb >= 2)
            launch(std::integral_constant<int, 4>());
        else
            launch(std::integral_constant<int, 1>());
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
    return job_workspace_bytes(pl, l, 1, rows_per_pass(M));
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
    size_t need = job_workspace_bytes(a, w1, 2 * n_experts, rows_per_pass(M));
    W3Plan single;
    if (n_experts == 1 && make_plan(w1, M, 1, single)) {
        const size_t one = job_workspace_bytes(single, w1, 1, rows_per_pass(M));
        need = one > need ? one : need;
    }
    const size_t gb = job_workspace_bytes(b, w2, 1, rows_per_pass(M));
    need = gb > need ? gb : need;
    W3Plan c;
    if (n_experts == 2 && make_plan(w2, M, 2, c)) { // both down projections in one launch
        const size_t gc = job_workspace_bytes(c, w2, 2, rows_per_pass(M));
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
    W3Plan pl, single;
    if (!make_plan(w1, M, 2, pl))
        return 0;
    const size_t both = job_workspace_bytes(pl, w1, 2, rows_per_pass(M));
    const size_t one = make_plan(w1, M, 1, single) ? job_workspace_bytes(single, w1, 1, rows_per_pass(M)) : 0;
    return both > one ? both : one; // (five rows and more run the projections one after the other)
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
    W3Plan single;
    if (M >= 5 && !ix && n_experts == 1 && make_plan(w1, M, 1, single) && make_plan(w3, M, 1, single) &&
        ws_bytes >= job_workspace_bytes(single, w1, 1, rows_per_pass(M))) {
        // Five rows and more, a block per compute unit: the two projections together would need two rounds of blocks and
        // partial sums in memory; one after the other each covers the chip once and meets in the exchange words.
        W3Job a = j, b = j;
        a.NL = b.NL = 1;
        b.layers[0] = w3, b.y = ab + ab_lstride;
        const int rc = run_job(a, M, ws, ws_bytes, s);
        return rc != HQQ_OK ? rc : run_job(b, M, ws, ws_bytes, s);
    }
    return run_job(j, M, ws, ws_bytes, s);
}

// h: M * K halves of scratch.  Batches go through it (silu(a) * b in a launch of its own, then the batch kernel, which
// takes its activations as they are); a single row builds them in the kernel's loads.
int launch_vec3_down(const hqq_linear *w2, const f16 *a, const f16 *b, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                     const SmallBatchEpilogue &ep, hipStream_t s, f16 *h, const StripIndex *ix)
{
    W3Job j = {};
    j.layers[0] = w2, j.NL = 1, j.ix = ix, j.lper = 1;
    j.y = y, j.ep = ep;
    if (M >= 2) {
        if (!h)
            return HQQ_E_NULL;
        const int rc = launch_silu_mul(a, b, h, M * w2->K, s);
        if (rc != HQQ_OK)
            return rc;
        j.x = h;
    } else {
        j.xa = a, j.xb = b;
    }
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

#ifdef HQQ_TUNING_BUILD
extern "C" void hqq_tuning_w3_stamps(void *buf) { hqq::g_w3_stamps = static_cast<unsigned long long *>(buf); }
#endif
