// Decode-time GEMV (batch M <= 4) for 2- and 4-bit codes, one launch per matmul or per fused w1/w3 gate.
//
// Algebra (shared with the small-batch kernel): the 16 output rows n = F*(jp + r*GP) + i, r = 16*rb .. 16*rb+15,
// of field i use the same scale and zero in every column, so the scale is folded into the activations,
//     y[n, m] = sum_k q[n, k] * xs[i, k, m]  -  sum_k z[i, k] * xs[i, k, m],      xs = 32 * s[i, k] * x[m, k]  (fp16),
// and the only per-weight work left is to present the code as an fp16 number.  That takes one v_and: the field,
// masked in place, is the fp16 subnormal q * 2^(pos - 24), which v_mfma_f32_16x16x32_f16 multiplies exactly.
//
// Work split.  A block owns one tile (jp, rb) of every layer of the launch (two for the gate).  Its waves split K:
// wave (layer, ks) walks S consecutive slabs of 256 columns and keeps the MFMA accumulators in registers across
// them, so partial sums meet only once per wave, in LDS.  All loads of a slab are 128 bits wide -- four code loads
// per lane, and for the table lanes 16 scale bytes, 16 zero bytes, their fp16 meta values and x -- and the loads of
// up to D slabs are in flight before the first arithmetic.  When the block holds all of K (BK == 1: every Mixtral
// projection with K = 4096, gate included) it applies the epilogue itself: no workspace, no atomics.  Otherwise
// (K = 14336) the BK blocks of a tile add their results into one 64-bit accumulation slot per output (fixed point,
// so the sum is exact and independent of the order of arrival) with a returning device-scope atomic; the block
// whose addition completes a slot writes that output.  The gate epilogue with K over several blocks (not a
// Mixtral shape) instead stores fp32 partial sums with device-scope stores, and the block that arrives last at the
// tile's counter adds them in a fixed order.
//
// A gate of three or four rows whose blocks hold all of K is launched as two passes of the two-row kernel (batch
// rows 0-1 and 2-3) in one grid, the two passes of a tile next to each other in launch order.
//
// Lane roles inside a slab, batches of two and four rows.  Code lanes: (rr = lane & 15, kg = lane >> 4) own packed
// row jp + (16*rb + rr)*GP, bytes 64*s + 16*kg .. +15 for step s.  Table lanes: (ti = lane >> 4 < F, kq = lane & 15)
// own table row F*jp + ti, columns 16*kq .. 16*kq+15, i.e. step kq >> 2, MFMA lane group kq & 3.
//
// Single rows (the decode step) use another layout, in which neither the codes nor the folded activations pass
// through LDS.  A lane (phi = lane & 3, rho = (lane >> 2) & 3, g = lane >> 4) owns the 16 columns 64*g + 16*phi .. +15
// of the slab: as a code lane of the tile rows 4*R + rho (R = 0..3, one 128-bit load each: four consecutive lanes read
// 64 consecutive bytes, a wave load covers 256 contiguous bytes of four rows), as a table lane of table row
// F*jp + rho.  The MFMA's sixteen A rows are (rho, phi): four tile rows, each at four column phases; its sixteen B
// columns are (field, phi), the lane's own 16 folded activations.  Output (row (rho, phi), column (i, phi)) of the
// MFMA whose A operand is field i masked in place is the partial sum of tile row rho, field i, over the columns of
// phase phi; the other columns pair a field with another field's scales and are never read.  So one B operand
// serves all four fields and all four row groups, a lane builds it from the table entries it loaded itself, and the
// four phases of a row are added once per wave, at the end.
#include "attention_parts.hpp"
#include "chain_parts.hpp"
#include "gemv_parts.hpp"
#include "hqq_common.hpp"
#include "norm_route.hpp"

#include <cstdlib>
#include <type_traits>

namespace hqq {
using namespace gemv;
namespace {

using StripLayer = LayerRecord;

// A launch may hold several groups of layers: group g covers blockIdx.z = z_begin .. z_begin + GP - 1 and has its
// own output.  Groups share K, the code width and the group size, not N (q, k and v projections in one launch;
// the gates of two experts in one launch).
constexpr int kMaxGroups = 4;
struct StripGroup {
    int z_begin, GP, N;
    int slot_begin; // first accumulation slot of the group: slot (slot_begin + n * MT + m) belongs to output (m, n)
    f16 *y;
    const f16 *bias;
    float *part[2]; // [BK][M][N] per layer
};

struct StripParams {
    StripLayer layer[kMaxGroups]; // record of (group g, layer l) at g * NL + l
    // Indexed launch (table != null): the layer records are read from a device table instead, record
    // table[sel[g * sel_gstride + l * sel_lstride] * table_stride + table_first + l * first_lstride], so that which
    // expert runs is decided on the device.
    const StripLayer *table;
    const int *sel;
    int table_stride, table_first;
    int sel_gstride, sel_lstride, first_lstride;
    StripGroup grp[kMaxGroups];
    const f16 *x;
    int x_lstride; // layer l reads x + l * x_lstride (0: every layer reads the same activations)
    int M, K;
    int passes; // 2 (two-row kernel only): the launch holds every tile twice, the second copy working on batch rows 2, 3
    int RB;
    int NS;       // K / 256
    int KS;       // waves per layer in a block
    int BK;       // blocks along K per tile
    int NL;       // layers per block (2: fused gate, or the down projections of two experts)
    int *counter; // one per tile, zero between launches
    unsigned long long *slots; // EPI 0 and 2 with K over several blocks: accumulation slots instead of partial sums (or null)
    const f16 *row_scale;
    int rs_lstride; // EPI 2: layer l scales by row_scale[l * rs_lstride + m]
    int accumulate;
    // NORM launches: the activations are weight * rmsnorm(x + delta) of the single row x (delta may be null), computed
    // by every block for itself; block (0, 0, 0) also writes x + delta to x_sum.
    const f16 *norm_delta, *norm_weight;
    f16 *x_sum;
    float norm_eps;
    // ROUTED launches (the gates of both active experts): the router runs in the block's prologue on the normed row
    // and its choice replaces sel; block (0, 0, 0) also writes the choice and the routing weights out.
    const f16 *gate_w;
    int n_experts;
    int *sel_out;
    f16 *rw_out;
    // Chained launches (the work of several launches in one grid, handed over through device words, see
    // chain_parts.hpp): the words of the chain and how many blocks of the launch have this one's role.
    int *chain;
    int chain_blocks;
#ifdef HQQ_TUNING_BUILD
    int skip; // timing experiments (results are then wrong): 1 leaves out the code phase, 2 the table phase
    unsigned long long *stamps; // per-wave time stamps, [block][16 waves][16], or null
#endif
};
#ifdef HQQ_TUNING_BUILD
#define HQQ_SKIP(p, bit) (((p).skip & (bit)) != 0)
#define STRIP_STAMP(i) do { if (p.stamps) st[i] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define HQQ_SKIP(p, bit) false
#define STRIP_STAMP(i)
#endif

template <int MT, int SKIND, int ZKIND> struct SlabRegs {
    Raw16<SKIND> s;
    Raw16<ZKIND> z;
    // the slab's activations.  Staged (MT <= 2): xw[j], lanes 0..31 hold 8 columns each of batch row 2j, lanes 32..63 of
    // row 2j+1.  Direct (MT = 4): xw[2m], xw[2m+1] are the table lane's own 16 columns of batch row m.
    u32x4 xw[MT <= 2 ? (MT + 1) / 2 : 2 * MT];
    u32x4 cw[4];             // codes: load i holds rows 4i .. 4i+3 of the tile, 16 lanes x 16 bytes per row
    uint32_t sms, smz, zms, zmz; // whole-tensor meta values, raw fp16 bits
    u32x4 xd, xg;            // NORM launches: the slab's pieces of delta and of the norm weight
};

// EPI: 0 y = o (+ bias) (* row_scale) (+ y);  1 y = silu(o0) * o1;  2 y = (y +) o0 * row_scale[0] + o1 * row_scale[1]
// NORM: 0 the activations are x; 1 weight * rmsnorm(x + delta), the mean of squares added up while the weights travel;
// 2 the same with the router of the normed row in the prologue, whose choice picks the experts of the launch
// The block (bx, by, bzi) of the launch described by p.  chain (a constant at every call site): CHAIN_NONE for a launch
// of its own; CHAIN_FIRST when later blocks of the same grid read this block's output (stored at device scope, then
// counted); CHAIN_LAST when the activations are produced by earlier blocks of the same grid: the weights are requested
// first, the activations read (at device scope) once the producers have been counted, and a NORM instantiation then
// uses them as they are.
template <int NBITS, int MT, int S, int D, int WAVES, int SKIND, int ZKIND, int EPI, bool GROUPED, int NORM>
__device__ __forceinline__ void strip_block(const StripParams &p, const int bx, const int by, const int bzi, const int chain)
{
    static_assert(!NORM || (MT == 1 && WAVES >= 4), "the fused norm is for single rows and blocks of four waves and more");
#ifdef HQQ_TUNING_BUILD
    unsigned long long st[16] = {};
#endif
    STRIP_STAMP(0);
    // Every kernel argument the prologue reads is fetched here, in one batch: read where they are used, they come in
    // four or five scalar loads one after the other (each waits for the branch before it), 0.15 us apiece before the
    // first weight load can be issued.
    {
        const StripLayer &A = p.layer[0], &B = p.layer[1];
        asm volatile("" ::"s"(p.table), "s"(p.sel), "s"(p.x), "s"(p.x_lstride), "s"(p.K), "s"(p.M), "s"(p.passes), "s"(p.RB),
                     "s"(p.NS), "s"(p.KS), "s"(p.BK), "s"(p.NL), "s"(p.grp[0].z_begin), "s"(p.grp[0].GP), "s"(p.grp[0].N),
                     "s"(p.grp[1].z_begin), "s"(p.grp[2].z_begin), "s"(p.grp[3].z_begin), "s"(p.table_stride), "s"(p.table_first),
                     "s"(p.sel_gstride), "s"(p.sel_lstride), "s"(p.first_lstride));
        if constexpr (!GROUPED)
            asm volatile("" ::"s"(A.codes), "s"(A.sq), "s"(A.zq), "s"(A.s_ms), "s"(A.s_mz), "s"(A.z_ms), "s"(A.z_mz), "s"(A.s_cols),
                         "s"(A.s_inv), "s"(B.codes), "s"(B.sq), "s"(B.zq), "s"(B.s_ms), "s"(B.s_mz), "s"(B.z_ms), "s"(B.z_mz),
                         "s"(B.s_cols), "s"(B.s_inv));
    }
    const bool origin = bx == 0 && by == 0 && bzi == 0;
    const bool normed = NORM != 0 && chain != CHAIN_LAST; // whether the activations go through the norm
    if (chain == CHAIN_FIRST)
        CHAIN_STAMP(p.chain, 0);
    constexpr bool ROUTED = NORM == 2;
    constexpr int F = 8 / NBITS;
    constexpr int ENTRY = 8; // halves per B-operand entry (16 bytes)
    constexpr int STEP_HALVES = F * 2 * 4 * MT * ENTRY;
    constexpr int XS_HALVES = 4 * STEP_HALVES;
    // Codes are staged through LDS for batches of one and two rows; at four rows the activation staging already
    // takes most of the LDS a wave can have, and there the codes are loaded straight into the MFMA layout.
    constexpr bool PHASE = MT == 1; // single rows: the (row, phase) x (field, phase) layout, nothing but x through LDS
    constexpr bool STAGE = MT == 2; // codes staged through LDS
    constexpr bool XSTAGE = MT <= 2; // x reaches the table lanes through LDS
    constexpr int CODE_PITCH = kSlab + 16; // bytes per tile row in the staging buffer: the pad spreads the rows over the banks
    __shared__ __attribute__((aligned(16))) f16 xs_lds[PHASE ? 1 : WAVES][PHASE ? 8 : XS_HALVES];
    __shared__ __attribute__((aligned(16))) uint8_t code_lds[STAGE ? WAVES : 1][STAGE ? 16 * CODE_PITCH : 16];
    __shared__ __attribute__((aligned(16))) f16 xw_lds[XSTAGE ? WAVES : 1][XSTAGE ? 2 * ((MT + 1) / 2) : 1][XSTAGE ? kSlab : 8];
    __shared__ float bias_lds[WAVES][F][MT];
    __shared__ __attribute__((aligned(16))) float red_lds[WAVES][16][MT][F];
    __shared__ __attribute__((aligned(16))) float fin_lds[2][16][MT][F];
    __shared__ int ticket_lds;
    __shared__ float norm_lds[4];
    __shared__ int sel_lds[2];
    __shared__ f16 rw_lds[2];
    // ROUTED launches: the normed row, written once by the prologue and read by every slab (hidden <= 4096)
    __shared__ __attribute__((aligned(16))) f16 xn_lds[ROUTED ? 4096 : 8];
    // ROUTED launches: the records of both gate projections of every expert, fetched while the router runs, so that
    // the chosen ones are at hand when it is done (one trip to memory less in front of the first weight load)
    constexpr int REC_WORDS = sizeof(StripLayer) / 4, REC_ALL = 8 * 2 * REC_WORDS;
    constexpr int REC_PER = (REC_ALL + WAVES * 64 - 1) / (WAVES * 64);
    __shared__ uint32_t rec_lds[ROUTED ? REC_ALL : 1];

    const int lane = threadIdx.x & 63;
    // the wave index as a scalar: what depends on it (the layer, its record, the K range) then lives in scalar
    // registers, and the record is picked from the kernel arguments without a memory access of its own
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kb = bx, rb = by;
    // Batches of three and four rows run as two passes of the two-row kernel inside one launch: blocks 2z and 2z + 1
    // are the two passes of tile z, so both ask for the tile's weights at about the same time and memory delivers
    // them once (how far apart the two are in launch order, 1 to 32 workgroups, made no difference when measured).
    int bz = bzi, pass = 0;
    if constexpr (MT == 2) {
        if (p.passes == 2) {
            pass = bz & 1;
            bz >>= 1;
        }
    }
    int g = 0;
    if constexpr (GROUPED) // absent groups begin at INT_MAX
        g = (bz >= p.grp[1].z_begin) + (bz >= p.grp[2].z_begin) + (bz >= p.grp[3].z_begin);
    const StripGroup &Gd = p.grp[g]; // g is uniform: the record comes from the kernel arguments by scalar loads
    const int jp = bz - Gd.z_begin;
    const int GP = Gd.GP, N = Gd.N;
    const int layer = wave >= p.KS ? 1 : 0;
    const int ks = wave - layer * p.KS;
    const bool wave_on = wave < p.KS * p.NL;
    float rnorm = 1.0f; // NORM launches: 1 / sqrt(mean(x^2) + eps), known once the block has added the row up
    if constexpr (ROUTED) {
        // every block routes for itself (the router's rows come from L2): which records to read is known only then
        const bool writer = origin;
        __shared__ __attribute__((aligned(16))) uint8_t route_raw[ROUTED ? sizeof(NormRouteLds<8>) : 16];
        NormRouteLds<8> &route_lds = *reinterpret_cast<NormRouteLds<8> *>(&route_raw[0]);
        uint32_t recw[REC_PER];
#pragma unroll
        for (int q = 0; q < REC_PER; ++q) {
            const int t = (int)threadIdx.x + q * WAVES * 64;
            const int tc = t < p.n_experts * 2 * REC_WORDS ? t : 0; // spare threads repeat word 0
            const int ex = tc / (2 * REC_WORDS), rem = tc - ex * 2 * REC_WORDS, ly = rem / REC_WORDS, w = rem - ly * REC_WORDS;
            recw[q] = gload<uint32_t>(reinterpret_cast<const uint32_t *>(p.table + (ex * p.table_stride + p.table_first + ly * p.first_lstride)) + w);
        }
        rnorm = norm_route_block<2, 8>(p.x, p.norm_delta, p.norm_weight, p.norm_eps, writer ? p.x_sum : nullptr, xn_lds, p.K,
                                       p.gate_w, p.n_experts, sel_lds, rw_lds, nullptr, route_lds);
#pragma unroll
        for (int q = 0; q < REC_PER; ++q) {
            const int t = (int)threadIdx.x + q * WAVES * 64;
            if (t < p.n_experts * 2 * REC_WORDS)
                rec_lds[t] = recw[q];
        }
        __syncthreads();
        if (writer && threadIdx.x < 2) {
            p.sel_out[threadIdx.x] = sel_lds[threadIdx.x];
            p.rw_out[threadIdx.x] = rw_lds[threadIdx.x];
        }
    }
    // both layer records come from the kernel arguments and are selected in registers: no dependent loads
    StripLayer L;
    if (p.table) {
        // one word of the record per lane, then broadcast: the record's address is known only now
        const int sel_at = g * p.sel_gstride + layer * p.sel_lstride;
        const int e = __builtin_amdgcn_readfirstlane(ROUTED ? sel_lds[sel_at] : p.sel[sel_at]);
        uint32_t word;
        if constexpr (ROUTED) {
            word = rec_lds[(e * 2 + layer) * REC_WORDS + (lane < 18 ? lane : 0)];
        } else {
            const uint32_t *src =
                reinterpret_cast<const uint32_t *>(p.table + (e * p.table_stride + p.table_first + layer * p.first_lstride));
            word = src[lane < 18 ? lane : 0];
        }
        uint32_t rec[18];
#pragma unroll
        for (int i = 0; i < 18; ++i)
            rec[i] = __builtin_amdgcn_readlane(word, i);
        __builtin_memcpy(&L, rec, sizeof(L));
    } else if constexpr (GROUPED) {
        L = p.layer[__builtin_amdgcn_readfirstlane(g * p.NL + layer)];
    } else {
        const StripLayer &A = p.layer[0], &B = p.layer[1];
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
    }
    const int slab0 = (kb * p.KS + ks) * S;
    const int K = p.K;
    const int M = MT == 1 ? 1 : (p.M - 2 * pass < MT ? p.M - 2 * pass : MT);

    const int rr = lane & 15, kg = lane >> 4;
    // table lane: table row ti of the tile, columns 16*kq .. 16*kq+15 of the slab
    const int ti = PHASE ? (lane >> 2) & 3 : lane >> 4;
    const int kq = PHASE ? 4 * (lane >> 4) + (lane & 3) : lane & 15;
    const bool tlane = ti < F;     // lanes that own table entries (all of them for 2-bit codes)
    const int ti_l = ti & (F - 1); // the other lanes repeat a table lane's loads, so that issuing loads never diverges

    const uint32_t trow = (uint32_t)(F * jp + ti_l) * (uint32_t)K + (uint32_t)(16 * kq);
    // Weight loads walk the tile row by row -- four consecutive lanes read 64 consecutive bytes, which is the unit the
    // address pipeline of the memory path handles per cycle -- and reach the MFMA layout (lane = row + 16 * k group)
    // through an LDS staging buffer.  Loading straight into that layout puts four different rows into every group of
    // four lanes and costs four times the address cycles; with twelve loads per slab that pipeline, not HBM, then
    // bounds the kernel.
    // Single rows read the same way, and because an MFMA row may be any (tile row, column phase) pair they need no
    // staging: the lane's 16 bytes of tile rows 4*i + ti are its A operands as they arrive.
    const int lrow = PHASE ? ti : lane >> 4, lchunk = PHASE ? kq : lane & 15;
    const uint32_t crow = STAGE || PHASE ? ((uint32_t)jp + (uint32_t)(16 * rb + lrow) * (uint32_t)GP) * (uint32_t)K + (uint32_t)(16 * lchunk)
                                         : ((uint32_t)jp + (uint32_t)(16 * rb + rr) * (uint32_t)GP) * (uint32_t)K + (uint32_t)(16 * kg);
    const uint32_t crow_step = STAGE || PHASE ? 4u * (uint32_t)GP * (uint32_t)K : 64u; // four tile rows further / next step
    const f16 *xl = p.x + layer * p.x_lstride + pass * 2 * K;

    auto issue = [&](SlabRegs<MT, SKIND, ZKIND> &r, int slab) __attribute__((always_inline)) {
        const uint32_t k0 = (uint32_t)slab * kSlab;
        const uint32_t c = trow + k0;
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
        load16<SKIND>(r.s, L.sq, L.s_ms, L.s_mz, c, scm);
        load16<ZKIND>(r.z, L.zq, L.z_ms, L.z_mz, c, zcm);
        // x: one coalesced piece per pair of batch rows (16 bytes per lane, 32 lanes per row)
        if constexpr (ROUTED) {
            // the row is in LDS already
        } else if constexpr (XSTAGE) {
            if (chain != CHAIN_LAST) { // (the last role reads its activations after the wait)
#pragma unroll
                for (int j = 0; j < (MT + 1) / 2; ++j) {
                    int m = 2 * j + (lane >> 5);
                    m = m < M ? m : 0;
                    r.xw[j] = gload<u32x4>(xl + (k0 + (uint32_t)(8 * (lane & 31)) + (uint32_t)(m * K)));
                }
            }
            if (NORM == 1 && normed) {
                r.xg = gload<u32x4>(p.norm_weight + (k0 + (uint32_t)(8 * (lane & 31))));
                // unconditional (a launch without delta re-reads x and ignores the value): a load under a branch
                // would make every later wait a wait for all loads
                r.xd = gload<u32x4>((p.norm_delta ? p.norm_delta : p.x) + (k0 + (uint32_t)(8 * (lane & 31))));
            }
        } else {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const u32x4 *xp = reinterpret_cast<const u32x4 *>(xl + (k0 + (uint32_t)(16 * kq) + (uint32_t)((m < M ? m : 0) * K)));
                r.xw[2 * m] = gload<u32x4>(xp);
                r.xw[2 * m + 1] = gload<u32x4>(xp + 1);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            r.cw[i] = gload<u32x4>(L.codes + (crow + k0 + (uint32_t)i * crow_step));
        // Whole-tensor meta values ride with the slab, after its weight loads.  Their address is the same in every
        // lane, but it is written so that the compiler does not see that (lane >> 6 is zero): a load it knows to be
        // uniform is moved to scalar registers at once, and that move waits for it before any weight load is issued.
        const int zero_off = lane >> 6;
        r.sms = r.smz = r.zms = r.zmz = 0;
        if constexpr (SKIND == TK_U8_SCALAR) {
            r.sms = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.s_ms) + zero_off);
            r.smz = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.s_mz) + zero_off);
        }
        if constexpr (ZKIND == TK_U8_SCALAR) {
            r.zms = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.z_ms) + zero_off);
            r.zmz = gload<uint16_t>(reinterpret_cast<const uint16_t *>(L.z_mz) + zero_off);
        }
    };

    // B operand of lane (mcol, kg) for (step s, field i, half h): entry ((s*F + i)*2 + h)*4 + kg, batch column mcol.
    // Column m of the MFMA result depends on column m of B only, and columns m >= M are never read back, so lanes
    // past the batch simply re-read a valid column instead of needing zeros.
    const int mcol = lane & 15;
    f16 *xs_w = &xs_lds[PHASE ? 0 : wave][0];
    const f16 *xs_r = xs_w + (kg * MT + (mcol < M ? mcol : 0)) * ENTRY;

    // single rows: one accumulator per (row group R, field i) at acc[R * F + i]
    constexpr int NACC = PHASE ? 4 * F : F;
    f32x4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i)
        acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float bias_acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        bias_acc[m] = 0.f;
    // Single rows, 8-bit zeros under one whole-tensor meta pair: sum z * xs = zms * (sum zq * xs - zmz * sum xs), and
    // both sums go to the matrix cores.  The zero bytes, masked in place like the codes (fp16 subnormals zq * 2^-24),
    // are the A operand and the lane's own B operand the other: the diagonal of the result holds the lane's products
    // added over the four lane groups; a second MFMA with A = 1 adds up xs alone.  (The zero is then not rounded to
    // fp16 twice on the way, as the reference's is: the difference is below the rounding of the weights themselves.)
    constexpr bool ZMFMA = PHASE && ZKIND == TK_U8_SCALAR;
    f32x4 accz = {0.f, 0.f, 0.f, 0.f}, accx = {0.f, 0.f, 0.f, 0.f};
    uint32_t zmeta_s = 0, zmeta_z = 0; // raw fp16 bits of the zero table's meta pair

    uint8_t *code_w = &code_lds[STAGE ? wave : 0][0];
    auto compute = [&](const SlabRegs<MT, SKIND, ZKIND> &r, int slab) __attribute__((always_inline)) {
        // ------------------------------------------------------------ staging: x and the codes change lanes through LDS
        if constexpr (XSTAGE) {
#pragma unroll
            for (int j = 0; j < (ROUTED ? 0 : (MT + 1) / 2); ++j) {
                u32x4 xv = r.xw[j];
                if (NORM == 1 && normed) { // weight * fp16(fp32(x + delta) * r): the roundings of the stand-alone norm kernel
                    f16x8 v = __builtin_bit_cast(f16x8, xv);
                    const f16x8 vd = v + __builtin_bit_cast(f16x8, r.xd);
                    v = p.norm_delta ? vd : v;
                    const f16x8 g = __builtin_bit_cast(f16x8, r.xg);
                    f16x8 o;
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        o[t] = g[t] * (f16)((float)v[t] * rnorm);
                    xv = __builtin_bit_cast(u32x4, o);
                }
                *reinterpret_cast<u32x4 *>(&xw_lds[wave][2 * j + (lane >> 5)][8 * (lane & 31)]) = xv;
            }
        }
        if constexpr (STAGE) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<u32x4 *>(code_w + (4 * i + lrow) * CODE_PITCH + 16 * lchunk) = r.cw[i];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ------------------------------------------------------------ table phase, once per slab
        f16x8 Bop[2] = {}; // single rows: the lane's own B operands, columns 0-7 and 8-15 of its 16
        if (tlane && !HQQ_SKIP(p, 2)) {
            f16x2 sv[8], zv[8];
            const f16x2 sms = as_h2(r.sms * 0x10001u), smz = as_h2(r.smz * 0x10001u);
            const f16x2 zms = as_h2(r.zms * 0x10001u), zmz = as_h2(r.zmz * 0x10001u);
            decode16<SKIND>(r.s, sms, smz, sv);
            if constexpr (!ZMFMA)
                decode16<ZKIND>(r.z, zms, zmz, zv);
            const f16x2 k32 = {(f16)kXsScale, (f16)kXsScale};
#pragma unroll
            for (int t = 0; t < 8; ++t)
                sv[t] = sv[t] * k32;
            // lane's 16 columns are step kq>>2, lane group kq&3, halves h = 0 (cols 0-7) and 1 (cols 8-15)
            f16 *dst = xs_w + (kq >> 2) * STEP_HALVES + ((ti * 2) * 4 + (kq & 3)) * MT * ENTRY;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    u32x4 x0, x1;
                    if constexpr (ROUTED) {
                        const u32x4 *xp = reinterpret_cast<const u32x4 *>(&xn_lds[slab * kSlab + 16 * kq]);
                        x0 = xp[0], x1 = xp[1];
                    } else if constexpr (XSTAGE) {
                        const u32x4 *xp = reinterpret_cast<const u32x4 *>(&xw_lds[wave][m][16 * kq]);
                        x0 = xp[0], x1 = xp[1];
                    } else {
                        x0 = r.xw[MT <= 2 ? 0 : 2 * m], x1 = r.xw[MT <= 2 ? 0 : 2 * m + 1];
                    }
                    f16x2 a[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        a[t] = sv[t] * as_h2(t < 4 ? x0[t & 3] : x1[t & 3]);
                        if constexpr (!ZMFMA)
                            bias_acc[m] = __builtin_amdgcn_fdot2(zv[t], a[t], bias_acc[m], false);
                    }
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        // B-operand order inside an 8-column block: columns (0,2,1,3,4,6,5,7)
                        const f16x2 *q = &a[4 * h];
                        const f16x8 o = {q[0].x, q[1].x, q[0].y, q[1].y, q[2].x, q[3].x, q[2].y, q[3].y};
                        if constexpr (PHASE)
                            Bop[h] = o;
                        else
                            *reinterpret_cast<f16x8 *>(dst + (h * 4 * MT + m) * ENTRY) = o;
                    }
                }
            }
        }
        if constexpr (ZMFMA) {
            zmeta_s = r.zms, zmeta_z = r.zmz;
            const u32x4 ones = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t z0 = r.z.q[2 * h], z1 = r.z.q[2 * h + 1];
                const u32x4 Az = {z0 & 0x00FF00FFu, (z0 >> 8) & 0x00FF00FFu, z1 & 0x00FF00FFu, (z1 >> 8) & 0x00FF00FFu};
                accz = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, Az), Bop[h], accz, 0, 0, 0);
                accx = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, ones), Bop[h], accx, 0, 0, 0);
            }
        }
        if constexpr (PHASE) {
            // -------------------------------------------------------- code phase, single rows: 4 row groups x 2 halves x F MFMAs
            // straight from the registers the loads filled; B is the lane's own
#pragma unroll
            for (int R = 0; R < 4; ++R) {
                if (HQQ_SKIP(p, 1))
                    break;
                const uint32_t d[4] = {r.cw[R].x, r.cw[R].y, r.cw[R].z, r.cw[R].w};
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t d0 = d[2 * h], d1 = d[2 * h + 1];
                    const uint32_t d0s = d0 >> 8, d1s = d1 >> 8;
#pragma unroll
                    for (int i = 0; i < F; ++i) {
                        const uint32_t mk = Field<NBITS>::mask(i);
                        const u32x4 Au = {d0 & mk, d0s & mk, d1 & mk, d1s & mk};
                        acc[R * F + i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, Au), Bop[h], acc[R * F + i], 0, 0, 0);
                    }
                }
            }
            // the next slab's x overwrites this one's in LDS: keep that behind the table phase's reads
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            return;
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
            u32x4 cws = r.cw[s];
            if constexpr (STAGE)
                cws = *reinterpret_cast<const u32x4 *>(code_w + rr * CODE_PITCH + 16 * (4 * s + kg));
            const uint32_t d[4] = {cws.x, cws.y, cws.z, cws.w};
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
        // the next slab's table phase overwrites xs: keep it behind these reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // ---------------------------------------------------------------- S slabs, D of them in flight
    // A slab past the end of K is issued all the same (it re-reads the last slab and is never used): with a fixed
    // number of loads the compiler waits for exactly the loads a slab needs and leaves the later ones in flight.
    SlabRegs<MT, SKIND, ZKIND> regs[D];
    const int last = p.NS - 1;
    // NORM launches: the row (x + delta) for the mean of squares is requested first, by the first four waves, two
    // pieces of eight elements per thread and pass (rows of up to 4096 elements take one pass); loads retire in issue
    // order, so these must go out before the weights for the sum to be ready while the weights still travel.
    constexpr int NPIECE = 2;
    f16x8 nv[NPIECE];
    if (NORM == 1 && normed) {
#pragma unroll
        for (int c = 0; c < NPIECE; ++c) {
            const int k = ((int)threadIdx.x + c * 256) * 8;
            const int kc = threadIdx.x < 256 && k < K ? k : 0;
            nv[c] = gload<f16x8>(p.x + kc);
            if (p.norm_delta)
                nv[c] = nv[c] + gload<f16x8>(p.norm_delta + kc);
        }
    }
    STRIP_STAMP(1);
    if (wave_on) {
#pragma unroll
        for (int i = 0; i < D; ++i)
            issue(regs[i], slab0 + i < p.NS ? slab0 + i : last);
    }
    STRIP_STAMP(2);
    if (chain == CHAIN_LAST) {
        // the weights are on their way; now the activations: wait for the blocks that produce them, then read the slabs'
        // pieces at device scope (they may have been written through another XCD's L2)
        CHAIN_STAMP(p.chain, 0);
        chain_wait(p.chain, CHAIN_GO_MID, kChainGoMid);
        CHAIN_STAMP(p.chain, 1);
        if (threadIdx.x == 0)
            chain_passed(p.chain, p.chain_blocks);
        if constexpr (XSTAGE && !ROUTED) {
            if (wave_on) {
#pragma unroll
                for (int i = 0; i < D; ++i) {
                    const int slab = slab0 + i < p.NS ? slab0 + i : last;
#pragma unroll
                    for (int j = 0; j < (MT + 1) / 2; ++j) {
                        int m = 2 * j + (lane >> 5);
                        m = m < M ? m : 0;
                        regs[i].xw[j] = chain_load16(xl + ((uint32_t)slab * kSlab + (uint32_t)(8 * (lane & 31)) + (uint32_t)(m * K)));
                    }
                }
            }
        }
    }
    if (NORM == 1 && normed) {
        // the sum in the order the stand-alone norm kernel adds it (256 threads, 8 elements each per pass), so that both
        // give the same bits
        float ss = 0.f;
        if (threadIdx.x < 256) {
            const bool writer = origin;
#pragma unroll
            for (int c = 0; c < NPIECE; ++c) {
                const int k = ((int)threadIdx.x + c * 256) * 8;
                if (k < K) {
                    if (writer)
                        *reinterpret_cast<f16x8 *>(p.x_sum + k) = nv[c];
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        ss += (float)nv[c][t] * (float)nv[c][t];
                }
            }
            for (int k = ((int)threadIdx.x + NPIECE * 256) * 8; k < K; k += 256 * 8) { // longer rows: the rest, late
                f16x8 v = gload<f16x8>(p.x + k);
                if (p.norm_delta)
                    v = v + gload<f16x8>(p.norm_delta + k);
                if (writer)
                    *reinterpret_cast<f16x8 *>(p.x_sum + k) = v;
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    ss += (float)v[t] * (float)v[t];
            }
            ss = wave_sum(ss);
            if (lane == 0)
                norm_lds[wave] = ss;
        }
        __syncthreads();
        const float mean = (norm_lds[0] + norm_lds[1] + norm_lds[2] + norm_lds[3]) / (float)K;
        rnorm = 1.0f / __builtin_sqrtf(mean + p.norm_eps);
    }
    if (wave_on) {
#pragma unroll
        for (int i = 0; i < S; ++i) {
            if (slab0 + i < p.NS)
                compute(regs[i % D], slab0 + i);
            if (i + D < S)
                issue(regs[i % D], slab0 + i + D < p.NS ? slab0 + i + D : last);
            if (i < 8)
                STRIP_STAMP(3 + i);
        }
    }

    // ---------------------------------------------------------------- wave tile -> LDS (zero term removed, unscaled)
    if constexpr (PHASE) {
        // The zero term of the lane's field: its 16 lanes are the four phases (neighbours) in each of the four lane groups.
        const int phi = lane & 3, gq = lane >> 4;
        float bz;
        if constexpr (ZMFMA) {
            // diagonal element (row = column) of lane (c, gq): gq == c >> 2, element c & 3; its four phases are neighbours
            float zs = phi == 0 ? accz[0] : (phi == 1 ? accz[1] : (phi == 2 ? accz[2] : accz[3]));
            float xsum = phi == 0 ? accx[0] : (phi == 1 ? accx[1] : (phi == 2 ? accx[2] : accx[3]));
            const float zmsf = (float)__builtin_bit_cast(f16, (uint16_t)zmeta_s), zmzf = (float)__builtin_bit_cast(f16, (uint16_t)zmeta_z);
            bz = zmsf * (zs * 16777216.0f - zmzf * xsum);
            bz += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, bz), 0xB1, 0xF, 0xF, true));
            bz += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, bz), 0x4E, 0xF, 0xF, true));
            bz = __shfl(bz, (lane & 15) + 16 * ti, kWave); // from the lane group that holds the field's diagonal
        } else {
            bz = bias_acc[0];
            bz += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, bz), 0xB1, 0xF, 0xF, true));
            bz += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, bz), 0x4E, 0xF, 0xF, true));
            bz += __shfl_xor(bz, 16, kWave);
            bz += __shfl_xor(bz, 32, kWave);
        }
        bz *= 1.0f / kXsScale;
        // Lane (column c = lane & 15, group gq = lane >> 4) holds rows (rho = gq, phi = v) of column c in element v; the sum
        // it wants is the one whose phase is the column's own, of the field the column belongs to.
        float un = Field<NBITS>::unscale(0);
#pragma unroll
        for (int i = 1; i < F; ++i)
            un = ti == i ? Field<NBITS>::unscale(i) : un;
#pragma unroll
        for (int R = 0; R < 4; ++R) {
            f32x4 t = acc[R * F];
#pragma unroll
            for (int i = 1; i < F; ++i)
                t = ti == i ? acc[R * F + i] : t;
            float e = phi == 0 ? t[0] : (phi == 1 ? t[1] : (phi == 2 ? t[2] : t[3]));
            e += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, e), 0xB1, 0xF, 0xF, true));
            e += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, e), 0x4E, 0xF, 0xF, true));
            if (phi == 0 && tlane)
                red_lds[wave][4 * R + gq][0][ti] = __builtin_fmaf(e, un, -bz);
        }
    }
#pragma unroll
    for (int m = 0; m < (PHASE ? 0 : MT); ++m) {
        const float v = row16_sum(bias_acc[m]);
        if (tlane && kq == 0)
            bias_lds[wave][ti][m] = v * (1.0f / kXsScale);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (!PHASE && mcol < MT) {
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
    STRIP_STAMP(11);
    __syncthreads();
    STRIP_STAMP(12);

    const bool alone = p.BK == 1;
    const int tile = bz * p.RB + rb;
    f16 *const y_rows = Gd.y + (int64_t)pass * 2 * N; // the pass's first batch row
    // both projections rounded to fp16, SiLU in fp32 rounded once, product in fp16: as the reference's ops do
    auto gate = [](float a, float b) __attribute__((always_inline)) -> f16 {
        const float u = (float)(f16)a;
        const f16 act = (f16)(u / (1.0f + __expf(-u)));
        return act * (f16)b;
    };
    // two down projections, each rounded to fp16 and scaled by its routing weight, added in layer order: the bits
    // two launches with row_scale (the second accumulating) would give
    auto both = [&](float a, float b, int m, f16 prev) __attribute__((always_inline)) -> f16 {
        const f16 t0 = (f16)a * p.row_scale[m], t1 = (f16)b * p.row_scale[p.rs_lstride + m];
        return p.accumulate ? (f16)((f16)(prev + t0) + t1) : (f16)(t0 + t1);
    };

#ifdef HQQ_TUNING_BUILD
    auto write_stamps = [&]() __attribute__((always_inline)) {
        if (p.stamps && lane == 0) {
            unsigned long long *d = p.stamps + ((size_t)((bzi * gridDim.y + by) * gridDim.x + bx) * 16 + wave) * 16;
            for (int i = 0; i < 14; ++i)
                d[i] = st[i];
            d[14] = __builtin_amdgcn_s_getreg((31 << 11) | 4);  // HW_ID: wave, SIMD, CU, shader array and engine
            d[15] = __builtin_amdgcn_s_getreg((31 << 11) | 20); // XCC_ID
        }
    };
#endif
    // ---------------------------------------------------------------- a block that holds all of K finishes its tile
    // A thread per (tile row, batch row) adds the waves' sums in wave order and applies the epilogue.
    if (alone) {
        for (int u = threadIdx.x; u < 16 * MT; u += WAVES * 64) {
            const int r_t = u / MT, m_t = u % MT;
            if (m_t >= M)
                continue;
            float o[2][F];
#pragma unroll
            for (int i = 0; i < F; ++i)
                o[0][i] = o[1][i] = 0.f;
            for (int w = 0; w < p.KS; ++w) {
#pragma unroll
                for (int l = 0; l < (EPI == 0 ? 1 : 2); ++l) {
                    const float *src = &red_lds[l * p.KS + w][r_t][m_t][0];
#pragma unroll
                    for (int i = 0; i < F; ++i)
                        o[l][i] += src[i];
                }
            }
            const int r = 16 * rb + r_t;
            const int64_t n = (int64_t)F * (jp + (int64_t)r * GP); // outputs n .. n+F-1
            f16 *dst = y_rows + (int64_t)m_t * N + n;
            f16 hv[F];
#pragma unroll
            for (int i = 0; i < F; ++i) {
                if constexpr (EPI == 1) {
                    hv[i] = gate(o[0][i], o[1][i]);
                } else if constexpr (EPI == 2) {
                    hv[i] = both(o[0][i], o[1][i], m_t, p.accumulate ? dst[i] : (f16)0);
                } else {
                    f16 val = (f16)o[0][i];
                    if (Gd.bias)
                        val = val + Gd.bias[n + i];
                    if (p.row_scale)
                        val = val * p.row_scale[m_t];
                    if (p.accumulate)
                        val = dst[i] + val;
                    hv[i] = val;
                }
            }
            if (EPI == 0 && chain == CHAIN_FIRST) { // read by later blocks of this grid, on any XCD: stored at device scope
                if constexpr (F == 4)
                    chain_store(dst, (f16x4){hv[0], hv[1], hv[2], hv[3]});
                else
                    chain_store(dst, (f16x2){hv[0], hv[1]});
            } else if constexpr (F == 4) {
                *reinterpret_cast<f16x4 *>(dst) = (f16x4){hv[0], hv[1], hv[2], hv[3]};
            } else {
                *reinterpret_cast<f16x2 *>(dst) = (f16x2){hv[0], hv[1]};
            }
        }
#ifdef HQQ_TUNING_BUILD
        STRIP_STAMP(13);
        write_stamps();
#endif
        if (chain == CHAIN_FIRST) {
            CHAIN_STAMP(p.chain, 2);
            chain_signal(p.chain, CHAIN_FIRST_DONE, p.chain_blocks, CHAIN_GO_FIRST, kChainGoFirst);
        }
        if (chain != CHAIN_NONE)
            CHAIN_STAMP(p.chain, 3);
        return;
    }


    // ---------------------------------------------------------------- block tile: 16 lanes per (layer, row, batch row)
    for (int t = threadIdx.x; t < p.NL * 16 * MT * 16; t += WAVES * 64) {
        const int w = t & 15, u = t >> 4;
        const int l_t = u / (16 * MT), r_t = (u / MT) & 15, m_t = u % MT;
        float o[F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            o[i] = 0.f;
        if (w < p.KS) {
            const float *src = &red_lds[l_t * p.KS + w][r_t][m_t][0];
#pragma unroll
            for (int i = 0; i < F; ++i)
                o[i] = src[i];
        }
#pragma unroll
        for (int i = 0; i < F; ++i)
            o[i] = row16_sum(o[i]);
        if (w != 0 || m_t >= M)
            continue;
        const int r = 16 * rb + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * GP); // outputs n .. n+F-1
        if (EPI == 1 || !p.slots) {
            // device-scope stores: written through the (per-XCD, mutually non-coherent) L2 so that the finishing
            // block, which may run on another XCD, can read them without any cache-wide flush
            float *dst = (l_t ? Gd.part[1] : Gd.part[0]) + ((int64_t)kb * M + m_t) * N + n;
#pragma unroll
            for (int i = 0; i < F; ++i)
                __hip_atomic_store(dst + i, o[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        float *dst = &fin_lds[l_t][r_t][m_t][0];
#pragma unroll
        for (int i = 0; i < F; ++i)
            dst[i] = o[i];
    }

    // ---------------------------------------------------------------- accumulation slots: one atomic per output
    if constexpr (EPI != 1) {
        if (p.slots) {
            __syncthreads();
            for (int u = threadIdx.x; u < 16 * MT * F; u += WAVES * 64) {
                const int i = u % F, m_t = (u / F) % MT, r_t = u / (F * MT);
                if (m_t >= M)
                    continue;
                const int r = 16 * rb + r_t;
                const int64_t n = (int64_t)F * (jp + (int64_t)r * GP) + i;
                unsigned long long *slot = p.slots + (Gd.slot_begin + n * MT + m_t);
                // EPI 2: the routing weights are applied to the block's partial results in fp32, so the two experts
                // share a slot and the weighted sum is rounded to fp16 once
                float term = fin_lds[0][r_t][m_t][i];
                if constexpr (EPI == 2)
                    term = term * (float)p.row_scale[m_t] + fin_lds[1][r_t][m_t][i] * (float)p.row_scale[p.rs_lstride + m_t];
                const unsigned long long mine = slot_term(term);
                const unsigned long long before = __hip_atomic_fetch_add(slot, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (slot_count(before) != p.BK - 1)
                    continue;
                // this addition completed the slot: leave it ready for the next launch, write the output
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                f16 val = (f16)slot_total(before + mine, p.BK);
                if constexpr (EPI == 0) {
                    if (Gd.bias)
                        val = val + Gd.bias[n];
                    if (p.row_scale)
                        val = val * p.row_scale[m_t];
                }
                f16 *dst = y_rows + (int64_t)m_t * N + n;
                *dst = p.accumulate ? (f16)(*dst + val) : val;
            }
#ifdef HQQ_TUNING_BUILD
            STRIP_STAMP(13);
            write_stamps();
#endif
            return;
        }
    }

    // ---------------------------------------------------------------- the block that arrives last finishes the tile
    // The partial sums were stored at device scope; once those stores are acknowledged the arrival is counted
    // with a device-scope atomic.  No cache-wide write-back or invalidate is involved (a __threadfence here
    // flushes the whole L2 of the XCD and costs more than the matmul).
    __builtin_amdgcn_s_waitcnt(0); // vmcnt(0) expcnt(0) lgkmcnt(0): every store of this thread is acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(&p.counter[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == p.BK - 1) // every contributor has arrived: leave the counter ready for the next launch
            __hip_atomic_store(&p.counter[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket_lds = prev;
    }
    __syncthreads();
    if (ticket_lds != p.BK - 1)
        return;
    for (int u = threadIdx.x; u < 16 * MT; u += WAVES * 64) {
        const int r_t = u / MT, m_t = u % MT;
        if (m_t >= M)
            continue;
        const int r = 16 * rb + r_t;
        const int64_t n = (int64_t)F * (jp + (int64_t)r * GP);
        float a[F], b[F];
#pragma unroll
        for (int i = 0; i < F; ++i)
            a[i] = b[i] = 0.f;
        for (int s = 0; s < p.BK; ++s) { // fixed order: results do not depend on which block came last
            const int64_t off = ((int64_t)s * M + m_t) * N + n;
#pragma unroll
            for (int i = 0; i < F; ++i) {
                a[i] += __hip_atomic_load(Gd.part[0] + off + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if constexpr (EPI != 0)
                    b[i] += __hip_atomic_load(Gd.part[1] + off + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        f16 *dst = y_rows + (int64_t)m_t * N + n;
        f16 hv[F];
#pragma unroll
        for (int i = 0; i < F; ++i) {
            if constexpr (EPI == 1) {
                hv[i] = gate(a[i], b[i]);
            } else if constexpr (EPI == 2) {
                hv[i] = both(a[i], b[i], m_t, p.accumulate ? dst[i] : (f16)0);
            } else {
                f16 val = (f16)a[i];
                if (Gd.bias)
                    val = val + Gd.bias[n + i];
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

// (single rows, several slabs per wave, one in flight: the form chosen for launches of more blocks than compute
// units, which must fit four waves to a SIMD, i.e. stay within 128 registers, for two blocks to share a unit)
template <int NBITS, int MT, int S, int D, int WAVES, int SKIND, int ZKIND, int EPI, bool GROUPED = false, int NORM = 0>
__global__ __launch_bounds__(WAVES * 64, (MT == 1 && S > 1 && D == 1 && WAVES == 8) ? 4 : 1) void gemv_strip_kernel(StripParams p)
{
    strip_block<NBITS, MT, S, D, WAVES, SKIND, ZKIND, EPI, GROUPED, NORM>(p, (int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z, CHAIN_NONE);
}

// The attention part of a decoder layer at one token as ONE grid (chain_parts.hpp): blocks [0, nA) are the grouped
// q/k/v projections with the residual add and the input norm in front (first role), blocks [nA, nA + heads) one
// query head each (middle role), the rest the output projection (last role), which has its weights in registers by
// the time the heads are done.  Every block is 16 waves; a head uses the first NT threads.
struct ChainAttentionArgs {
    const f16 *q, *k, *v; // written by the first role, read by the middle one
    const f16 *cos_t, *sin_t;
    const int64_t *pos;
    f16 *cache_k, *cache_v;
    int64_t max_len;
    int group, heads;
    f16 *out; // written by the middle role, read by the last one (as its activations)
};
struct ChainParams {
    StripParams a, c;
    ChainAttentionArgs att;
    int nA;
};

template <int NBITS, int SKIND, int ZKIND, int HD, int NT>
__global__ __launch_bounds__(1024) void attention_chain_kernel(ChainParams P)
{
    const int L = (int)blockIdx.x;
    if (L < P.nA) {
        strip_block<NBITS, 1, 1, 1, 16, SKIND, ZKIND, 0, true, 1>(P.a, 0, L % P.a.RB, L / P.a.RB, CHAIN_FIRST);
    } else if (L < P.nA + P.att.heads) {
        if ((int)threadIdx.x < NT)
            attention_head<HD, NT>(P.att.q, P.att.k, P.att.v, P.att.cos_t, P.att.sin_t, P.att.pos, P.att.cache_k, P.att.cache_v,
                                   P.att.max_len, P.att.group, P.att.out, L - P.nA, CHAIN_MID, P.a.chain, P.att.heads);
    } else {
        const int c = L - P.nA - P.att.heads;
        strip_block<NBITS, 1, 1, 1, 16, SKIND, ZKIND, 0, true, 1>(P.c, 0, c % P.c.RB, c / P.c.RB, CHAIN_LAST);
    }
}

__global__ void zero_words_kernel(uint32_t *p, size_t n)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        p[i] = 0;
}

#ifdef HQQ_TUNING_BUILD
unsigned long long *g_strip_stamps = nullptr; // device buffer the launches write their waves' time stamps to
#endif

struct StripPlan {
    int F, GP, RB, NS, MT, S, D, WAVES, KS, BK, SKIND, ZKIND;
};

// tiles_all: tiles of the whole launch when it holds more groups than this layer's (0: this layer alone)
bool make_plan(const hqq_linear *l, int64_t M, int NL, StripPlan &pl, int64_t tiles_all = 0)
{
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
    pl.NS = (int)(l->K / kSlab);
    pl.MT = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
    if (pl.GP > 65535 || pl.RB > 65535 || (int64_t)pl.GP * pl.RB * sizeof(int) > kTileCounterBytes)
        return false;
    // Shape of the split: S slabs per wave, KS waves per layer, BK blocks along K.
    const int64_t tiles = tiles_all > 0 ? tiles_all : (int64_t)pl.GP * pl.RB;
    if (tiles * sizeof(int) > kTileCounterBytes)
        return false;
    const int max_waves = pl.MT == 1 ? 16 : 8; // wider batches need more registers and LDS staging per wave
    int S = 1, BK = 1;
    int KS = pl.NS;
    if (pl.MT <= 2) {
        // One and two rows (measured on the Mixtral projections): as many waves as the slabs of a compute unit's share
        // fill, one slab each, while that share is at most 16 slabs; beyond that two or four slabs per wave, the
        // later ones loaded while the earlier are worked on.  Two-layer blocks run best as eight waves of four
        // slabs, two blocks to a compute unit.  K is split over blocks when a block cannot hold it, or when there
        // would be fewer than about a hundred blocks.
        const int64_t share = tiles * pl.NS * NL / 256;
        S = NL == 2 ? 4 : (share <= 16 ? 1 : (share <= 32 ? 2 : 4));
        while (S > 1 && S > pl.NS)
            S /= 2;
        const int cap = NL == 2 && S == 4 ? 4 : max_waves / NL;
        const int groups = (pl.NS + S - 1) / S;
        KS = groups;
        while (KS > cap || (tiles * BK < 100 && KS > 4 && BK < 16)) {
            ++BK;
            KS = (groups + BK - 1) / BK;
        }
    } else {
        // One slab per wave unless a block that holds all of K would then need more than eight waves; K is split over
        // several blocks only when a single block cannot hold it or there would be too few blocks to cover the chip.
        // (two-layer blocks always take two slabs per wave: half the blocks along K, half the partial sums)
        if (KS * NL > max_waves && ((pl.NS + 1) / 2 * NL <= max_waves || (NL == 2 && pl.NS >= 2))) {
            S = 2;
            KS = (pl.NS + 1) / 2;
        }
        while (KS * NL > max_waves || (tiles * BK < 200 && KS > 4 && BK < 16)) {
            ++BK;
            KS = ((pl.NS + S - 1) / S + BK - 1) / BK;
        }
    }
    if (tuning_int("HQQ_STRIP_K", (int)l->K) == (int)l->K && tuning_int("HQQ_STRIP_NL", NL) == NL) {
        S = tuning_int("HQQ_STRIP_S", S);
        KS = tuning_int("HQQ_STRIP_KS", KS);
        BK = tuning_int("HQQ_STRIP_BK", BK);
    }
    if (S != 1 && S != 2 && !(S == 4 && pl.MT <= 2))
        return false;
    if (KS < 1 || KS * NL > max_waves || BK < 1 || BK > 65535)
        return false;
    if ((int64_t)S * KS * BK < pl.NS)
        return false;
    pl.S = S, pl.KS = KS, pl.BK = BK;
    pl.WAVES = KS * NL > 8 ? 16 : (KS * NL > 4 ? 8 : 4);
    // Slabs of a wave in flight at once: two, with one block to a compute unit; one when the launch has more blocks
    // than the chip has compute units (the gates of a token's two experts: 448), so that two blocks fit into a unit
    // (under 128 registers a wave) and cover each other's waits (measured on the 32-layer decode step: 440 -> 483 tok/s).
    pl.D = S < 2 ? S : 2;
    if (pl.MT == 1 && S > 1)
        pl.D = tuning_int("HQQ_STRIP_D", tiles * BK > 256 ? 1 : 2) == 1 ? 1 : 2;
    return true;
}

void fill_layer(StripLayer &L, const hqq_linear *l) { fill_layer_record(L, l); }

template <int NBITS, int MT, int S, int D, int WAVES, int EPI, bool GROUPED>
void launch_kinds(const StripParams &p, const StripPlan &pl, dim3 grid, hipStream_t s)
{
    if constexpr (GROUPED && EPI == 0 && MT == 1 && WAVES >= 4) {
        if (p.norm_weight) { // the fused norm exists for the grouped single-row projections only
            if (pl.SKIND == TK_F16)
                gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_F16, TK_F16, EPI, true, 1><<<grid, dim3(WAVES * 64), 0, s>>>(p);
            else
                gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_U8_COLS, TK_U8_SCALAR, EPI, true, 1><<<grid, dim3(WAVES * 64), 0, s>>>(p);
            return;
        }
    }
    if constexpr (GROUPED && EPI == 1 && MT == 1 && WAVES >= 4) {
        if (p.gate_w) { // the routed gate of the decode step
            if (pl.SKIND == TK_F16)
                gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_F16, TK_F16, EPI, true, 2><<<grid, dim3(WAVES * 64), 0, s>>>(p);
            else
                gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_U8_COLS, TK_U8_SCALAR, EPI, true, 2><<<grid, dim3(WAVES * 64), 0, s>>>(p);
            return;
        }
    }
    if (pl.SKIND == TK_F16)
        gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_F16, TK_F16, EPI, GROUPED><<<grid, dim3(WAVES * 64), 0, s>>>(p);
    else
        gemv_strip_kernel<NBITS, MT, S, D, WAVES, TK_U8_COLS, TK_U8_SCALAR, EPI, GROUPED><<<grid, dim3(WAVES * 64), 0, s>>>(p);
}

template <int NBITS, int MT, int S, int D, int EPI, bool GROUPED>
void launch_waves(const StripParams &p, const StripPlan &pl, dim3 grid, hipStream_t s)
{
    if constexpr (MT == 1) {
        if (pl.WAVES == 16) {
            launch_kinds<NBITS, MT, S, D, 16, EPI, GROUPED>(p, pl, grid, s);
            return;
        }
    }
    if (pl.WAVES >= 8)
        launch_kinds<NBITS, MT, S, D, 8, EPI, GROUPED>(p, pl, grid, s);
    else
        launch_kinds<NBITS, MT, S, D, 4, EPI, GROUPED>(p, pl, grid, s);
}

template <int NBITS, int MT, int EPI, bool GROUPED>
void launch_depth(const StripParams &p, const StripPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.S == 1)
        launch_waves<NBITS, MT, 1, 1, EPI, GROUPED>(p, pl, grid, s);
    else if (pl.S == 2 && (MT > 1 || pl.D == 2))
        launch_waves<NBITS, MT, 2, 2, EPI, GROUPED>(p, pl, grid, s);
    else if (pl.S == 2) {
        if constexpr (MT == 1)
            launch_waves<NBITS, MT, 2, 1, EPI, GROUPED>(p, pl, grid, s);
    } else if (MT > 1 || pl.D == 2) {
        if constexpr (MT <= 2)
            launch_waves<NBITS, MT, 4, 2, EPI, GROUPED>(p, pl, grid, s);
    } else {
        if constexpr (MT == 1)
            launch_waves<NBITS, MT, 4, 1, EPI, GROUPED>(p, pl, grid, s);
    }
}

// several groups in one launch and the two-expert sum exist for single-row batches only (the decode step)
template <int NBITS, int EPI, bool GROUPED>
void launch_batch(const StripParams &p, const StripPlan &pl, dim3 grid, hipStream_t s)
{
    if (pl.MT == 1) {
        launch_depth<NBITS, 1, EPI, GROUPED>(p, pl, grid, s);
        return;
    }
    if constexpr (!GROUPED && EPI != 2) {
        if (pl.MT == 2)
            launch_depth<NBITS, 2, EPI, false>(p, pl, grid, s);
        else
            launch_depth<NBITS, 4, EPI, false>(p, pl, grid, s);
    }
}

// What one launch covers: NG groups of NL layers each.  Shapes come from shape[g * NL + l]; the records come from
// the same descriptors, or from a device table when ix is given.
struct StripJob {
    const hqq_linear *shape[kMaxGroups];
    int NG, NL, EPI;
    const StripIndex *ix;
    int sel_gstride, sel_lstride, first_lstride;
    const f16 *x;
    int64_t x_lstride;
    f16 *y[kMaxGroups];
    const f16 *row_scale;
    int rs_lstride, accumulate;
    const f16 *norm_delta, *norm_weight; // norm_weight != null: activations = norm_weight * rmsnorm(x + norm_delta)
    f16 *x_sum;
    float norm_eps;
    const f16 *gate_w; // != null: routed gate launch (needs the norm fields and an index table)
    int n_experts;
    int *sel_out;
    f16 *rw_out;
};

bool same_family(const hqq_linear *a, const hqq_linear *b)
{
    return a->K == b->K && a->nbits == b->nbits && a->group_size == b->group_size &&
           table_kind(a->scale) == table_kind(b->scale) && table_kind(a->zero) == table_kind(b->zero);
}

// plan of the whole job (the split along K is common to every group) and the bytes of partial sums it needs
bool plan_job(const StripJob &j, int64_t M, StripPlan &pl, StripPlan *per_group, size_t &part_bytes)
{
    if (j.NG < 1 || j.NL < 1 || j.NL > 2 || j.NG * j.NL > kMaxGroups)
        return false;
    int64_t tiles = 0;
    for (int g = 0; g < j.NG; ++g) {
        StripPlan t;
        for (int l = 0; l < j.NL; ++l) {
            const hqq_linear *a = j.shape[g * j.NL + l];
            if (!a || !make_plan(a, M, j.NL, t) || !same_family(a, j.shape[0]) || a->N != j.shape[g * j.NL]->N)
                return false;
        }
        tiles += (int64_t)t.GP * t.RB;
    }
    if ((j.NG > 1 || j.EPI == 2) && M != 1)
        return false;
    part_bytes = 0;
    for (int g = 0; g < j.NG; ++g) {
        if (!make_plan(j.shape[g * j.NL], M, j.NL, per_group[g], tiles))
            return false;
        part_bytes += (size_t)j.NL * (size_t)per_group[g].BK * (size_t)M * (size_t)j.shape[g * j.NL]->N * sizeof(float);
    }
    pl = per_group[0];
    if (pl.BK == 1)
        part_bytes = 0;
    return true;
}

// the launch parameters, plan and grid of a job
int build_job(const StripJob &j, int64_t M, void *ws, size_t ws_bytes, StripParams &p, StripPlan &pl, dim3 &grid)
{
    StripPlan per_group[kMaxGroups];
    size_t part_bytes = 0;
    // A gate of three or four rows whose blocks hold all of K runs as two passes of the two-row kernel in one launch.
    int passes = 1;
    if ((M == 3 || M == 4) && j.EPI == 1 && j.NL == 2 && j.NG == 1 && !j.norm_weight &&
        !tuning_flag("HQQ_STRIP_NOPASS") && plan_job(j, 2, pl, per_group, part_bytes) &&
        pl.BK == 1 && 2 * per_group[0].GP <= 65535)
        passes = 2;
    if (passes == 1 && !plan_job(j, M, pl, per_group, part_bytes))
        return HQQ_E_UNSUPPORTED;
    const bool alone = pl.BK == 1;
    if (!alone && (!ws || ws_bytes < kHeadBytes + part_bytes))
        return HQQ_E_WORKSPACE;
    if (j.EPI == 2 && !j.row_scale)
        return HQQ_E_NULL;
    p = StripParams{};
    char *base = static_cast<char *>(ws);
    char *part = base + kHeadBytes;
    int z = 0;
    int64_t slot = 0;
    for (int g = 0; g < kMaxGroups; ++g) {
        StripGroup &G = p.grp[g];
        if (g >= j.NG) {
            G.z_begin = 0x7fffffff;
            continue;
        }
        const hqq_linear *a = j.shape[g * j.NL];
        G.z_begin = z, G.GP = per_group[g].GP, G.N = (int)a->N;
        G.slot_begin = (int)slot;
        slot += a->N * pl.MT;
        G.y = j.y[g];
        G.bias = j.EPI == 0 ? static_cast<const f16 *>(a->bias) : nullptr;
        for (int l = 0; l < j.NL; ++l) {
            fill_layer(p.layer[g * j.NL + l], j.shape[g * j.NL + l]);
            if (!alone) {
                G.part[l] = reinterpret_cast<float *>(part);
                part += (size_t)pl.BK * (size_t)M * (size_t)a->N * sizeof(float);
            }
        }
        z += per_group[g].GP;
    }
    if (j.NL == 1) // the single-group kernel picks between records 0 and 1 by the wave's layer
        for (int g = j.NG; g < kMaxGroups; ++g)
            p.layer[g] = p.layer[0];
    if (z > 65535)
        return HQQ_E_UNSUPPORTED;
    if (j.ix) {
        p.table = static_cast<const StripLayer *>(j.ix->table);
        p.sel = j.ix->sel;
        p.table_stride = j.ix->stride, p.table_first = j.ix->first;
        p.sel_gstride = j.sel_gstride, p.sel_lstride = j.sel_lstride, p.first_lstride = j.first_lstride;
    }
    p.x = j.x, p.x_lstride = (int)j.x_lstride, p.M = (int)M, p.K = (int)j.shape[0]->K;
    p.passes = passes;
    p.RB = pl.RB, p.NS = pl.NS, p.KS = pl.KS, p.BK = pl.BK, p.NL = j.NL;
    p.counter = reinterpret_cast<int *>(base);
    // plain or weighted-pair epilogue, K over at most eight blocks, every output of the launch has a slot: no
    // partial sums
    if (!alone && ((j.EPI == 0 && j.NL == 1) || (j.EPI == 2 && j.NL == 2 && j.NG == 1)) && pl.BK <= 8 && slot * (int64_t)sizeof(unsigned long long) <= (int64_t)kSlotBytes)
        p.slots = reinterpret_cast<unsigned long long *>(base + kCounterBytes);
    p.row_scale = j.row_scale, p.rs_lstride = j.rs_lstride, p.accumulate = j.accumulate;
#ifdef HQQ_TUNING_BUILD
    p.skip = tuning_int("HQQ_STRIP_SKIP", 0);
    p.stamps = g_strip_stamps;
#endif
    if (j.norm_weight) {
        // every launch shape the planner can pick for these jobs has the fused-norm form except blocks under four waves
        const bool plain = j.EPI == 0 && j.NL == 1 && !j.gate_w;
        const bool routed = j.EPI == 1 && j.NL == 2 && j.NG == 2 && j.gate_w && j.ix && j.sel_out && j.rw_out &&
                            j.n_experts >= 2 && j.n_experts <= 8 && j.shape[0]->K <= 4096 && j.shape[0]->K % 8 == 0;
        if ((!plain && !routed) || M != 1 || pl.WAVES < 4 || !j.x_sum)
            return HQQ_E_UNSUPPORTED;
        p.norm_delta = j.norm_delta, p.norm_weight = j.norm_weight, p.x_sum = j.x_sum, p.norm_eps = j.norm_eps;
        p.gate_w = j.gate_w, p.n_experts = j.n_experts, p.sel_out = j.sel_out, p.rw_out = j.rw_out;
    }
    grid = dim3((unsigned)pl.BK, (unsigned)pl.RB, (unsigned)(z * passes));
    return HQQ_OK;
}

int run_job(const StripJob &j, int64_t M, void *ws, size_t ws_bytes, hipStream_t s)
{
    StripParams p;
    StripPlan pl;
    dim3 grid;
    const int rc = build_job(j, M, ws, ws_bytes, p, pl, grid);
    if (rc != HQQ_OK)
        return rc;
    const bool two = j.shape[0]->nbits == 2;
    if (j.NG > 1 || j.norm_weight) {
        if (j.EPI == 0 && j.NL == 1)
            two ? launch_batch<2, 0, true>(p, pl, grid, s) : launch_batch<4, 0, true>(p, pl, grid, s);
        else if (j.EPI == 1 && j.NL == 2)
            two ? launch_batch<2, 1, true>(p, pl, grid, s) : launch_batch<4, 1, true>(p, pl, grid, s);
        else
            return HQQ_E_UNSUPPORTED;
    } else if (j.EPI == 0 && j.NL == 1) {
        two ? launch_batch<2, 0, false>(p, pl, grid, s) : launch_batch<4, 0, false>(p, pl, grid, s);
    } else if (j.EPI == 1 && j.NL == 2) {
        two ? launch_batch<2, 1, false>(p, pl, grid, s) : launch_batch<4, 1, false>(p, pl, grid, s);
    } else if (j.EPI == 2 && j.NL == 2) {
        two ? launch_batch<2, 2, false>(p, pl, grid, s) : launch_batch<4, 2, false>(p, pl, grid, s);
    } else {
        return HQQ_E_UNSUPPORTED;
    }
    return launch_status();
}

} // namespace

// Batches of three rows and more go to the batch kernel (gemv_batch.hip) where it takes the shape.
static bool use_batch(const hqq_linear *l, int64_t M) { return M >= 3 && !tuning_flag("HQQ_BATCH_OFF") && batch_supported(l, M); }

bool strip_supported(const hqq_linear *l, int64_t M)
{
    StripPlan pl;
    return make_plan(l, M, 1, pl) || use_batch(l, M);
}

bool strip_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    if (M >= 3 && !tuning_flag("HQQ_BATCH_OFF") && batch_gate_supported(w1, w3, M))
        return true;
    StripPlan a, b;
    return make_plan(w1, M, 2, a) && make_plan(w3, M, 2, b) && same_family(w1, w3) && w1->N == w3->N;
}

size_t strip_workspace_bytes(const hqq_linear *l, int64_t M)
{
    StripPlan pl;
    if (!make_plan(l, M, 1, pl))
        return use_batch(l, M) ? batch_workspace_bytes(l, M) : 0;
    // sized for the worst split the planner may choose for this shape (one slab per wave and block)
    return kHeadBytes + (size_t)pl.NS * (size_t)M * (size_t)l->N * sizeof(float);
}

int launch_strip_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                        const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix)
{
    if (use_batch(l, M))
        return launch_batch_matmul(l, x, M, y, ws, ws_bytes, ep, s, ix);
    StripJob j = {};
    j.shape[0] = l, j.NG = 1, j.NL = 1, j.EPI = 0, j.ix = ix, j.first_lstride = 1;
    j.x = x, j.y[0] = y, j.row_scale = ep.row_scale, j.accumulate = ep.accumulate;
    return run_job(j, M, ws, ws_bytes, s);
}

size_t strip_record_bytes() { return sizeof(StripLayer); }

void strip_fill_record(void *dst, const hqq_linear *l) { fill_layer(*static_cast<StripLayer *>(dst), l); }

int launch_strip_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                         size_t ws_bytes, hipStream_t s, const StripIndex *ix)
{
    if (M >= 3 && !tuning_flag("HQQ_BATCH_OFF") && batch_gate_supported(w1, w3, M))
        return launch_batch_gate_up(w1, w3, x, M, h, ws, ws_bytes, s, ix);
    StripJob j = {};
    j.shape[0] = w1, j.shape[1] = w3, j.NG = 1, j.NL = 2, j.EPI = 1, j.ix = ix, j.first_lstride = 1;
    j.x = x, j.y[0] = h;
    return run_job(j, M, ws, ws_bytes, s);
}

// The gates of the experts sel[0] and sel[1] of a record table in one launch: h[e] = silu(w1_e x) * w3_e x.
int launch_strip_gate_up_pair(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, f16 *h0, f16 *h1, void *ws,
                              size_t ws_bytes, hipStream_t s, const StripIndex &ix)
{
    StripJob j = {};
    j.shape[0] = j.shape[2] = w1, j.shape[1] = j.shape[3] = w3;
    j.NG = 2, j.NL = 2, j.EPI = 1, j.ix = &ix, j.sel_gstride = 1, j.first_lstride = 1;
    j.x = x, j.y[0] = h0, j.y[1] = h1;
    return run_job(j, 1, ws, ws_bytes, s);
}

// The same launch with the post-attention norm and the router in front of it: every block forms
// weight * rmsnorm(x + delta), routes it over gate_w (n_experts x K) and takes the gates of the two experts chosen;
// x + delta goes to x_sum, the choice to sel_out[2] and the routing weights to rw_out[2].
int launch_strip_gate_up_pair_routed(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, const StripNorm &norm,
                                     const f16 *gate_w, int n_experts, int *sel_out, f16 *rw_out, f16 *h0, f16 *h1,
                                     void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix)
{
    StripJob j = {};
    j.shape[0] = j.shape[2] = w1, j.shape[1] = j.shape[3] = w3;
    j.NG = 2, j.NL = 2, j.EPI = 1, j.ix = &ix, j.sel_gstride = 1, j.first_lstride = 1;
    j.x = x, j.y[0] = h0, j.y[1] = h1;
    j.norm_delta = norm.delta, j.norm_weight = norm.weight, j.x_sum = norm.x_sum, j.norm_eps = norm.eps;
    j.gate_w = gate_w, j.n_experts = n_experts, j.sel_out = sel_out, j.rw_out = rw_out;
    if (!norm.weight || !gate_w)
        return HQQ_E_NULL;
    return run_job(j, 1, ws, ws_bytes, s);
}

// y (+)= w2_{sel[0]} h0 * row_scale[0] + w2_{sel[1]} h1 * row_scale[1] in one launch; h1 = h0 + h_stride.
int launch_strip_down_pair(const hqq_linear *w2, const f16 *h0, int64_t h_stride, f16 *y, const f16 *row_scale,
                           int accumulate, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix)
{
    StripJob j = {};
    j.shape[0] = j.shape[1] = w2;
    j.NG = 1, j.NL = 2, j.EPI = 2, j.ix = &ix, j.sel_lstride = 1, j.first_lstride = 0;
    j.x = h0, j.x_lstride = h_stride, j.y[0] = y, j.row_scale = row_scale, j.rs_lstride = 1, j.accumulate = accumulate;
    return run_job(j, 1, ws, ws_bytes, s);
}

// Up to four projections of the same K, code width and group size applied to the same single row in one launch.
// With norm: the row is norm->weight * rmsnorm(x + norm->delta), and x + delta is written to norm->x_sum.
int launch_strip_group(const hqq_linear *const *layers, int count, const f16 *x, f16 *const *ys, void *ws,
                       size_t ws_bytes, hipStream_t s, const StripNorm *norm)
{
    if (count < 1 || count > kMaxGroups)
        return HQQ_E_UNSUPPORTED;
    StripJob j = {};
    for (int g = 0; g < count; ++g)
        j.shape[g] = layers[g], j.y[g] = ys[g];
    j.NG = count, j.NL = 1, j.EPI = 0, j.x = x;
    if (norm) {
        if (!norm->weight || !norm->x_sum || layers[0]->K % 8 != 0)
            return HQQ_E_UNSUPPORTED;
        j.norm_delta = norm->delta, j.norm_weight = norm->weight, j.x_sum = norm->x_sum, j.norm_eps = norm->eps;
    }
    return run_job(j, 1, ws, ws_bytes, s);
}

// The attention part of a decoder layer at one token in one launch (attention_chain_kernel).  Taken for the shapes
// the decode step has: 4-bit projections whose blocks hold all of K in 16 waves of one slab each, heads of 128.
static int plan_attention_chain(const AttentionChain &c, void *ws, size_t ws_bytes, ChainParams &P, int &blocks, int &nt)
{
    if (!c.q || !c.k || !c.v || !c.o)
        return HQQ_E_NULL;
    // (caches the attention launch splits over several blocks per head are left to it: the chain has one block per head)
    if (c.head_dim != 128 || c.n_heads < 1 || c.n_kv_heads < 1 || c.n_heads % c.n_kv_heads != 0 || c.max_len < 1 ||
        attention_parts(c.max_len) != 1)
        return HQQ_E_UNSUPPORTED;
    if (c.q->N != (int64_t)c.n_heads * c.head_dim || c.k->N != (int64_t)c.n_kv_heads * c.head_dim || c.v->N != c.k->N ||
        c.o->K != c.q->N || c.q->nbits != 4 || !same_family(c.q, c.o))
        return HQQ_E_UNSUPPORTED;
    if (c.q->bias || c.k->bias || c.v->bias || c.o->bias || c.q->K % 8 != 0)
        return HQQ_E_UNSUPPORTED;
    StripJob ja = {};
    ja.shape[0] = c.q, ja.shape[1] = c.k, ja.shape[2] = c.v;
    ja.y[0] = c.q_out, ja.y[1] = c.k_out, ja.y[2] = c.v_out;
    ja.NG = 3, ja.NL = 1, ja.EPI = 0, ja.x = c.x;
    ja.norm_delta = c.delta, ja.norm_weight = c.norm_weight, ja.x_sum = c.x_sum, ja.norm_eps = c.eps;
    StripJob jc = {};
    jc.shape[0] = c.o, jc.y[0] = c.y, jc.NG = 1, jc.NL = 1, jc.EPI = 0, jc.x = c.att_out;
    StripPlan pa, pc;
    dim3 ga, gc;
    int rc;
    if ((rc = build_job(ja, 1, ws, ws_bytes, P.a, pa, ga)) != HQQ_OK || (rc = build_job(jc, 1, ws, ws_bytes, P.c, pc, gc)) != HQQ_OK)
        return rc;
    for (const StripPlan *pl : {&pa, &pc})
        if (pl->MT != 1 || pl->S != 1 || pl->D != 1 || pl->WAVES != 16 || pl->BK != 1)
            return HQQ_E_UNSUPPORTED;
    if (pa.SKIND != pc.SKIND || pa.ZKIND != pc.ZKIND)
        return HQQ_E_UNSUPPORTED;
    if (!ws || ws_bytes < kHeadBytes)
        return HQQ_E_WORKSPACE;
    // the chain's counters: the last words of the counter region (tile counters are not used by blocks that hold all of K)
    static_assert(CHAIN_WORDS * sizeof(int) <= kChainBytes, "the chain's words fit the space kept for them");
    int *chain = reinterpret_cast<int *>(static_cast<char *>(ws) + kCounterBytes) - CHAIN_WORDS;
    P.nA = (int)(ga.y * ga.z);
    const int nC = (int)(gc.y * gc.z);
    P.a.chain = P.c.chain = chain;
    P.a.chain_blocks = P.nA, P.c.chain_blocks = nC;
    P.att = ChainAttentionArgs{c.q_out, c.k_out, c.v_out, c.cos_t, c.sin_t, c.pos, c.cache_k, c.cache_v, c.max_len,
                               c.n_heads / c.n_kv_heads, c.n_heads, c.att_out};
    if (!aligned16(c.cache_k) || !aligned16(c.cache_v) || !aligned16(c.att_out) || (reinterpret_cast<uintptr_t>(c.q_out) & 3u) ||
        (reinterpret_cast<uintptr_t>(c.k_out) & 3u) || (reinterpret_cast<uintptr_t>(c.v_out) & 3u))
        return HQQ_E_ALIGN;
    blocks = P.nA + c.n_heads + nC;
    nt = attention_block_threads(c.max_len);
    return HQQ_OK;
}

size_t attention_chain_error_offset() { return kCounterBytes - (CHAIN_WORDS - CHAIN_ERROR) * sizeof(int); }

int launch_attention_chain(const AttentionChain &c, void *ws, size_t ws_bytes, hipStream_t s)
{
    ChainParams P;
    int blocks = 0, nt = 0;
    const int rc = plan_attention_chain(c, ws, ws_bytes, P, blocks, nt);
    if (rc != HQQ_OK)
        return rc;
    const size_t lds = (size_t)c.max_len * sizeof(float);
    const bool f16_tables = table_kind(c.q->scale) == TK_F16;
    if (nt == 256) {
        if (f16_tables)
            attention_chain_kernel<4, TK_F16, TK_F16, 128, 256><<<blocks, 1024, lds, s>>>(P);
        else
            attention_chain_kernel<4, TK_U8_COLS, TK_U8_SCALAR, 128, 256><<<blocks, 1024, lds, s>>>(P);
    } else {
        if (f16_tables)
            attention_chain_kernel<4, TK_F16, TK_F16, 128, 1024><<<blocks, 1024, lds, s>>>(P);
        else
            attention_chain_kernel<4, TK_U8_COLS, TK_U8_SCALAR, 128, 1024><<<blocks, 1024, lds, s>>>(P);
    }
    return launch_status();
}

// bytes of workspace the three launches above can need for these shapes (0 when the strip kernel does not take them)
size_t strip_job_workspace_bytes(const hqq_linear *const *layers, int count, int NL, int64_t M)
{
    if (count < 1 || count > kMaxGroups)
        return 0;
    StripJob j = {};
    for (int g = 0; g < count; ++g)
        j.shape[g] = layers[g];
    j.NL = NL, j.NG = count / NL;
    StripPlan pl, per_group[kMaxGroups];
    size_t part = 0;
    if (!plan_job(j, M, pl, per_group, part))
        return 0;
    return kHeadBytes + part;
}

int launch_zero_workspace_head(void *ws, size_t ws_bytes, hipStream_t s)
{
    const size_t n = (ws_bytes < kHeadBytes ? ws_bytes : kHeadBytes) / 4;
    if (n == 0)
        return HQQ_OK;
    zero_words_kernel<<<16, 256, 0, s>>>(static_cast<uint32_t *>(ws), n);
    return launch_status();
}

size_t workspace_head_bytes() { return kHeadBytes; }

#ifdef HQQ_TUNING_BUILD
extern "C" void hqq_tuning_strip_stamps(void *buf) { g_strip_stamps = static_cast<unsigned long long *>(buf); }
#endif

} // namespace hqq
