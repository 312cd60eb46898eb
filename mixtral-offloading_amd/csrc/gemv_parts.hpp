// Pieces shared by the decode GEMV kernels: table decoding (16 entries per lane, 128-bit loads), the in-place
// "code as fp16 subnormal" fields and the 16-lane DPP sum.
#pragma once

#include "hqq_common.hpp"

namespace hqq {
namespace gemv {

constexpr int kSlab = 256;           // columns per wave
constexpr float kXsScale = 32.0f;    // xs = 32 * s * x keeps small activations out of the fp16 subnormal range
// Head of every workspace, zero between launches: one arrival counter per tile, then the accumulation slots of the
// split-K decode launches (one 64-bit word per output of the launch).
constexpr size_t kCounterBytes = 64 * 1024;
// the last 4 KB of the counter region hold the words of chained launches (chain_parts.hpp): tile counters stay below
constexpr size_t kChainBytes = 4 * 1024;
constexpr size_t kTileCounterBytes = kCounterBytes - kChainBytes;
constexpr size_t kSlotBytes = 512 * 1024;
constexpr size_t kHeadBytes = kCounterBytes + kSlotBytes;
// A slot holds the sum of the K blocks' partial results as a fixed-point number (26 fractional bits, kept in bits
// 8..55; magnitudes up to 2^17 per contribution, at most 15 of them) and, above bit 56, the number of blocks that
// have added theirs.  Integer addition is exact, so the total does not depend on the order of arrival; the block whose
// addition completes a slot reads the total out of the value its own atomic returns, writes the output and clears the
// slot: one trip to memory instead of three (partial sums, arrival counter, partial sums again).
// A contribution that has no fixed-point form is counted instead, in the low byte: bits 0..3 count those beyond
// +2^17 (the fp16 result is +inf whatever the others add), bits 4..7 those beyond -2^17, and a NaN counts in both --
// the total is then +inf, -inf, or NaN when both kinds met, as a floating-point sum of the same terms would be.
constexpr int kSlotFracBits = 26;
constexpr float kSlotLimit = 131071.0f;
constexpr unsigned long long kSlotOne = 1ull << 56;
__device__ __forceinline__ unsigned long long slot_term(float v)
{
    if (!(v <= kSlotLimit)) // beyond +2^17, or NaN
        return kSlotOne + (v != v ? 0x11ull : 0x01ull);
    if (v < -kSlotLimit)
        return kSlotOne + 0x10ull;
    const long long fx = (long long)__builtin_rintf(v * (float)(1u << kSlotFracBits)) * 256; // exact scaling by 2^26
    return kSlotOne + (unsigned long long)fx;
}
__device__ __forceinline__ int slot_count(unsigned long long word) { return (int)((word + (1ull << 55)) >> 56); }
__device__ __forceinline__ float slot_total(unsigned long long word, int count)
{
    const unsigned flags = (unsigned)word & 0xFFu;
    if (flags) {
        const bool pos = (flags & 0x0Fu) != 0, neg = (flags & 0xF0u) != 0;
        return pos && neg ? __builtin_nanf("") : (pos ? __builtin_inff() : -__builtin_inff());
    }
    const long long fx = (long long)(word - ((unsigned long long)count << 56));
    return (float)((double)fx * (1.0 / (double)(1ull << (kSlotFracBits + 8))));
}

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

// Load through a pointer known to be device memory.  A pointer that reaches the kernel inside a record (selected
// between two kernel arguments, or read from a table) has lost its address space, and the compiler then emits flat
// loads: those count on both memory counters, so the first wait for an LDS operation would also wait for every
// weight load still in flight.
template <typename T> __device__ __forceinline__ T gload(const void *p)
{
    return *(const T __attribute__((address_space(1))) *)(p);
}

template <int KIND>
__device__ __forceinline__ void load16(Raw16<KIND> &r, const uint8_t *tab, const f16 *ms, const f16 *mz, uint32_t c,
                                       uint32_t cm)
{
    if constexpr (KIND == TK_F16) {
        const u32x4 *p = reinterpret_cast<const u32x4 *>(reinterpret_cast<const f16 *>(tab) + c);
        r.q = gload<u32x4>(p);
        r.q_hi = gload<u32x4>(p + 1);
    } else {
        r.q = gload<u32x4>(tab + c);
        if constexpr (KIND == TK_U8_COLS) {
            const u32x4 *a = reinterpret_cast<const u32x4 *>(ms + cm);
            const u32x4 *b = reinterpret_cast<const u32x4 *>(mz + cm);
            r.ms[0] = gload<u32x4>(a), r.ms[1] = gload<u32x4>(a + 1);
            r.mz[0] = gload<u32x4>(b), r.mz[1] = gload<u32x4>(b + 1);
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


inline int table_kind(const hqq_table &t) { return t.kind == HQQ_TABLE_F16 ? TK_F16 : (t.meta_cols == 1 ? TK_U8_SCALAR : TK_U8_COLS); }

} // namespace gemv
} // namespace hqq
