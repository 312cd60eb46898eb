// Reader of (G, K) scale / zero tables, four columns per lane: shared by the kernels that walk K in 64-column steps.
#pragma once

#include "hqq_common.hpp"

namespace hqq {

// How the two tables of a layer are stored; the common cases get branch-free code.
enum { TM_GENERIC = 0, TM_HQQ8 = 1 /* scale: u8 + per-column meta, zero: u8 + scalar meta */, TM_F16 = 2 };

// Reader of one (G, K) table for the four columns a lane owns.  KIND: 0 runtime flags, 1 u8 with per-column
// meta, 2 u8 with scalar meta, 3 fp16.
template <int KIND> struct TableCursor {
    const uint8_t *u8;
    const f16 *f;
    const f16 *ms, *mz;
    uint32_t c;    // flat index j*K + k of the lane's first column
    uint32_t cm;   // c % meta_cols
    uint32_t cols; // meta_cols
    bool is_u8, scalar;
    f16x2 ms_s, mz_s; // scalar meta, splat

    __device__ __forceinline__ void init(const Table &t, uint32_t c0, uint32_t cols_inv)
    {
        is_u8 = KIND == 0 ? t.kind == HQQ_TABLE_U8 : KIND != 3;
        u8 = static_cast<const uint8_t *>(t.data);
        f = static_cast<const f16 *>(t.data);
        ms = t.ms, mz = t.mz;
        cols = (uint32_t)t.meta_cols;
        scalar = KIND == 0 ? (is_u8 && cols == 1) : KIND == 2;
        c = c0;
        cm = 0;
        if (is_u8 && !scalar) { // c0 mod cols: the quotient estimate is at most 2 short
            cm = c0 - __umulhi(c0, cols_inv) * cols;
            if (cm >= cols)
                cm -= cols;
            if (cm >= cols)
                cm -= cols;
        }
        if (scalar) {
            ms_s = (f16x2){ms[0], ms[0]};
            mz_s = (f16x2){mz[0], mz[0]};
        }
    }
    __device__ __forceinline__ void advance(uint32_t d)
    {
        c += d;
        if (is_u8 && !scalar) {
            cm += d; // d <= cols
            if (cm >= cols)
                cm -= cols;
        }
    }
};

struct TableRaw {
    u32x2 data;  // 4 bytes (u8 table) or 4 halves (fp16 table)
    u32x2 ms, mz; // 4 halves each (u8 table with per-column meta)
};

template <int KIND> __device__ __forceinline__ TableRaw table_load(const TableCursor<KIND> &t)
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
template <int KIND>
__device__ __forceinline__ void table_decode(const TableCursor<KIND> &t, const TableRaw &r, f16x2 &lo, f16x2 &hi)
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

} // namespace hqq
