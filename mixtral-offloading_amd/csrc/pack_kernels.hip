// Bit packers, 8-bit table expansion and the bit-exact de-quantiser.
//
// These are streaming byte kernels, bounded by HBM: every thread moves whole
// 32-bit or 128-bit words and does its bit work on four codes per lane-op.
// Layouts follow the reference packers (src/packing.py:10-97).
#include "gemv_parts.hpp"
#include "hqq_common.hpp"
#include "table_reader.hpp"

namespace hqq {
namespace {

constexpr int kThreads = 256;

// the same byte mask in every byte of a word, for scalar bytes and 128-bit words
template <typename WordT> __device__ __forceinline__ WordT byte_mask(uint32_t b)
{
    if constexpr (sizeof(WordT) == 1) {
        return (WordT)b;
    } else {
        const uint32_t m = b * 0x01010101u;
        WordT r = {m, m, m, m};
        return r;
    }
}

// ---------------------------------------------------------------- 4 / 2 bit
// One thread handles VEC consecutive columns of one packed row.
template <int NBITS, typename WordT>
__global__ __launch_bounds__(kThreads) void unpack_u8_kernel(const uint8_t *__restrict__ in, int64_t prows,
                                                             int64_t cols, uint8_t *__restrict__ out)
{
    constexpr int F = 8 / NBITS;
    constexpr int VEC = sizeof(WordT);
    const int64_t chunks = cols / VEC;
    const int64_t total = prows * chunks;
    for (int64_t idx = blockIdx.x * (int64_t)kThreads + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * kThreads) {
        const int64_t p = idx / chunks, c = (idx - p * chunks) * VEC;
        const WordT w = *reinterpret_cast<const WordT *>(in + p * cols + c);
#pragma unroll
        for (int i = 0; i < F; ++i) {
            WordT v;
            if constexpr (NBITS == 4)
                v = (WordT)(w >> (4 * (1 - i))) & byte_mask<WordT>(0x0Fu);
            else
                v = (WordT)(w >> (2 * (3 - i))) & byte_mask<WordT>(0x03u);
            *reinterpret_cast<WordT *>(out + (F * p + i) * cols + c) = v;
        }
    }
}

template <int NBITS, typename WordT>
__global__ __launch_bounds__(kThreads) void pack_u8_kernel(const uint8_t *__restrict__ q, int64_t prows, int64_t cols,
                                                           uint8_t *__restrict__ out)
{
    constexpr int F = 8 / NBITS;
    constexpr int VEC = sizeof(WordT);
    const int64_t chunks = cols / VEC;
    const int64_t total = prows * chunks;
    for (int64_t idx = blockIdx.x * (int64_t)kThreads + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * kThreads) {
        const int64_t p = idx / chunks, c = (idx - p * chunks) * VEC;
        WordT acc = byte_mask<WordT>(0);
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const WordT v = *reinterpret_cast<const WordT *>(q + (F * p + i) * cols + c);
            // uint8 shift as in the reference: bits pushed past bit 7 are lost, the last row is OR-ed unmasked
            const int sh = NBITS * (F - 1 - i);
            acc |= (WordT)(v << sh) & byte_mask<WordT>((0xFFu << sh) & 0xFFu);
        }
        *reinterpret_cast<WordT *>(out + p * cols + c) = acc;
    }
}

// ------------------------------------------------------------------- 3 bit
// One thread handles VEC consecutive columns of one word row: VEC words in,
// VEC bytes to each of ten unpacked rows (or the reverse).
template <int VEC>
__global__ __launch_bounds__(kThreads) void unpack3_kernel(const uint32_t *__restrict__ in, int64_t words,
                                                           int64_t cols, uint8_t *__restrict__ out)
{
    const int64_t chunks = cols / VEC;
    const int64_t total = words * chunks;
    for (int64_t idx = blockIdx.x * (int64_t)kThreads + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * kThreads) {
        const int64_t p = idx / chunks, c = (idx - p * chunks) * VEC;
        uint32_t w[VEC];
        if constexpr (VEC == 4) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(in + p * cols + c);
            w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
        } else {
            w[0] = in[p * cols + c];
        }
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            const int sh = 3 * (9 - i);
            uint8_t *dst = out + (10 * p + i) * cols + c;
            if constexpr (VEC == 4) {
                const uint32_t b = ((w[0] >> sh) & 7u) | (((w[1] >> sh) & 7u) << 8) | (((w[2] >> sh) & 7u) << 16) |
                                   (((w[3] >> sh) & 7u) << 24);
                *reinterpret_cast<uint32_t *>(dst) = b;
            } else {
                *dst = (uint8_t)((w[0] >> sh) & 7u);
            }
        }
    }
}

template <int VEC>
__global__ __launch_bounds__(kThreads) void pack3_kernel(const uint8_t *__restrict__ q, int64_t rows, int64_t cols,
                                                         uint32_t *__restrict__ out)
{
    const int64_t words = (rows + 9) / 10;
    const int64_t chunks = cols / VEC;
    const int64_t total = words * chunks;
    for (int64_t idx = blockIdx.x * (int64_t)kThreads + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * kThreads) {
        const int64_t p = idx / chunks, c = (idx - p * chunks) * VEC;
        uint32_t w[VEC] = {};
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            const int64_t r = 10 * p + i;
            if (r < rows) { // lanes past the last row stay zero
                const int sh = 3 * (9 - i);
                if constexpr (VEC == 4) {
                    const uint32_t b = *reinterpret_cast<const uint32_t *>(q + r * cols + c);
                    // codes are widened to 32 bits and shifted unmasked, as the reference does
                    w[0] |= (b & 0xFFu) << sh;
                    w[1] |= ((b >> 8) & 0xFFu) << sh;
                    w[2] |= ((b >> 16) & 0xFFu) << sh;
                    w[3] |= (b >> 24) << sh;
                } else {
                    w[0] |= (uint32_t)q[r * cols + c] << sh;
                }
            }
        }
        if constexpr (VEC == 4) {
            u32x4 v;
            v.x = w[0], v.y = w[1], v.z = w[2], v.w = w[3];
            *reinterpret_cast<u32x4 *>(out + p * cols + c) = v;
        } else {
            out[p * cols + c] = w[0];
        }
    }
}

// ------------------------------------------------------- table -> fp16
__global__ __launch_bounds__(kThreads) void table_to_f16_kernel(Table t, int64_t count, f16 *__restrict__ out)
{
    for (int64_t i = blockIdx.x * (int64_t)kThreads + threadIdx.x; i < count; i += (int64_t)gridDim.x * kThreads)
        out[i] = table_at(t, i);
}

// ------------------------------------------------------- de-quantise
// W[n,k] = fp16(fp16(q - Z[n%G,k]) * S[n%G,k]); one thread per (word, 4 columns).
template <int NBITS>
__global__ __launch_bounds__(kThreads) void dequantize_kernel(const void *__restrict__ codes, Table sc, Table zr,
                                                              int64_t N, int64_t K, int64_t G, f16 *__restrict__ w)
{
    constexpr int F = NBITS == 3 ? 10 : 8 / NBITS;
    const int64_t prows = (N + F - 1) / F;
    const int64_t kchunks = (K + 3) / 4;
    const int64_t total = prows * kchunks;
    for (int64_t idx = blockIdx.x * (int64_t)kThreads + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * kThreads) {
        const int64_t p = idx / kchunks, k0 = (idx - p * kchunks) * 4;
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const int64_t n = F * p + i;
            if (n >= N)
                break;
            const int64_t j = n % G;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t k = k0 + e;
                if (k < K) {
                    const f16 q = (f16)(float)code_at<NBITS>(codes, n, k, K);
                    const f16 d = q - table_at(zr, j * K + k); // first rounding
                    w[n * K + k] = d * table_at(sc, j * K + k); // second rounding
                }
            }
        }
    }
}

// The same values for the usual shapes, moving whole words: one thread owns four columns of one packed row, turns
// the row's codes into fp16 with byte permutes (0x6400 | b is 1024 + b), reads four entries of each table per
// weight row and stores four halves per weight row.  Needs K % 4 == 0, G*K < 2^32 and, for 8-bit tables with
// per-column meta, meta_cols % 4 == 0 (a chunk of four columns then never wraps).
template <int NBITS, int SKIND, int ZKIND>
__global__ __launch_bounds__(kThreads) void dequantize_words_kernel(const void *__restrict__ codes, Table sc, Table zr,
                                                                    uint32_t sc_inv, uint32_t zr_inv, uint32_t N,
                                                                    uint32_t K, uint32_t G, f16 *__restrict__ w)
{
    constexpr uint32_t F = NBITS == 3 ? 10 : 8 / NBITS;
    const uint32_t prows = (N + F - 1) / F;
    const uint32_t kchunks = K / 4;
    const uint32_t total = prows * kchunks;
    const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
    for (uint32_t idx = blockIdx.x * kThreads + threadIdx.x; idx < total; idx += gridDim.x * kThreads) {
        const uint32_t p = idx / kchunks, k0 = (idx - p * kchunks) * 4;
        u32x4 w3 = {0, 0, 0, 0};
        uint32_t w8 = 0;
        if constexpr (NBITS == 3)
            w3 = *reinterpret_cast<const u32x4 *>(static_cast<const uint32_t *>(codes) + (size_t)p * K + k0);
        else
            w8 = *reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(codes) + (size_t)p * K + k0);
        uint32_t j = (F * p) % G;
#pragma unroll
        for (uint32_t i = 0; i < F; ++i) {
            const uint32_t n = F * p + i;
            if (n >= N)
                break;
            TableCursor<SKIND> cs;
            TableCursor<ZKIND> cz;
            cs.init(sc, j * K + k0, sc_inv);
            cz.init(zr, j * K + k0, zr_inv);
            f16x2 s01, s23, z01, z23;
            table_decode(cs, table_load(cs), s01, s23);
            table_decode(cz, table_load(cz), z01, z23);
            uint32_t b; // the four codes of row n, one per byte
            if constexpr (NBITS == 3) {
                const uint32_t sh = 3 * (9 - i);
                b = ((w3.x >> sh) & 7u) | (((w3.y >> sh) & 7u) << 8) | (((w3.z >> sh) & 7u) << 16) |
                    (((w3.w >> sh) & 7u) << 24);
            } else {
                b = (w8 >> (NBITS * (F - 1 - i))) & ((1u << NBITS) - 1) * 0x01010101u;
            }
            const f16x2 q01 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, b, 0x04010400u)) - k1024;
            const f16x2 q23 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, b, 0x04030402u)) - k1024;
            const f16x2 d01 = q01 - z01, d23 = q23 - z23; // first rounding
            u32x2 o;
            o.x = __builtin_bit_cast(uint32_t, d01 * s01); // second rounding
            o.y = __builtin_bit_cast(uint32_t, d23 * s23);
            *reinterpret_cast<u32x2 *>(w + (size_t)n * K + k0) = o;
            if (++j == G)
                j = 0;
        }
    }
}

// ------------------------------------------------------- small elementwise
__global__ __launch_bounds__(kThreads) void silu_mul_kernel(const f16 *__restrict__ a, const f16 *__restrict__ b,
                                                            f16 *__restrict__ h, int64_t count)
{
    for (int64_t i = blockIdx.x * (int64_t)kThreads + threadIdx.x; i < count; i += (int64_t)gridDim.x * kThreads) {
        const float x = (float)a[i];
        const f16 act = (f16)(x / (1.0f + __expf(-x))); // silu in fp32, one rounding
        h[i] = act * b[i];
    }
}

__global__ __launch_bounds__(kThreads) void scale_store_kernel(const f16 *__restrict__ src, f16 *__restrict__ dst,
                                                               const f16 *__restrict__ row_scale, int accumulate,
                                                               int64_t M, int64_t N)
{
    for (int64_t i = blockIdx.x * (int64_t)kThreads + threadIdx.x; i < M * N; i += (int64_t)gridDim.x * kThreads) {
        f16 v = src[i];
        if (row_scale)
            v = v * row_scale[i / N];
        dst[i] = accumulate ? (f16)(dst[i] + v) : v;
    }
}

inline int grid_for(int64_t total)
{
    int64_t b = (total + kThreads - 1) / kThreads;
    if (b < 1)
        b = 1;
    if (b > 256 * 32)
        b = 256 * 32;
    return (int)b;
}

template <int NBITS>
int unpack_u8(const uint8_t *in, int64_t prows, int64_t cols, uint8_t *out, hipStream_t s)
{
    if (prows < 0 || cols < 0)
        return HQQ_E_SHAPE;
    if (prows == 0 || cols == 0) // empty input: nothing to do, and an empty tensor may well have no address
        return HQQ_OK;
    if (!in || !out)
        return HQQ_E_NULL;
    if (cols % 16 == 0 && aligned16(in) && aligned16(out))
        unpack_u8_kernel<NBITS, u32x4><<<grid_for(prows * cols / 16), kThreads, 0, s>>>(in, prows, cols, out);
    else
        unpack_u8_kernel<NBITS, uint8_t><<<grid_for(prows * cols), kThreads, 0, s>>>(in, prows, cols, out);
    return launch_status();
}

template <int NBITS>
int pack_u8(const uint8_t *q, int64_t rows, int64_t cols, uint8_t *out, hipStream_t s)
{
    constexpr int F = 8 / NBITS;
    if (rows < 0 || cols < 0 || rows % F != 0) // reference asserts an even height for 4 bit (src/packing.py:12)
        return HQQ_E_SHAPE;
    if (rows == 0 || cols == 0)
        return HQQ_OK;
    if (!q || !out)
        return HQQ_E_NULL;
    const int64_t prows = rows / F;
    if (cols % 16 == 0 && aligned16(q) && aligned16(out))
        pack_u8_kernel<NBITS, u32x4><<<grid_for(prows * cols / 16), kThreads, 0, s>>>(q, prows, cols, out);
    else
        pack_u8_kernel<NBITS, uint8_t><<<grid_for(prows * cols), kThreads, 0, s>>>(q, prows, cols, out);
    return launch_status();
}

// table kinds of TableCursor: 1 u8 with per-column meta, 2 u8 with scalar meta, 3 fp16; 0 = not a word-path table
inline int words_table_kind(const hqq_table &t)
{
    if (t.kind == HQQ_TABLE_F16)
        return aligned16(t.data) ? 3 : 0;
    if ((reinterpret_cast<uintptr_t>(t.data) & 3u) != 0)
        return 0;
    if (t.meta_cols == 1)
        return 2;
    const bool meta_ok = (reinterpret_cast<uintptr_t>(t.meta_scale) & 7u) == 0 && (reinterpret_cast<uintptr_t>(t.meta_zero) & 7u) == 0;
    return t.meta_cols % 4 == 0 && meta_ok ? 1 : 0;
}

template <int NBITS, int SKIND>
void dequantize_words_z(int zk, int grid, const hqq_linear *l, const Table &sc, const Table &zr, uint32_t si, uint32_t zi,
                        uint32_t G, f16 *w, hipStream_t s)
{
    const uint32_t N = (uint32_t)l->N, K = (uint32_t)l->K;
    if (zk == 1)
        dequantize_words_kernel<NBITS, SKIND, 1><<<grid, kThreads, 0, s>>>(l->codes, sc, zr, si, zi, N, K, G, w);
    else if (zk == 2)
        dequantize_words_kernel<NBITS, SKIND, 2><<<grid, kThreads, 0, s>>>(l->codes, sc, zr, si, zi, N, K, G, w);
    else
        dequantize_words_kernel<NBITS, SKIND, 3><<<grid, kThreads, 0, s>>>(l->codes, sc, zr, si, zi, N, K, G, w);
}

template <int NBITS>
void dequantize_words_s(int sk, int zk, int grid, const hqq_linear *l, const Table &sc, const Table &zr, uint32_t si,
                        uint32_t zi, uint32_t G, f16 *w, hipStream_t s)
{
    if (sk == 1)
        dequantize_words_z<NBITS, 1>(zk, grid, l, sc, zr, si, zi, G, w, s);
    else if (sk == 2)
        dequantize_words_z<NBITS, 2>(zk, grid, l, sc, zr, si, zi, G, w, s);
    else
        dequantize_words_z<NBITS, 3>(zk, grid, l, sc, zr, si, zi, G, w, s);
}

// The same values again for HQQ's two table layouts (8-bit scale with per-column meta and 8-bit zero with one meta
// pair, or both fp16) when K and the meta columns are multiples of 16: one thread owns sixteen columns of one packed
// row, so every access is 128 bits wide (codes, tables, meta, and two stores per weight row) and a wave writes 2 KB
// of a weight row at a time.
template <int NBITS, int SKIND, int ZKIND>
__global__ __launch_bounds__(kThreads) void dequantize_chunks_kernel(const uint8_t *__restrict__ codes, const uint8_t *__restrict__ sq,
                                                                     const uint8_t *__restrict__ zq, const f16 *__restrict__ s_ms,
                                                                     const f16 *__restrict__ s_mz, const f16 *__restrict__ z_ms,
                                                                     const f16 *__restrict__ z_mz, uint32_t s_cols, uint32_t s_inv,
                                                                     uint32_t N, uint32_t K, uint32_t G, f16 *__restrict__ w)
{
    using namespace gemv;
    constexpr uint32_t F = NBITS == 3 ? 10 : 8 / NBITS;
    const uint32_t prows = (N + F - 1) / F, kchunks = K / 16;
    const uint32_t idx = blockIdx.x * kThreads + threadIdx.x;
    if (idx >= prows * kchunks)
        return;
    const uint32_t p = idx / kchunks, k0 = (idx - p * kchunks) * 16;
    u32x4 cw[NBITS == 3 ? 4 : 1];
    if constexpr (NBITS == 3) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            cw[q] = gload<u32x4>(reinterpret_cast<const uint32_t *>(codes) + (size_t)p * K + k0 + 4 * q);
    } else {
        cw[0] = gload<u32x4>(codes + (size_t)p * K + k0);
    }
    f16x2 zms = {(f16)1.0f, (f16)1.0f}, zmz = {(f16)0.0f, (f16)0.0f};
    if constexpr (ZKIND == TK_U8_SCALAR)
        zms = (f16x2){z_ms[0], z_ms[0]}, zmz = (f16x2){z_mz[0], z_mz[0]};
    const f16x2 k1024 = {(f16)1024.0f, (f16)1024.0f};
    uint32_t j = (F * p) % G;
#pragma unroll
    for (uint32_t i = 0; i < F; ++i) {
        const uint32_t n = F * p + i;
        if (n >= N)
            break;
        const uint32_t ce = j * K + k0;
        uint32_t cm = 0;
        if constexpr (SKIND == TK_U8_COLS) {
            cm = ce - __umulhi(ce, s_inv) * s_cols; // ce mod cols; the quotient estimate is at most 2 short
            cm -= cm >= s_cols ? s_cols : 0;
            cm -= cm >= s_cols ? s_cols : 0;
        }
        Raw16<SKIND> rs;
        Raw16<ZKIND> rz;
        load16<SKIND>(rs, sq, s_ms, s_mz, ce, cm);
        load16<ZKIND>(rz, zq, nullptr, nullptr, ce, 0);
        f16x2 sv[8], zv[8];
        decode16<SKIND>(rs, zms, zmz, sv);
        decode16<ZKIND>(rz, zms, zmz, zv);
        u32x4 o[2];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t b; // the codes of row n at columns 4q .. 4q+3, one per byte
            if constexpr (NBITS == 3) {
                const uint32_t sh = 3 * (9 - i);
                b = ((cw[q].x >> sh) & 7u) | (((cw[q].y >> sh) & 7u) << 8) | (((cw[q].z >> sh) & 7u) << 16) |
                    (((cw[q].w >> sh) & 7u) << 24);
            } else {
                b = (cw[0][q] >> (NBITS * (F - 1 - i))) & ((1u << NBITS) - 1) * 0x01010101u;
            }
            const f16x2 q01 = as_h2(__builtin_amdgcn_perm(0x64646464u, b, 0x04010400u)) - k1024;
            const f16x2 q23 = as_h2(__builtin_amdgcn_perm(0x64646464u, b, 0x04030402u)) - k1024;
            const f16x2 d01 = q01 - zv[2 * q], d23 = q23 - zv[2 * q + 1]; // first rounding
            o[q >> 1][2 * (q & 1)] = as_u32(d01 * sv[2 * q]);             // second rounding
            o[q >> 1][2 * (q & 1) + 1] = as_u32(d23 * sv[2 * q + 1]);
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(w + (size_t)n * K + k0);
        dst[0] = o[0], dst[1] = o[1]; // plain stores: the GEMM that follows finds much of the layer in the last-level cache
        if (++j == G)
            j = 0;
    }
}

template <int NBITS> bool dequantize_chunks(const hqq_linear *l, f16 *w, hipStream_t s)
{
    const int sk = gemv::table_kind(l->scale), zk = gemv::table_kind(l->zero);
    const bool q8 = sk == gemv::TK_U8_COLS && zk == gemv::TK_U8_SCALAR, f16t = sk == gemv::TK_F16 && zk == gemv::TK_F16;
    const int64_t G = l->N / l->group_size;
    constexpr int F = NBITS == 3 ? 10 : 8 / NBITS;
    const int64_t prows = (l->N + F - 1) / F, threads = prows * (l->K / 16);
    if ((!q8 && !f16t) || l->K % 16 != 0 || G * l->K >= (1ll << 32) || threads >= (1ll << 31) ||
        !aligned16(w) || !aligned16(l->codes) || !aligned16(l->scale.data) || !aligned16(l->zero.data))
        return false;
    if (q8 && (l->scale.meta_cols % 16 != 0 || !aligned16(l->scale.meta_scale) || !aligned16(l->scale.meta_zero)))
        return false;
    const uint32_t s_cols = q8 ? (uint32_t)l->scale.meta_cols : 1;
    const uint32_t s_inv = (uint32_t)(0xFFFFFFFFull / (uint64_t)s_cols);
    const unsigned grid = (unsigned)((threads + kThreads - 1) / kThreads);
    const uint8_t *codes = static_cast<const uint8_t *>(l->codes), *sq = static_cast<const uint8_t *>(l->scale.data),
                  *zq = static_cast<const uint8_t *>(l->zero.data);
    const f16 *sms = static_cast<const f16 *>(l->scale.meta_scale), *smz = static_cast<const f16 *>(l->scale.meta_zero),
              *zms = static_cast<const f16 *>(l->zero.meta_scale), *zmz = static_cast<const f16 *>(l->zero.meta_zero);
    if (q8)
        dequantize_chunks_kernel<NBITS, gemv::TK_U8_COLS, gemv::TK_U8_SCALAR><<<grid, kThreads, 0, s>>>(
            codes, sq, zq, sms, smz, zms, zmz, s_cols, s_inv, (uint32_t)l->N, (uint32_t)l->K, (uint32_t)G, w);
    else
        dequantize_chunks_kernel<NBITS, gemv::TK_F16, gemv::TK_F16><<<grid, kThreads, 0, s>>>(
            codes, sq, zq, sms, smz, zms, zmz, s_cols, s_inv, (uint32_t)l->N, (uint32_t)l->K, (uint32_t)G, w);
    return true;
}

// launches the word-path de-quantiser when the layer fits it; false = the caller takes the per-element kernel
bool dequantize_words(const hqq_linear *l, const Table &sc, const Table &zr, f16 *w, hipStream_t s)
{
    if (l->nbits == 4 ? dequantize_chunks<4>(l, w, s) : l->nbits == 2 ? dequantize_chunks<2>(l, w, s) : dequantize_chunks<3>(l, w, s))
        return true;
    const int sk = words_table_kind(l->scale), zk = words_table_kind(l->zero);
    const int64_t G = l->N / l->group_size;
    const int F = l->nbits == 3 ? 10 : 8 / l->nbits;
    const int64_t prows = (l->N + F - 1) / F;
    if (!sk || !zk || l->K % 4 != 0 || G * l->K >= (1ll << 32) || prows * (l->K / 4) >= (1ll << 31) ||
        (reinterpret_cast<uintptr_t>(w) & 7u) != 0 || !aligned16(l->codes))
        return false;
    const uint32_t si = l->scale.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->scale.meta_cols) : 0;
    const uint32_t zi = l->zero.meta_cols > 0 ? (uint32_t)(0xFFFFFFFFull / (uint64_t)l->zero.meta_cols) : 0;
    const int grid = grid_for(prows * (l->K / 4));
    if (l->nbits == 4)
        dequantize_words_s<4>(sk, zk, grid, l, sc, zr, si, zi, (uint32_t)G, w, s);
    else if (l->nbits == 2)
        dequantize_words_s<2>(sk, zk, grid, l, sc, zr, si, zi, (uint32_t)G, w, s);
    else
        dequantize_words_s<3>(sk, zk, grid, l, sc, zr, si, zi, (uint32_t)G, w, s);
    return true;
}

} // namespace

int launch_silu_mul(const f16 *a, const f16 *b, f16 *h, int64_t count, hipStream_t s)
{
    if (count <= 0)
        return HQQ_OK;
    silu_mul_kernel<<<grid_for(count), kThreads, 0, s>>>(a, b, h, count);
    return launch_status();
}

int launch_scale_store(const f16 *src, f16 *dst, const f16 *row_scale, int accumulate, int64_t M, int64_t N,
                       hipStream_t s)
{
    if (M * N <= 0)
        return HQQ_OK;
    scale_store_kernel<<<grid_for(M * N), kThreads, 0, s>>>(src, dst, row_scale, accumulate, M, N);
    return launch_status();
}

} // namespace hqq

using namespace hqq;

extern "C" {

int hqq_pack_4bit_u8(const uint8_t *q, int64_t rows, int64_t cols, uint8_t *out, void *stream)
{
    return pack_u8<4>(q, rows, cols, out, (hipStream_t)stream);
}
int hqq_pack_2bit_u8(const uint8_t *q, int64_t rows, int64_t cols, uint8_t *out, void *stream)
{
    return pack_u8<2>(q, rows, cols, out, (hipStream_t)stream);
}
int hqq_unpack_4bit_u8(const uint8_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream)
{
    return unpack_u8<4>(in, rows, cols, q, (hipStream_t)stream);
}
int hqq_unpack_2bit_u8(const uint8_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream)
{
    return unpack_u8<2>(in, rows, cols, q, (hipStream_t)stream);
}

int hqq_pack_3bit_i32(const uint8_t *q, int64_t rows, int64_t cols, int32_t *out, void *stream)
{
    if (rows < 0 || cols < 0)
        return HQQ_E_SHAPE;
    if (rows == 0 || cols == 0)
        return HQQ_OK;
    if (!q || !out)
        return HQQ_E_NULL;
    const int64_t words = (rows + 9) / 10;
    hipStream_t s = (hipStream_t)stream;
    if (cols % 4 == 0 && aligned16(out) && (reinterpret_cast<uintptr_t>(q) & 3u) == 0)
        pack3_kernel<4><<<grid_for(words * cols / 4), kThreads, 0, s>>>(q, rows, cols, (uint32_t *)out);
    else
        pack3_kernel<1><<<grid_for(words * cols), kThreads, 0, s>>>(q, rows, cols, (uint32_t *)out);
    return launch_status();
}

int hqq_unpack_3bit_i32(const int32_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream)
{
    if (rows < 0 || cols < 0)
        return HQQ_E_SHAPE;
    if (rows == 0 || cols == 0)
        return HQQ_OK;
    if (!in || !q)
        return HQQ_E_NULL;
    hipStream_t s = (hipStream_t)stream;
    if (cols % 4 == 0 && aligned16(in) && (reinterpret_cast<uintptr_t>(q) & 3u) == 0)
        unpack3_kernel<4><<<grid_for(rows * cols / 4), kThreads, 0, s>>>((const uint32_t *)in, rows, cols, q);
    else
        unpack3_kernel<1><<<grid_for(rows * cols), kThreads, 0, s>>>((const uint32_t *)in, rows, cols, q);
    return launch_status();
}

int hqq_table_to_f16(const hqq_table *t, int64_t count, void *out_f16, void *stream)
{
    if (!t || !t->data || !out_f16)
        return HQQ_E_NULL;
    if (t->kind == HQQ_TABLE_U8 && (!t->meta_scale || !t->meta_zero))
        return HQQ_E_NULL;
    if (count < 0 || (t->kind == HQQ_TABLE_U8 && t->meta_cols < 1) || (t->kind != HQQ_TABLE_U8 && t->kind != HQQ_TABLE_F16))
        return HQQ_E_SHAPE;
    if (count == 0)
        return HQQ_OK;
    table_to_f16_kernel<<<grid_for(count), kThreads, 0, (hipStream_t)stream>>>(make_table(*t), count, (f16 *)out_f16);
    return launch_status();
}

int hqq_dequantize(const hqq_linear *l, void *w_out_f16, void *stream)
{
    int rc = validate_linear(l);
    if (rc != HQQ_OK)
        return rc;
    if (!w_out_f16)
        return HQQ_E_NULL;
    const int64_t G = l->N / l->group_size;
    const int F = l->nbits == 3 ? 10 : 8 / l->nbits;
    const int64_t total = ((l->N + F - 1) / F) * ((l->K + 3) / 4);
    hipStream_t s = (hipStream_t)stream;
    const Table sc = make_table(l->scale), zr = make_table(l->zero);
    if (dequantize_words(l, sc, zr, (f16 *)w_out_f16, s))
        return launch_status();
    if (l->nbits == 4)
        dequantize_kernel<4><<<grid_for(total), kThreads, 0, s>>>(l->codes, sc, zr, l->N, l->K, G, (f16 *)w_out_f16);
    else if (l->nbits == 2)
        dequantize_kernel<2><<<grid_for(total), kThreads, 0, s>>>(l->codes, sc, zr, l->N, l->K, G, (f16 *)w_out_f16);
    else
        dequantize_kernel<3><<<grid_for(total), kThreads, 0, s>>>(l->codes, sc, zr, l->N, l->K, G, (f16 *)w_out_f16);
    return launch_status();
}

} // extern "C"
