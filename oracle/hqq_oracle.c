/*
 * Plain-C restatement of the reference's HQQ quantized-linear path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP library and the "port"
 * CPU baseline.  Nothing shipped links or loads this file.
 *
 * fp16 values travel as raw uint16_t bit patterns and every fp16 operation is
 * done as: widen to float (exact), operate in float (exact for one fp16
 * subtraction or multiplication: 24 >= 2*11+2), round to nearest-even with
 * integer arithmetic only.  That makes this file independent of numpy's and
 * the GPU's half arithmetic, which is what pins them.
 *
 * Citations are into the reference tree (src/...).
 */
#include <stdint.h>
#include <string.h>
#include <stddef.h>

static float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0u));
    if (absx >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (absx < 0x33000001u) /* <= 2^-25: rounds to zero (tie goes to even = 0) */
        return sign;
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q++;
    return (uint16_t)(sign | (base + q)); /* mantissa carry bumps the exponent */
}

uint16_t oracle_f2h(float f) { return f2h(f); }
float oracle_h2f(uint16_t h) { return h2f(h); }

/* src/packing.py:10-17 */
void oracle_pack_4bit_u8(const uint8_t *q, int64_t h, int64_t w, uint8_t *out)
{
    for (int64_t p = 0; p < h / 2; ++p)
        for (int64_t c = 0; c < w; ++c)
            out[p * w + c] = (uint8_t)((uint8_t)(q[(2 * p) * w + c] << 4) | q[(2 * p + 1) * w + c]);
}

/* src/packing.py:19-27 */
void oracle_unpack_4bit_u8(const uint8_t *in, int64_t hp, int64_t w, uint8_t *q)
{
    for (int64_t p = 0; p < hp; ++p)
        for (int64_t c = 0; c < w; ++c) {
            uint8_t b = in[p * w + c];
            q[(2 * p) * w + c] = b >> 4;
            q[(2 * p + 1) * w + c] = b & 0x0F;
        }
}

/* src/packing.py:36-41 */
void oracle_pack_2bit_u8(const uint8_t *q, int64_t h, int64_t w, uint8_t *out)
{
    for (int64_t p = 0; p < h / 4; ++p)
        for (int64_t c = 0; c < w; ++c)
            out[p * w + c] = (uint8_t)((uint8_t)(q[(4 * p) * w + c] << 6) | (uint8_t)(q[(4 * p + 1) * w + c] << 4) |
                                       (uint8_t)(q[(4 * p + 2) * w + c] << 2) | q[(4 * p + 3) * w + c]);
}

/* src/packing.py:43-53 */
void oracle_unpack_2bit_u8(const uint8_t *in, int64_t hp, int64_t w, uint8_t *q)
{
    for (int64_t p = 0; p < hp; ++p)
        for (int64_t c = 0; c < w; ++c) {
            uint8_t b = in[p * w + c];
            for (int i = 0; i < 4; ++i)
                q[(4 * p + i) * w + c] = (b >> (2 * (3 - i))) & 3;
        }
}

/* src/packing.py:62-81: h rows in, ceil(h/10) words out, missing lanes zero */
void oracle_pack_3bit_i32(const uint8_t *q, int64_t h, int64_t w, int32_t *out)
{
    int64_t words = (h + 9) / 10;
    for (int64_t p = 0; p < words; ++p)
        for (int64_t c = 0; c < w; ++c) {
            uint32_t v = 0;
            for (int i = 0; i < 10; ++i) {
                int64_t r = 10 * p + i;
                if (r < h)
                    v |= (uint32_t)q[r * w + c] << (3 * (9 - i));
            }
            out[p * w + c] = (int32_t)v;
        }
}

/* src/packing.py:83-97: always 10 rows per word */
void oracle_unpack_3bit_i32(const int32_t *in, int64_t words, int64_t w, uint8_t *q)
{
    for (int64_t p = 0; p < words; ++p)
        for (int64_t c = 0; c < w; ++c) {
            int32_t v = in[p * w + c];
            for (int i = 0; i < 10; ++i)
                q[(10 * p + i) * w + c] = (uint8_t)((v >> (3 * (9 - i))) & 7);
        }
}

/* code of weight (n,k) as the reference kernels read it:
 * src/triton_kernels.py:84,91 / :272,279 / :462,469 */
static inline unsigned code_at(const void *codes, int nbits, int64_t n, int64_t k, int64_t K)
{
    if (nbits == 4)
        return (((const uint8_t *)codes)[(n / 2) * K + k] >> (((n + 1) % 2) * 4)) & 0xFu;
    if (nbits == 2)
        return (((const uint8_t *)codes)[(n / 4) * K + k] >> ((3 - n % 4) * 2)) & 0x3u;
    return ((uint32_t)((const int32_t *)codes)[(n / 10) * K + k] >> ((9 - n % 10) * 3)) & 0x7u;
}

/* src/custom_layers.py:63-66 (-> formula at :111): 8-bit table -> fp16 table.
 * q is (rows, cols) row-major; ms/mz have `cols` entries (or 1 when scalar). */
void oracle_meta_dequant(const uint8_t *q, int64_t rows, int64_t cols, const uint16_t *ms, const uint16_t *mz,
                         int scalar_meta, uint16_t *out)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            int64_t m = scalar_meta ? 0 : c;
            uint16_t t = f2h((float)q[r * cols + c] - h2f(mz[m]));
            out[r * cols + c] = f2h(h2f(t) * h2f(ms[m]));
        }
}

/* src/custom_layers.py:95-116 / src/triton_kernels.py:109-118:
 * W[n,k] = fp16(fp16(q - Z[n%G,k]) * S[n%G,k]); tables are fp16 (G,K). */
void oracle_dequantize(const void *codes, int nbits, int64_t N, int64_t K, int64_t gs, const uint16_t *scale,
                       const uint16_t *zero, uint16_t *w_out)
{
    int64_t G = N / gs;
    for (int64_t n = 0; n < N; ++n) {
        const uint16_t *s = scale + (n % G) * K, *z = zero + (n % G) * K;
        for (int64_t k = 0; k < K; ++k) {
            uint16_t t = f2h((float)code_at(codes, nbits, n, k, K) - h2f(z[k]));
            w_out[n * K + k] = f2h(h2f(t) * h2f(s[k]));
        }
    }
}

/* src/triton_kernels.py:103-131: C[m,n] = sum_k A[m,k] * W[n,k], here in
 * double, rounded once to fp16; w is the dequantised fp16 (N,K) matrix. */
void oracle_matmul_transpose(const uint16_t *x, int64_t M, const uint16_t *w, int64_t N, int64_t K, uint16_t *y)
{
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)h2f(x[m * K + k]) * (double)h2f(w[n * K + k]);
            y[m * N + n] = f2h((float)acc);
        }
}
