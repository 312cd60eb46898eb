// The attention of one new token for one query head, shared by the stand-alone kernel and the chained launch of a
// decoder layer's attention part.
#pragma once
#include "chain_parts.hpp"
#include "hqq_common.hpp"

namespace hqq {

// Threads per head.  256 only for caches that never hold more than a hundred-odd positions: from there on the block of
// 1024 is faster (sixteen lanes per cache row, so 64 rows per pass instead of 16), at 200 positions by 4 us.  The
// stand-alone kernel and the chained launch use the same count, so both add in the same order.
inline int attention_block_threads(int64_t max_len) { return max_len <= tuning_int("HQQ_ATT_SMALL", 128) ? 256 : 1024; }

// Rotary embedding, KV-cache append and attention of ONE new token (the reference takes them from HF transformers'
// Mixtral attention): one block per query head.  Roundings follow the fp16 torch ops they replace: rope terms
// rounded separately, scores = fp16(q . k) then / sqrt(hd) in fp32, softmax in fp32, probabilities cast to fp16,
// output accumulated in fp32.  The current position is read from device memory, so the launch can be replayed
// from a graph; positions 0 .. pos are attended (the new key and value are taken from registers, and also
// written to the cache by the first head of each KV group).
// One block of NT threads per head: 256 for caches of up to 512 positions, 1024 beyond (the block walks the head's
// cache rows, so a long cache wants more threads and a short one fewer reduction steps).
// chain (a constant at every call site): CHAIN_NONE for the stand-alone kernel.  CHAIN_MID when q, k and v are produced
// by earlier blocks of the same grid and the output is read by later ones: what only needs the position (rope row,
// the first cached key rows) is requested first, then the block waits for the producers, reads q, k and v at device
// scope, and at the end stores its output at device scope and counts itself (chain_blocks heads in all).  The arithmetic is the same.
template <int HD, int NT>
__device__ __forceinline__ void attention_head(const f16 *__restrict__ q_in, const f16 *__restrict__ k_in,
                                               const f16 *__restrict__ v_in, const f16 *__restrict__ cos_t,
                                               const f16 *__restrict__ sin_t, const int64_t *__restrict__ pos_p,
                                               f16 *__restrict__ cache_k, f16 *__restrict__ cache_v, int64_t max_len, int group,
                                               f16 *__restrict__ out, const int h, const int chain, int *chain_words,
                                               int chain_blocks)
{
    extern __shared__ float score_lds[]; // [pos + 1]
    __shared__ __attribute__((aligned(16))) f16 q_lds[HD];
    __shared__ __attribute__((aligned(16))) f16 k_lds[HD];
    constexpr int NW = NT / 64;
    __shared__ float red_lds[2 * NW];
    __shared__ float acc_lds[NT / (HD / 8)][HD];
    __shared__ __attribute__((aligned(16))) f16 raw_lds[3][HD]; // chained: q, k and v of the head as they arrive
    const int kv = h / group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the new token's q, k and v do not depend on the position: their loads go out before it is waited for
    const int d = tid < HD ? tid : 0, dr = d < HD / 2 ? d + HD / 2 : d - HD / 2;
    f16 qa = (f16)0, qb = (f16)0, ka = (f16)0, kb = (f16)0, vnew = (f16)0;
    if (chain == CHAIN_NONE) {
        qa = q_in[h * HD + d], qb = q_in[h * HD + dr];
        ka = k_in[kv * HD + d], kb = k_in[kv * HD + dr];
        vnew = v_in[kv * HD + d];
    }
    const int64_t pos_raw = pos_p[0];
    // the position lives in device memory: a step past the cache must not write past it
    const bool live = pos_raw >= 0 && pos_raw < max_len;
    if (chain == CHAIN_NONE && !live)
        return;
    const int64_t pos = live ? pos_raw : 0;
    const f16 *cs = cos_t + pos * HD, *sn = sin_t + pos * HD;
    const f16 cs_d = cs[d], sn_d = sn[d];
    // the cached key rows of the first four passes only need the position: requested before the rope table arrives
    // (the row of the new token itself is taken from LDS later)
    constexpr int LPK = HD / 8, KROWS = NT / LPK;
    const int ksub = tid / LPK, kc = tid % LPK;
    f16x8 kfirst[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t l = u * KROWS + ksub;
        const int64_t lc = l <= pos ? l : pos;
        kfirst[u] = *reinterpret_cast<const f16x8 *>(cache_k + ((int64_t)kv * max_len + lc) * HD + 8 * kc);
    }
    if (chain == CHAIN_MID) {
        CHAIN_STAMP(chain_words, 0);
        chain_wait(chain_words, CHAIN_GO_FIRST, kChainGoFirst);
        CHAIN_STAMP(chain_words, 1);
        if (!live) { // nothing to attend: still counted, so that the blocks that wait for this one go on
            chain_signal(chain_words, CHAIN_MID_DONE, chain_blocks, CHAIN_GO_MID, kChainGoMid);
            return;
        }
        static_assert(NT >= 3 * HD / 2, "one thread per pair of elements of q, k and v");
        if (tid < 3 * HD / 2) {
            const int which = tid / (HD / 2), e = 2 * (tid % (HD / 2));
            const f16 *src = which == 0 ? q_in + h * HD : (which == 1 ? k_in + kv * HD : v_in + kv * HD);
            *reinterpret_cast<uint32_t *>(&raw_lds[which][e]) = chain_load4(src + e);
        }
        __syncthreads();
        qa = raw_lds[0][d], qb = raw_lds[0][dr];
        ka = raw_lds[1][d], kb = raw_lds[1][dr];
        vnew = raw_lds[2][d];
    }
    if (tid < HD) {
        const f16 qr = d < HD / 2 ? -qb : qb, kr = d < HD / 2 ? -kb : kb;
        const f16 qrot = (f16)(qa * cs_d) + (f16)(qr * sn_d);
        const f16 krot = (f16)(ka * cs_d) + (f16)(kr * sn_d);
        q_lds[d] = qrot;
        k_lds[d] = krot;
        if (h % group == 0) {
            cache_k[((int64_t)kv * max_len + pos) * HD + d] = krot;
            cache_v[((int64_t)kv * max_len + pos) * HD + d] = vnew;
        }
    }
    __syncthreads();

    // scores: LPK threads share a key row (16 bytes each, so a wave's load covers whole rows), four passes of
    // KROWS rows in flight; the pieces of a dot product meet through lane exchanges
    const float inv = 1.0f / __builtin_sqrtf((float)HD);
    float mx = -3.0e38f;
    {
        const f16x8 qq = *reinterpret_cast<const f16x8 *>(q_lds + 8 * kc);
        for (int64_t l0 = 0; l0 <= pos; l0 += 4 * KROWS) {
            f16x8 kk[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t l = l0 + u * KROWS + ksub;
                const int64_t lc = l <= pos ? l : pos;
                if (lc == pos)
                    kk[u] = *reinterpret_cast<const f16x8 *>(k_lds + 8 * kc);
                else if (l0 == 0)
                    kk[u] = kfirst[u];
                else
                    kk[u] = *reinterpret_cast<const f16x8 *>(cache_k + ((int64_t)kv * max_len + lc) * HD + 8 * kc);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float acc = 0.f;
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    acc += (float)kk[u][t] * (float)qq[t];
#pragma unroll
                for (int off = LPK / 2; off > 0; off >>= 1)
                    acc += __shfl_xor(acc, off, 64);
                const int64_t l = l0 + u * KROWS + ksub;
                if (kc == 0 && l <= pos) {
                    const float sc = (float)(f16)acc * inv;
                    score_lds[l] = sc;
                    mx = fmaxf(mx, sc);
                }
            }
        }
    }
    // the value rows of the first four passes do not depend on the scores: requested now, used after the softmax
    constexpr int LPR = HD / 8, ROWS = NT / LPR;
    const int rsub = tid / LPR, c8 = tid % LPR;
    // eight elements of value row lc <= pos; the new token's row is not in the cache yet for the other heads of its group
    auto value_row = [&](int64_t lc) __attribute__((always_inline)) -> f16x8 {
        if (chain == CHAIN_NONE) {
            const f16 *vrow = lc == pos ? v_in + kv * HD : cache_v + ((int64_t)kv * max_len + lc) * HD;
            return *reinterpret_cast<const f16x8 *>(vrow + 8 * c8);
        }
        const int64_t lr = lc < pos ? lc : (pos > 0 ? pos - 1 : 0);
        f16x8 v = *reinterpret_cast<const f16x8 *>(cache_v + ((int64_t)kv * max_len + lr) * HD + 8 * c8);
        if (lc == pos)
            v = *reinterpret_cast<const f16x8 *>(&raw_lds[2][8 * c8]);
        return v;
    };
    f16x8 vfirst[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t l = u * ROWS + rsub;
        const int64_t lc = l <= pos ? l : pos;
        vfirst[u] = value_row(lc);
    }
    // block max
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    if (lane == 0)
        red_lds[wave] = mx;
    __syncthreads();
    mx = red_lds[0];
#pragma unroll
    for (int w = 1; w < NW; ++w)
        mx = fmaxf(mx, red_lds[w]);
    float sum = 0.f;
    for (int64_t l = tid; l <= pos; l += NT) {
        const float e = __expf(score_lds[l] - mx);
        score_lds[l] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0)
        red_lds[NW + wave] = sum;
    __syncthreads();
    sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w)
        sum += red_lds[NW + w];
    const float rs = 1.0f / sum;

    // output: LPR threads share a value row (16 bytes each), the block covers ROWS rows per pass and four passes
    // are in flight; the ROWS partial outputs meet in LDS
    float o[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
        o[t] = 0.f;
    for (int64_t l0 = 0; l0 <= pos; l0 += 4 * ROWS) {
        f16x8 vv[4];
        float pr[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t l = l0 + u * ROWS + rsub;
            const int64_t lc = l <= pos ? l : pos;
            if (l0 == 0) {
                vv[u] = vfirst[u];
            } else {
                vv[u] = value_row(lc);
            }
            pr[u] = l <= pos ? (float)(f16)(score_lds[lc] * rs) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < 8; ++t)
                o[t] += pr[u] * (float)vv[u][t];
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
        acc_lds[rsub][8 * c8 + t] = o[t];
    __syncthreads();
    // the ROWS partial outputs: sixteen at a time by HD threads each, then the sums of the sixteens in order
    constexpr int NPART = ROWS / 16;
    static_assert(ROWS % 16 == 0 && NT >= HD * NPART, "one thread per column and group of sixteen partial outputs");
    if constexpr (NPART > 1) {
        if (tid < HD * NPART) {
            const int pt = tid / HD, dcol = tid % HD;
            float a = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                a += acc_lds[16 * pt + r][dcol];
            acc_lds[16 * pt][dcol] = a;
        }
        __syncthreads();
    }
    auto column = [&](int dcol) __attribute__((always_inline)) -> float {
        float a = 0.f;
        if constexpr (NPART > 1) {
#pragma unroll
            for (int pt = 0; pt < NPART; ++pt)
                a += acc_lds[16 * pt][dcol];
        } else {
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                a += acc_lds[r][dcol];
        }
        return a;
    };
    if (chain == CHAIN_MID) {
        if (tid < HD / 2)
            chain_store(out + h * HD + 2 * tid, (f16x2){(f16)column(2 * tid), (f16)column(2 * tid + 1)});
        CHAIN_STAMP(chain_words, 2);
        chain_signal(chain_words, CHAIN_MID_DONE, chain_blocks, CHAIN_GO_MID, kChainGoMid);
        CHAIN_STAMP(chain_words, 3);
        return;
    }
    if (tid < HD)
        out[h * HD + tid] = (f16)column(tid);
}


} // namespace hqq
