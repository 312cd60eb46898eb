// Residual add, RMSNorm and router of one token as a block-level routine: used by the stand-alone kernel and by the
// gate launch of the decode step, so that both give the same bits.
#pragma once

#include "hqq_common.hpp"

namespace hqq {

constexpr int kMaxExperts = 16;

// softmax over the fp16-rounded logits in fp32, the two largest probabilities renormalised by their sum and cast to
// fp16 (reference src/custom_layers.py:277-282).  Called by the first sixteen threads of the block (one wave): thread
// i takes the exponential of expert i, thread 0 adds them up in expert order and picks the two largest, so the
// result does not depend on how many threads helped.  prob_lds: kMaxExperts floats.
__device__ __forceinline__ void route_top2(const float *logit_lds, float *prob_lds, int n_experts, int *sel, f16 *weights,
                                           f16 *logits_out)
{
    const int i = threadIdx.x;
    float mx = logit_lds[0];
    for (int e = 1; e < n_experts; ++e)
        mx = fmaxf(mx, logit_lds[e]);
    if (i < n_experts) {
        prob_lds[i] = __expf(logit_lds[i] - mx);
        if (logits_out)
            logits_out[i] = (f16)logit_lds[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (i != 0)
        return;
    float sum = 0.f;
    for (int e = 0; e < n_experts; ++e)
        sum += prob_lds[e];
    int b0 = 0, b1 = -1;
    float p0 = prob_lds[0] / sum, p1 = 0.f;
    for (int e = 1; e < n_experts; ++e) {
        const float pe = prob_lds[e] / sum;
        if (pe > p0)
            b0 = e, p0 = pe;
    }
    for (int e = 0; e < n_experts; ++e) {
        const float pe = prob_lds[e] / sum;
        if (e != b0 && (b1 < 0 || pe > p1))
            b1 = e, p1 = pe;
    }
    const float tot = p0 + p1;
    sel[0] = b0, sel[1] = b1;
    weights[0] = (f16)(p0 / tot);
    weights[1] = (f16)(p1 / tot);
}

// LDS the routine needs (NE = 8 or 16 experts)
template <int NE> struct NormRouteLds {
    float part[4];
    float dot[NE][256 + 4];
    float logit[kMaxExperts];
    float prob[kMaxExperts];
};

// For hidden <= CH * 2048 and at most NE experts, with every global load issued before the first use: the token, the
// norm weight and the thread's pieces of all router rows travel together, so the block waits for memory once.
// Threads 0..255 of the block work (thread t owns elements (c * 256 + t) * 8 .. + 7 of chunk c); every thread of the
// block must call, because the routine synchronises the block.  x_sum (may be x itself, or null) receives
// x + delta, y (or null) the normed row; sel / weights / logits_out may point anywhere (thread 0 writes them).
// Returns 1 / sqrt(mean((x + delta)^2) + eps).
template <int CH, int NE, bool DELTA>
__device__ __forceinline__ float norm_route_body(const f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *x_sum,
                                                 f16 *y, int hidden, const f16 *gate_w, int n_experts, int *sel,
                                                 f16 *weights, f16 *logits_out, NormRouteLds<NE> &lds)
{
    const int tid = threadIdx.x;
    const bool worker = tid < 256;
    f16x8 xv[CH], dv[CH], wv[CH], gv[CH][NE];
    bool on[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int k = (c * 256 + tid) * 8;
        on[c] = worker && k < hidden;
        const int kc = on[c] ? k : 0;
        xv[c] = *reinterpret_cast<const f16x8 *>(x + kc);
        if constexpr (DELTA) // a compile-time choice: every load of the routine is then issued in one batch
            dv[c] = *reinterpret_cast<const f16x8 *>(delta + kc);
        wv[c] = *reinterpret_cast<const f16x8 *>(weight + kc);
#pragma unroll
        for (int e = 0; e < NE; ++e)
            gv[c][e] = *reinterpret_cast<const f16x8 *>(gate_w + (int64_t)(e < n_experts ? e : 0) * hidden + kc);
    }
    if constexpr (DELTA) {
#pragma unroll
        for (int c = 0; c < CH; ++c)
            xv[c] = xv[c] + dv[c];
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if (on[c]) {
            if (x_sum && (DELTA || x_sum != x))
                *reinterpret_cast<f16x8 *>(x_sum + (c * 256 + tid) * 8) = xv[c];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                ss += (float)xv[c][t] * (float)xv[c][t];
        }
    }
    ss = wave_sum(ss);
    if (worker && (tid & 63) == 0)
        lds.part[tid >> 6] = ss;
    __syncthreads();
    const float mean = (lds.part[0] + lds.part[1] + lds.part[2] + lds.part[3]) / (float)hidden;
    const float r = 1.0f / __builtin_sqrtf(mean + eps);
    float dot[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e)
        dot[e] = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if (on[c]) {
            f16x8 o;
#pragma unroll
            for (int t = 0; t < 8; ++t)
                o[t] = wv[c][t] * (f16)((float)xv[c][t] * r);
            if (y)
                *reinterpret_cast<f16x8 *>(y + (c * 256 + tid) * 8) = o;
#pragma unroll
            for (int e = 0; e < NE; ++e)
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    dot[e] += (float)o[t] * (float)gv[c][e][t];
        }
    }
    if (worker) {
#pragma unroll
        for (int e = 0; e < NE; ++e)
            lds.dot[e][tid] = dot[e];
    }
    __syncthreads();
    // sixteen threads per expert: each adds sixteen of the 256 partial sums, then the sixteen meet by lane shuffles
    const int e = tid >> 4, i = tid & 15;
    if (worker && e < NE) {
        float a = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j)
            a += lds.dot[e][16 * j + i];
#pragma unroll
        for (int off = 8; off > 0; off >>= 1)
            a += __shfl_xor(a, off, 64);
        if (i == 0 && e < n_experts)
            lds.logit[e] = (float)(f16)a;
    }
    __syncthreads();
    if (tid < kMaxExperts)
        route_top2(lds.logit, lds.prob, n_experts, sel, weights, logits_out);
    return r;
}

template <int CH, int NE>
__device__ __forceinline__ float norm_route_block(const f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *x_sum,
                                                  f16 *y, int hidden, const f16 *gate_w, int n_experts, int *sel,
                                                  f16 *weights, f16 *logits_out, NormRouteLds<NE> &lds)
{
    if (delta)
        return norm_route_body<CH, NE, true>(x, delta, weight, eps, x_sum, y, hidden, gate_w, n_experts, sel, weights,
                                             logits_out, lds);
    return norm_route_body<CH, NE, false>(x, nullptr, weight, eps, x_sum, y, hidden, gate_w, n_experts, sel, weights,
                                          logits_out, lds);
}

} // namespace hqq
