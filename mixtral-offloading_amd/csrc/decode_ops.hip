// Small decode-step kernels around the quantized linears: the router (reference src/custom_layers.py:276-282)
// and the residual add + RMSNorm of the decoder layer.  One block each: at batch 1 they are latency, not bandwidth.
#include "hqq_common.hpp"

namespace hqq {
namespace {

constexpr int kMaxExperts = 16;

// logits = fp16(x W^T) (fp32 accumulation, one rounding, as a half linear does); softmax in fp32; the two largest
// probabilities, renormalised by their sum, cast to fp16 (reference src/custom_layers.py:277-282).
__global__ __launch_bounds__(64 * kMaxExperts) void router_top2_kernel(const f16 *__restrict__ x, const f16 *__restrict__ w,
                                                                       int n_experts, int hidden, int *__restrict__ sel,
                                                                       f16 *__restrict__ weights, f16 *__restrict__ logits_out)
{
    __shared__ float logit_lds[kMaxExperts];
    const int lane = threadIdx.x & 63, e = threadIdx.x >> 6;
    if (e < n_experts) {
        const f16 *row = w + (int64_t)e * hidden;
        float acc = 0.f;
        for (int k = lane * 8; k < hidden; k += 64 * 8) {
            const f16x8 a = *reinterpret_cast<const f16x8 *>(x + k);
            const f16x8 b = *reinterpret_cast<const f16x8 *>(row + k);
#pragma unroll
            for (int t = 0; t < 8; ++t)
                acc += (float)a[t] * (float)b[t];
        }
        acc = wave_sum(acc);
        if (lane == 0)
            logit_lds[e] = (float)(f16)acc;
    }
    __syncthreads();
    if (threadIdx.x != 0)
        return;
    float mx = logit_lds[0];
    for (int i = 1; i < n_experts; ++i)
        mx = fmaxf(mx, logit_lds[i]);
    float prob[kMaxExperts], sum = 0.f;
    for (int i = 0; i < n_experts; ++i) {
        prob[i] = __expf(logit_lds[i] - mx);
        sum += prob[i];
    }
    int b0 = 0, b1 = -1;
    for (int i = 0; i < n_experts; ++i) {
        prob[i] /= sum;
        if (logits_out)
            logits_out[i] = (f16)logit_lds[i];
    }
    for (int i = 1; i < n_experts; ++i)
        if (prob[i] > prob[b0])
            b0 = i;
    for (int i = 0; i < n_experts; ++i)
        if (i != b0 && (b1 < 0 || prob[i] > prob[b1]))
            b1 = i;
    const float tot = prob[b0] + prob[b1];
    sel[0] = b0, sel[1] = b1;
    weights[0] = (f16)(prob[b0] / tot);
    weights[1] = (f16)(prob[b1] / tot);
}

// x += delta (fp16 add, when delta is given; x is written back), then y = weight * fp16(x * rsqrt(mean(x^2) + eps))
// with the statistics in fp32: the decoder layer's residual add and RMSNorm in one pass.
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(f16 *__restrict__ x, const f16 *__restrict__ delta,
                                                          const f16 *__restrict__ weight, float eps, f16 *__restrict__ y,
                                                          int hidden)
{
    __shared__ float part_lds[4];
    const int tid = threadIdx.x;
    float ss = 0.f;
    for (int k = tid * 8; k < hidden; k += 256 * 8) {
        f16x8 v = *reinterpret_cast<const f16x8 *>(x + k);
        if (delta) {
            v = v + *reinterpret_cast<const f16x8 *>(delta + k);
            *reinterpret_cast<f16x8 *>(x + k) = v;
        }
#pragma unroll
        for (int t = 0; t < 8; ++t)
            ss += (float)v[t] * (float)v[t];
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0)
        part_lds[tid >> 6] = ss;
    __syncthreads();
    const float mean = (part_lds[0] + part_lds[1] + part_lds[2] + part_lds[3]) / (float)hidden;
    const float r = 1.0f / __builtin_sqrtf(mean + eps);
    for (int k = tid * 8; k < hidden; k += 256 * 8) {
        const f16x8 v = *reinterpret_cast<const f16x8 *>(x + k); // this thread's own writes
        const f16x8 w = *reinterpret_cast<const f16x8 *>(weight + k);
        f16x8 o;
#pragma unroll
        for (int t = 0; t < 8; ++t)
            o[t] = w[t] * (f16)((float)v[t] * r);
        *reinterpret_cast<f16x8 *>(y + k) = o;
    }
}

} // namespace

int launch_router_top2(const f16 *x, const f16 *w, int n_experts, int64_t hidden, int *sel, f16 *weights, f16 *logits,
                       hipStream_t s)
{
    if (n_experts < 2 || n_experts > kMaxExperts || hidden % 8 != 0 || hidden <= 0 || hidden > (1 << 24))
        return HQQ_E_SHAPE;
    if (!aligned16(x) || !aligned16(w))
        return HQQ_E_ALIGN;
    router_top2_kernel<<<1, 64 * kMaxExperts, 0, s>>>(x, w, n_experts, (int)hidden, sel, weights, logits);
    return launch_status();
}

int launch_add_rmsnorm(f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *y, int64_t hidden, hipStream_t s)
{
    if (hidden % 8 != 0 || hidden <= 0 || hidden > (1 << 24))
        return HQQ_E_SHAPE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || (delta && !aligned16(delta)))
        return HQQ_E_ALIGN;
    add_rmsnorm_kernel<<<1, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden);
    return launch_status();
}

} // namespace hqq
