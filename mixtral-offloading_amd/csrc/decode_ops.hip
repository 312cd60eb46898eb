// Small decode-step kernels around the quantized linears: the router (reference src/custom_layers.py:276-282)
// and the residual add + RMSNorm of the decoder layer.  One block each: at batch 1 they are latency, not bandwidth.
#include "attention_parts.hpp"
#include "hqq_common.hpp"
#include "norm_route.hpp"

namespace hqq {
namespace {

// logits = fp16(x W^T) (fp32 accumulation, one rounding, as a half linear does); softmax in fp32; the two largest
// probabilities, renormalised by their sum, cast to fp16 (reference src/custom_layers.py:277-282).
__global__ __launch_bounds__(64 * kMaxExperts) void router_top2_kernel(const f16 *__restrict__ x, const f16 *__restrict__ w,
                                                                       int n_experts, int hidden, int *__restrict__ sel,
                                                                       f16 *__restrict__ weights, f16 *__restrict__ logits_out)
{
    __shared__ float logit_lds[kMaxExperts];
    __shared__ float prob_lds[kMaxExperts];
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
    if (threadIdx.x < kMaxExperts)
        route_top2(logit_lds, prob_lds, n_experts, sel, weights, logits_out);
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

// add_rmsnorm_kernel followed by router_top2_kernel on its output, in one block: the post-attention norm of a decoder
// layer feeds the router directly (reference src/custom_layers.py:276-282 on the normed hidden state).
__global__ __launch_bounds__(256) void add_rmsnorm_router_kernel(f16 *__restrict__ x, const f16 *__restrict__ delta,
                                                                 const f16 *__restrict__ weight, float eps,
                                                                 f16 *__restrict__ y, int hidden,
                                                                 const f16 *__restrict__ gate_w, int n_experts,
                                                                 int *__restrict__ sel, f16 *__restrict__ weights,
                                                                 f16 *__restrict__ logits_out)
{
    __shared__ float part_lds[4];
    __shared__ float dot_lds[4][kMaxExperts];
    __shared__ float logit_lds[kMaxExperts];
    __shared__ float prob_lds[kMaxExperts];
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
    float dot[kMaxExperts];
#pragma unroll
    for (int e = 0; e < kMaxExperts; ++e)
        dot[e] = 0.f;
    for (int k = tid * 8; k < hidden; k += 256 * 8) {
        const f16x8 v = *reinterpret_cast<const f16x8 *>(x + k); // this thread's own writes
        const f16x8 w = *reinterpret_cast<const f16x8 *>(weight + k);
        f16x8 o;
#pragma unroll
        for (int t = 0; t < 8; ++t)
            o[t] = w[t] * (f16)((float)v[t] * r);
        *reinterpret_cast<f16x8 *>(y + k) = o;
#pragma unroll
        for (int e = 0; e < kMaxExperts; ++e) {
            if (e < n_experts) {
                const f16x8 g = *reinterpret_cast<const f16x8 *>(gate_w + (int64_t)e * hidden + k);
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    dot[e] += (float)o[t] * (float)g[t];
            }
        }
    }
#pragma unroll
    for (int e = 0; e < kMaxExperts; ++e) {
        if (e < n_experts) {
            const float d = wave_sum(dot[e]);
            if ((tid & 63) == 0)
                dot_lds[tid >> 6][e] = d;
        }
    }
    __syncthreads();
    if (tid < n_experts)
        logit_lds[tid] = (float)(f16)(dot_lds[0][tid] + dot_lds[1][tid] + dot_lds[2][tid] + dot_lds[3][tid]);
    __syncthreads();
    if (tid < kMaxExperts)
        route_top2(logit_lds, prob_lds, n_experts, sel, weights, logits_out);
}

// The same computation for hidden <= CH * 2048 and at most NE experts with every global load issued before the
// first use: the token, the norm weight and the thread's pieces of all router rows travel together, so the block
// waits for memory once.  Thread t owns elements (c * 256 + t) * 8 .. + 7 of chunk c.
template <int CH, int NE>
__global__ __launch_bounds__(256) void add_rmsnorm_router_once_kernel(f16 *__restrict__ x, const f16 *__restrict__ delta,
                                                                      const f16 *__restrict__ weight, float eps,
                                                                      f16 *__restrict__ y, int hidden,
                                                                      const f16 *__restrict__ gate_w, int n_experts,
                                                                      int *__restrict__ sel, f16 *__restrict__ weights,
                                                                      f16 *__restrict__ logits_out)
{
    __shared__ NormRouteLds<NE> lds;
    norm_route_block<CH, NE>(x, delta, weight, eps, x, y, hidden, gate_w, n_experts, sel, weights, logits_out, lds);
}

// One block of NT threads per head (attention_parts.hpp): 256 for caches of up to 512 positions, 1024 beyond.
template <int HD, int NT>
__global__ __launch_bounds__(NT) void attention_decode_kernel(const f16 *__restrict__ q_in, const f16 *__restrict__ k_in,
                                                               const f16 *__restrict__ v_in, const f16 *__restrict__ cos_t,
                                                               const f16 *__restrict__ sin_t, const int64_t *__restrict__ pos_p,
                                                               f16 *__restrict__ cache_k, f16 *__restrict__ cache_v,
                                                               int64_t max_len, int group, f16 *__restrict__ out)
{
    attention_head<HD, NT>(q_in, k_in, v_in, cos_t, sin_t, pos_p, cache_k, cache_v, max_len, group, out, (int)blockIdx.x,
                           CHAIN_NONE, nullptr, 0);
}

} // namespace

int launch_attention_decode(const f16 *q, const f16 *k, const f16 *v, const f16 *cos_t, const f16 *sin_t, const int64_t *pos,
                            f16 *cache_k, f16 *cache_v, int64_t max_len, int n_heads, int n_kv_heads, int head_dim, f16 *out,
                            hipStream_t s)
{
    if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || max_len < 1 || max_len > 16000)
        return HQQ_E_SHAPE;
    if (head_dim != 64 && head_dim != 128)
        return HQQ_E_UNSUPPORTED;
    if (!aligned16(cache_k) || !aligned16(cache_v))
        return HQQ_E_ALIGN;
    const size_t lds = (size_t)max_len * sizeof(float);
    const int group = n_heads / n_kv_heads;
    const int64_t small = attention_block_threads(max_len) == 256 ? max_len : 0;
    if (head_dim == 128 && max_len <= small)
        attention_decode_kernel<128, 256><<<n_heads, 256, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    else if (head_dim == 128)
        attention_decode_kernel<128, 1024><<<n_heads, 1024, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    else if (max_len <= small)
        attention_decode_kernel<64, 256><<<n_heads, 256, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    else
        attention_decode_kernel<64, 1024><<<n_heads, 1024, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    return launch_status();
}

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

int launch_add_rmsnorm_router(f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *y, int64_t hidden,
                              const f16 *gate_w, int n_experts, int *sel, f16 *weights, f16 *logits, hipStream_t s)
{
    if (hidden % 8 != 0 || hidden <= 0 || hidden > (1 << 24) || n_experts < 2 || n_experts > kMaxExperts)
        return HQQ_E_SHAPE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || (delta && !aligned16(delta)) || !aligned16(gate_w))
        return HQQ_E_ALIGN;
    if (n_experts <= 8 && hidden <= 2048)
        add_rmsnorm_router_once_kernel<1, 8><<<1, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden, gate_w, n_experts, sel,
                                                               weights, logits);
    else if (n_experts <= 8 && hidden <= 4096)
        add_rmsnorm_router_once_kernel<2, 8><<<1, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden, gate_w, n_experts, sel,
                                                               weights, logits);
    else if (hidden <= 2048)
        add_rmsnorm_router_once_kernel<1, 16><<<1, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden, gate_w, n_experts, sel,
                                                                weights, logits);
    else
        add_rmsnorm_router_kernel<<<1, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden, gate_w, n_experts, sel, weights,
                                                    logits);
    return launch_status();
}

} // namespace hqq
