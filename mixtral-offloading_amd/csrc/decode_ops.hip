// Small decode-step kernels around the quantized linears: the router (reference src/custom_layers.py:276-282)
// and the residual add + RMSNorm of the decoder layer.  One block each: at batch 1 they are latency, not bandwidth.
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

// Rotary embedding, KV-cache append and attention of ONE new token (the reference takes them from HF transformers'
// Mixtral attention): one block per query head.  Roundings follow the fp16 torch ops they replace: rope terms
// rounded separately, scores = fp16(q . k) then / sqrt(hd) in fp32, softmax in fp32, probabilities cast to fp16,
// output accumulated in fp32.  The current position is read from device memory, so the launch can be replayed
// from a graph; positions 0 .. pos are attended (the new key and value are taken from registers, and also
// written to the cache by the first head of each KV group).
// One block of NT threads per head: 256 for caches of up to 512 positions, 1024 beyond (the block walks the head's
// cache rows, so a long cache wants more threads and a short one fewer reduction steps).
template <int HD, int NT>
__global__ __launch_bounds__(NT) void attention_decode_kernel(const f16 *__restrict__ q_in, const f16 *__restrict__ k_in,
                                                               const f16 *__restrict__ v_in, const f16 *__restrict__ cos_t,
                                                               const f16 *__restrict__ sin_t, const int64_t *__restrict__ pos_p,
                                                               f16 *__restrict__ cache_k, f16 *__restrict__ cache_v,
                                                               int64_t max_len, int group, f16 *__restrict__ out)
{
    extern __shared__ float score_lds[]; // [pos + 1]
    __shared__ __attribute__((aligned(16))) f16 q_lds[HD];
    __shared__ __attribute__((aligned(16))) f16 k_lds[HD];
    constexpr int NW = NT / 64;
    __shared__ float red_lds[2 * NW];
    __shared__ float acc_lds[NT / (HD / 8)][HD];
    const int h = blockIdx.x, kv = h / group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the new token's q, k and v do not depend on the position: their loads go out before it is waited for
    const int d = tid < HD ? tid : 0, dr = d < HD / 2 ? d + HD / 2 : d - HD / 2;
    const f16 qa = q_in[h * HD + d], qb = q_in[h * HD + dr];
    const f16 ka = k_in[kv * HD + d], kb = k_in[kv * HD + dr];
    const f16 vnew = v_in[kv * HD + d];
    const int64_t pos = pos_p[0];
    if (pos < 0 || pos >= max_len) // the position lives in device memory: a step past the cache must not write past it
        return;
    const f16 *cs = cos_t + pos * HD, *sn = sin_t + pos * HD;
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
    if (tid < HD) {
        const f16 qr = d < HD / 2 ? -qb : qb, kr = d < HD / 2 ? -kb : kb;
        const f16 qrot = (f16)(qa * cs[d]) + (f16)(qr * sn[d]);
        const f16 krot = (f16)(ka * cs[d]) + (f16)(kr * sn[d]);
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
    f16x8 vfirst[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t l = u * ROWS + rsub;
        const int64_t lc = l <= pos ? l : pos;
        const f16 *vrow = lc == pos ? v_in + kv * HD : cache_v + ((int64_t)kv * max_len + lc) * HD;
        vfirst[u] = *reinterpret_cast<const f16x8 *>(vrow + 8 * c8);
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
                const f16 *vrow = lc == pos ? v_in + kv * HD : cache_v + ((int64_t)kv * max_len + lc) * HD;
                vv[u] = *reinterpret_cast<const f16x8 *>(vrow + 8 * c8);
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
    if (tid < HD) {
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
            a += acc_lds[r][tid];
        out[h * HD + tid] = (f16)a;
    }
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
    if (head_dim == 128 && max_len <= 512)
        attention_decode_kernel<128, 256><<<n_heads, 256, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    else if (head_dim == 128)
        attention_decode_kernel<128, 1024><<<n_heads, 1024, lds, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len, group, out);
    else if (max_len <= 512)
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
