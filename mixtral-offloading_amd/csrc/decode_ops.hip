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
    // one block per token (row)
    x += (int64_t)blockIdx.x * hidden;
    sel += 2 * blockIdx.x, weights += 2 * blockIdx.x;
    if (logits_out)
        logits_out += (int64_t)blockIdx.x * n_experts;
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
    // one block per token (row)
    x += (int64_t)blockIdx.x * hidden, y += (int64_t)blockIdx.x * hidden;
    if (delta)
        delta += (int64_t)blockIdx.x * hidden;
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

// Long caches: the positions of a head are split over several blocks, so that the walk over the cache is shared by
// more compute units than there are heads.  Block (head, part) attends its share of positions 0 .. pos and leaves the
// largest score m, the sum l of exp(score - m) and the un-normalised output sum(exp(score - m) * v) of that share in
// the workspace (device-scope stores); the block of a head that counts itself last adds the shares up,
//     out = sum_p o_p * exp(m_p - m) / sum_p l_p * exp(m_p - m),   m = max_p m_p,
// so nobody waits for anybody.  Scores are rounded as in the one-block kernel (fp16(q . k) / sqrt(hd)); the
// probabilities stay fp32 here (a share does not know the whole sum, so they cannot be rounded to fp16 before they
// multiply the values as the one-block kernel does): the results agree within fp16 rounding, not bit for bit.
constexpr int kSplitRecord(int hd) { return hd + 2; } // floats a block leaves: m, l, o[hd]
constexpr int64_t kSplitRows = 1024;                   // positions per block from which a split pays

template <int HD>
__global__ __launch_bounds__(1024) void attention_split_kernel(const f16 *__restrict__ q_in, const f16 *__restrict__ k_in,
                                                                const f16 *__restrict__ v_in, const f16 *__restrict__ cos_t,
                                                                const f16 *__restrict__ sin_t, const int64_t *__restrict__ pos_p,
                                                                f16 *__restrict__ cache_k, f16 *__restrict__ cache_v,
                                                                int64_t max_len, int group, int parts, float *part_out,
                                                                int *counters, f16 *__restrict__ out)
{
    constexpr int NT = 1024, NW = NT / 64, LP = HD / 8, ROWS = NT / LP, NPART = ROWS / 16;
    extern __shared__ float score_lds[]; // the share's scores, then their exponentials
    __shared__ __attribute__((aligned(16))) f16 q_lds[HD];
    __shared__ __attribute__((aligned(16))) f16 k_lds[HD];
    __shared__ float red_lds[2 * NW];
    __shared__ float acc_lds[ROWS][HD];
    __shared__ int last_lds;
    const int h = (int)blockIdx.x / parts, sp = (int)blockIdx.x - h * parts, kv = h / group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int d = tid < HD ? tid : 0, dr = d < HD / 2 ? d + HD / 2 : d - HD / 2;
    const f16 qa = q_in[h * HD + d], qb = q_in[h * HD + dr];
    const f16 ka = k_in[kv * HD + d], kb = k_in[kv * HD + dr];
    const f16 vnew = v_in[kv * HD + d];
    const int64_t pos = pos_p[0];
    if (pos < 0 || pos >= max_len) // (every block of the launch leaves alike: no counter is touched)
        return;
    const f16 cs_d = cos_t[pos * HD + d], sn_d = sin_t[pos * HD + d];
    // as many blocks as the positions so far give a thousand rows each (handing shares over costs about as much as
    // walking a thousand rows): the others leave at once, and a single block writes the output itself
    const int64_t n = pos + 1;
    const int64_t want = (n + kSplitRows - 1) / kSplitRows;
    const int eff = want < parts ? (int)want : parts;
    if (sp >= eff)
        return;
    const int64_t chunk = (n + eff - 1) / eff;
    const int64_t lo = (int64_t)sp * chunk, hi = lo + chunk < n ? lo + chunk : n; // empty when lo >= n
    if (tid < HD) {
        const f16 qr = d < HD / 2 ? -qb : qb, kr = d < HD / 2 ? -kb : kb;
        const f16 qrot = (f16)(qa * cs_d) + (f16)(qr * sn_d);
        const f16 krot = (f16)(ka * cs_d) + (f16)(kr * sn_d);
        q_lds[d] = qrot;
        k_lds[d] = krot;
        if (sp == 0 && h % group == 0) { // (block 0 of a head always works)
            cache_k[((int64_t)kv * max_len + pos) * HD + d] = krot;
            cache_v[((int64_t)kv * max_len + pos) * HD + d] = vnew;
        }
    }
    __syncthreads();
    const int rsub = tid / LP, c8 = tid % LP; // LP lanes share a cache row, 16 bytes each
    const float inv = 1.0f / __builtin_sqrtf((float)HD);
    float mx = -3.0e38f;
    {
        const f16x8 qq = *reinterpret_cast<const f16x8 *>(q_lds + 8 * c8);
        for (int64_t l0 = lo; l0 < hi; l0 += 4 * ROWS) {
            f16x8 kk[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int64_t l = l0 + u * ROWS + rsub;
                const int64_t lc = l < hi ? l : hi - 1;
                if (lc == pos) // the new token's key is not in the cache yet for the other heads of its group
                    kk[u] = *reinterpret_cast<const f16x8 *>(k_lds + 8 * c8);
                else
                    kk[u] = *reinterpret_cast<const f16x8 *>(cache_k + ((int64_t)kv * max_len + lc) * HD + 8 * c8);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float acc = 0.f;
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    acc += (float)kk[u][t] * (float)qq[t];
#pragma unroll
                for (int off = LP / 2; off > 0; off >>= 1)
                    acc += __shfl_xor(acc, off, 64);
                const int64_t l = l0 + u * ROWS + rsub;
                if (c8 == 0 && l < hi) {
                    const float sc = (float)(f16)acc * inv;
                    score_lds[l - lo] = sc;
                    mx = fmaxf(mx, sc);
                }
            }
        }
    }
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
    for (int64_t i = tid; i < hi - lo; i += NT) {
        const float e = __expf(score_lds[i] - mx);
        score_lds[i] = e;
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

    float o[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
        o[t] = 0.f;
    for (int64_t l0 = lo; l0 < hi; l0 += 4 * ROWS) {
        f16x8 vv[4];
        float pr[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t l = l0 + u * ROWS + rsub;
            const int64_t lc = l < hi ? l : hi - 1;
            const f16 *vrow = lc == pos ? v_in + kv * HD : cache_v + ((int64_t)kv * max_len + lc) * HD;
            vv[u] = *reinterpret_cast<const f16x8 *>(vrow + 8 * c8);
            pr[u] = l < hi ? score_lds[lc - lo] : 0.f;
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
    static_assert(ROWS % 16 == 0 && NT >= HD * NPART, "one thread per column and group of sixteen partial outputs");
    if (tid < HD * NPART) {
        const int pt = tid / HD, dcol = tid % HD;
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            a += acc_lds[16 * pt + r][dcol];
        acc_lds[16 * pt][dcol] = a;
    }
    __syncthreads();
    if (eff == 1) {
        if (tid < HD) {
            float a = 0.f;
#pragma unroll
            for (int pt = 0; pt < NPART; ++pt)
                a += acc_lds[16 * pt][tid];
            out[h * HD + tid] = (f16)(a / sum);
        }
        return;
    }
    // the share's record, at device scope: the block that adds the shares up may run on another XCD
    float *const mine = part_out + ((int64_t)h * parts + sp) * kSplitRecord(HD);
    if (tid < HD) {
        float a = 0.f;
#pragma unroll
        for (int pt = 0; pt < NPART; ++pt)
            a += acc_lds[16 * pt][tid];
        __hip_atomic_store(mine + 2 + tid, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid == 0) {
        __hip_atomic_store(mine, mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(mine + 1, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0); // every store of this thread is acknowledged
    __syncthreads();
    if (tid == 0) {
        const int prev = __hip_atomic_fetch_add(&counters[h], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == eff - 1) // every share is there: leave the counter ready for the next launch
            __hip_atomic_store(&counters[h], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_lds = prev == eff - 1;
    }
    __syncthreads();
    if (!last_lds || tid >= HD)
        return;
    const float *const rec = part_out + (int64_t)h * parts * kSplitRecord(HD);
    // every share's record requested in one batch (at most eight), then added up in a fixed order: the result does not
    // depend on which block came last
    constexpr int kMaxParts = 8;
    float ms[kMaxParts], ls[kMaxParts], os[kMaxParts];
#pragma unroll
    for (int p = 0; p < kMaxParts; ++p) {
        const float *r = rec + (p < eff ? p : 0) * kSplitRecord(HD);
        ms[p] = __hip_atomic_load(r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ls[p] = __hip_atomic_load(r + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        os[p] = __hip_atomic_load(r + 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float m = -3.0e38f;
#pragma unroll
    for (int p = 0; p < kMaxParts; ++p)
        m = p < eff ? fmaxf(m, ms[p]) : m;
    float tot = 0.f, acc = 0.f;
#pragma unroll
    for (int p = 0; p < kMaxParts; ++p) {
        const float f = p < eff ? __expf(ms[p] - m) : 0.f;
        tot += ls[p] * f;
        acc += os[p] * f;
    }
    out[h * HD + tid] = (f16)(acc / tot);
}

// Rotary embedding and KV-cache append for `rows` new tokens of one sequence at positions start .. start + rows - 1
// (the prompt pass): q (rows, n_heads * hd) is rotated in place, the rotated keys and the values go to
// cache_k / cache_v [n_kv][max_len][hd].  Block (token, head), head < n_heads a query head, else a key/value head;
// the arithmetic is the one-token kernel's: fp16(x * cos) + fp16(rotate_half(x) * sin), three fp16 roundings.
__global__ __launch_bounds__(256) void rope_append_rows_kernel(f16 *__restrict__ q, const f16 *__restrict__ k,
                                                               const f16 *__restrict__ v, const f16 *__restrict__ cos_t,
                                                               const f16 *__restrict__ sin_t, int64_t start, int n_heads,
                                                               int n_kv, int hd, f16 *__restrict__ cache_k,
                                                               f16 *__restrict__ cache_v, int64_t max_len)
{
    const int t = blockIdx.x, hh = blockIdx.y, d = threadIdx.x;
    const int64_t pos = start + t;
    const bool on = d < hd;
    const int dc = on ? d : 0;
    const int dr = dc < hd / 2 ? dc + hd / 2 : dc - hd / 2;
    const f16 cs = cos_t[pos * hd + dc], sn = sin_t[pos * hd + dc];
    if (hh < n_heads) {
        f16 *row = q + ((int64_t)t * n_heads + hh) * hd;
        const f16 a = row[dc], b = row[dr];
        __syncthreads(); // every element is read before any is overwritten
        const f16 r = dc < hd / 2 ? -b : b;
        if (on)
            row[dc] = (f16)(a * cs) + (f16)(r * sn);
    } else {
        const int kvh = hh - n_heads;
        const f16 *row = k + ((int64_t)t * n_kv + kvh) * hd;
        const f16 a = row[dc], b = row[dr];
        const f16 r = dc < hd / 2 ? -b : b;
        if (on) {
            cache_k[((int64_t)kvh * max_len + pos) * hd + dc] = (f16)(a * cs) + (f16)(r * sn);
            cache_v[((int64_t)kvh * max_len + pos) * hd + dc] = v[((int64_t)t * n_kv + kvh) * hd + dc];
        }
    }
}

} // namespace

// blocks per head: one up to 1024 positions (the one-block kernel, whose roundings are the reference ops'), then one
// per thousand positions of the cache, eight at most; how many of them a launch uses follows the position
int attention_parts(int64_t max_len)
{
    const int forced = tuning_int("HQQ_ATT_PARTS", 0);
    if (forced > 0)
        return forced < 8 ? forced : 8;
    const int64_t want = (max_len + kSplitRows - 1) / kSplitRows;
    return want < 1 ? 1 : (want > 8 ? 8 : (int)want);
}

size_t attention_workspace_bytes(int64_t max_len, int n_heads, int head_dim)
{
    const int parts = attention_parts(max_len);
    if (parts <= 1)
        return 0;
    return 256 + (((size_t)n_heads * sizeof(int) + 255) & ~(size_t)255) + (size_t)n_heads * parts * kSplitRecord(head_dim) * sizeof(float);
}

int launch_attention_decode(const f16 *q, const f16 *k, const f16 *v, const f16 *cos_t, const f16 *sin_t, const int64_t *pos,
                            f16 *cache_k, f16 *cache_v, int64_t max_len, int n_heads, int n_kv_heads, int head_dim, f16 *out,
                            hipStream_t s, void *ws, size_t ws_bytes)
{
    if (n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || max_len < 1 || max_len > 16000)
        return HQQ_E_SHAPE;
    if (head_dim != 64 && head_dim != 128)
        return HQQ_E_UNSUPPORTED;
    if (!aligned16(cache_k) || !aligned16(cache_v))
        return HQQ_E_ALIGN;
    const int group = n_heads / n_kv_heads;
    const int parts = attention_parts(max_len);
    // with a workspace (zero-filled once; the counters in it are left at zero) long caches are split over blocks
    if (parts > 1 && ws && ws_bytes >= attention_workspace_bytes(max_len, n_heads, head_dim) &&
        (reinterpret_cast<uintptr_t>(ws) & 255u) == 0 && (int64_t)n_heads * parts <= 65535) {
        int *counters = reinterpret_cast<int *>(static_cast<char *>(ws) + 256);
        float *part_out = reinterpret_cast<float *>(static_cast<char *>(ws) + 256 + (((size_t)n_heads * sizeof(int) + 255) & ~(size_t)255));
        // a block's share: the cache over all blocks, or everything so far while that is a thousand rows or fewer
        const int64_t even = (max_len + parts - 1) / parts, few = max_len < kSplitRows ? max_len : kSplitRows;
        const size_t lds_part = (size_t)(even > few ? even : few) * sizeof(float);
        if (head_dim == 128)
            attention_split_kernel<128><<<n_heads * parts, 1024, lds_part, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len,
                                                                                  group, parts, part_out, counters, out);
        else
            attention_split_kernel<64><<<n_heads * parts, 1024, lds_part, s>>>(q, k, v, cos_t, sin_t, pos, cache_k, cache_v, max_len,
                                                                                 group, parts, part_out, counters, out);
        return launch_status();
    }
    const size_t lds = (size_t)max_len * sizeof(float);
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
                       hipStream_t s, int64_t rows)
{
    if (rows < 1 || rows > 0x7fffffff)
        return HQQ_E_SHAPE;
    if (n_experts < 2 || n_experts > kMaxExperts || hidden % 8 != 0 || hidden <= 0 || hidden > (1 << 24))
        return HQQ_E_SHAPE;
    if (!aligned16(x) || !aligned16(w))
        return HQQ_E_ALIGN;
    router_top2_kernel<<<(unsigned)rows, 64 * kMaxExperts, 0, s>>>(x, w, n_experts, (int)hidden, sel, weights, logits);
    return launch_status();
}

// The (token, slot) pairs of a prompt pass grouped by expert: a stable counting sort of pair p = 2 * token + slot by
// sel[p], in one block.  Thread t owns the pairs t * chunk .. (t + 1) * chunk - 1: it counts them per expert, thread e
// turns the counts of expert e into each thread's first place (the experts one after the other, the threads in
// order), and every thread places its pairs in order.  Out: counts[e]; for row r of the grouped order the token it
// came from (64-bit, as index_add_ takes it) and its routing weight.
constexpr int kGroupThreads = 256;
__global__ __launch_bounds__(kGroupThreads) void moe_group_pairs_kernel(const int *__restrict__ sel,
                                                                          const f16 *__restrict__ weights, int pairs,
                                                                          int n_experts, int *__restrict__ counts,
                                                                          long long *__restrict__ token_of_row,
                                                                          f16 *__restrict__ scale_of_row)
{
    __shared__ int first[kGroupThreads][kMaxExperts + 1]; // (+1: the threads of a wave fall into different banks)
    __shared__ int base[kMaxExperts];
    __shared__ int total;
    const int t = threadIdx.x;
    const int chunk = (pairs + kGroupThreads - 1) / kGroupThreads;
    const int lo = t * chunk < pairs ? t * chunk : pairs, hi = lo + chunk < pairs ? lo + chunk : pairs;
    for (int e = 0; e < n_experts; ++e)
        first[t][e] = 0;
    for (int p = lo; p < hi; ++p) {
        const int e = sel[p];
        if (e >= 0 && e < n_experts)
            ++first[t][e];
    }
    __syncthreads();
    if (t < n_experts) {
        int run = 0;
        for (int u = 0; u < kGroupThreads; ++u) {
            const int c = first[u][t];
            first[u][t] = run;
            run += c;
        }
        counts[t] = run;
        base[t] = run;
    }
    __syncthreads();
    if (t == 0) {
        int run = 0;
        for (int e = 0; e < n_experts; ++e) {
            const int c = base[e];
            base[e] = run;
            run += c;
        }
        total = run;
    }
    __syncthreads();
    for (int p = lo; p < hi; ++p) {
        const int e = sel[p];
        if (e < 0 || e >= n_experts)
            continue;
        const int row = base[e] + first[t][e]++;
        token_of_row[row] = p >> 1;
        scale_of_row[row] = weights[p];
    }
    // pairs whose expert is out of range are left out of the counts; the rows that stay free at the end name token 0
    // with weight zero, so that a caller who indexes with all of them reads valid memory and adds nothing
    for (int row = total + t; row < pairs; row += kGroupThreads) {
        token_of_row[row] = 0;
        scale_of_row[row] = (f16)0.0f;
    }
}

int launch_moe_group_pairs(const int *sel, const f16 *weights, int64_t tokens, int n_experts, int *counts,
                           long long *token_of_row, f16 *scale_of_row, hipStream_t s)
{
    if (tokens < 1 || tokens > (1 << 28) || n_experts < 2 || n_experts > kMaxExperts)
        return HQQ_E_SHAPE;
    moe_group_pairs_kernel<<<1, kGroupThreads, 0, s>>>(sel, weights, (int)(2 * tokens), n_experts, counts, token_of_row,
                                                       scale_of_row);
    return launch_status();
}

int launch_add_rmsnorm(f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *y, int64_t hidden, hipStream_t s,
                       int64_t rows)
{
    if (hidden % 8 != 0 || hidden <= 0 || hidden > (1 << 24) || rows < 1 || rows > 0x7fffffff)
        return HQQ_E_SHAPE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || (delta && !aligned16(delta)))
        return HQQ_E_ALIGN;
    add_rmsnorm_kernel<<<(unsigned)rows, 256, 0, s>>>(x, delta, weight, eps, y, (int)hidden);
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

int launch_rope_append_rows(f16 *q, const f16 *k, const f16 *v, const f16 *cos_t, const f16 *sin_t, int64_t start,
                            int64_t rows, f16 *cache_k, f16 *cache_v, int64_t max_len, int n_heads, int n_kv_heads,
                            int head_dim, hipStream_t s)
{
    if (head_dim < 2 || head_dim > 256 || head_dim % 2 != 0 || n_heads < 1 || n_kv_heads < 1 || n_heads + n_kv_heads > 65535 ||
        rows < 1 || rows > 0x7fffffff || start < 0 || start + rows > max_len)
        return HQQ_E_SHAPE;
    const dim3 grid((unsigned)rows, (unsigned)(n_heads + n_kv_heads));
    rope_append_rows_kernel<<<grid, 256, 0, s>>>(q, k, v, cos_t, sin_t, start, n_heads, n_kv_heads, head_dim, cache_k,
                                                 cache_v, max_len);
    return launch_status();
}

} // namespace hqq
