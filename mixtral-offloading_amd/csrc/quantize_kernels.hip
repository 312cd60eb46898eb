// HQQ's quantiser (hqq Quantizer.quantize / optimize_weights, called at src/custom_layers.py:35-39 and
// src/build_model.py:108-120) for the grouping this path uses: the tensor seen as a row-major (rows, cols) matrix
// whose COLUMNS are the groups (axis 0: rows = group size, cols = N*K / group size), and the one-group form used for
// the zero table's 8-bit meta (min and max over the whole tensor).
//
//   scale = min((2^b - 1) / (max - min), 2e4),  zero = -min * scale  (rounded when asked),
//   optionally refined by the half-quadratic solver (shrinkage of the residual in the l_p norm, p < 1, and the
//   closed-form zero update, beta growing by kappa per iteration, stopped by the mean absolute error of the whole
//   tensor),  q = clamp(round(w * scale + zero), 0, 2^b - 1),  outputs q, 1 / scale, zero.
//
// One thread owns CP neighbouring groups (4, 2 or 1, by what the registers hold) and keeps their values in registers,
// so every iteration of the solver is register arithmetic; consecutive threads read consecutive pieces of a row, so
// every row is a coalesced streaming read of 4 to 16 bytes per thread.  The solver
// stops for the WHOLE tensor at once: a first pass adds up the error of every iteration (fp64 atomics), a one-thread
// kernel finds the iteration the host loop would have stopped at, and a second pass repeats that many iterations and
// writes the result.  All arithmetic is fp32 with separate multiplies and adds, as the tensor ops it replaces.
#include "hqq_common.hpp"

#include <cmath>

namespace hqq {
namespace {

constexpr int kQThreads = 256;
constexpr int kQMaxIters = 64;

struct QuantParams {
    const void *w;
    int fp32_in;
    int64_t rows, cols;
    float max_v;
    int round_zero;
    int iters;
    float lp;
    double beta, kappa; // doubles, as in the host loop they restate
    uint8_t *codes;   // (rows, cols)
    float *inv_scale; // (cols)
    float *zero;      // (cols)
    double *err;      // [kQMaxIters] sums of |w - w_r| per iteration
    int *stop;        // [1] iterations the second pass runs
};

// CP consecutive values starting at element `at` (a multiple of CP)
template <int CP> __device__ __forceinline__ void load_w(const QuantParams &p, int64_t at, float (&out)[CP])
{
    if (p.fp32_in) {
        typedef float vec __attribute__((ext_vector_type(CP)));
        const vec v = *reinterpret_cast<const vec *>(static_cast<const float *>(p.w) + at);
#pragma unroll
        for (int j = 0; j < CP; ++j)
            out[j] = CP == 1 ? reinterpret_cast<const float *>(&v)[0] : v[j];
    } else {
        typedef _Float16 vec __attribute__((ext_vector_type(CP)));
        const vec v = *reinterpret_cast<const vec *>(static_cast<const f16 *>(p.w) + at);
#pragma unroll
        for (int j = 0; j < CP; ++j)
            out[j] = (float)(CP == 1 ? reinterpret_cast<const f16 *>(&v)[0] : v[j]);
    }
}

// sign(x) * relu(|x| - (1 / beta) * (|x| + 1e-8)^(p - 1))
__device__ __forceinline__ float shrink_lp(float x, float inv_beta, float pm1)
{
    const float a = __builtin_fabsf(x);
    const float t = a - inv_beta * __builtin_powf(a + 1e-8f, pm1);
    const float r = t > 0.f ? t : 0.f;
    return x > 0.f ? r : (x < 0.f ? -r : 0.f);
}

// PASS 0: no refinement, write the result.  PASS 1: add up the error of every iteration.  PASS 2: run *p.stop
// iterations, write the result.
template <int GS, int CP, int PASS> __global__ __launch_bounds__(kQThreads) void quantize_groups_kernel(QuantParams p)
{
    const int64_t c = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * CP; // first group of the thread
    const bool on = c < p.cols;
    const int64_t cc = on ? c : p.cols - CP;
    float w[GS][CP];
#pragma unroll
    for (int r = 0; r < GS; ++r)
        load_w<CP>(p, (int64_t)r * p.cols + cc, w[r]);
    float scale[CP], zero[CP];
#pragma unroll
    for (int j = 0; j < CP; ++j) {
        float mn = w[0][j], mx = w[0][j];
#pragma unroll
        for (int r = 1; r < GS; ++r) {
            mn = __builtin_fminf(mn, w[r][j]);
            mx = __builtin_fmaxf(mx, w[r][j]);
        }
        float sc = p.max_v / (mx - mn);
        scale[j] = sc < 2e4f ? sc : 2e4f; // (a constant group gives inf, clamped like any other large value)
        zero[j] = -mn * scale[j];
        if (p.round_zero)
            zero[j] = __builtin_rintf(zero[j]);
    }
    if constexpr (PASS != 0) {
        const int iters = PASS == 1 ? p.iters : *p.stop;
        __shared__ double red[kQThreads / 64];
        double beta = p.beta; // the host loop keeps beta as a double and hands 1 / beta to fp32 tensor ops
        const float pm1 = p.lp - 1.0f;
        for (int it = 0; it < iters; ++it) {
            const float inv_beta = (float)(1.0 / beta);
            float e = 0.f;
#pragma unroll
            for (int j = 0; j < CP; ++j) {
                float ej = 0.f, acc = 0.f;
#pragma unroll
                for (int r = 0; r < GS; ++r) {
                    float q = __builtin_rintf(w[r][j] * scale[j] + zero[j]);
                    q = __builtin_fminf(__builtin_fmaxf(q, 0.f), p.max_v);
                    const float wr = (q - zero[j]) / scale[j];
                    const float d = w[r][j] - wr;
                    ej += __builtin_fabsf(d);
                    const float we = shrink_lp(d, inv_beta, pm1);
                    acc += q - (w[r][j] - we) * scale[j];
                }
                zero[j] = acc / (float)GS;
                e += ej;
            }
            beta *= p.kappa;
            if constexpr (PASS == 1) {
                double s = on ? (double)e : 0.0;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1)
                    s += __shfl_xor(s, off, 64);
                if ((threadIdx.x & 63) == 0)
                    red[threadIdx.x >> 6] = s;
                __syncthreads();
                if (threadIdx.x == 0) {
                    double t = 0.0;
                    for (int i = 0; i < kQThreads / 64; ++i)
                        t += red[i];
                    atomicAdd(&p.err[it], t);
                }
                __syncthreads();
            }
        }
    }
    if constexpr (PASS != 1) {
        if (on) {
            typedef uint8_t bvec __attribute__((ext_vector_type(CP)));
#pragma unroll
            for (int r = 0; r < GS; ++r) {
                uint8_t qb[CP];
#pragma unroll
                for (int j = 0; j < CP; ++j) {
                    float q = __builtin_rintf(w[r][j] * scale[j] + zero[j]);
                    q = __builtin_fminf(__builtin_fmaxf(q, 0.f), p.max_v);
                    qb[j] = (uint8_t)q;
                }
                if constexpr (CP == 1) {
                    p.codes[(int64_t)r * p.cols + c] = qb[0];
                } else {
                    bvec v;
#pragma unroll
                    for (int j = 0; j < CP; ++j)
                        v[j] = qb[j];
                    *reinterpret_cast<bvec *>(p.codes + (int64_t)r * p.cols + c) = v;
                }
            }
#pragma unroll
            for (int j = 0; j < CP; ++j) {
                p.inv_scale[c + j] = 1.0f / scale[j];
                p.zero[c + j] = zero[j];
            }
        }
    }
}

// the iteration count of the host loop: it updates zero, then stops at the first iteration whose error (taken before
// the update) is not below the best so far
__global__ void quantize_stop_kernel(const double *err, int iters, double numel, int *stop)
{
    float best = 1e4f;
    int n = iters;
    for (int it = 0; it < iters; ++it) {
        const float e = (float)(err[it] / numel);
        if (e < best) {
            best = e;
        } else {
            n = it + 1;
            break;
        }
    }
    *stop = n;
}

__global__ void quantize_clear_kernel(double *err, int *stop)
{
    if (threadIdx.x < kQMaxIters)
        err[threadIdx.x] = 0.0;
    if (threadIdx.x == 0)
        *stop = 0;
}

// One group for the whole tensor (channel_wise = False).  Three launches: the extremes are cleared, every block
// folds its share of the tensor into them (floats ordered as integers, so that integer atomics find min and max),
// then every element is coded.
__device__ __forceinline__ int ordered(float v) // monotonic map of fp32 onto int32
{
    const int b = __builtin_bit_cast(int, v);
    return b >= 0 ? b : b ^ 0x7fffffff;
}
__device__ __forceinline__ float unordered(int o) { return __builtin_bit_cast(float, o >= 0 ? o : o ^ 0x7fffffff); }

__global__ void whole_clear_kernel(int *extremes)
{
    extremes[0] = 0x7fffffff; // min
    extremes[1] = (int)0x80000000; // max
}

__global__ __launch_bounds__(256) void whole_extremes_kernel(const float *x, int64_t n, int *extremes)
{
    __shared__ float mn_s[4], mx_s[4];
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x;
    float mn = x[first < n ? first : 0], mx = mn;
    for (int64_t i = first; i < n; i += (int64_t)gridDim.x * 256) {
        mn = __builtin_fminf(mn, x[i]);
        mx = __builtin_fmaxf(mx, x[i]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        mn = __builtin_fminf(mn, __shfl_xor(mn, off, 64));
        mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, 64));
    }
    if ((threadIdx.x & 63) == 0)
        mn_s[threadIdx.x >> 6] = mn, mx_s[threadIdx.x >> 6] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; ++i) {
            mn = __builtin_fminf(mn, mn_s[i]);
            mx = __builtin_fmaxf(mx, mx_s[i]);
        }
        atomicMin(&extremes[0], ordered(mn));
        atomicMax(&extremes[1], ordered(mx));
    }
}

__global__ __launch_bounds__(256) void whole_codes_kernel(const float *x, int64_t n, float max_v, const int *extremes,
                                                          uint8_t *codes, float *inv_scale, float *zero_out)
{
    const float mn = unordered(extremes[0]), mx = unordered(extremes[1]);
    float scale = max_v / (mx - mn);
    scale = scale < 2e4f ? scale : 2e4f;
    const float zero = -mn * scale;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        float q = __builtin_rintf(x[i] * scale + zero);
        q = __builtin_fminf(__builtin_fmaxf(q, 0.f), max_v);
        codes[i] = (uint8_t)q;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *inv_scale = 1.0f / scale;
        *zero_out = zero;
    }
}

template <int GS, int CP> int run_groups_cp(const QuantParams &p, hipStream_t s)
{
    const int64_t per_block = (int64_t)kQThreads * CP;
    const unsigned blocks = (unsigned)((p.cols + per_block - 1) / per_block);
    if (p.iters == 0) {
        quantize_groups_kernel<GS, CP, 0><<<blocks, kQThreads, 0, s>>>(p);
        return launch_status();
    }
    quantize_clear_kernel<<<1, 64, 0, s>>>(p.err, p.stop);
    quantize_groups_kernel<GS, CP, 1><<<blocks, kQThreads, 0, s>>>(p);
    quantize_stop_kernel<<<1, 1, 0, s>>>(p.err, p.iters, (double)p.rows * (double)p.cols, p.stop);
    quantize_groups_kernel<GS, CP, 2><<<blocks, kQThreads, 0, s>>>(p);
    return launch_status();
}

// groups per thread: as many as GS * CP values fit the registers, the column count and the pointers' alignment allow
template <int GS> int run_groups(const QuantParams &p, hipStream_t s)
{
    const int elem = p.fp32_in ? 4 : 2;
    auto fits = [&](int cp) {
        return p.cols % cp == 0 && (reinterpret_cast<uintptr_t>(p.w) % (size_t)(cp * elem)) == 0 &&
               (reinterpret_cast<uintptr_t>(p.codes) % (size_t)cp) == 0;
    };
    if constexpr (GS <= 32) {
        if (fits(4))
            return run_groups_cp<GS, 4>(p, s);
    }
    if constexpr (GS <= 64) {
        if (fits(2))
            return run_groups_cp<GS, 2>(p, s);
    }
    return run_groups_cp<GS, 1>(p, s);
}

} // namespace

size_t quantize_workspace_bytes() { return kQMaxIters * sizeof(double) + 64; }

int launch_quantize_groups(const void *w, int fp32_in, int64_t rows, int64_t cols, int nbits, int round_zero, int iters,
                           float lp, double beta, double kappa, uint8_t *codes, float *inv_scale, float *zero, void *ws,
                           size_t ws_bytes, hipStream_t s)
{
    if (rows < 1 || cols < 1 || nbits < 1 || nbits > 8 || iters < 0 || iters > kQMaxIters)
        return HQQ_E_SHAPE;
    if (cols >= (1ll << 31) * (int64_t)kQThreads)
        return HQQ_E_UNSUPPORTED;
    if (iters > 0 && (!ws || ws_bytes < quantize_workspace_bytes() || (reinterpret_cast<uintptr_t>(ws) & 7u)))
        return HQQ_E_WORKSPACE;
    QuantParams p = {};
    p.w = w, p.fp32_in = fp32_in, p.rows = rows, p.cols = cols;
    p.max_v = (float)((1 << nbits) - 1), p.round_zero = round_zero, p.iters = iters;
    p.lp = lp, p.beta = beta, p.kappa = kappa;
    p.codes = codes, p.inv_scale = inv_scale, p.zero = zero;
    p.err = static_cast<double *>(ws);
    p.stop = reinterpret_cast<int *>(static_cast<char *>(ws) + kQMaxIters * sizeof(double));
    switch (rows) {
    case 8: return run_groups<8>(p, s);
    case 16: return run_groups<16>(p, s);
    case 32: return run_groups<32>(p, s);
    case 64: return run_groups<64>(p, s);
    case 128: return run_groups<128>(p, s);
    default: return HQQ_E_UNSUPPORTED; // group sizes of the reference's configurations and of the 8-bit meta tables
    }
}

int launch_quantize_whole(const float *x, int64_t n, int nbits, uint8_t *codes, float *inv_scale, float *zero, void *ws,
                          size_t ws_bytes, hipStream_t s)
{
    if (n < 1 || nbits < 1 || nbits > 8)
        return HQQ_E_SHAPE;
    if (!ws || ws_bytes < quantize_workspace_bytes() || (reinterpret_cast<uintptr_t>(ws) & 7u))
        return HQQ_E_WORKSPACE;
    int *extremes = static_cast<int *>(ws);
    int64_t blocks = (n + 256 * 8 - 1) / (256 * 8);
    blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    whole_clear_kernel<<<1, 1, 0, s>>>(extremes);
    whole_extremes_kernel<<<(unsigned)blocks, 256, 0, s>>>(x, n, extremes);
    whole_codes_kernel<<<(unsigned)blocks, 256, 0, s>>>(x, n, (float)((1 << nbits) - 1), extremes, codes, inv_scale, zero);
    return launch_status();
}

} // namespace hqq
