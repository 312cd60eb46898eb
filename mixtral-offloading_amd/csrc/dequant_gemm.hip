// Wide batches: the weights de-quantised once per call into the workspace (hqq_dequantize: bit for bit the
// reference's dequantize(), src/custom_layers.py:95-116), then one library GEMM over the fp16 weights with fp32
// accumulation, which is the reference's own PyTorch path (dequantize, then torch.matmul).  From a few hundred rows
// on the de-quantising pass (one read of the codes, one write of N x K fp16) costs less than rebuilding the weights
// inside a matrix-core kernel once per batch tile, and a plain fp16 GEMM is what the vendor's library is tuned for.
#include "gemv_parts.hpp"
#include "hqq_common.hpp"

#include <rocblas/rocblas.h>

#include <mutex>

namespace hqq {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mutex;                  // a handle is used by one thread at a time
rocblas_handle g_handle[kMaxDevices]; // per device, created at the first call there

// y[m, n] += bias[n]; eight outputs per thread
__global__ __launch_bounds__(256) void add_bias_rows_kernel(f16 *__restrict__ y, const f16 *__restrict__ bias, int64_t M, int64_t N)
{
    const int64_t per_row = (N + 7) / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M * per_row)
        return;
    const int64_t m = i / per_row, n0 = (i - m * per_row) * 8;
    for (int64_t n = n0; n < n0 + 8 && n < N; ++n)
        y[m * N + n] = y[m * N + n] + bias[n];
}

} // namespace

// every validated layer can be de-quantised; the library call takes 32-bit sizes
bool dqgemm_supported(const hqq_linear *l, int64_t M)
{
    return M >= 1 && M < (1ll << 31) && l->N < (1ll << 31) && l->K < (1ll << 31);
}

// From how many rows on the de-quantise-then-GEMM form is the faster one (measured at Mixtral shapes, cache-cold: 2-
// and 4-bit layers with N >= K break even near 512 rows, with K > N near 1024, 3-bit layers, whose tile kernel pays
// for a rewrite of the codes as well, near 256; the thresholds sit a little above); small layers stay with the
// matrix-core kernels, whose launch is cheaper than two.
bool dqgemm_preferred(const hqq_linear *l, int64_t M)
{
    if (!dqgemm_supported(l, M) || l->N * l->K < (1ll << 22))
        return false;
    const int64_t from = l->nbits == 3 ? 320 : (l->N >= l->K ? 640 : 1280);
    return M >= from;
}

// The head of a workspace holds the other families' counters and accumulation slots, which they expect to find at
// zero: the de-quantised weights go behind it.
size_t dqgemm_workspace_bytes(const hqq_linear *l, int64_t)
{
    return gemv::kHeadBytes + (((size_t)l->N * (size_t)l->K * sizeof(f16) + 255u) & ~(size_t)255u);
}

int launch_dqgemm_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s)
{
    if (!dqgemm_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (!ws || ws_bytes < dqgemm_workspace_bytes(l, M))
        return HQQ_E_WORKSPACE;
    f16 *w = reinterpret_cast<f16 *>(static_cast<char *>(ws) + gemv::kHeadBytes);
    int rc = hqq_dequantize(l, w, s);
    if (rc != HQQ_OK)
        return rc;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return HQQ_E_UNSUPPORTED;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (!g_handle[dev] && rocblas_create_handle(&g_handle[dev]) != rocblas_status_success) {
            g_handle[dev] = nullptr;
            return HQQ_E_UNSUPPORTED;
        }
        if (rocblas_set_stream(g_handle[dev], s) != rocblas_status_success)
            return HQQ_E_UNSUPPORTED;
        // row-major y (M, N) = x (M, K) . w (N, K)^T is, column-major, y^T (N x M) = w^T-as-stored (K x N)^T . x^T (K x M)
        const float alpha = 1.0f, beta = 0.0f;
        const rocblas_status st = rocblas_gemm_ex(
            g_handle[dev], rocblas_operation_transpose, rocblas_operation_none, (rocblas_int)l->N, (rocblas_int)M,
            (rocblas_int)l->K, &alpha, w, rocblas_datatype_f16_r, (rocblas_int)l->K, x, rocblas_datatype_f16_r,
            (rocblas_int)l->K, &beta, y, rocblas_datatype_f16_r, (rocblas_int)l->N, y, rocblas_datatype_f16_r,
            (rocblas_int)l->N, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
        if (st != rocblas_status_success)
            return HQQ_E_UNSUPPORTED;
    }
    if (l->bias) {
        const int64_t threads = M * ((l->N + 7) / 8);
        add_bias_rows_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, s>>>(y, static_cast<const f16 *>(l->bias), M, l->N);
    }
    return launch_status();
}

} // namespace hqq
