// General kernel: any N, K, group size and batch, no alignment demands.
// One wavefront per output column n walks K one element per lane, rebuilding
// each weight exactly as the reference does.  It is the safety net for shapes
// the tuned kernels do not take, and the in-library cross-check for them.
#include "hqq_common.hpp"

namespace hqq {
namespace {

constexpr int kMT = 8; // batch rows per pass

template <int NBITS>
__global__ __launch_bounds__(256) void general_matmul_kernel(const void *__restrict__ codes, Table sc, Table zr,
                                                             const f16 *__restrict__ bias, const f16 *__restrict__ x,
                                                             int64_t M, int64_t N, int64_t K, int64_t G,
                                                             f16 *__restrict__ y)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t n = wave; n < N; n += nwaves) {
        const int64_t j = n % G;
        for (int64_t m0 = 0; m0 < M; m0 += kMT) {
            float acc[kMT];
#pragma unroll
            for (int m = 0; m < kMT; ++m)
                acc[m] = 0.f;
            for (int64_t k = lane; k < K; k += 64) {
                const f16 q = (f16)(float)code_at<NBITS>(codes, n, k, K);
                const f16 d = q - table_at(zr, j * K + k);
                const float w = (float)(f16)(d * table_at(sc, j * K + k));
#pragma unroll
                for (int m = 0; m < kMT; ++m)
                    if (m0 + m < M)
                        acc[m] = __builtin_fmaf((float)x[(m0 + m) * K + k], w, acc[m]);
            }
#pragma unroll
            for (int m = 0; m < kMT; ++m) {
                const float v = wave_sum(acc[m]);
                if (lane == 0 && m0 + m < M) {
                    f16 r = (f16)v;
                    if (bias)
                        r = r + bias[n]; // fp16 add after the cast, as `c + bias` in the reference wrappers
                    y[(m0 + m) * N + n] = r;
                }
            }
        }
    }
}

} // namespace

int launch_general_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, hipStream_t s)
{
    const int64_t G = l->N / l->group_size;
    int64_t blocks = (l->N + 3) / 4;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    const Table sc = make_table(l->scale), zr = make_table(l->zero);
    const f16 *bias = static_cast<const f16 *>(l->bias);
    if (l->nbits == 4)
        general_matmul_kernel<4><<<(int)blocks, 256, 0, s>>>(l->codes, sc, zr, bias, x, M, l->N, l->K, G, y);
    else if (l->nbits == 2)
        general_matmul_kernel<2><<<(int)blocks, 256, 0, s>>>(l->codes, sc, zr, bias, x, M, l->N, l->K, G, y);
    else
        general_matmul_kernel<3><<<(int)blocks, 256, 0, s>>>(l->codes, sc, zr, bias, x, M, l->N, l->K, G, y);
    return launch_status();
}

} // namespace hqq
