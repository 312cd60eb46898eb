// Shared declarations of the gfx950 HQQ library: the C ABI, vector types and
// the table accessors every kernel uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>

#include "hqq_mi355x.h"

namespace hqq {

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Device-side copy of hqq_table with typed pointers.
struct Table {
    const void *data;
    const f16 *ms;
    const f16 *mz;
    int64_t meta_cols;
    int kind;
};

inline Table make_table(const hqq_table &t)
{
    Table r;
    r.data = t.data;
    r.ms = static_cast<const f16 *>(t.meta_scale);
    r.mz = static_cast<const f16 *>(t.meta_zero);
    r.meta_cols = t.meta_cols;
    r.kind = t.kind;
    return r;
}

// fp16 value of table entry c: either stored, or fp16(fp16(q - mz) * ms) with
// two roundings exactly as the reference's meta de-quantisation
// (reference src/custom_layers.py:63-66, formula restated at :111).
__device__ __forceinline__ f16 table_at(const Table &t, int64_t c)
{
    if (t.kind == HQQ_TABLE_F16)
        return static_cast<const f16 *>(t.data)[c];
    const int64_t mc = (t.meta_cols == 1) ? 0 : (c % t.meta_cols);
    const f16 q = (f16)(float)static_cast<const uint8_t *>(t.data)[c];
    const f16 d = q - t.mz[mc];
    return d * t.ms[mc];
}

// Code of weight (n, k) in the kernel layout
// (reference src/triton_kernels.py:84,91 / :272,279 / :462,469).
template <int NBITS>
__device__ __forceinline__ uint32_t code_at(const void *codes, int64_t n, int64_t k, int64_t K)
{
    if constexpr (NBITS == 4)
        return (static_cast<const uint8_t *>(codes)[(n >> 1) * K + k] >> (((n + 1) & 1) * 4)) & 0xFu;
    else if constexpr (NBITS == 2)
        return (static_cast<const uint8_t *>(codes)[(n >> 2) * K + k] >> ((3 - (n & 3)) * 2)) & 0x3u;
    else
        return (static_cast<const uint32_t *>(codes)[(n / 10) * K + k] >> ((9 - n % 10) * 3)) & 0x7u;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, kWave);
    return v;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The library never reads the environment.  A tuning build (make TUNING=1, -DHQQ_TUNING_BUILD, a separate .so that
// experiments select through HQQ_MI355X_LIB) lets HQQ_* variables override launch shapes; in the normal build these
// helpers are constants and the override code folds away.
#ifdef HQQ_TUNING_BUILD
inline int tuning_int(const char *name, int dflt)
{
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : dflt;
}
inline bool tuning_flag(const char *name) { return std::getenv(name) != nullptr; }
#else
constexpr int tuning_int(const char *, int dflt) { return dflt; }
constexpr bool tuning_flag(const char *) { return false; }
#endif

// launch-status helper: kernels are launched with <<<>>> and checked once
inline int launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? HQQ_OK : static_cast<int>(e);
}

// implemented in the individual translation units
int validate_linear(const hqq_linear *l);
int launch_general_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, hipStream_t s);
bool smallbatch_supported(const hqq_linear *l, int64_t M);
size_t smallbatch_workspace_bytes(const hqq_linear *l, int64_t M);
// epilogue selector of the small-batch kernel
struct SmallBatchEpilogue {
    const f16 *row_scale = nullptr; // optional per-row multiplier (routing weight)
    int accumulate = 0;             // add into y instead of storing
};
int launch_smallbatch_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                             const SmallBatchEpilogue &ep, hipStream_t s);
// fused w1/w3 pass: h = silu(x w1^T) * (x w3^T), fp16 (M, N)
int launch_smallbatch_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                              size_t ws_bytes, hipStream_t s);
// strip kernel (M <= 4, K % 256 == 0): the decode path; part of the small-batch family.  A block per tile, one or two
// slabs of 256 columns per wave, in-block gate epilogue
bool strip_supported(const hqq_linear *l, int64_t M);
size_t strip_workspace_bytes(const hqq_linear *l, int64_t M);
// What a decode kernel needs to know of a layer besides its shape; also the record of a device-side expert table.
struct LayerRecord {
    const uint8_t *codes;
    const uint8_t *sq, *zq; // 8-bit tables, or fp16 tables
    const f16 *s_ms, *s_mz; // meta of the scale table
    const f16 *z_ms, *z_mz; // meta of the zero table
    uint32_t s_cols, z_cols, s_inv, z_inv; // meta columns and floor(2^32 / columns)
};
static_assert(sizeof(LayerRecord) == 72, "the record is read as 18 words");
inline void fill_layer_record(LayerRecord &L, const hqq_linear *l)
{
    L.codes = static_cast<const uint8_t *>(l->codes);
    L.sq = static_cast<const uint8_t *>(l->scale.data);
    L.zq = static_cast<const uint8_t *>(l->zero.data);
    L.s_ms = static_cast<const f16 *>(l->scale.meta_scale);
    L.s_mz = static_cast<const f16 *>(l->scale.meta_zero);
    L.z_ms = static_cast<const f16 *>(l->zero.meta_scale);
    L.z_mz = static_cast<const f16 *>(l->zero.meta_zero);
    L.s_cols = (uint32_t)l->scale.meta_cols;
    L.z_cols = (uint32_t)l->zero.meta_cols;
    L.s_inv = L.s_cols ? (uint32_t)(0xFFFFFFFFull / L.s_cols) : 0;
    L.z_inv = L.z_cols ? (uint32_t)(0xFFFFFFFFull / L.z_cols) : 0;
}

// Indexed launch: the layer records come from a device table of strip_record_bytes() records, record
// sel[0] * stride + first (+ 1 for the second projection of the gate); the descriptors passed alongside only give
// the shape, which every record of the table must share.
struct StripIndex {
    const void *table;
    const int *sel;
    int stride, first;
};
bool strip_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M); // the fused w1/w3 launch
// decode batches of 3 to 16 rows (gemv_batch.hip): reached through the strip entry points
bool batch_supported(const hqq_linear *l, int64_t M);
bool batch_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M);
size_t batch_workspace_bytes(const hqq_linear *l, int64_t M);
int launch_batch_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                        const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix = nullptr);
int launch_batch_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                         size_t ws_bytes, hipStream_t s, const StripIndex *ix = nullptr);
size_t strip_record_bytes();
void strip_fill_record(void *dst, const hqq_linear *l);
int launch_strip_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                        const SmallBatchEpilogue &ep, hipStream_t s, const StripIndex *ix = nullptr);
int launch_strip_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                         size_t ws_bytes, hipStream_t s, const StripIndex *ix = nullptr);
int launch_strip_gate_up_pair(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, f16 *h0, f16 *h1, void *ws,
                              size_t ws_bytes, hipStream_t s, const StripIndex &ix);
int launch_strip_down_pair(const hqq_linear *w2, const f16 *h0, int64_t h_stride, f16 *y, const f16 *row_scale,
                           int accumulate, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix);
// residual add and RMSNorm folded into a grouped launch: the row is weight * rmsnorm(x + delta) (delta may be null)
// and x + delta goes to x_sum
struct StripNorm {
    const f16 *delta, *weight;
    f16 *x_sum;
    float eps;
};
int launch_strip_group(const hqq_linear *const *layers, int count, const f16 *x, f16 *const *ys, void *ws,
                       size_t ws_bytes, hipStream_t s, const StripNorm *norm = nullptr);
int launch_strip_gate_up_pair_routed(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, const StripNorm &norm,
                                     const f16 *gate_w, int n_experts, int *sel_out, f16 *rw_out, f16 *h0, f16 *h1,
                                     void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix);
size_t strip_job_workspace_bytes(const hqq_linear *const *layers, int count, int NL, int64_t M);
// The attention part of a decoder layer at one token as one launch: q/k/v projections of weight * rmsnorm(x + delta)
// (x + delta to x_sum), rope + cache append + attention per head, output projection into y.  q_out, k_out, v_out and
// att_out are scratch rows the parts hand over through.  Needs the workspace head (zero between launches).
struct AttentionChain {
    const hqq_linear *q, *k, *v, *o;
    const f16 *x, *delta, *norm_weight;
    float eps;
    f16 *x_sum;
    f16 *q_out, *k_out, *v_out, *att_out;
    const f16 *cos_t, *sin_t;
    const int64_t *pos;
    f16 *cache_k, *cache_v;
    int64_t max_len;
    int n_heads, n_kv_heads, head_dim;
    f16 *y;
};
size_t attention_chain_error_offset(); // of the chain's error word inside the workspace
int launch_attention_chain(const AttentionChain &c, void *ws, size_t ws_bytes, hipStream_t s);
int launch_zero_workspace_head(void *ws, size_t ws_bytes, hipStream_t s);
// the quantiser (quantize_kernels.hip)
size_t quantize_workspace_bytes();
int launch_quantize_groups(const void *w, int fp32_in, int64_t rows, int64_t cols, int nbits, int round_zero, int iters,
                           float lp, double beta, double kappa, uint8_t *codes, float *inv_scale, float *zero, void *ws,
                           size_t ws_bytes, hipStream_t s);
int launch_quantize_whole(const float *x, int64_t n, int nbits, uint8_t *codes, float *inv_scale, float *zero, void *ws,
                          size_t ws_bytes, hipStream_t s);
size_t workspace_head_bytes();
bool tile_supported(const hqq_linear *l, int64_t M);
size_t tile_workspace_bytes(const hqq_linear *l, int64_t M);
int launch_tile_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                       const SmallBatchEpilogue *ep = nullptr);
bool tile_epilogue_supported(const hqq_linear *l, int64_t M);
// A tile launch whose finishing pass (the sum over its K blocks, bias, routing weight, accumulation) is left to the
// caller, who runs the passes of several launches as one (launch_tile_finish_group).
struct TileFinish {
    const float *part; // null: the launch has written its output itself
    int KSP, M, N, F;
    const f16 *bias;
    f16 *y;
    const f16 *row_scale;
    int accumulate;
};
constexpr int kTileFinishGroupMax = 16;
size_t tile_partial_bytes(const hqq_linear *l, int64_t M);
int launch_tile_matmul_deferred(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                                const SmallBatchEpilogue *ep, void *part_at, TileFinish *finish);
int launch_tile_finish_group(const TileFinish *f, int n, hipStream_t s);
bool tile_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M);
size_t tile_gate_workspace_bytes(const hqq_linear *w1, const hqq_linear *w3, int64_t M);
int launch_tile_gate_up(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *h, void *ws,
                        size_t ws_bytes, hipStream_t s);
// MFMA with the de-quantised weights staged in LDS (2-, 3- and 4-bit codes): the kernel of wide batches
bool ldsgemm_supported(const hqq_linear *l, int64_t M);
size_t ldsgemm_workspace_bytes(const hqq_linear *l, int64_t M);
int launch_ldsgemm_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s,
                          const SmallBatchEpilogue *ep = nullptr);
bool vec3_supported(const hqq_linear *l, int64_t M);
size_t vec3_workspace_bytes(const hqq_linear *l, int64_t M);
int launch_vec3_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s);
// 3-bit expert FFN in two launches: the gate projections of n_experts experts (ab: layer l at ab + l * ab_lstride,
// w1 then w3 of each expert; two experts only from a record table), then the down projection reading silu(a) * b
bool vec3_ffn_supported(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, int64_t M, int n_experts);
size_t vec3_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, int64_t M, int n_experts);
int launch_vec3_down_pair(const hqq_linear *w2, const f16 *ab, int64_t ab_lstride, f16 *y, const f16 *row_scale,
                          int accumulate, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex &ix);
bool vec3_gate_supported(const hqq_linear *w1, const hqq_linear *w3, int64_t M);
size_t vec3_gate_workspace_bytes(const hqq_linear *w1, int64_t M);
int launch_vec3_gate(const hqq_linear *w1, const hqq_linear *w3, const f16 *x, int64_t M, f16 *ab, int64_t ab_lstride,
                     int n_experts, void *ws, size_t ws_bytes, hipStream_t s, const StripIndex *ix = nullptr);
int launch_vec3_down(const hqq_linear *w2, const f16 *a, const f16 *b, int64_t M, f16 *y, void *ws, size_t ws_bytes,
                     const SmallBatchEpilogue &ep, hipStream_t s, f16 *h, const StripIndex *ix = nullptr);
int launch_router_top2(const f16 *x, const f16 *w, int n_experts, int64_t hidden, int *sel, f16 *weights, f16 *logits,
                       hipStream_t s, int64_t rows = 1);
int launch_moe_group_pairs(const int *sel, const f16 *weights, int64_t tokens, int n_experts, int *counts,
                           long long *token_of_row, f16 *scale_of_row, hipStream_t s);
int launch_add_rmsnorm(f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *y, int64_t hidden, hipStream_t s,
                       int64_t rows = 1);
int launch_rope_append_rows(f16 *q, const f16 *k, const f16 *v, const f16 *cos_t, const f16 *sin_t, int64_t start,
                            int64_t rows, f16 *cache_k, f16 *cache_v, int64_t max_len, int n_heads, int n_kv_heads,
                            int head_dim, hipStream_t s);
int launch_add_rmsnorm_router(f16 *x, const f16 *delta, const f16 *weight, float eps, f16 *y, int64_t hidden,
                              const f16 *gate_w, int n_experts, int *sel, f16 *weights, f16 *logits, hipStream_t s);
int launch_attention_decode(const f16 *q, const f16 *k, const f16 *v, const f16 *cos_t, const f16 *sin_t, const int64_t *pos,
                            f16 *cache_k, f16 *cache_v, int64_t max_len, int n_heads, int n_kv_heads, int head_dim, f16 *out,
                            hipStream_t s, void *ws = nullptr, size_t ws_bytes = 0);
int attention_parts(int64_t max_len); // blocks per head of the attention launch
size_t attention_workspace_bytes(int64_t max_len, int n_heads, int head_dim);
// dequant_gemm.hip: wide batches as hqq_dequantize into the workspace + one library GEMM
bool dqgemm_supported(const hqq_linear *l, int64_t M);
bool dqgemm_preferred(const hqq_linear *l, int64_t M);
size_t dqgemm_workspace_bytes(const hqq_linear *l, int64_t M);
int launch_dqgemm_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, hipStream_t s);
int launch_silu_mul(const f16 *a, const f16 *b, f16 *h, int64_t count, hipStream_t s);
int launch_scale_store(const f16 *src, f16 *dst, const f16 *row_scale, int accumulate, int64_t M, int64_t N,
                       hipStream_t s);

} // namespace hqq
