/*
 * hqq_mi355x -- C ABI of the MI355X (gfx950) HQQ quantized-linear library.
 *
 * Every entry point takes plain device pointers, sizes and a hipStream_t passed
 * as void*; nothing here depends on PyTorch.  All pointers are borrowed, the
 * caller allocates every output and workspace, no entry point synchronises the
 * stream or the device, and none of them calls hipMalloc / hipFree.
 *
 * Return value: 0 = success, negative = argument error (HQQ_E_*), positive =
 * the hipError_t of the failed runtime call.  hqq_error_string() explains both.
 *
 * "Reference" citations are into dvmazur/mixtral-offloading (src/...): each
 * entry point names the Python function of the reference that it replaces.
 */
#ifndef HQQ_MI355X_H
#define HQQ_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HQQ_ABI_VERSION 1

enum {
    HQQ_OK = 0,
    HQQ_E_NULL = -1,      /* a required pointer is NULL                       */
    HQQ_E_NBITS = -2,     /* nbits not in {2,3,4}                             */
    HQQ_E_SHAPE = -3,     /* sizes disagree (the reference's asserts)         */
    HQQ_E_ALIGN = -4,     /* pointer or row pitch not aligned as documented   */
    HQQ_E_WORKSPACE = -5, /* workspace too small (see hqq_workspace_bytes)    */
    HQQ_E_UNSUPPORTED = -6,
    HQQ_E_CACHE = -7      /* expert-cache policy error (see hqq_lru_*)        */
};

/* How a (G, K) scale or zero table is stored.
 *   HQQ_TABLE_F16 : fp16 values, G*K of them                                  (meta['scale'] / meta['zero'])
 *   HQQ_TABLE_U8  : uint8 values, G*K of them, with fp16 meta scale / zero of `meta_cols` entries; entry i of the table
 *                   de-quantises as fp16(fp16(q[i] - mz[i % meta_cols]) * ms[i % meta_cols]).  meta_cols == 1 is the
 *                   whole-tensor (scalar) case.                               (meta['scale_q'] + meta['meta_scale'])
 * Reference: src/custom_layers.py:62-66 expands HQQ_TABLE_U8 to fp16 on every forward.                               */
enum { HQQ_TABLE_F16 = 0, HQQ_TABLE_U8 = 1 };

typedef struct hqq_table {
    const void *data;      /* fp16[G*K] or uint8[G*K]                          */
    const void *meta_scale; /* fp16[meta_cols] (HQQ_TABLE_U8 only)             */
    const void *meta_zero;  /* fp16[meta_cols] (HQQ_TABLE_U8 only)             */
    int64_t meta_cols;
    int32_t kind;
    int32_t reserved;
} hqq_table;

/* One HQQ-quantised linear layer in the kernel layout of the reference
 * (src/custom_layers.py:41-47 `repack`, consumed at :68-86):
 *   nbits 4: codes uint8 (N/2, K), byte = q[2p] << 4 | q[2p+1]                        (src/packing.py:10-17)
 *   nbits 2: codes uint8 (N/4, K), byte = q[4p]<<6 | q[4p+1]<<4 | q[4p+2]<<2 | q[4p+3] (src/packing.py:36-41)
 *   nbits 3: codes int32 (ceil(N/10), K), code i of a word at bit 3*(9-i)              (src/packing.py:62-81)
 * Weight (n, k) uses table row n % G, G = N / group_size (src/triton_kernels.py:86-88).
 * codes must be 16-byte aligned and K a multiple of 16 for the fast kernels; other shapes take a slower general kernel. */
typedef struct hqq_linear {
    int32_t nbits;
    int32_t group_size;
    int64_t N; /* out features */
    int64_t K; /* in features  */
    const void *codes;
    hqq_table scale;
    hqq_table zero;
    const void *bias; /* fp16[N] or NULL */
} hqq_linear;

int hqq_abi_version(void);
const char *hqq_error_string(int code);

/* ---- bit packers: replace Quantizer.pack / Quantizer.unpack entries '4bit_u8', '2bit_u8', '3bit_32'
 *      installed by src/packing.py:105-111 (functions at :10-27, :36-53, :62-97).
 * `rows` is the height of the UNPACKED array for pack_* and of the PACKED array for unpack_*; `cols` is the product of
 * the trailing dimensions.  Unpacked codes are uint8.  unpack_3bit always writes 10*rows rows (spare rows are zero).  */
int hqq_pack_4bit_u8(const uint8_t *q, int64_t rows, int64_t cols, uint8_t *out, void *stream);
int hqq_pack_2bit_u8(const uint8_t *q, int64_t rows, int64_t cols, uint8_t *out, void *stream);
int hqq_pack_3bit_i32(const uint8_t *q, int64_t rows, int64_t cols, int32_t *out, void *stream);
int hqq_unpack_4bit_u8(const uint8_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream);
int hqq_unpack_2bit_u8(const uint8_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream);
int hqq_unpack_3bit_i32(const int32_t *in, int64_t rows, int64_t cols, uint8_t *q, void *stream);

/* ---- 8-bit table -> fp16 table: replaces Quantizer.dequantize(meta['scale_q'], meta['meta_scale']) and the same for
 *      zero at src/custom_layers.py:63-66.  out is fp16[count].                                                      */
int hqq_table_to_f16(const hqq_table *t, int64_t count, void *out_f16, void *stream);

/* ---- full de-quantisation to fp16 (N, K): replaces HQQLinearTritonSavable.dequantize, src/custom_layers.py:95-116.
 *      Bit-exact: W = fp16(fp16(q - z) * s).                                                                         */
int hqq_dequantize(const hqq_linear *l, void *w_out_f16, void *stream);

/* ---- y = x @ dequant(W).T (+ bias): replaces triton_matmul4_transpose / triton_matmul2_transpose /
 *      triton_matmul3_transpose (src/triton_kernels.py:133-191, 321-380, 511-564) together with the meta expansion of
 *      forward_triton (src/custom_layers.py:55-92).  x is fp16 (M, K) contiguous, y is fp16 (M, N).  fp32 accumulation.
 *      `workspace` must hold hqq_matmul_workspace_bytes(l, M) bytes, 256-byte aligned.  It holds split-K partial sums
 *      and, in its first 576 KiB, per-tile arrival counters and per-output accumulation slots that must start at
 *      zero: call hqq_workspace_init once after allocating it (or zero-fill it); every call leaves that head at zero
 *      again, so one workspace serves any sequence of calls that are ordered on a stream.  Calls that overlap in
 *      time need separate workspaces.                                                                               */
size_t hqq_matmul_workspace_bytes(const hqq_linear *l, int64_t M);
/* zero the head (counters and slots) of a workspace with a small fill kernel (safe under stream capture)            */
int hqq_workspace_init(void *workspace, size_t workspace_bytes, void *stream);
/* same, with the kernel family forced (-1 = automatic choice, else 0..5 as hqq_matmul_kernel_family reports):
 * HQQ_E_UNSUPPORTED when that family does not take the configuration.  For tests and profiling.  (Family 5 forced
 * on a batch smaller than it is chosen from needs 576 KiB + 2 * N * K bytes of workspace.)                          */
int hqq_matmul_transpose_ex(const hqq_linear *l, const void *x_f16, int64_t M, void *y_f16, void *workspace,
                            size_t workspace_bytes, int family, void *stream);
int hqq_matmul_transpose(const hqq_linear *l, const void *x_f16, int64_t M, void *y_f16, void *workspace,
                         size_t workspace_bytes, void *stream);

/* ---- y = w2( silu(w1 x) * (w3 x) ): replaces MixtralBLockSparseTop2MLP_HQQ.forward, src/custom_layers.py:253-256.
 *      x fp16 (M, hidden), y fp16 (M, hidden).  When `row_scale_f16` is not NULL, row m of the result is multiplied by
 *      row_scale_f16[m] (the routing weight, src/custom_layers.py:308) and when `accumulate` is non-zero the result is
 *      added to y in fp16 instead of stored (the index_add_ at :312 for a single row block).                          */
size_t hqq_expert_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, int64_t M);
int hqq_expert_ffn(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *x_f16, int64_t M,
                   void *y_f16, const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                   void *stream);

/* ---- the expert loop of SparseMoeWrapper.forward for several tokens (src/custom_layers.py:298-312: per expert a
 *      where / gather / expert / scale / index_add_) over rows the caller has already grouped by expert: rows
 *      row_start[g] .. row_start[g + 1] - 1 of x (fp16, hidden wide) go through expert g (w1[g], w2[g], w3[g]) and
 *      y[row] = row_scale_f16[row] * expert(x[row]) (row_scale_f16 may be NULL).  row_start is a HOST array of
 *      n_groups + 1 entries starting at 0; groups without rows may have NULL layers.  One call issues every group's
 *      launches in order on `stream` with one workspace of hqq_expert_groups_ffn_workspace_bytes(..) bytes (the
 *      largest group's need, then the partial sums of the down projections that split K: their finishing passes run
 *      as one launch at the end of the call; head zeroed as for hqq_matmul_transpose).  Results are
 *      hqq_expert_ffn's, bit for bit.                                                                              */
size_t hqq_expert_groups_ffn_workspace_bytes(const hqq_linear *const *w1, const hqq_linear *const *w2,
                                             const hqq_linear *const *w3, int32_t n_groups, const int64_t *row_start);
int hqq_expert_groups_ffn(const hqq_linear *const *w1, const hqq_linear *const *w2, const hqq_linear *const *w3,
                          int32_t n_groups, const int64_t *row_start, const void *x_f16, void *y_f16,
                          const void *row_scale_f16, void *workspace, size_t workspace_bytes, void *stream);

/* ---- hqq_expert_ffn for callers that cannot allocate or carry a workspace (code under HIP graph capture, tight
 *      serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The workspace is an
 *      array of HQQ_STATIC_SCRATCH_BYTES built into the library's device code (every GPU the library runs on holds it
 *      until the process ends); the call allocates nothing and returns HQQ_E_WORKSPACE when
 *      hqq_expert_ffn_workspace_bytes(w1, w2, w3, M) exceeds that size (Mixtral-8x7B experts: batches up to 4 rows at
 *      any code width, up to 16 rows for 2-bit codes).  Results are hqq_expert_ffn's, bit for bit.  All calls on one
 *      GPU share the array: calls that overlap in time on one GPU race (order them on one stream, or with events).
 *      The first call on a GPU records one extra small fill kernel on `stream`.                                    */
#define HQQ_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
int hqq_expert_ffn_static(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *x_f16, int64_t M,
                          void *y_f16, const void *row_scale_f16, int accumulate, void *stream);

/* ---- h = silu(w1 x) * (w3 x), fp16 (M, ffn): the first half of the expert FFN (src/custom_layers.py:254), both
 *      projections rounded to fp16 as the reference's two layers round them, SiLU in fp32 rounded once, the product in
 *      fp16.  One fused pass over both weight matrices where a kernel family has one for the batch (2- and 4-bit
 *      layers of one kind), else both projections followed by an elementwise pass.  Layers without bias.
 *      Workspace: hqq_gate_up_workspace_bytes(w1, w3, M), 256-byte aligned, head zeroed as for hqq_matmul_transpose.  */
size_t hqq_gate_up_workspace_bytes(const hqq_linear *w1, const hqq_linear *w3, int64_t M);
int hqq_gate_up(const hqq_linear *w1, const hqq_linear *w3, const void *x_f16, int64_t M, void *h_f16, void *workspace,
                size_t workspace_bytes, void *stream);

/* ---- expert FFN whose expert is chosen on the device: the same computation as hqq_expert_ffn, but the weights come
 *      from record expert_index[0] of a device-resident table, so that the router's choice (src/custom_layers.py:
 *      276-296: topk, then a host-side list of active experts) needs no host synchronisation when every expert of
 *      the layer is resident.  The table holds 3 records per expert in the order w1, w3, w2, each
 *      hqq_expert_record_bytes() long and written by hqq_expert_record_fill into HOST memory (the caller copies the
 *      table to the device once).  w1 / w2 / w3 describe the common shape of all experts (any one expert's
 *      descriptors).  Batches of at most 4 rows (2- and 4-bit experts) or 16 rows (3-bit experts, K a multiple of
 *      256 and at least ten groups down N).  Workspace as for hqq_expert_ffn.  expert_index[0] is read on the
 *      device and not checked: it must name an expert of the table.                                                 */
size_t hqq_expert_record_bytes(void);
int hqq_expert_record_fill(const hqq_linear *l, void *host_record);
int hqq_expert_ffn_indexed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *device_table,
                           const int32_t *expert_index, const void *x_f16, int64_t M, void *y_f16,
                           const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                           void *stream);

/* ---- both experts of one token in two launches instead of four: y (+)= sum over e < 2 of
 *      fp16(FFN_{expert_index[e]}(x)) * row_scale[e], the loop body of src/custom_layers.py:298-312 for the two
 *      active experts of a single token (what two hqq_expert_ffn_indexed calls give, the second accumulating, up to
 *      the order in which the fp32 partial sums over K are added and, where K of the down projection is split over
 *      blocks, up to one fp16 rounding: the weighted sum of both experts is then formed in higher precision and
 *      rounded once, where index_add_ on fp16 tensors rounds each product and the sum).  One launch
 *      computes silu(w1 x) * w3 x of both experts, one both down projections and their weighted sum (3-bit experts:
 *      the four gate projections, then both down projections, which apply silu(a) * b as they read them).  x is one row
 *      (hidden fp16), expert_index two device int32, row_scale two device fp16.  Table as for
 *      hqq_expert_ffn_indexed.  HQQ_E_UNSUPPORTED when the shapes do not fit the decode kernel (the workspace query
 *      then returns 0): call hqq_expert_ffn_indexed twice instead.                                                 */
size_t hqq_expert_pair_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3);
int hqq_expert_pair_ffn_indexed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3,
                                const void *device_table, const int32_t *expert_index, const void *x_f16, void *y_f16,
                                const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                                void *stream);

/* ---- the whole MoE block of one token in two launches: hqq_add_rmsnorm_router followed by
 *      hqq_expert_pair_ffn_indexed, with the norm and the router run by every block of the first launch in front of
 *      the gates (src/custom_layers.py:276-312 after the decoder layer's post-attention norm).  x + delta is written to
 *      x_sum (a buffer other than x), the router's choice to sel_out[2] and weights_f16_out[2] (device memory),
 *      y (+)= the weighted sum of the two experts' outputs.  hidden <= 4096, n_experts <= 8, 2- or 4-bit experts
 *      (HQQ_E_UNSUPPORTED otherwise: make the two calls); workspace as hqq_expert_pair_ffn_workspace_bytes.  Results
 *      are those of the two calls it replaces, bit for bit.                                                         */
int hqq_moe_pair_routed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *device_table,
                        const void *x_f16, const void *delta_f16, const void *norm_weight_f16, float eps, void *x_sum_f16,
                        const void *gate_w_f16, int32_t n_experts, int32_t *sel_out, void *weights_f16_out, void *y_f16,
                        int accumulate, void *workspace, size_t workspace_bytes, void *stream);

/* ---- up to four HQQLinearTritonSavable.forward_triton calls (src/custom_layers.py:100-118) on the same single row
 *      in one launch: ys[i] = x @ dequant(layers[i]).T (+ bias).  The layers share K, code width, group size and
 *      table kinds but not N -- the q, k and v projections of an attention block.  Results are those of
 *      hqq_matmul_transpose on each layer up to the order in which the fp32 partial sums over K are added.  HQQ_E_UNSUPPORTED (workspace query 0) when the layers do not fit: call
 *      hqq_matmul_transpose per layer instead.                                                                      */
size_t hqq_matmul_group_workspace_bytes(const hqq_linear *const *layers, int32_t count);
int hqq_matmul_group(const hqq_linear *const *layers, int32_t count, const void *x_f16, void *const *ys_f16,
                     void *workspace, size_t workspace_bytes, void *stream);

/* ---- hqq_add_rmsnorm folded into hqq_matmul_group: ys[i] = (norm_weight * rmsnorm(x + delta)) @ dequant(layers[i]).T,
 *      and x + delta is written to x_sum (a buffer other than x: every block reads x while one writes x_sum).  The
 *      input norm of a decoder layer and its q / k / v projections in one launch; delta may be NULL.  Results are
 *      those of hqq_add_rmsnorm followed by hqq_matmul_group, bit for bit.  All pointers 16-byte aligned.          */
int hqq_matmul_group_norm(const hqq_linear *const *layers, int32_t count, const void *x_f16, const void *delta_f16,
                          const void *norm_weight_f16, float eps, void *x_sum_f16, void *const *ys_f16, void *workspace,
                          size_t workspace_bytes, void *stream);

/* ---- router of one token: logits = fp16(x W^T), fp32 softmax, the two largest probabilities renormalised and cast
 *      to fp16 (src/custom_layers.py:276-282), written to device memory: sel_out[2] expert indices (largest
 *      first), weights_f16_out[2]; logits_f16_out[n_experts] when not NULL.  n_experts <= 16.                       */
int hqq_router_top2(const void *x_f16, const void *gate_w_f16, int32_t n_experts, int64_t hidden, int32_t *sel_out,
                    void *weights_f16_out, void *logits_f16_out, void *stream);

/* ---- residual add and RMSNorm of one token (the reference takes both from HF transformers' Mixtral decoder layer):
 *      x += delta in fp16 when delta is not NULL (x is written back), y = weight * fp16(x * rsqrt(mean(x^2) + eps)). */
int hqq_add_rmsnorm(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16, int64_t hidden,
                    void *stream);

/* ---- the same three for the `rows` tokens of a prompt pass (the reference runs HF transformers' Mixtral layer over
 *      the whole prompt, src/custom_layers.py:270-282 its router): row r of x / delta / y is r * hidden elements
 *      further, sel_out is [rows][2], weights_f16_out [rows][2], logits_f16_out [rows][n_experts] (or NULL).  Row by
 *      row the results are those of the one-token calls.                                                           */
int hqq_add_rmsnorm_rows(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16, int64_t rows,
                         int64_t hidden, void *stream);
int hqq_router_top2_rows(const void *x_f16, const void *gate_w_f16, int32_t n_experts, int64_t rows, int64_t hidden,
                         int32_t *sel_out, void *weights_f16_out, void *logits_f16_out, void *stream);

/* ---- the (token, slot) pairs of a prompt pass grouped by expert on the device (the reference builds an expert mask
 *      and runs torch.where per expert, src/custom_layers.py:288-301): sel [tokens][2] and weights_f16 [tokens][2] as
 *      hqq_router_top2_rows writes them.  Pair p = 2 * token + slot goes to the rows of expert sel[p], pairs of one
 *      expert in the order of p.  Out: counts_out[e] rows of expert e (the only figure the host needs before it
 *      launches the experts), and for row r of the grouped order token_of_row_out[r] (the token it came from) and
 *      scale_of_row_f16_out[r] (its routing weight).                                                                 */
int hqq_moe_group_pairs(const int32_t *sel, const void *weights_f16, int64_t tokens, int32_t n_experts, int32_t *counts_out,
                        int64_t *token_of_row_out, void *scale_of_row_f16_out, void *stream);

/* ---- rotary embedding and KV-cache append of `rows` new tokens at positions start .. start + rows - 1 (HF
 *      transformers' apply_rotary_pos_emb in the reference's Mixtral attention): q (rows, n_heads*head_dim) is rotated
 *      in place, the rotated k (rows, n_kv_heads*head_dim) and v are written to cache_k / cache_v
 *      [n_kv_heads][max_len][head_dim].  cos / sin are tables [positions][head_dim] at least start + rows long;
 *      start + rows <= max_len, head_dim even and <= 256.  Arithmetic as in hqq_attention_decode.                  */
int hqq_rope_append_rows(void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                         int64_t start, int64_t rows, void *cache_k_f16, void *cache_v_f16, int64_t max_len,
                         int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, void *stream);

/* ---- hqq_add_rmsnorm followed by hqq_router_top2 on its output y, in one launch: the post-attention norm of a
 *      decoder layer and the router that reads it (src/custom_layers.py:276-282).  x and y as hqq_add_rmsnorm gives
 *      them; logits as hqq_router_top2 up to the order of the fp32 sums.                                           */
int hqq_add_rmsnorm_router(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16,
                           int64_t hidden, const void *gate_w_f16, int32_t n_experts, int32_t *sel_out,
                           void *weights_f16_out, void *logits_f16_out, void *stream);

/* ---- rotary embedding, KV-cache append and attention of one new token (HF transformers' Mixtral attention in the
 *      reference): q (n_heads*head_dim), k and v (n_kv_heads*head_dim) are the un-rotated projections of the token;
 *      cos / sin are tables [positions][head_dim]; pos[0] (device memory) is the token's position; the rotated key
 *      and the value are written to cache_k / cache_v [n_kv_heads][max_len][head_dim] at pos and positions 0..pos
 *      are attended.  out is (n_heads*head_dim).  head_dim 64 or 128; the caller keeps pos < max_len <= 16000 and
 *      cos / sin at least max_len rows long (pos is read on the device and bounded by max_len only).               */
int hqq_attention_decode(const void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                         const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len, int32_t n_heads,
                         int32_t n_kv_heads, int32_t head_dim, void *out_f16, void *stream);

/* ---- the same with a workspace (256-byte aligned, zero-filled once, at least hqq_attention_decode_workspace_bytes()):
 *      for caches longer than 1024 positions the positions of a head are then split over up to 8 blocks (one per
 *      thousand positions attended so far), each leaving its share's maximum, sum and un-normalised output in the
 *      workspace, and the block that finishes last adds them up.  Probabilities stay fp32 in this form,
 *      so its results agree with hqq_attention_decode's within fp16 rounding, not bit for bit.  The workspace query
 *      returns 0 for caches the one-block kernel keeps (then both entry points are the same).                       */
size_t hqq_attention_decode_workspace_bytes(int64_t max_len, int32_t n_heads, int32_t head_dim);
int hqq_attention_decode_ws(const void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                            const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len, int32_t n_heads,
                            int32_t n_kv_heads, int32_t head_dim, void *out_f16, void *workspace, size_t workspace_bytes,
                            void *stream);

/* ---- the attention part of a decoder layer at one token as ONE launch: hqq_matmul_group_norm (input norm + q, k, v
 *      of x + delta, x + delta to x_sum), hqq_attention_decode and hqq_matmul_transpose (o_proj) into y, with the same
 *      bits as those three calls.  The parts run as blocks of one grid in that order and hand over through the scratch
 *      rows q/k/v/att (n_heads*head_dim, n_kv_heads*head_dim twice, n_heads*head_dim halves) and counters in the
 *      workspace head (hqq_workspace_init once; at least hqq_attention_chain_workspace_bytes()): the output projection
 *      has fetched its weights by the time the heads are done.  (HF transformers' Mixtral attention in the reference;
 *      the projections are src/custom_layers.py:55-92.)  HQQ_E_UNSUPPORTED for shapes outside it (then make the three
 *      calls): 4-bit projections without bias whose K fits one block (K <= 4096), head_dim 128, max_len <= 1024 (the
 *      caches the one-block attention kernel keeps).
 *      A wait that does not end (it cannot, by the order of the blocks) gives up after about a quarter of a second and
 *      sets the int at hqq_attention_chain_error_offset() bytes into the workspace, which is otherwise zero.          */
size_t hqq_attention_chain_workspace_bytes(void);
size_t hqq_attention_chain_error_offset(void);
int hqq_attention_chain(const hqq_linear *q, const hqq_linear *k, const hqq_linear *v, const hqq_linear *o, const void *x_f16,
                        const void *delta_f16, const void *norm_weight_f16, float eps, void *x_sum_f16, void *q_scratch_f16,
                        void *k_scratch_f16, void *v_scratch_f16, void *att_scratch_f16, const void *cos_f16,
                        const void *sin_f16, const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len,
                        int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, void *y_f16, void *workspace,
                        size_t workspace_bytes, void *stream);

/* ---- the quantiser: hqq's Quantizer.quantize as the reference calls it (src/custom_layers.py:35-39 through
 *      HQQLinear.quantize, src/build_model.py:108-120), for the grouping of this path: the tensor read as a row-major
 *      (rows, cols) matrix whose columns are the groups (axis 0; rows = group size 8, 16, 32, 64 or 128).  w is fp16
 *      (w_is_fp32 = 0) or fp32.  scale = min((2^nbits - 1) / (max - min), 2e4), zero = -min * scale (rounded when
 *      round_zero), refined by `iters` iterations at most of hqq's half-quadratic solver when iters > 0 (lp_norm 0.7,
 *      beta 10, kappa 1.01, 20 iterations are hqq's defaults; beta and kappa are doubles, as in the reference's host
 *      loop, so that beta takes the same sequence of values; the solver stops for the whole tensor when the mean
 *      absolute error no longer falls), then q = clamp(round(w * scale + zero), 0, 2^nbits - 1).  Outputs: codes
 *      uint8 (rows, cols), unpacked; inv_scale fp32 (cols) = 1 / scale; zero fp32 (cols).  The workspace (8-byte
 *      aligned, hqq_quantize_workspace_bytes()) is only needed when iters > 0.  hqq_quantize_whole is the one-group
 *      form (channel_wise = False, the zero table's 8-bit meta): min and max over all n fp32 values; it always needs
 *      the workspace.                                                                                              */
size_t hqq_quantize_workspace_bytes(void);
int hqq_quantize_groups(const void *w, int32_t w_is_fp32, int64_t rows, int64_t cols, int32_t nbits, int32_t round_zero,
                        int32_t iters, float lp_norm, double beta, double kappa, void *codes_u8, void *inv_scale_f32,
                        void *zero_f32, void *workspace, size_t workspace_bytes, void *stream);
int hqq_quantize_whole(const void *x_f32, int64_t n, int32_t nbits, void *codes_u8, void *inv_scale_f32, void *zero_f32,
                       void *workspace, size_t workspace_bytes, void *stream);

/* ---- which kernel family a call would use (for tests and profiles): 0 general, 1 MFMA small-batch, 2 MFMA tile,
 *      3 three-bit decode kernel (one to eight rows in a pass over the words), 4 MFMA kernel with weights dequantised
 *      into shared memory (reads 3-bit words as they are stored), 5 batches of hundreds of rows: hqq_dequantize into the workspace, then one fp16 GEMM of the
 *      vendor's library (rocBLAS) with fp32 accumulation, which is the reference's PyTorch path
 *      (src/custom_layers.py:95-116 and torch.matmul); hqq_matmul_workspace_bytes grows by 2 * N * K bytes there.
 *      The first such call on a device creates the library's handle (it allocates: not under stream capture).      */
int hqq_matmul_kernel_family(const hqq_linear *l, int64_t M);

/* ---- expert offload: replaces the two copies of ExpertCache._swap (src/expert_cache.py:186-189).
 *      Enqueues one asynchronous host-to-device copy of a whole expert slab from pinned host memory on `copy_stream`,
 *      records `done_event` (a hipEvent_t) after it when not NULL.  The reference's device-to-host copy of the evicted
 *      expert is not needed: weights are immutable and every expert keeps its pinned host copy.                       */
int hqq_slab_h2d_async(void *dst_device, const void *src_pinned, size_t bytes, void *copy_stream, void *done_event);
/* make `stream` wait for `event` without blocking the host */
int hqq_stream_wait_event(void *stream, void *event);

/* ---- LRU policy of one eviction group (host only, no GPU calls): replaces EvictionGroupInfo and the bookkeeping of
 *      ExpertCache.load_experts / _swap (src/expert_cache.py:20-52, 120-201).  Experts are integers 0..n_experts-1;
 *      `slots` device slots exist.                                                                                    */
typedef struct hqq_lru hqq_lru;
hqq_lru *hqq_lru_create(int32_t n_experts, int32_t slots);
void hqq_lru_destroy(hqq_lru *c);
/* place expert `e` into a free device slot at load time (src/expert_cache.py:102-110); returns the slot or HQQ_E_CACHE */
int hqq_lru_add_resident(hqq_lru *c, int32_t e);
/* Plan one load_experts(..., unordered=True) call for `n` distinct experts: marks every one used, then decides the
 * evictions.  Outputs, each of length n, in the order the experts must be run (resident first, then misses in request
 * order): order[i] = expert, slot[i] = device slot it will occupy, victim[i] = expert evicted to make room or -1 for a
 * hit.  Returns 0 or HQQ_E_CACHE (unknown expert, duplicates, more misses than slots).                               */
int hqq_lru_plan(hqq_lru *c, const int32_t *experts, int32_t n, int32_t *order, int32_t *slot, int32_t *victim);
/* Plan a speculative load (no counterpart in the reference, whose README.md:24-26 lists speculative loading as not
 * yet available): of the `n` distinct guessed experts, those that are resident are left alone (their place in the
 * eviction order does not change); each of the others takes the place of the least recently used resident that is
 * not one of the `n_keep` experts in `keep` (the experts a guess must not evict), or is dropped when there is none.
 * Hits and misses are not counted.  Outputs for the *count experts that are to be loaded, in request order: order[i]
 * = expert, slot[i] = device slot, victim[i] = the expert evicted.  Returns 0 or HQQ_E_CACHE / HQQ_E_NULL.          */
int hqq_lru_plan_guess(hqq_lru *c, const int32_t *experts, int32_t n, const int32_t *keep, int32_t n_keep,
                       int32_t *order, int32_t *slot, int32_t *victim, int32_t *count);
int64_t hqq_lru_hits(const hqq_lru *c);
int64_t hqq_lru_misses(const hqq_lru *c);
/* device slot of expert e, or -1 when it is not resident */
int hqq_lru_slot_of(const hqq_lru *c, int32_t e);

#ifdef __cplusplus
}
#endif
#endif /* HQQ_MI355X_H */
