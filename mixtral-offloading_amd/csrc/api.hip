// C ABI: argument checks (the reference's asserts become error codes),
// kernel-family dispatch and workspace carving.
#include "hqq_common.hpp"

#include <mutex>

namespace hqq {

static int validate_table(const hqq_table &t)
{
    if (!t.data)
        return HQQ_E_NULL;
    if (t.kind == HQQ_TABLE_F16)
        return HQQ_OK;
    if (t.kind != HQQ_TABLE_U8)
        return HQQ_E_SHAPE;
    if (!t.meta_scale || !t.meta_zero)
        return HQQ_E_NULL;
    if (t.meta_cols < 1)
        return HQQ_E_SHAPE;
    return HQQ_OK;
}

int validate_linear(const hqq_linear *l)
{
    if (!l || !l->codes)
        return HQQ_E_NULL;
    if (l->nbits != 2 && l->nbits != 3 && l->nbits != 4) // reference src/custom_layers.py:24
        return HQQ_E_NBITS;
    if (l->N <= 0 || l->K <= 0 || l->group_size <= 0)
        return HQQ_E_SHAPE;
    if (l->N % l->group_size != 0) // table row n % G needs G = N / group_size to be whole
        return HQQ_E_SHAPE;
    if ((l->nbits == 4 && l->N % 2) || (l->nbits == 2 && l->N % 4))
        return HQQ_E_SHAPE;
    int rc = validate_table(l->scale);
    if (rc != HQQ_OK)
        return rc;
    return validate_table(l->zero);
}

static inline size_t align256(size_t v) { return (v + 255u) & ~(size_t)255u; }

enum { FAM_GENERAL = 0, FAM_SMALLBATCH = 1, FAM_TILE = 2, FAM_VEC3 = 3, FAM_LDS = 4, FAM_DQGEMM = 5 };
constexpr int64_t kSmallBatchMax = 16;

// a batch wider than the small-batch kernels take, run as slices of 16 rows (the weights of the later slices come
// from L2 / Infinity Cache); used where the tile kernel does not take the shape
static bool sliced_supported(const hqq_linear *l, int64_t M) { return M > kSmallBatchMax && smallbatch_supported(l, kSmallBatchMax); }

static int pick_family(const hqq_linear *l, int64_t M)
{
    if (dqgemm_preferred(l, M)) // hundreds of rows: de-quantise once, then a library GEMM
        return FAM_DQGEMM;
    if (strip_supported(l, M)) // decode batches: part of the small-batch family
        return FAM_SMALLBATCH;
    if (l->nbits == 3 && M <= 8 && vec3_supported(l, M)) // up to eight rows in one pass over the 3-bit words
        return FAM_VEC3;
    if (l->nbits == 3 && M >= 5 && M <= kSmallBatchMax && ldsgemm_supported(l, M)) // 3-bit words read as they are stored
        return FAM_LDS;
    if (l->nbits == 3 && tile_supported(l, M)) // wider batches: 3-bit codes rewritten as 4-bit ones, then the tile kernel
        return FAM_TILE;
    if (vec3_supported(l, M))
        return FAM_VEC3;
    if (tile_supported(l, M)) // five rows and more: weights rebuilt once per batch tile on the matrix cores
        return FAM_TILE;
    if (smallbatch_supported(l, M))
        return FAM_SMALLBATCH;
    if (sliced_supported(l, M))
        return FAM_SMALLBATCH;
    if (M >= 5 && ldsgemm_supported(l, M)) // e.g. 3-bit layers whose group count the tile kernel does not take
        return FAM_LDS;
    return FAM_GENERAL;
}

static size_t family_workspace(const hqq_linear *l, int64_t M, int fam)
{
    if (fam == FAM_SMALLBATCH)
        return smallbatch_workspace_bytes(l, M > kSmallBatchMax ? kSmallBatchMax : M);
    if (fam == FAM_VEC3)
        return vec3_workspace_bytes(l, M);
    if (fam == FAM_TILE)
        return tile_workspace_bytes(l, M);
    if (fam == FAM_LDS)
        return ldsgemm_workspace_bytes(l, M);
    if (fam == FAM_DQGEMM)
        return dqgemm_workspace_bytes(l, M);
    return 0;
}

static int run_matmul(const hqq_linear *l, const f16 *x, int64_t M, f16 *y, void *ws, size_t ws_bytes, int fam,
                      hipStream_t s)
{
    if (M == 0)
        return HQQ_OK;
    switch (fam) {
    case FAM_SMALLBATCH:
        if (M > kSmallBatchMax) {
            for (int64_t m0 = 0; m0 < M; m0 += kSmallBatchMax) {
                const int64_t mb = M - m0 < kSmallBatchMax ? M - m0 : kSmallBatchMax;
                int rc = launch_smallbatch_matmul(l, x + m0 * l->K, mb, y + m0 * l->N, ws, ws_bytes, SmallBatchEpilogue{}, s);
                if (rc != HQQ_OK)
                    return rc;
            }
            return HQQ_OK;
        }
        return launch_smallbatch_matmul(l, x, M, y, ws, ws_bytes, SmallBatchEpilogue{}, s);
    case FAM_VEC3:
        return launch_vec3_matmul(l, x, M, y, ws, ws_bytes, s);
    case FAM_TILE:
        return launch_tile_matmul(l, x, M, y, ws, ws_bytes, s);
    case FAM_LDS:
        return launch_ldsgemm_matmul(l, x, M, y, ws, ws_bytes, s);
    case FAM_DQGEMM:
        return launch_dqgemm_matmul(l, x, M, y, ws, ws_bytes, s);
    default:
        return launch_general_matmul(l, x, M, y, s);
    }
}

} // namespace hqq

using namespace hqq;

extern "C" {

int hqq_abi_version(void) { return HQQ_ABI_VERSION; }

const char *hqq_error_string(int code)
{
    switch (code) {
    case HQQ_OK: return "ok";
    case HQQ_E_NULL: return "a required pointer is NULL";
    case HQQ_E_NBITS: return "nbits must be 2, 3 or 4";
    case HQQ_E_SHAPE: return "sizes disagree";
    case HQQ_E_ALIGN: return "pointer or pitch is not aligned as documented";
    case HQQ_E_WORKSPACE: return "workspace is too small or misaligned";
    case HQQ_E_UNSUPPORTED: return "configuration not supported by the requested kernel family";
    case HQQ_E_CACHE: return "expert cache policy error";
    default: break;
    }
    if (code > 0)
        return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error";
}

int hqq_matmul_kernel_family(const hqq_linear *l, int64_t M)
{
    int rc = validate_linear(l);
    if (rc != HQQ_OK)
        return rc;
    return pick_family(l, M);
}

size_t hqq_matmul_workspace_bytes(const hqq_linear *l, int64_t M)
{
    if (validate_linear(l) != HQQ_OK || M <= 0)
        return 0;
    // large enough for whichever family is chosen or forced
    const int64_t Ms = M > kSmallBatchMax ? kSmallBatchMax : M;
    size_t a = smallbatch_supported(l, Ms) ? 2 * smallbatch_workspace_bytes(l, Ms) : 0;
    size_t b = vec3_supported(l, M) ? vec3_workspace_bytes(l, M) : 0;
    const size_t c = tile_supported(l, M) ? tile_workspace_bytes(l, M) : 0;
    if (c > b)
        b = c;
    const size_t d = ldsgemm_supported(l, M) ? ldsgemm_workspace_bytes(l, M) : 0;
    if (d > b)
        b = d;
    const size_t e = dqgemm_preferred(l, M) ? dqgemm_workspace_bytes(l, M) : 0; // (forced on fewer rows it needs 2 * N * K bytes)
    if (e > b)
        b = e;
    return align256(a > b ? a : b);
}

int hqq_workspace_init(void *workspace, size_t workspace_bytes, void *stream)
{
    if (!workspace)
        return HQQ_E_NULL;
    if (reinterpret_cast<uintptr_t>(workspace) & 255u)
        return HQQ_E_WORKSPACE;
    return launch_zero_workspace_head(workspace, workspace_bytes, (hipStream_t)stream);
}

int hqq_matmul_transpose_ex(const hqq_linear *l, const void *x_f16, int64_t M, void *y_f16, void *workspace,
                            size_t workspace_bytes, int family, void *stream)
{
    int rc = validate_linear(l);
    if (rc != HQQ_OK)
        return rc;
    if (M < 0)
        return HQQ_E_SHAPE;
    if (M == 0)
        return HQQ_OK;
    if (!x_f16 || !y_f16)
        return HQQ_E_NULL;
    int fam = family < 0 ? pick_family(l, M) : family;
    if (fam == FAM_SMALLBATCH && !smallbatch_supported(l, M) && !sliced_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (fam == FAM_VEC3 && !vec3_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (fam == FAM_TILE && !tile_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (fam == FAM_LDS && !ldsgemm_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (fam == FAM_DQGEMM && !dqgemm_supported(l, M))
        return HQQ_E_UNSUPPORTED;
    if (fam < 0 || fam > FAM_DQGEMM)
        return HQQ_E_UNSUPPORTED;
    const size_t need = family_workspace(l, M, fam);
    if (need > 0 && (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)))
        return HQQ_E_WORKSPACE;
    return run_matmul(l, (const f16 *)x_f16, M, (f16 *)y_f16, workspace, workspace_bytes, fam, (hipStream_t)stream);
}

int hqq_matmul_transpose(const hqq_linear *l, const void *x_f16, int64_t M, void *y_f16, void *workspace,
                         size_t workspace_bytes, void *stream)
{
    return hqq_matmul_transpose_ex(l, x_f16, M, y_f16, workspace, workspace_bytes, -1, stream);
}

// workspace of the FFN: [matmul scratch, counters first][h: M x ffn fp16][t: M x hidden fp16][a, b: M x ffn fp16
// each (unfused path only)]
static size_t ffn_matmul_scratch(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, int64_t M)
{
    size_t mm = hqq_matmul_workspace_bytes(w1, M); // already sized for the fused gate pass over two layers
    const size_t m2 = hqq_matmul_workspace_bytes(w2, M), m3 = hqq_matmul_workspace_bytes(w3, M);
    if (m2 > mm)
        mm = m2;
    if (m3 > mm)
        mm = m3;
    const size_t g = tile_gate_workspace_bytes(w1, w3, M);
    if (g > mm)
        mm = g;
    const size_t v = vec3_ffn_workspace_bytes(w1, w2, M, 1);
    if (v > mm)
        mm = v;
    return align256(mm);
}

size_t hqq_expert_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, int64_t M)
{
    if (validate_linear(w1) != HQQ_OK || validate_linear(w2) != HQQ_OK || validate_linear(w3) != HQQ_OK || M <= 0)
        return 0;
    return ffn_matmul_scratch(w1, w2, w3, M) + 3 * align256((size_t)M * w1->N * 2) + align256((size_t)M * w2->N * 2);
}

// workspace of the gate: [matmul scratch, counters first][a, b: M x N fp16 each (unfused paths only)]
static size_t gate_matmul_scratch(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    size_t mm = hqq_matmul_workspace_bytes(w1, M); // already sized for the fused decode pass over two layers
    const size_t m3 = hqq_matmul_workspace_bytes(w3, M), g = tile_gate_workspace_bytes(w1, w3, M);
    mm = m3 > mm ? m3 : mm;
    mm = g > mm ? g : mm;
    const size_t v = vec3_gate_workspace_bytes(w1, M);
    mm = v > mm ? v : mm;
    return align256(mm);
}

size_t hqq_gate_up_workspace_bytes(const hqq_linear *w1, const hqq_linear *w3, int64_t M)
{
    if (validate_linear(w1) != HQQ_OK || validate_linear(w3) != HQQ_OK || M <= 0 || w1->N != w3->N || w1->K != w3->K)
        return 0;
    return gate_matmul_scratch(w1, w3, M) + 2 * align256((size_t)M * w1->N * 2);
}

int hqq_gate_up(const hqq_linear *w1, const hqq_linear *w3, const void *x_f16, int64_t M, void *h_f16, void *workspace,
                size_t workspace_bytes, void *stream)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (M < 0 || w1->N != w3->N || w1->K != w3->K)
        return HQQ_E_SHAPE;
    if (M == 0)
        return HQQ_OK;
    if (!x_f16 || !h_f16)
        return HQQ_E_NULL;
    if (w1->bias || w3->bias)
        return HQQ_E_UNSUPPORTED; // the reference's experts have none (src/custom_layers.py:253-256)
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    const f16 *x = (const f16 *)x_f16;
    f16 *h = (f16 *)h_f16;
    const bool alike = w1->nbits == w3->nbits && w1->group_size == w3->group_size;
    // one fused launch where a kernel family has one for the batch; the decode kernels need no more workspace than
    // they check for themselves
    const bool wide = pick_family(w1, M) == FAM_DQGEMM || pick_family(w3, M) == FAM_DQGEMM; // two plain projections
    const bool prefer_tile = !wide && tile_supported(w1, M) && tile_supported(w3, M) && !strip_gate_supported(w1, w3, M) &&
                             pick_family(w1, M) != FAM_LDS && pick_family(w3, M) != FAM_LDS && pick_family(w1, M) != FAM_VEC3 &&
                             pick_family(w3, M) != FAM_VEC3;
    if (alike && !wide && !prefer_tile && smallbatch_supported(w1, M) && smallbatch_supported(w3, M))
        return launch_smallbatch_gate_up(w1, w3, x, M, h, workspace, workspace_bytes, s);
    if (prefer_tile && tile_gate_supported(w1, w3, M))
        return launch_tile_gate_up(w1, w3, x, M, h, workspace, workspace_bytes, s);
    // otherwise both projections (3-bit decode batches: in one launch), then silu(a) * b
    if (workspace_bytes < hqq_gate_up_workspace_bytes(w1, w3, M))
        return HQQ_E_WORKSPACE;
    char *p = static_cast<char *>(workspace);
    const size_t mm_bytes = gate_matmul_scratch(w1, w3, M), mid = align256((size_t)M * w1->N * 2);
    f16 *a = (f16 *)(p + mm_bytes), *b = (f16 *)(p + mm_bytes + mid);
    if (pick_family(w1, M) == FAM_VEC3 && pick_family(w3, M) == FAM_VEC3 && vec3_gate_supported(w1, w3, M)) {
        if ((rc = launch_vec3_gate(w1, w3, x, M, a, (int64_t)(mid / 2), 1, p, mm_bytes, s)) != HQQ_OK)
            return rc;
    } else {
        if ((rc = run_matmul(w1, x, M, a, p, mm_bytes, pick_family(w1, M), s)) != HQQ_OK)
            return rc;
        if ((rc = run_matmul(w3, x, M, b, p, mm_bytes, pick_family(w3, M), s)) != HQQ_OK)
            return rc;
    }
    return launch_silu_mul(a, b, h, M * w1->N, s);
}

// whether the down projection of an expert FFN at M rows is a tile launch whose finishing pass can be left to the caller
static bool down_finish_deferrable(const hqq_linear *w2, int64_t M)
{
    return M > kSmallBatchMax && pick_family(w2, M) == FAM_TILE && tile_epilogue_supported(w2, M) && tile_partial_bytes(w2, M) > 0;
}

// down_part / defer: see launch_tile_matmul_deferred; used when down_finish_deferrable(w2, M)
static int expert_ffn_impl(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *x_f16, int64_t M,
                           void *y_f16, const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                           void *stream, void *down_part, TileFinish *defer)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w2)) != HQQ_OK ||
        (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (M < 0 || w1->N != w3->N || w1->K != w3->K || w2->K != w1->N || w2->N != w1->K)
        return HQQ_E_SHAPE;
    if (M == 0)
        return HQQ_OK;
    if (!x_f16 || !y_f16)
        return HQQ_E_NULL;
    const size_t need = hqq_expert_ffn_workspace_bytes(w1, w2, w3, M);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *p = static_cast<char *>(workspace);
    const size_t mid = align256((size_t)M * w1->N * 2), outb = align256((size_t)M * w2->N * 2);
    const size_t mm_bytes = ffn_matmul_scratch(w1, w2, w3, M);
    void *mm = p; // first, so that hqq_workspace_init finds the counters at the head of the workspace
    f16 *h = (f16 *)(p + mm_bytes);
    f16 *t = (f16 *)(p + mm_bytes + mid);
    f16 *a = (f16 *)(p + mm_bytes + mid + outb);
    f16 *b = (f16 *)(p + mm_bytes + 2 * mid + outb);
    const f16 *x = (const f16 *)x_f16;
    f16 *y = (f16 *)y_f16;

    // 3-bit decode batches: both gate projections in one launch, silu(a) * b folded into the down projection's loads
    if (pick_family(w1, M) == FAM_VEC3 && pick_family(w2, M) == FAM_VEC3 && vec3_ffn_supported(w1, w2, w3, M, 1)) {
        if ((rc = launch_vec3_gate(w1, w3, x, M, a, (int64_t)(mid / 2), 1, mm, mm_bytes, s)) != HQQ_OK)
            return rc;
        SmallBatchEpilogue ep;
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        return launch_vec3_down(w2, a, b, M, y, mm, mm_bytes, ep, s, h);
    }
    // fused gate: decode batches always; wider ones only where the tile kernel does not take the shape
    const bool wide = pick_family(w1, M) == FAM_DQGEMM || pick_family(w3, M) == FAM_DQGEMM; // two plain projections
    const bool prefer_tile = !wide && tile_supported(w1, M) && tile_supported(w3, M) && !strip_gate_supported(w1, w3, M) &&
                             pick_family(w1, M) != FAM_LDS && pick_family(w3, M) != FAM_LDS && pick_family(w1, M) != FAM_VEC3 &&
                             pick_family(w3, M) != FAM_VEC3;
    const bool fast13 = !wide && !prefer_tile && smallbatch_supported(w1, M) && smallbatch_supported(w3, M) && !w1->bias &&
                        !w3->bias && w1->nbits == w3->nbits && w1->group_size == w3->group_size;
    if (fast13) {
        rc = launch_smallbatch_gate_up(w1, w3, x, M, h, mm, mm_bytes, s);
        if (rc != HQQ_OK)
            return rc;
    } else if (prefer_tile && tile_gate_supported(w1, w3, M)) {
        // both projections in one launch of the tile kernel, silu(a) * b in its finishing pass
        if ((rc = launch_tile_gate_up(w1, w3, x, M, h, mm, mm_bytes, s)) != HQQ_OK)
            return rc;
    } else {
        if ((rc = run_matmul(w1, x, M, a, mm, mm_bytes, pick_family(w1, M), s)) != HQQ_OK)
            return rc;
        if ((rc = run_matmul(w3, x, M, b, mm, mm_bytes, pick_family(w3, M), s)) != HQQ_OK)
            return rc;
        if ((rc = launch_silu_mul(a, b, h, M * w1->N, s)) != HQQ_OK)
            return rc;
    }
    if (M <= kSmallBatchMax && smallbatch_supported(w2, M) && pick_family(w2, M) == FAM_SMALLBATCH) {
        SmallBatchEpilogue ep;
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        return launch_smallbatch_matmul(w2, h, M, y, mm, mm_bytes, ep, s);
    }
    if (defer && down_finish_deferrable(w2, M)) {
        SmallBatchEpilogue ep;
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        return launch_tile_matmul_deferred(w2, h, M, y, mm, mm_bytes, s, &ep, down_part, defer);
    }
    if (!row_scale_f16 && !accumulate)
        return run_matmul(w2, h, M, y, mm, mm_bytes, pick_family(w2, M), s);
    if (pick_family(w2, M) == FAM_LDS) {
        SmallBatchEpilogue ep; // applied by the kernel's finishing pass over its partial sums
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        return launch_ldsgemm_matmul(w2, h, M, y, mm, mm_bytes, s, &ep);
    }
    if (pick_family(w2, M) == FAM_TILE && tile_epilogue_supported(w2, M)) {
        SmallBatchEpilogue ep; // the routing weight and the accumulation in the matmul's own epilogue
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        return launch_tile_matmul(w2, h, M, y, mm, mm_bytes, s, &ep);
    }
    if ((rc = run_matmul(w2, h, M, t, mm, mm_bytes, pick_family(w2, M), s)) != HQQ_OK)
        return rc;
    return launch_scale_store(t, y, (const f16 *)row_scale_f16, accumulate, M, w2->N, s);
}

int hqq_expert_ffn(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *x_f16, int64_t M,
                   void *y_f16, const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                   void *stream)
{
    return expert_ffn_impl(w1, w2, w3, x_f16, M, y_f16, row_scale_f16, accumulate, workspace, workspace_bytes, stream,
                           nullptr, nullptr);
}

// ---- the experts of one MoE layer over rows already grouped by expert: hqq_expert_ffn once per group, from one call
// Workspace of the grouped call: what the largest group needs, then the partial sums of every group whose down
// projection leaves its finishing pass to the end of the call.
static size_t groups_common_bytes(const hqq_linear *const *w1, const hqq_linear *const *w2, const hqq_linear *const *w3,
                                  int32_t n_groups, const int64_t *row_start, size_t *parts)
{
    size_t need = 0;
    *parts = 0;
    for (int g = 0; g < n_groups; ++g) {
        const int64_t M = row_start[g + 1] - row_start[g];
        if (M <= 0)
            continue;
        if (!w1[g] || !w2[g] || !w3[g])
            return 0;
        const size_t one = hqq_expert_ffn_workspace_bytes(w1[g], w2[g], w3[g], M);
        if (one == 0)
            return 0;
        need = one > need ? one : need;
        if (down_finish_deferrable(w2[g], M))
            *parts += tile_partial_bytes(w2[g], M);
    }
    return align256(need);
}

size_t hqq_expert_groups_ffn_workspace_bytes(const hqq_linear *const *w1, const hqq_linear *const *w2,
                                             const hqq_linear *const *w3, int32_t n_groups, const int64_t *row_start)
{
    if (!w1 || !w2 || !w3 || !row_start || n_groups <= 0)
        return 0;
    size_t parts = 0;
    const size_t common = groups_common_bytes(w1, w2, w3, n_groups, row_start, &parts);
    return common ? common + parts : 0;
}

int hqq_expert_groups_ffn(const hqq_linear *const *w1, const hqq_linear *const *w2, const hqq_linear *const *w3,
                          int32_t n_groups, const int64_t *row_start, const void *x_f16, void *y_f16,
                          const void *row_scale_f16, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!w1 || !w2 || !w3 || !row_start)
        return HQQ_E_NULL;
    if (n_groups < 0 || row_start[0] != 0)
        return HQQ_E_SHAPE;
    for (int g = 0; g < n_groups; ++g) {
        if (row_start[g + 1] < row_start[g])
            return HQQ_E_SHAPE;
        if (row_start[g + 1] > row_start[g] && (!w1[g] || !w2[g] || !w3[g]))
            return HQQ_E_NULL;
    }
    // The down projections that split K write their partial sums to a place of their own behind the common workspace,
    // and one launch at the end finishes them all (sum over the K blocks, routing weight, store): between the experts
    // no finishing launch waits for its projection to drain.
    size_t parts = 0;
    const size_t common = groups_common_bytes(w1, w2, w3, n_groups, row_start, &parts);
    const bool defer = workspace && common > 0 && parts > 0 && workspace_bytes >= common + parts;
    TileFinish fin[kTileFinishGroupMax];
    int nf = 0;
    char *part_at = static_cast<char *>(workspace) + common;
    for (int g = 0; g < n_groups; ++g) {
        const int64_t lo = row_start[g], M = row_start[g + 1] - lo;
        if (M == 0)
            continue;
        const char *x = static_cast<const char *>(x_f16) + (size_t)lo * (size_t)w1[g]->K * 2;
        char *y = static_cast<char *>(y_f16) + (size_t)lo * (size_t)w2[g]->N * 2;
        const char *rs = row_scale_f16 ? static_cast<const char *>(row_scale_f16) + (size_t)lo * 2 : nullptr;
        const bool later = defer && nf < kTileFinishGroupMax && down_finish_deferrable(w2[g], M);
        if (later)
            fin[nf] = TileFinish{};
        const int rc = expert_ffn_impl(w1[g], w2[g], w3[g], x_f16 ? x : nullptr, M, y_f16 ? y : nullptr, rs, 0, workspace,
                                       defer ? common : workspace_bytes, stream, later ? part_at : nullptr,
                                       later ? &fin[nf] : nullptr);
        if (rc != HQQ_OK)
            return rc;
        if (later && fin[nf].part) {
            part_at += tile_partial_bytes(w2[g], M);
            ++nf;
        }
    }
    return nf ? launch_tile_finish_group(fin, nf, (hipStream_t)stream) : HQQ_OK;
}

// ---- the expert FFN for callers that cannot allocate.  The workspace is a file-scope device array; each GPU holds
// its own copy at its own address, found once per device with hipGetSymbolAddress (the array's name is only a
// host-side handle, never a device address).
constexpr size_t kStaticScratchBytes = HQQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static void *scratch_ptr[kMaxDevices]; // per device, null until the first call there

// The device address of `scratch` on the current device.  Nothing is cleared here: a file-scope device array is
// zero when the module is loaded, and every launch leaves the head (counters, accumulation slots) at zero again.  (A
// fill recorded on the first caller's stream would not be ordered against a first call on another stream, and a
// captured one would be replayed with every graph launch.)
static int static_scratch(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices)
        return HQQ_E_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return static_cast<int>(e);
        if (!ptr || (reinterpret_cast<uintptr_t>(ptr) & 255u))
            return HQQ_E_ALIGN;
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return HQQ_OK;
}

int hqq_expert_ffn_static(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *x_f16, int64_t M,
                          void *y_f16, const void *row_scale_f16, int accumulate, void *stream)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w2)) != HQQ_OK ||
        (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (M < 0 || w1->N != w3->N || w1->K != w3->K || w2->K != w1->N || w2->N != w1->K)
        return HQQ_E_SHAPE;
    if (M == 0)
        return HQQ_OK;
    if (hqq_expert_ffn_workspace_bytes(w1, w2, w3, M) > kStaticScratchBytes)
        return HQQ_E_WORKSPACE; // beyond the built-in scratch: use hqq_expert_ffn with a workspace of the caller's
    void *ws = nullptr;
    if ((rc = static_scratch(&ws)) != HQQ_OK)
        return rc;
    return hqq_expert_ffn(w1, w2, w3, x_f16, M, y_f16, row_scale_f16, accumulate, ws, kStaticScratchBytes, stream);
}

size_t hqq_expert_record_bytes(void) { return strip_record_bytes(); }

int hqq_expert_record_fill(const hqq_linear *l, void *host_record)
{
    int rc = validate_linear(l);
    if (rc != HQQ_OK)
        return rc;
    if (!host_record)
        return HQQ_E_NULL;
    if (!strip_supported(l, 1) && !vec3_supported(l, 1))
        return HQQ_E_UNSUPPORTED;
    strip_fill_record(host_record, l);
    return HQQ_OK;
}

int hqq_expert_ffn_indexed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *device_table,
                           const int32_t *expert_index, const void *x_f16, int64_t M, void *y_f16,
                           const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w2)) != HQQ_OK ||
        (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (M < 0 || w1->N != w3->N || w1->K != w3->K || w2->K != w1->N || w2->N != w1->K)
        return HQQ_E_SHAPE;
    if (M == 0)
        return HQQ_OK;
    if (!x_f16 || !y_f16 || !device_table || !expert_index)
        return HQQ_E_NULL;
    const bool three = w1->nbits == 3 && vec3_ffn_supported(w1, w2, w3, M, 1);
    if (!three && (!strip_supported(w1, M) || !strip_supported(w3, M) || !strip_supported(w2, M)))
        return HQQ_E_UNSUPPORTED;
    const size_t need = hqq_expert_ffn_workspace_bytes(w1, w2, w3, M);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *p = static_cast<char *>(workspace);
    const size_t mm_bytes = ffn_matmul_scratch(w1, w2, w3, M);
    f16 *h = (f16 *)(p + mm_bytes);
    if (three) {
        const size_t mid = align256((size_t)M * w1->N * 2), outb = align256((size_t)M * w2->N * 2);
        f16 *a = (f16 *)(p + mm_bytes + mid + outb), *b = (f16 *)(p + mm_bytes + 2 * mid + outb);
        const StripIndex gate3 = {device_table, expert_index, 3, 0}, down3 = {device_table, expert_index, 3, 2};
        if ((rc = launch_vec3_gate(w1, w3, (const f16 *)x_f16, M, a, (int64_t)(mid / 2), 1, p, mm_bytes, s, &gate3)) != HQQ_OK)
            return rc;
        SmallBatchEpilogue ep3;
        ep3.row_scale = (const f16 *)row_scale_f16;
        ep3.accumulate = accumulate;
        return launch_vec3_down(w2, a, b, M, (f16 *)y_f16, p, mm_bytes, ep3, s, h, &down3);
    }
    const StripIndex gate = {device_table, expert_index, 3, 0}, down = {device_table, expert_index, 3, 2};
    if ((rc = launch_strip_gate_up(w1, w3, (const f16 *)x_f16, M, h, p, mm_bytes, s, &gate)) != HQQ_OK)
        return rc;
    SmallBatchEpilogue ep;
    ep.row_scale = (const f16 *)row_scale_f16;
    ep.accumulate = accumulate;
    return launch_strip_matmul(w2, h, M, (f16 *)y_f16, p, mm_bytes, ep, s, &down);
}

// workspace of the two-expert step: [strip scratch, counters first][h of expert 0][h of expert 1]
static size_t pair_scratch(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3)
{
    if (w1->nbits == 3)
        return vec3_ffn_supported(w1, w2, w3, 1, 2) ? align256(vec3_ffn_workspace_bytes(w1, w2, 1, 2)) : 0;
    const hqq_linear *gate[4] = {w1, w3, w1, w3}, *down[2] = {w2, w2};
    const size_t a = strip_job_workspace_bytes(gate, 4, 2, 1), b = strip_job_workspace_bytes(down, 2, 2, 1);
    if (a == 0 || b == 0)
        return 0;
    return align256(a > b ? a : b);
}

size_t hqq_expert_pair_ffn_workspace_bytes(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3)
{
    if (validate_linear(w1) != HQQ_OK || validate_linear(w2) != HQQ_OK || validate_linear(w3) != HQQ_OK)
        return 0;
    const size_t mm = pair_scratch(w1, w2, w3);
    // h of both experts; 3-bit layers keep the two gate projections of each apart (silu(a) * b is applied on load)
    return mm ? mm + (w1->nbits == 3 ? 4 : 2) * align256((size_t)w1->N * 2) : 0;
}

int hqq_expert_pair_ffn_indexed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3,
                                const void *device_table, const int32_t *expert_index, const void *x_f16, void *y_f16,
                                const void *row_scale_f16, int accumulate, void *workspace, size_t workspace_bytes,
                                void *stream)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w2)) != HQQ_OK ||
        (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (w1->N != w3->N || w1->K != w3->K || w2->K != w1->N || w2->N != w1->K)
        return HQQ_E_SHAPE;
    if (!x_f16 || !y_f16 || !device_table || !expert_index || !row_scale_f16)
        return HQQ_E_NULL;
    const size_t mm_bytes = pair_scratch(w1, w2, w3);
    if (mm_bytes == 0)
        return HQQ_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < hqq_expert_pair_ffn_workspace_bytes(w1, w2, w3) ||
        (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *p = static_cast<char *>(workspace);
    const size_t mid = align256((size_t)w1->N * 2);
    f16 *h0 = (f16 *)(p + mm_bytes), *h1 = (f16 *)(p + mm_bytes + mid);
    const StripIndex gate = {device_table, expert_index, 3, 0}, down = {device_table, expert_index, 3, 2};
    if (w1->nbits == 3) {
        // a0, b0, a1, b1 from one launch, then one down projection per expert, the second adding into y
        const int64_t ls = (int64_t)(mid / 2);
        if ((rc = launch_vec3_gate(w1, w3, (const f16 *)x_f16, 1, h0, ls, 2, p, mm_bytes, s, &gate)) != HQQ_OK)
            return rc;
        // both down projections in one launch where K is split over blocks (their results then meet in the
        // outputs' accumulation slots), else one launch per expert, the second adding into y
        rc = launch_vec3_down_pair(w2, h0, ls, (f16 *)y_f16, (const f16 *)row_scale_f16, accumulate, p, mm_bytes, s, down);
        if (rc != HQQ_E_UNSUPPORTED)
            return rc;
        const StripIndex down1 = {device_table, expert_index + 1, 3, 2};
        SmallBatchEpilogue ep;
        ep.row_scale = (const f16 *)row_scale_f16;
        ep.accumulate = accumulate;
        if ((rc = launch_vec3_down(w2, h0, h0 + ls, 1, (f16 *)y_f16, p, mm_bytes, ep, s, nullptr, &down)) != HQQ_OK)
            return rc;
        ep.row_scale = (const f16 *)row_scale_f16 + 1;
        ep.accumulate = 1;
        return launch_vec3_down(w2, h0 + 2 * ls, h0 + 3 * ls, 1, (f16 *)y_f16, p, mm_bytes, ep, s, nullptr, &down1);
    }
    if ((rc = launch_strip_gate_up_pair(w1, w3, (const f16 *)x_f16, h0, h1, p, mm_bytes, s, gate)) != HQQ_OK)
        return rc;
    return launch_strip_down_pair(w2, h0, (int64_t)(mid / 2), (f16 *)y_f16, (const f16 *)row_scale_f16, accumulate, p,
                                  mm_bytes, s, down);
}

int hqq_moe_pair_routed(const hqq_linear *w1, const hqq_linear *w2, const hqq_linear *w3, const void *device_table,
                        const void *x_f16, const void *delta_f16, const void *norm_weight_f16, float eps, void *x_sum_f16,
                        const void *gate_w_f16, int32_t n_experts, int32_t *sel_out, void *weights_f16_out, void *y_f16,
                        int accumulate, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc;
    if ((rc = validate_linear(w1)) != HQQ_OK || (rc = validate_linear(w2)) != HQQ_OK ||
        (rc = validate_linear(w3)) != HQQ_OK)
        return rc;
    if (w1->N != w3->N || w1->K != w3->K || w2->K != w1->N || w2->N != w1->K)
        return HQQ_E_SHAPE;
    if (!x_f16 || !y_f16 || !device_table || !norm_weight_f16 || !x_sum_f16 || !gate_w_f16 || !sel_out || !weights_f16_out)
        return HQQ_E_NULL;
    if (n_experts < 2 || n_experts > 8 || w1->K > 4096 || w1->K % 8 != 0 || w1->nbits == 3)
        return HQQ_E_UNSUPPORTED; // 3-bit experts: hqq_add_rmsnorm_router, then hqq_expert_pair_ffn_indexed
    if ((reinterpret_cast<uintptr_t>(x_f16) | reinterpret_cast<uintptr_t>(delta_f16) | reinterpret_cast<uintptr_t>(gate_w_f16) |
         reinterpret_cast<uintptr_t>(norm_weight_f16) | reinterpret_cast<uintptr_t>(x_sum_f16)) & 15u)
        return HQQ_E_ALIGN;
    const size_t mm_bytes = pair_scratch(w1, w2, w3);
    if (mm_bytes == 0)
        return HQQ_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < hqq_expert_pair_ffn_workspace_bytes(w1, w2, w3) ||
        (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *p = static_cast<char *>(workspace);
    const size_t mid = align256((size_t)w1->N * 2);
    f16 *h0 = (f16 *)(p + mm_bytes), *h1 = (f16 *)(p + mm_bytes + mid);
    // the first launch chooses the experts and leaves its choice in sel_out, which the second one reads
    const StripIndex gate = {device_table, nullptr, 3, 0}, down = {device_table, sel_out, 3, 2};
    const StripNorm norm = {(const f16 *)delta_f16, (const f16 *)norm_weight_f16, (f16 *)x_sum_f16, eps};
    if ((rc = launch_strip_gate_up_pair_routed(w1, w3, (const f16 *)x_f16, norm, (const f16 *)gate_w_f16, n_experts, sel_out,
                                               (f16 *)weights_f16_out, h0, h1, p, mm_bytes, s, gate)) != HQQ_OK)
        return rc;
    return launch_strip_down_pair(w2, h0, (int64_t)(mid / 2), (f16 *)y_f16, (const f16 *)weights_f16_out, accumulate, p,
                                  mm_bytes, s, down);
}

size_t hqq_matmul_group_workspace_bytes(const hqq_linear *const *layers, int32_t count)
{
    if (!layers || count < 1 || count > 4)
        return 0;
    for (int i = 0; i < count; ++i)
        if (validate_linear(layers[i]) != HQQ_OK)
            return 0;
    return strip_job_workspace_bytes(layers, count, 1, 1);
}

int hqq_matmul_group(const hqq_linear *const *layers, int32_t count, const void *x_f16, void *const *ys_f16,
                     void *workspace, size_t workspace_bytes, void *stream)
{
    if (!layers || !ys_f16 || !x_f16)
        return HQQ_E_NULL;
    if (count < 1 || count > 4)
        return HQQ_E_SHAPE;
    int rc;
    for (int i = 0; i < count; ++i) {
        if ((rc = validate_linear(layers[i])) != HQQ_OK)
            return rc;
        if (!ys_f16[i])
            return HQQ_E_NULL;
        if (layers[i]->K != layers[0]->K)
            return HQQ_E_SHAPE;
    }
    const size_t need = strip_job_workspace_bytes(layers, count, 1, 1);
    if (need == 0)
        return HQQ_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    return launch_strip_group(layers, count, (const f16 *)x_f16, reinterpret_cast<f16 *const *>(ys_f16), workspace,
                              workspace_bytes, (hipStream_t)stream);
}

int hqq_matmul_group_norm(const hqq_linear *const *layers, int32_t count, const void *x_f16, const void *delta_f16,
                          const void *norm_weight_f16, float eps, void *x_sum_f16, void *const *ys_f16, void *workspace,
                          size_t workspace_bytes, void *stream)
{
    if (!layers || !ys_f16 || !x_f16 || !norm_weight_f16 || !x_sum_f16)
        return HQQ_E_NULL;
    if (count < 1 || count > 4)
        return HQQ_E_SHAPE;
    int rc;
    for (int i = 0; i < count; ++i) {
        if ((rc = validate_linear(layers[i])) != HQQ_OK)
            return rc;
        if (!ys_f16[i])
            return HQQ_E_NULL;
        if (layers[i]->K != layers[0]->K)
            return HQQ_E_SHAPE;
    }
    const size_t need = strip_job_workspace_bytes(layers, count, 1, 1);
    if (need == 0)
        return HQQ_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return HQQ_E_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(x_f16) | reinterpret_cast<uintptr_t>(delta_f16) |
         reinterpret_cast<uintptr_t>(norm_weight_f16) | reinterpret_cast<uintptr_t>(x_sum_f16)) & 15u)
        return HQQ_E_ALIGN;
    const StripNorm norm = {(const f16 *)delta_f16, (const f16 *)norm_weight_f16, (f16 *)x_sum_f16, eps};
    return launch_strip_group(layers, count, (const f16 *)x_f16, reinterpret_cast<f16 *const *>(ys_f16), workspace,
                              workspace_bytes, (hipStream_t)stream, &norm);
}

int hqq_router_top2(const void *x_f16, const void *gate_w_f16, int32_t n_experts, int64_t hidden, int32_t *sel_out,
                    void *weights_f16_out, void *logits_f16_out, void *stream)
{
    if (!x_f16 || !gate_w_f16 || !sel_out || !weights_f16_out)
        return HQQ_E_NULL;
    return launch_router_top2((const f16 *)x_f16, (const f16 *)gate_w_f16, n_experts, hidden, sel_out,
                              (f16 *)weights_f16_out, (f16 *)logits_f16_out, (hipStream_t)stream);
}

int hqq_add_rmsnorm(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16, int64_t hidden,
                    void *stream)
{
    if (!x_f16 || !weight_f16 || !y_f16)
        return HQQ_E_NULL;
    return launch_add_rmsnorm((f16 *)x_f16, (const f16 *)delta_f16, (const f16 *)weight_f16, eps, (f16 *)y_f16, hidden,
                              (hipStream_t)stream);
}

int hqq_add_rmsnorm_rows(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16, int64_t rows,
                         int64_t hidden, void *stream)
{
    if (!x_f16 || !weight_f16 || !y_f16)
        return HQQ_E_NULL;
    return launch_add_rmsnorm((f16 *)x_f16, (const f16 *)delta_f16, (const f16 *)weight_f16, eps, (f16 *)y_f16, hidden,
                              (hipStream_t)stream, rows);
}

int hqq_router_top2_rows(const void *x_f16, const void *gate_w_f16, int32_t n_experts, int64_t rows, int64_t hidden,
                         int32_t *sel_out, void *weights_f16_out, void *logits_f16_out, void *stream)
{
    if (!x_f16 || !gate_w_f16 || !sel_out || !weights_f16_out)
        return HQQ_E_NULL;
    return launch_router_top2((const f16 *)x_f16, (const f16 *)gate_w_f16, n_experts, hidden, sel_out,
                              (f16 *)weights_f16_out, (f16 *)logits_f16_out, (hipStream_t)stream, rows);
}

int hqq_moe_group_pairs(const int32_t *sel, const void *weights_f16, int64_t tokens, int32_t n_experts, int32_t *counts_out,
                        int64_t *token_of_row_out, void *scale_of_row_f16_out, void *stream)
{
    if (!sel || !weights_f16 || !counts_out || !token_of_row_out || !scale_of_row_f16_out)
        return HQQ_E_NULL;
    return launch_moe_group_pairs(sel, (const f16 *)weights_f16, tokens, n_experts, counts_out,
                                  reinterpret_cast<long long *>(token_of_row_out), (f16 *)scale_of_row_f16_out,
                                  (hipStream_t)stream);
}

int hqq_rope_append_rows(void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                         int64_t start, int64_t rows, void *cache_k_f16, void *cache_v_f16, int64_t max_len,
                         int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, void *stream)
{
    if (!q_f16 || !k_f16 || !v_f16 || !cos_f16 || !sin_f16 || !cache_k_f16 || !cache_v_f16)
        return HQQ_E_NULL;
    return launch_rope_append_rows((f16 *)q_f16, (const f16 *)k_f16, (const f16 *)v_f16, (const f16 *)cos_f16,
                                   (const f16 *)sin_f16, start, rows, (f16 *)cache_k_f16, (f16 *)cache_v_f16, max_len,
                                   n_heads, n_kv_heads, head_dim, (hipStream_t)stream);
}

int hqq_add_rmsnorm_router(void *x_f16, const void *delta_f16, const void *weight_f16, float eps, void *y_f16,
                           int64_t hidden, const void *gate_w_f16, int32_t n_experts, int32_t *sel_out,
                           void *weights_f16_out, void *logits_f16_out, void *stream)
{
    if (!x_f16 || !weight_f16 || !y_f16 || !gate_w_f16 || !sel_out || !weights_f16_out)
        return HQQ_E_NULL;
    return launch_add_rmsnorm_router((f16 *)x_f16, (const f16 *)delta_f16, (const f16 *)weight_f16, eps, (f16 *)y_f16,
                                     hidden, (const f16 *)gate_w_f16, n_experts, sel_out, (f16 *)weights_f16_out,
                                     (f16 *)logits_f16_out, (hipStream_t)stream);
}

int hqq_attention_decode(const void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                         const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len, int32_t n_heads,
                         int32_t n_kv_heads, int32_t head_dim, void *out_f16, void *stream)
{
    if (!q_f16 || !k_f16 || !v_f16 || !cos_f16 || !sin_f16 || !pos || !cache_k_f16 || !cache_v_f16 || !out_f16)
        return HQQ_E_NULL;
    return launch_attention_decode((const f16 *)q_f16, (const f16 *)k_f16, (const f16 *)v_f16, (const f16 *)cos_f16,
                                   (const f16 *)sin_f16, pos, (f16 *)cache_k_f16, (f16 *)cache_v_f16, max_len, n_heads,
                                   n_kv_heads, head_dim, (f16 *)out_f16, (hipStream_t)stream);
}

size_t hqq_quantize_workspace_bytes(void) { return quantize_workspace_bytes(); }

int hqq_quantize_groups(const void *w, int32_t w_is_fp32, int64_t rows, int64_t cols, int32_t nbits, int32_t round_zero,
                        int32_t iters, float lp_norm, double beta, double kappa, void *codes_u8, void *inv_scale_f32,
                        void *zero_f32, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!w || !codes_u8 || !inv_scale_f32 || !zero_f32)
        return HQQ_E_NULL;
    return launch_quantize_groups(w, w_is_fp32, rows, cols, nbits, round_zero, iters, lp_norm, beta, kappa,
                                  static_cast<uint8_t *>(codes_u8), static_cast<float *>(inv_scale_f32),
                                  static_cast<float *>(zero_f32), workspace, workspace_bytes, (hipStream_t)stream);
}

int hqq_quantize_whole(const void *x_f32, int64_t n, int32_t nbits, void *codes_u8, void *inv_scale_f32, void *zero_f32,
                       void *workspace, size_t workspace_bytes, void *stream)
{
    if (!x_f32 || !codes_u8 || !inv_scale_f32 || !zero_f32)
        return HQQ_E_NULL;
    return launch_quantize_whole(static_cast<const float *>(x_f32), n, nbits, static_cast<uint8_t *>(codes_u8),
                                 static_cast<float *>(inv_scale_f32), static_cast<float *>(zero_f32), workspace,
                                 workspace_bytes, (hipStream_t)stream);
}

size_t hqq_attention_chain_workspace_bytes(void) { return workspace_head_bytes(); }

size_t hqq_attention_chain_error_offset(void) { return attention_chain_error_offset(); }

int hqq_attention_chain(const hqq_linear *q, const hqq_linear *k, const hqq_linear *v, const hqq_linear *o, const void *x_f16,
                        const void *delta_f16, const void *norm_weight_f16, float eps, void *x_sum_f16, void *q_scratch_f16,
                        void *k_scratch_f16, void *v_scratch_f16, void *att_scratch_f16, const void *cos_f16,
                        const void *sin_f16, const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len,
                        int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, void *y_f16, void *workspace,
                        size_t workspace_bytes, void *stream)
{
    int rc;
    if ((rc = validate_linear(q)) != HQQ_OK || (rc = validate_linear(k)) != HQQ_OK || (rc = validate_linear(v)) != HQQ_OK ||
        (rc = validate_linear(o)) != HQQ_OK)
        return rc;
    if (!x_f16 || !norm_weight_f16 || !x_sum_f16 || !q_scratch_f16 || !k_scratch_f16 || !v_scratch_f16 || !att_scratch_f16 ||
        !cos_f16 || !sin_f16 || !pos || !cache_k_f16 || !cache_v_f16 || !y_f16)
        return HQQ_E_NULL;
    if (q->K != k->K || q->K != v->K || o->N != q->K)
        return HQQ_E_SHAPE;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u) || workspace_bytes < workspace_head_bytes())
        return HQQ_E_WORKSPACE;
    AttentionChain c = {};
    c.q = q, c.k = k, c.v = v, c.o = o;
    c.x = (const f16 *)x_f16, c.delta = (const f16 *)delta_f16, c.norm_weight = (const f16 *)norm_weight_f16, c.eps = eps;
    c.x_sum = (f16 *)x_sum_f16;
    c.q_out = (f16 *)q_scratch_f16, c.k_out = (f16 *)k_scratch_f16, c.v_out = (f16 *)v_scratch_f16;
    c.att_out = (f16 *)att_scratch_f16;
    c.cos_t = (const f16 *)cos_f16, c.sin_t = (const f16 *)sin_f16, c.pos = pos;
    c.cache_k = (f16 *)cache_k_f16, c.cache_v = (f16 *)cache_v_f16, c.max_len = max_len;
    c.n_heads = n_heads, c.n_kv_heads = n_kv_heads, c.head_dim = head_dim;
    c.y = (f16 *)y_f16;
    return launch_attention_chain(c, workspace, workspace_bytes, (hipStream_t)stream);
}

size_t hqq_attention_decode_workspace_bytes(int64_t max_len, int32_t n_heads, int32_t head_dim)
{
    if (max_len < 1 || n_heads < 1 || (head_dim != 64 && head_dim != 128))
        return 0;
    return attention_workspace_bytes(max_len, n_heads, head_dim);
}

int hqq_attention_decode_ws(const void *q_f16, const void *k_f16, const void *v_f16, const void *cos_f16, const void *sin_f16,
                            const int64_t *pos, void *cache_k_f16, void *cache_v_f16, int64_t max_len, int32_t n_heads,
                            int32_t n_kv_heads, int32_t head_dim, void *out_f16, void *workspace, size_t workspace_bytes,
                            void *stream)
{
    if (!q_f16 || !k_f16 || !v_f16 || !cos_f16 || !sin_f16 || !pos || !cache_k_f16 || !cache_v_f16 || !out_f16)
        return HQQ_E_NULL;
    const size_t need = hqq_attention_decode_workspace_bytes(max_len, n_heads, head_dim);
    if (need > 0 && (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)))
        return HQQ_E_WORKSPACE;
    return launch_attention_decode((const f16 *)q_f16, (const f16 *)k_f16, (const f16 *)v_f16, (const f16 *)cos_f16,
                                   (const f16 *)sin_f16, pos, (f16 *)cache_k_f16, (f16 *)cache_v_f16, max_len, n_heads,
                                   n_kv_heads, head_dim, (f16 *)out_f16, (hipStream_t)stream, workspace, workspace_bytes);
}

} // extern "C"
