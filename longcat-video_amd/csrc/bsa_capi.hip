// C ABI of the engine: argument validation, workspace carving, kernel
// sequencing.  Nothing here allocates device memory or waits for the GPU.
#include "bsa_common.h"

#include <atomic>
#include <mutex>
#include <cmath>
#include <cstdarg>
#include <cstdio>

namespace bsa {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

inline int hip_fail(hipError_t e, const char* what) {
    return set_error(BSA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Row pitch rules shared by the data-movement kernels: rows are moved in
// 16-byte pieces by groups of lanes whose count divides the workgroup.
int check_row(int D, int dtype) {
    const int es = dtype_size(dtype);
    if (es == 0) return set_error(BSA_ERR_UNSUPPORTED, "unknown dtype %d", dtype);
    if (D <= 0) return set_error(BSA_ERR_BAD_ARG, "head dim %d must be positive", D);
    const int bytes = D * es;
    if (bytes % 16 != 0) return set_error(BSA_ERR_UNSUPPORTED, "row of %d bytes is not a multiple of 16", bytes);
    const int cpr = bytes / 16;
    if (cpr > 256 || (256 % cpr) != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "head dim %d: row pieces (%d) must divide 256", D, cpr);
    return BSA_OK;
}

int check_grid(int B, int Hn, int T, int H, int W, int t, int h, int w) {
    if (B <= 0 || Hn <= 0 || T <= 0 || H <= 0 || W <= 0 || t <= 0 || h <= 0 || w <= 0)
        return set_error(BSA_ERR_BAD_ARG, "sizes must be positive (B=%d heads=%d grid=%dx%dx%d chunk=%dx%dx%d)",
                         B, Hn, T, H, W, t, h, w);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads = %lld exceeds 65535", (long long)B * Hn);
    return BSA_OK;
}

int check_strides(const int64_t s[3], int D, int dtype, const char* name) {
    if (s == nullptr) return set_error(BSA_ERR_BAD_ARG, "%s strides are null", name);
    const int es = dtype_size(dtype);
    for (int i = 0; i < 3; ++i) {
        if (s[i] < 0) return set_error(BSA_ERR_BAD_ARG, "%s stride %d is negative", name, i);
        if ((s[i] * es) % 16 != 0)
            return set_error(BSA_ERR_BAD_ARG, "%s stride %d (%lld elements) breaks 16-byte row alignment", name, i, (long long)s[i]);
    }
    if (s[2] < D) return set_error(BSA_ERR_BAD_ARG, "%s token stride %lld is smaller than head dim %d", name, (long long)s[2], D);
    return BSA_OK;
}

}  // namespace
}  // namespace bsa

using namespace bsa;

#define BSA_TRY(expr)                   \
    do {                                \
        const int rc_ = (expr);         \
        if (rc_ != BSA_OK) return rc_;  \
    } while (0)

extern "C" {

int bsa_version(void) { return 100; }

const char* bsa_last_error(void) { return g_err; }

int bsa_num_selected(double sparsity, int n_kv_blocks) {
    return (int)((1.0 - sparsity) * (double)n_kv_blocks);
}

int64_t bsa_padded_tokens(int T, int H, int W, int t, int h, int w) {
    if (T <= 0 || H <= 0 || W <= 0 || t <= 0 || h <= 0 || w <= 0) return -1;
    const Grid3 g = make_grid(T, H, W, t, h, w);
    return (int64_t)g.blocks() * g.chunk();
}

int bsa_permute_thw_to_blocks(const void* src, const int64_t src_strides[3], void* dst, void* pooled,
                              uint64_t* tile_valid, int B, int Hn, int T, int H, int W, int t, int h,
                              int w, int D, int dtype, void* stream) {
    if (!src || !dst) return set_error(BSA_ERR_BAD_ARG, "permute: src/dst is null");
    BSA_TRY(check_row(D, dtype));
    BSA_TRY(check_grid(B, Hn, T, H, W, t, h, w));
    BSA_TRY(check_strides(src_strides, D, dtype, "src"));
    if (!aligned16(src) || !aligned16(dst)) return set_error(BSA_ERR_BAD_ARG, "permute: pointers must be 16-byte aligned");
    const Grid3 g = make_grid(T, H, W, t, h, w);
    if (tile_valid && g.chunk() % 64 != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "tile validity needs a chunk of a multiple of 64 tokens, got %d", g.chunk());
    const hipError_t e = launch_permute(src, src_strides, dst, pooled, tile_valid, B, Hn, g, D, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "permute launch");
}

int bsa_unpermute_blocks_to_thw(const void* src, void* dst, const int64_t dst_strides[3], int B, int Hn,
                                int T, int H, int W, int t, int h, int w, int D, int dtype, void* stream) {
    if (!src || !dst) return set_error(BSA_ERR_BAD_ARG, "unpermute: src/dst is null");
    BSA_TRY(check_row(D, dtype));
    BSA_TRY(check_grid(B, Hn, T, H, W, t, h, w));
    BSA_TRY(check_strides(dst_strides, D, dtype, "dst"));
    if (!aligned16(src) || !aligned16(dst)) return set_error(BSA_ERR_BAD_ARG, "unpermute: pointers must be 16-byte aligned");
    const Grid3 g = make_grid(T, H, W, t, h, w);
    const hipError_t e = launch_unpermute(src, dst, dst_strides, B, Hn, g, D, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "unpermute launch");
}

int bsa_mean_pool(const void* x, void* out, int B, int Hn, int64_t S, int block, int D, int dtype, void* stream) {
    if (!x || !out) return set_error(BSA_ERR_BAD_ARG, "mean_pool: x/out is null");
    BSA_TRY(check_row(D, dtype));
    if (B <= 0 || Hn <= 0 || S <= 0 || block <= 0)
        return set_error(BSA_ERR_BAD_ARG, "mean_pool: sizes must be positive (B=%d heads=%d S=%lld block=%d)", B, Hn, (long long)S, block);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (!aligned16(x)) return set_error(BSA_ERR_BAD_ARG, "mean_pool: x must be 16-byte aligned");
    const hipError_t e = launch_mean_pool(x, out, B, Hn, S, block, D, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "mean_pool launch");
}

static int check_topk(int B, int Hn, int nbq, int nbk, int k_sel, int dtype) {
    if (dtype_size(dtype) == 0) return set_error(BSA_ERR_UNSUPPORTED, "unknown dtype %d", dtype);
    if (B <= 0 || Hn <= 0 || nbq <= 0 || nbk <= 0)
        return set_error(BSA_ERR_BAD_ARG, "top-k: sizes must be positive (B=%d heads=%d nbq=%d nbk=%d)", B, Hn, nbq, nbk);
    if (k_sel < 0 || k_sel > nbk) return set_error(BSA_ERR_SHAPE, "top-k: k_sel=%d outside [0, %d]", k_sel, nbk);
    if (nbk > 4096) return set_error(BSA_ERR_UNSUPPORTED, "top-k: %d KV blocks exceed the limit of 4096", nbk);
    return BSA_OK;
}

int bsa_topk_from_score(const void* score, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out, int B,
                        int Hn, int nbq, int nbk, int k_sel, int dtype, void* stream) {
    if (!score || !lens_out || (!idx_out && !idx_sorted_out)) return set_error(BSA_ERR_BAD_ARG, "top-k: null pointer");
    BSA_TRY(check_topk(B, Hn, nbq, nbk, k_sel, dtype));
    const hipError_t e = launch_topk(score, idx_out, idx_sorted_out, lens_out, (int64_t)B * Hn * nbq, nbk, k_sel, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "top-k launch");
}

int bsa_visit_order(const int32_t* idx_sorted, const int32_t* lens, int32_t* idx_out, int64_t rows, int nbk,
                    int idx_stride, void* stream) {
    if (!idx_sorted || !lens || !idx_out) return set_error(BSA_ERR_BAD_ARG, "visit_order: null pointer");
    if (rows < 0 || rows > 0x7fffffff || nbk <= 0 || idx_stride <= 0 || idx_stride > 4096)
        return set_error(BSA_ERR_BAD_ARG, "visit_order: rows in [0, 2^31), nbk > 0 and 0 < idx_stride <= 4096 wanted");
    const hipError_t e = launch_pace_order(idx_sorted, idx_out, lens, rows, nbk, idx_stride, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "visit order");
    return BSA_OK;
}

int bsa_score_topk(const void* q_cmp, const void* k_cmp, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out,
                   void* score_out, int B, int Hn, int nbq, int nbk, int D, int k_sel, int dtype, void* stream) {
    if (!q_cmp || !k_cmp || !lens_out || (!idx_out && !idx_sorted_out)) return set_error(BSA_ERR_BAD_ARG, "score_topk: null pointer");
    if (!score_out) return set_error(BSA_ERR_BAD_ARG, "score_topk: a score buffer of B*heads*nbq*nbk elements is required");
    BSA_TRY(check_topk(B, Hn, nbq, nbk, k_sel, dtype));
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "score: head dim %d is not built (only 128)", D);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (!aligned16(q_cmp) || !aligned16(k_cmp)) return set_error(BSA_ERR_BAD_ARG, "score: pooled tensors must be 16-byte aligned");
    hipError_t e = launch_score(q_cmp, k_cmp, score_out, B * Hn, nbq, nbk, D, dtype, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "score launch");
    e = launch_topk(score_out, idx_out, idx_sorted_out, lens_out, (int64_t)B * Hn * nbq, nbk, k_sel, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "top-k launch");
}

static int check_cdf(float thr, float scale, int k_min, int idx_stride, int nbk) {
    if (!(thr > 0.f) || !std::isfinite(thr)) return set_error(BSA_ERR_BAD_ARG, "cdf: threshold must be positive and finite");
    if (!(scale > 0.f) || !std::isfinite(scale)) return set_error(BSA_ERR_BAD_ARG, "cdf: sm_scale must be positive and finite");
    if (idx_stride <= 0 || idx_stride > nbk || idx_stride > 4096)
        return set_error(BSA_ERR_SHAPE, "cdf: idx_stride=%d outside [1, min(%d, 4096)]", idx_stride, nbk);
    if (k_min < 0 || k_min > idx_stride) return set_error(BSA_ERR_SHAPE, "cdf: k_min=%d outside [0, %d]", k_min, idx_stride);
    return BSA_OK;
}

int bsa_cdf_from_score(const void* score, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out, int B, int Hn,
                       int nbq, int nbk, float cdf_threshold, float sm_scale, int k_min, int idx_stride, int dtype,
                       void* stream) {
    if (!score || !lens_out || (!idx_out && !idx_sorted_out)) return set_error(BSA_ERR_BAD_ARG, "cdf: null pointer");
    BSA_TRY(check_topk(B, Hn, nbq, nbk, 0, dtype));
    BSA_TRY(check_cdf(cdf_threshold, sm_scale, k_min, idx_stride, nbk));
    const int64_t rows = (int64_t)B * Hn * nbq;
    hipError_t e = launch_cdf_count(score, lens_out, rows, nbk, cdf_threshold, sm_scale, k_min, idx_stride, dtype, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "cdf count launch");
    e = launch_topk(score, idx_out, idx_sorted_out, lens_out, rows, nbk, 0, dtype, (hipStream_t)stream, lens_out, idx_stride);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "top-k launch");
}

int bsa_score_cdf(const void* q_cmp, const void* k_cmp, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out,
                  void* score_out, int B, int Hn, int nbq, int nbk, int D, float cdf_threshold, float sm_scale, int k_min,
                  int idx_stride, int dtype, void* stream) {
    if (!q_cmp || !k_cmp || !lens_out || (!idx_out && !idx_sorted_out)) return set_error(BSA_ERR_BAD_ARG, "score_cdf: null pointer");
    if (!score_out) return set_error(BSA_ERR_BAD_ARG, "score_cdf: a score buffer of B*heads*nbq*nbk elements is required");
    BSA_TRY(check_topk(B, Hn, nbq, nbk, 0, dtype));
    BSA_TRY(check_cdf(cdf_threshold, sm_scale, k_min, idx_stride, nbk));
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "score: head dim %d is not built (only 128)", D);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (!aligned16(q_cmp) || !aligned16(k_cmp)) return set_error(BSA_ERR_BAD_ARG, "score: pooled tensors must be 16-byte aligned");
    const hipError_t e = launch_score(q_cmp, k_cmp, score_out, B * Hn, nbq, nbk, D, dtype, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "score launch");
    return bsa_cdf_from_score(score_out, idx_out, idx_sorted_out, lens_out, B, Hn, nbq, nbk, cdf_threshold, sm_scale, k_min,
                              idx_stride, dtype, stream);
}

int bsa_fwd(const void* q, const void* k, const void* v, const int32_t* idx, const int32_t* lens,
            const uint64_t* tile_valid, void* o, float* lse, int B, int Hn, int64_t Sq, int64_t Sk, int D,
            int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype, void* stream) {
    if (!q || !k || !v || !idx || !lens || !o) return set_error(BSA_ERR_BAD_ARG, "fwd: null pointer");
    if (dtype_size(dtype) == 0) return set_error(BSA_ERR_UNSUPPORTED, "unknown dtype %d", dtype);
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "fwd: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || Sq <= 0 || Sk <= 0 || idx_stride < 0)
        return set_error(BSA_ERR_BAD_ARG, "fwd: sizes must be positive (B=%d heads=%d Sq=%lld Sk=%lld)", B, Hn, (long long)Sq, (long long)Sk);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (bs_q <= 0 || bs_k <= 0 || bs_q % 64 != 0 || bs_k % 64 != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "fwd: chunk sizes %d/%d must be multiples of 64", bs_q, bs_k);
    if (Sq % bs_q != 0 || Sk % bs_k != 0)
        return set_error(BSA_ERR_SHAPE, "fwd: Sq=%lld / Sk=%lld are not multiples of the chunk sizes %d / %d", (long long)Sq, (long long)Sk, bs_q, bs_k);
    if (!(sm_scale > 0.f) || !std::isfinite(sm_scale)) return set_error(BSA_ERR_BAD_ARG, "fwd: sm_scale must be positive and finite");
    if ((Sq / 64) * (int64_t)B * Hn > 0x7fffffffLL || Sk > 0x7fffffffLL || (dtype != BSA_F32 && Sk >= (1 << 24)))
        return set_error(BSA_ERR_UNSUPPORTED, "fwd: problem too large (32-bit work item indices, 24-bit key rows for the 16-bit types)");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
        return set_error(BSA_ERR_BAD_ARG, "fwd: q/k/v/o must be 16-byte aligned");
    const hipError_t e = launch_fwd(q, k, v, idx, lens, tile_valid, o, lse, B, Hn, Sq, Sk, bs_q, bs_k, idx_stride,
                                    sm_scale, dtype, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "fwd launch");
}

// ---- the fragment-order kernel for blocked-order callers --------------------------------------------------
static int check_fwd_fragment(const void* q, const void* k, const void* v, const int32_t* idx, const int32_t* lens, void* o,
                              int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride, float sm_scale,
                              int dtype) {
    if (dtype != BSA_BF16 && dtype != BSA_F16)
        return set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: dtype %d is not built (bf16, fp16; fp32 runs through bsa_fwd)", dtype);
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || Sq <= 0 || Sk <= 0 || idx_stride < 0)
        return set_error(BSA_ERR_BAD_ARG, "fwd_fragment: sizes must be positive (B=%d heads=%d Sq=%lld Sk=%lld)", B, Hn, (long long)Sq, (long long)Sk);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (bs_q <= 0 || bs_k <= 0 || bs_q % 64 != 0 || bs_k % 64 != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: chunk sizes %d/%d must be multiples of 64", bs_q, bs_k);
    if (Sq % bs_q != 0 || Sk % bs_k != 0)
        return set_error(BSA_ERR_SHAPE, "fwd_fragment: Sq=%lld / Sk=%lld are not multiples of the chunk sizes %d / %d", (long long)Sq, (long long)Sk, bs_q, bs_k);
    if (idx_stride > 4096) return set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: lists of %d entries exceed the limit of 4096", idx_stride);
    if ((Sq / 64) * (int64_t)B * Hn > 0x7fffffffLL || Sk / 64 > 0x7fffff)
        return set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: problem too large (32-bit work item indices, 2^23 KV tiles per head)");
    return BSA_OK;
}

namespace {
struct FragmentWs { size_t kv, norms, fallback, total; };
FragmentWs fragment_ws(int B, int Hn, int64_t Sq, int64_t Sk, int D) {
    auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
    FragmentWs w;
    w.kv = up((size_t)B * Hn * (size_t)Sk * D * 2);
    w.norms = up(frag_key_norm_floats(B, Hn, Sk / 64) * sizeof(float));
    w.fallback = up(frag_fallback_ints((int64_t)B * Hn * (Sq / 64)) * sizeof(int32_t));
    w.total = 2 * w.kv + w.norms + w.fallback;       // K, V, key norms, the list of items left to the second kernel
    return w;
}
}  // namespace

size_t bsa_fwd_fragment_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int D, int dtype) {
    if ((dtype != BSA_BF16 && dtype != BSA_F16) || D != 128 || B <= 0 || Hn <= 0 || Sq <= 0 || Sq % 64 != 0 || Sk <= 0 || Sk % 64 != 0) {
        set_error(BSA_ERR_UNSUPPORTED, "fwd_fragment: bf16 / fp16, head dim 128, Sq and Sk positive multiples of 64");
        return 0;
    }
    return fragment_ws(B, Hn, Sq, Sk, D).total;
}

int bsa_fwd_fragment(const void* q, const void* k, const void* v, const int32_t* idx, const int32_t* lens,
                     const uint64_t* tile_valid, void* o, float* lse, int B, int Hn, int64_t Sq, int64_t Sk, int D,
                     int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype, void* workspace,
                     size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !lens || !o || !workspace || (!idx && idx_stride > 0)) return set_error(BSA_ERR_BAD_ARG, "fwd_fragment: null pointer");
    BSA_TRY(check_fwd_fragment(q, k, v, idx, lens, o, B, Hn, Sq, Sk, D, bs_q, bs_k, idx_stride, sm_scale, dtype));
    if (!(sm_scale > 0.f) || !std::isfinite(sm_scale)) return set_error(BSA_ERR_BAD_ARG, "fwd_fragment: sm_scale must be positive and finite");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return set_error(BSA_ERR_BAD_ARG, "fwd_fragment: q/k/v/o must be 16-byte aligned, the workspace 256-byte aligned");
    const FragmentWs fw = fragment_ws(B, Hn, Sq, Sk, D);
    const size_t need = fw.total;
    if (workspace_bytes < need) return set_error(BSA_ERR_WORKSPACE, "fwd_fragment: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    // a blocked-order tensor is a (Sk / 64, 8, 8) grid cut into (1, 8, 8) chunks: tile i = rows 64 i .. 64 i + 63
    const Grid3 g = make_grid((int)(Sk / 64), 8, 8, 1, 8, 8);
    const int64_t kv_st[3] = {(int64_t)Hn * Sk * D, Sk * D, D};
    const int64_t q_st[3] = {(int64_t)Hn * Sq * D, Sq * D, D};
    char* kf = static_cast<char*>(workspace);
    char* vf = kf + fw.kv;
    float* knorm = reinterpret_cast<float*>(vf + fw.kv);
    int32_t* fallback = reinterpret_cast<int32_t*>(vf + fw.kv + fw.norms);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = launch_frag(k, kv_st, kf, B, Hn, g, dtype, false, st, nullptr, nullptr, nullptr, knorm);
    if (e == hipSuccess) e = launch_frag(v, kv_st, vf, B, Hn, g, dtype, true, st);
    if (e == hipSuccess)
        e = launch_fwd_frag(q, kf, vf, idx, lens, tile_valid, o, lse, B, Hn, Sq, Sk, bs_q, bs_k, idx_stride, sm_scale, dtype, st,
                            nullptr, q_st, q_st, Sq, nullptr, nullptr, knorm, fallback);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "fwd_fragment");
}

static int check_bwd_shape(int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int dtype) {
    if (dtype != BSA_BF16 && dtype != BSA_F16) return set_error(BSA_ERR_UNSUPPORTED, "bwd: dtype %d is not built (bf16, fp16)", dtype);
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "bwd: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || Sq <= 0 || Sk <= 0)
        return set_error(BSA_ERR_BAD_ARG, "bwd: sizes must be positive (B=%d heads=%d Sq=%lld Sk=%lld)", B, Hn, (long long)Sq, (long long)Sk);
    if ((int64_t)B * Hn > 65535) return set_error(BSA_ERR_UNSUPPORTED, "B*heads exceeds 65535");
    if (bs_q <= 0 || bs_k <= 0 || bs_q % 64 != 0 || bs_k % 64 != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "bwd: chunk sizes %d/%d must be multiples of 64", bs_q, bs_k);
    if (Sq % bs_q != 0 || Sk % bs_k != 0)
        return set_error(BSA_ERR_SHAPE, "bwd: Sq=%lld / Sk=%lld are not multiples of the chunk sizes %d / %d", (long long)Sq, (long long)Sk, bs_q, bs_k);
    if ((Sq / 32) * (int64_t)B * Hn > 0x7fffffffLL || (Sk / 32) * (int64_t)B * Hn > 0x7fffffffLL)
        return set_error(BSA_ERR_UNSUPPORTED, "bwd: problem too large (32-bit work item indices)");
    if (Sq / bs_q > bwd_max_query_blocks())
        return set_error(BSA_ERR_UNSUPPORTED, "bwd: %lld query blocks exceed the %d whose list the dK / dV kernel can hold in LDS",
                         (long long)(Sq / bs_q), bwd_max_query_blocks());
    return BSA_OK;
}

size_t bsa_bwd_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride, int dtype) {
    if (check_bwd_shape(B, Hn, Sq, Sk, D, bs_q, bs_k, dtype) != BSA_OK) return 0;
    if (idx_stride <= 0 || idx_stride > 4096) { set_error(BSA_ERR_BAD_ARG, "bwd: idx_stride=%d outside [1, 4096]", idx_stride); return 0; }
    return bwd_workspace_bytes(B, Hn, Sq, Sk, bs_q, bs_k, idx_stride);
}

int bsa_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
            const int32_t* idx, const int32_t* lens, const uint64_t* tile_valid, void* dq, void* dk, void* dv, int B,
            int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype,
            void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !o || !d_o || !lse || !idx || !lens || !dq || !dk || !dv || !workspace)
        return set_error(BSA_ERR_BAD_ARG, "bwd: null pointer");
    BSA_TRY(check_bwd_shape(B, Hn, Sq, Sk, D, bs_q, bs_k, dtype));
    if (idx_stride <= 0 || idx_stride > 4096) return set_error(BSA_ERR_BAD_ARG, "bwd: idx_stride=%d outside [1, 4096]", idx_stride);
    if (!(sm_scale > 0.f) || !std::isfinite(sm_scale)) return set_error(BSA_ERR_BAD_ARG, "bwd: sm_scale must be positive and finite");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) ||
        !aligned16(dv) || (reinterpret_cast<uintptr_t>(workspace) & 255u))
        return set_error(BSA_ERR_BAD_ARG, "bwd: tensors must be 16-byte aligned, the workspace 256-byte aligned");
    const size_t need = bwd_workspace_bytes(B, Hn, Sq, Sk, bs_q, bs_k, idx_stride);
    if (workspace_bytes < need) return set_error(BSA_ERR_WORKSPACE, "bwd: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    const hipError_t e = launch_bwd(q, k, v, o, d_o, lse, idx, lens, tile_valid, dq, dk, dv, B, Hn, Sq, Sk, bs_q, bs_k, idx_stride,
                                    sm_scale, dtype, workspace, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "bwd launch");
}

// ---- whole operator -------------------------------------------------------
namespace {
struct Plan {
    Grid3 gq, gk;
    int64_t Sqp, Skp;
    int nbq, nbk, es;
    int sel_width;        // columns of the index lists: k_sel, or the cap of the CDF rule
    bool cdf;
    bool direct_qo, direct_kv;
    bool frag;            // k and v are rewritten in fragment order for fwd_frag_kernel (bsa_fwd_frag.hip)
    size_t off_qp, off_kp, off_vp, off_op, off_qc, off_kc, off_score, off_idx, off_idx_sorted, off_lens, off_valid, off_qrows, off_ktiles, off_order, off_queue, off_knorm, off_fallback, total;
};
inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

// compact: keep the workspace small (k and v are gathered where they lie by fwd_mfma_kernel, only the chunks at the
// padded edge are copied) instead of rewriting k and v in fragment order for the faster fwd_frag_kernel.
int make_plan(const bsa_3d_params* p, Plan* pl, bool compact = false) {
    if (!p) return set_error(BSA_ERR_BAD_ARG, "params are null");
    BSA_TRY(check_row(p->D, p->dtype));
    BSA_TRY(check_grid(p->B, p->Hn, p->Tq, p->Hq, p->Wq, p->tq, p->hq, p->wq));
    BSA_TRY(check_grid(p->B, p->Hn, p->Tk, p->Hk, p->Wk, p->tk, p->hk, p->wk));
    if (p->D != 128) return set_error(BSA_ERR_UNSUPPORTED, "head dim %d is not built (only 128)", p->D);
    pl->gq = make_grid(p->Tq, p->Hq, p->Wq, p->tq, p->hq, p->wq);
    pl->gk = make_grid(p->Tk, p->Hk, p->Wk, p->tk, p->hk, p->wk);
    if (pl->gq.chunk() % 64 != 0 || pl->gk.chunk() % 64 != 0)
        return set_error(BSA_ERR_UNSUPPORTED, "chunk sizes %d/%d must be multiples of 64 tokens", pl->gq.chunk(), pl->gk.chunk());
    pl->nbq = pl->gq.blocks();
    pl->nbk = pl->gk.blocks();
    BSA_TRY(check_topk(p->B, p->Hn, pl->nbq, pl->nbk, p->k_sel, p->dtype));
    pl->cdf = p->cdf_threshold > 0.f;
    pl->sel_width = pl->cdf ? pl->nbk : p->k_sel;       // the CDF rule may keep every block of a row (nbk <= 4096)
    if (pl->cdf && !std::isfinite(p->cdf_threshold)) return set_error(BSA_ERR_BAD_ARG, "cdf_threshold must be finite");
    if (!(p->sm_scale > 0.f) || !std::isfinite(p->sm_scale)) return set_error(BSA_ERR_BAD_ARG, "sm_scale must be positive and finite");
    pl->Sqp = (int64_t)pl->nbq * pl->gq.chunk();
    pl->Skp = (int64_t)pl->nbk * pl->gk.chunk();
    pl->es = dtype_size(p->dtype);
    if ((pl->Sqp / 64) * (int64_t)p->B * p->Hn > 0x7fffffffLL || (p->dtype != BSA_F32 && pl->Skp >= (1 << 24)) || pl->Skp > 0x7fffffffLL)
        return set_error(BSA_ERR_UNSUPPORTED, "problem too large (32-bit work item indices, 24-bit key rows for the 16-bit types)");
    const size_t bh = (size_t)p->B * p->Hn;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up256(bytes); return o; };
    // The MFMA kernel reads q and writes o in THW order itself, and gathers k and v tiles from THW
    // order when the kv grid allows it; blocked copies are only made for the fp32 kernel and for
    // kv grids that do not qualify.
    pl->direct_qo = p->dtype != BSA_F32;
    pl->frag = pl->direct_qo && !compact;
    pl->direct_kv = pl->direct_qo && !pl->frag && kv_direct_ok(pl->gk, (int64_t)p->D * pl->es);
    pl->off_qp = take(pl->direct_qo ? 0 : bh * pl->Sqp * p->D * pl->es);
    // fragment order is a permutation of the padded blocked order: the same size
    const size_t kv_rows = pl->direct_kv ? (size_t)edge_count(pl->gk) * pl->gk.chunk() : (size_t)pl->Skp;
    pl->off_kp = take(bh * kv_rows * p->D * pl->es);
    pl->off_vp = take(bh * kv_rows * p->D * pl->es);
    pl->off_op = take(pl->direct_qo ? 0 : bh * pl->Sqp * p->D * pl->es);
    pl->off_qc = take(bh * pl->nbq * p->D * pl->es);
    pl->off_kc = take(bh * pl->nbk * p->D * pl->es);
    pl->off_score = take(bh * pl->nbq * (size_t)pl->nbk * pl->es);
    pl->off_idx = take(bh * pl->nbq * (size_t)(pl->sel_width > 0 ? pl->sel_width : 1) * sizeof(int32_t));
    pl->off_idx_sorted = take(bh * pl->nbq * (size_t)(pl->sel_width > 0 ? pl->sel_width : 1) * sizeof(int32_t));
    pl->off_lens = take(bh * pl->nbq * sizeof(int32_t));
    pl->off_valid = take((size_t)(pl->Skp / 64) * sizeof(uint64_t));
    pl->off_qrows = take(pl->direct_qo ? (size_t)pl->Sqp * sizeof(int32_t) : 0);
    pl->off_ktiles = take(pl->direct_kv ? (size_t)(pl->Skp / 64) * sizeof(uint32_t) : 0);
    // lists of unequal length (the CDF rule): work items by descending length, and the counter they are drawn with
    pl->off_order = take(pl->cdf && pl->direct_qo ? bh * (size_t)(pl->Sqp / 64) * sizeof(int32_t) : 0);
    pl->off_queue = take(pl->cdf && pl->direct_qo ? 2 * sizeof(uint32_t) : 0);    // the counter and the choice of schedule
    pl->off_knorm = take(pl->frag ? frag_key_norm_floats(p->B, p->Hn, pl->Skp / 64) * sizeof(float) : 0);   // key norms per head and tile
    pl->off_fallback = take(pl->frag ? frag_fallback_ints((int64_t)bh * (pl->Sqp / 64)) * sizeof(int32_t) : 0);
    pl->total = off;
    return BSA_OK;
}
}  // namespace

size_t bsa_workspace_bytes(const bsa_3d_params* p) {
    Plan pl;
    if (make_plan(p, &pl) != BSA_OK) return 0;
    return pl.total;
}

namespace {
struct Ws {
    void *qp, *kp, *vp, *op, *qc, *kc, *score;
    int32_t *idx, *idx_sorted, *lens, *qrows, *order;
    uint32_t *ktiles, *queue;
    uint64_t* valid;
    float* knorm;
    int32_t* fallback;
};
int carve(const Plan& pl, void* workspace, size_t workspace_bytes, const char* who, Ws* w) {
    if (!workspace) return set_error(BSA_ERR_BAD_ARG, "%s: workspace is null", who);
    if (workspace_bytes < pl.total)
        return set_error(BSA_ERR_WORKSPACE, "%s: workspace of %zu bytes is smaller than the %zu required", who, workspace_bytes, pl.total);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return set_error(BSA_ERR_BAD_ARG, "%s: workspace must be 256-byte aligned", who);
    char* ws = static_cast<char*>(workspace);
    w->qp = ws + pl.off_qp; w->kp = ws + pl.off_kp; w->vp = ws + pl.off_vp; w->op = ws + pl.off_op;
    w->qc = ws + pl.off_qc; w->kc = ws + pl.off_kc; w->score = ws + pl.off_score;
    w->idx = reinterpret_cast<int32_t*>(ws + pl.off_idx);
    w->idx_sorted = reinterpret_cast<int32_t*>(ws + pl.off_idx_sorted);
    w->lens = reinterpret_cast<int32_t*>(ws + pl.off_lens);
    w->valid = reinterpret_cast<uint64_t*>(ws + pl.off_valid);
    w->qrows = pl.direct_qo ? reinterpret_cast<int32_t*>(ws + pl.off_qrows) : nullptr;
    w->ktiles = pl.direct_kv ? reinterpret_cast<uint32_t*>(ws + pl.off_ktiles) : nullptr;
    w->order = pl.cdf && pl.direct_qo ? reinterpret_cast<int32_t*>(ws + pl.off_order) : nullptr;
    w->queue = pl.cdf && pl.direct_qo ? reinterpret_cast<uint32_t*>(ws + pl.off_queue) : nullptr;
    w->knorm = pl.frag ? reinterpret_cast<float*>(ws + pl.off_knorm) : nullptr;
    w->fallback = pl.frag ? reinterpret_cast<int32_t*>(ws + pl.off_fallback) : nullptr;
    return BSA_OK;
}
bool kv_padded(const bsa_3d_params* p) { return (p->Tk % p->tk) || (p->Hk % p->hk) || (p->Wk % p->wk); }

int check_kv_views(const Plan& pl, const int64_t k_strides[3], const int64_t v_strides[3], const char* who) {
    if (pl.direct_kv && (k_strides[2] != v_strides[2] || !kv_direct_ok(pl.gk, k_strides[2] * pl.es)))
        return set_error(BSA_ERR_UNSUPPORTED, "%s: k and v must share one token stride (got %lld and %lld elements) small "
                         "enough for 32-bit offsets inside a tile; pass contiguous copies",
                         who, (long long)k_strides[2], (long long)v_strides[2]);
    return BSA_OK;
}

// Everything the attention kernel needs besides the selection, for the 16-bit types: the row table
// of q, and for k and v the tile table, the validity words and the copies of the edge chunks (or
// of all chunks when the kv grid does not allow gathering).  With `pool`, q and k are also read in
// full and their chunk means stored (one pass over each).
hipError_t prepare_thw(const Plan& pl, const bsa_3d_params* p, const Ws& w, const void* q, const int64_t q_strides[3],
                       const void* k, const int64_t k_strides[3], const void* v, const int64_t v_strides[3], bool pool,
                       hipStream_t st, const RowTransform* trq = nullptr, const RowTransform* trk = nullptr) {
    hipError_t e;
    const bool padded_k = kv_padded(p);
    if (pool && !(pl.frag && pl.gq.chunk() == 64))
        e = launch_permute(q, q_strides, nullptr, w.qc, nullptr, p->B, p->Hn, pl.gq, p->D, p->dtype, st, false, w.qrows, nullptr);
    else    // tables only: one (batch, head) slice of workgroups, no row is read
        e = launch_permute(q, q_strides, nullptr, nullptr, nullptr, 1, 1, pl.gq, p->D, p->dtype, st, false, w.qrows, nullptr);
    if (e != hipSuccess) return e;
    if (pool && pl.frag && pl.gq.chunk() == 64) {
        // chunk means of q from a read-only pass (the same sums); with a row transform, from the fragment pass run
        // without a destination, which applies it
        if (trq == nullptr && p->D == 128) e = launch_pool_tiles(q, q_strides, w.qrows, w.qc, p->B, p->Hn, pl.gq, p->dtype, st);
        else e = launch_frag(q, q_strides, nullptr, p->B, p->Hn, pl.gq, p->dtype, false, st, w.qc, nullptr, trq);
        if (e != hipSuccess) return e;
    }
    if (pl.frag) {
        // 64-slot chunks: one pass over k gives its fragment order, its chunk means and the validity words
        if (pl.gk.chunk() == 64) {
            e = launch_frag(k, k_strides, w.kp, p->B, p->Hn, pl.gk, p->dtype, false, st, pool ? w.kc : nullptr,
                            padded_k ? w.valid : nullptr, trk, w.knorm);
            if (e != hipSuccess) return e;
            return launch_frag(v, v_strides, w.vp, p->B, p->Hn, pl.gk, p->dtype, true, st);
        }
        // larger chunks: pooled means and validity words of k by the pooling pass, then k and v in fragment order
        if (pool || padded_k) {
            if (pool)
                e = launch_permute(k, k_strides, nullptr, w.kc, padded_k ? w.valid : nullptr, p->B, p->Hn, pl.gk, p->D, p->dtype, st);
            else
                e = launch_permute(k, k_strides, nullptr, nullptr, w.valid, 1, 1, pl.gk, p->D, p->dtype, st);
            if (e != hipSuccess) return e;
        }
        e = launch_frag(k, k_strides, w.kp, p->B, p->Hn, pl.gk, p->dtype, false, st, nullptr, nullptr, nullptr, w.knorm);
        if (e != hipSuccess) return e;
        return launch_frag(v, v_strides, w.vp, p->B, p->Hn, pl.gk, p->dtype, true, st);
    }
    // gathering: the pass over k copies the edge chunks of v along with those of k
    e = launch_permute(k, k_strides, w.kp, pool ? w.kc : nullptr, padded_k ? w.valid : nullptr, p->B, p->Hn, pl.gk, p->D,
                       p->dtype, st, pl.direct_kv, nullptr, w.ktiles, pl.direct_kv && padded_k ? v : nullptr, v_strides, w.vp);
    if (e != hipSuccess) return e;
    if (!pl.direct_kv)
        e = launch_permute(v, v_strides, w.vp, nullptr, nullptr, p->B, p->Hn, pl.gk, p->D, p->dtype, st);
    return e;
}

hipError_t attention_thw(const Plan& pl, const bsa_3d_params* p, const Ws& w, const void* q, const int64_t q_strides[3],
                         const void* k, const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
                         const int64_t o_strides[3], const int32_t* idx, const int32_t* lens, int idx_stride, float* lse,
                         hipStream_t st, bool by_length = false) {
    if (pl.frag)
        return launch_fwd_frag(q, w.kp, w.vp, idx, lens, kv_padded(p) ? w.valid : nullptr, o, lse, p->B, p->Hn, pl.Sqp, pl.Skp,
                               pl.gq.chunk(), pl.gk.chunk(), idx_stride, p->sm_scale, p->dtype, st, w.qrows, q_strides, o_strides,
                               (int64_t)p->Tq * p->Hq * p->Wq, by_length ? w.order : nullptr, by_length ? w.queue : nullptr, w.knorm, w.fallback);
    FwdLayout L;
    L.q_rows = w.qrows;
    L.k_tiles = w.ktiles;
    L.k_edge = w.kp;
    L.v_edge = w.vp;
    for (int i = 0; i < 3; ++i) { L.q_st[i] = q_strides[i]; L.o_st[i] = o_strides[i]; }
    if (pl.direct_kv) {
        for (int i = 0; i < 3; ++i) { L.k_st[i] = k_strides[i]; L.v_st[i] = v_strides[i]; }
        L.kw = pl.gk.w; L.kh = pl.gk.h; L.kH = pl.gk.H; L.kW = pl.gk.W;
    } else {
        L.k_st[0] = L.v_st[0] = (int64_t)p->Hn * pl.Skp * p->D;
        L.k_st[1] = L.v_st[1] = pl.Skp * p->D;
        L.k_st[2] = L.v_st[2] = p->D;
        L.kw = 4; L.kh = 16; L.kH = 16; L.kW = 4;
    }
    return launch_fwd(q, pl.direct_kv ? k : w.kp, pl.direct_kv ? v : w.vp, idx, lens, kv_padded(p) ? w.valid : nullptr, o, lse,
                      p->B, p->Hn, pl.Sqp, pl.Skp, pl.gq.chunk(), pl.gk.chunk(), idx_stride, p->sm_scale, p->dtype, st, &L,
                      (int64_t)p->Tq * p->Hq * p->Wq, (int64_t)edge_count(pl.gk) * pl.gk.chunk() * p->D * pl.es,
                      by_length ? w.order : nullptr, by_length ? w.queue : nullptr);
}

int check_tensor(const void* x, const int64_t strides[3], const bsa_3d_params* p, const char* name) {
    if (!x) return set_error(BSA_ERR_BAD_ARG, "%s is null", name);
    BSA_TRY(check_strides(strides, p->D, p->dtype, name));
    if (!aligned16(x)) return set_error(BSA_ERR_BAD_ARG, "%s must be 16-byte aligned", name);
    return BSA_OK;
}
}  // namespace

int bsa_thw_prepare(const bsa_3d_params* p, const void* k, const int64_t k_strides[3], const void* v,
                    const int64_t v_strides[3], void* workspace, size_t workspace_bytes, void* stream) {
    Plan pl;
    Ws w;
    BSA_TRY(make_plan(p, &pl));
    if (!pl.direct_qo) return set_error(BSA_ERR_UNSUPPORTED, "thw_prepare: bf16 and fp16 only (fp32 runs through bsa_fwd_3d)");
    BSA_TRY(carve(pl, workspace, workspace_bytes, "thw_prepare", &w));
    BSA_TRY(check_tensor(k, k_strides, p, "k"));
    BSA_TRY(check_tensor(v, v_strides, p, "v"));
    BSA_TRY(check_kv_views(pl, k_strides, v_strides, "thw_prepare"));
    const int64_t none[3] = {0, 0, p->D};
    const hipError_t e = prepare_thw(pl, p, w, k, none, k, k_strides, v, v_strides, false, (hipStream_t)stream);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "thw_prepare");
}

int bsa_fwd_thw(const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k,
                const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
                const int64_t o_strides[3], const int32_t* idx, const int32_t* lens, int idx_stride, float* lse,
                void* workspace, size_t workspace_bytes, void* stream) {
    Plan pl;
    Ws w;
    BSA_TRY(make_plan(p, &pl));
    if (!pl.direct_qo) return set_error(BSA_ERR_UNSUPPORTED, "fwd_thw: bf16 and fp16 only (fp32 runs through bsa_fwd_3d)");
    BSA_TRY(carve(pl, workspace, workspace_bytes, "fwd_thw", &w));
    BSA_TRY(check_tensor(q, q_strides, p, "q"));
    BSA_TRY(check_tensor(k, k_strides, p, "k"));
    BSA_TRY(check_tensor(v, v_strides, p, "v"));
    BSA_TRY(check_tensor(o, o_strides, p, "o"));
    BSA_TRY(check_kv_views(pl, k_strides, v_strides, "fwd_thw"));
    if (!lens || idx_stride < 0 || (!idx && idx_stride > 0)) return set_error(BSA_ERR_BAD_ARG, "fwd_thw: selection is missing");
    hipError_t e = hipSuccess;
    // p->cdf_threshold > 0 declares lists of unequal length: work items by length, both schedules enqueued
    if (pl.cdf && idx_stride > 0)
        e = launch_order_by_length(lens, w.order, p->B * p->Hn, pl.nbq, pl.gq.chunk() / 64, idx_stride, (hipStream_t)stream);
    if (e == hipSuccess)
        e = attention_thw(pl, p, w, q, q_strides, k, k_strides, v, v_strides, o, o_strides, idx, lens, idx_stride, lse,
                          (hipStream_t)stream, pl.cdf && idx_stride > 0);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "fwd_thw");
}

}  // extern "C"

namespace {
int fwd_3d_impl(const Plan& pl, const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k,
                const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
                const int64_t o_strides[3], void* workspace, size_t workspace_bytes, int32_t* idx_out,
                int32_t* lens_out, void* score_out, void* stream, const bsa_qk_norm* qkn = nullptr, void* q_normed = nullptr,
                const int64_t* qn_strides = nullptr, float* lse_out = nullptr, int32_t* walk_out = nullptr) {
    Ws w;
    if (!q || !k || !v || !o || !workspace) return set_error(BSA_ERR_BAD_ARG, "fwd_3d: null pointer");
    BSA_TRY(carve(pl, workspace, workspace_bytes, "fwd_3d", &w));
    BSA_TRY(check_tensor(q, q_strides, p, "q"));
    BSA_TRY(check_tensor(k, k_strides, p, "k"));
    BSA_TRY(check_tensor(v, v_strides, p, "v"));
    BSA_TRY(check_tensor(o, o_strides, p, "o"));
    BSA_TRY(check_kv_views(pl, k_strides, v_strides, "fwd_3d"));

    const bool padded_k = kv_padded(p);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e;
#define BSA_HIP(call, what) do { e = (call); if (e != hipSuccess) return hip_fail(e, what); } while (0)
    if (qkn != nullptr) {
        // q and k as the projection left them: the pass that takes q's chunk means also normalises and rotates its
        // rows into q_normed (what the attention kernel then reads), the pass that rewrites k in fragment order
        // normalises and rotates on the way
        RowTransform trq = {qkn->q_weight, qkn->rope_table, qkn->t_offset_q, qkn->table_T, qkn->eps, q_normed, qn_strides[0], qn_strides[1], qn_strides[2]};
        RowTransform trk = {qkn->k_weight, qkn->rope_table, qkn->t_offset_k, qkn->table_T, qkn->eps, nullptr, 0, 0, 0};
        BSA_HIP(prepare_thw(pl, p, w, q, q_strides, k, k_strides, v, v_strides, true, st, &trq, &trk), "pool, norm, rotate and prepare");
        q = q_normed;
        q_strides = qn_strides;
    } else if (pl.direct_qo) {
        BSA_HIP(prepare_thw(pl, p, w, q, q_strides, k, k_strides, v, v_strides, true, st), "pool and prepare");
    } else {
        BSA_HIP(launch_permute(q, q_strides, w.qp, w.qc, nullptr, p->B, p->Hn, pl.gq, p->D, p->dtype, st), "permute q");
        BSA_HIP(launch_permute(k, k_strides, w.kp, w.kc, padded_k ? w.valid : nullptr, p->B, p->Hn, pl.gk, p->D, p->dtype, st), "permute k");
        BSA_HIP(launch_permute(v, v_strides, w.vp, nullptr, nullptr, p->B, p->Hn, pl.gk, p->D, p->dtype, st), "permute v");
    }
    BSA_HIP(launch_score(w.qc, w.kc, w.score, p->B * p->Hn, pl.nbq, pl.nbk, p->D, p->dtype, st), "score");
    // the lists the attention kernel walks come out in ascending block order and, for the fragment-order
    // kernel, are then put in its visiting order (L2 locality); the score order is only produced when the
    // caller asks for the selection
    const int64_t sel_rows = (int64_t)p->B * p->Hn * pl.nbq;
    if (pl.cdf) {
        BSA_HIP(launch_cdf_count(w.score, w.lens, sel_rows, pl.nbk, p->cdf_threshold, p->sm_scale, p->k_sel < pl.sel_width ? p->k_sel : pl.sel_width,
                                 pl.sel_width, p->dtype, st), "cdf count");
        BSA_HIP(launch_topk(w.score, idx_out ? w.idx : nullptr, w.idx_sorted, w.lens, sel_rows, pl.nbk, 0, p->dtype, st, w.lens, pl.sel_width), "top-k");
    } else {
        BSA_HIP(launch_topk(w.score, idx_out ? w.idx : nullptr, w.idx_sorted, w.lens, sel_rows, pl.nbk, p->k_sel, p->dtype, st), "top-k");
    }
    if (pl.frag && pl.sel_width > 0)
        BSA_HIP(launch_pace_order(w.idx_sorted, w.idx_sorted, w.lens, sel_rows, pl.nbk, pl.sel_width, st), "visit order");
    if (pl.direct_qo) {
        // lists of unequal length: one launch whose workgroups draw the items, longest lists first
        if (pl.cdf)
            BSA_HIP(launch_order_by_length(w.lens, w.order, p->B * p->Hn, pl.nbq, pl.gq.chunk() / 64, pl.sel_width, st), "order by length");
        BSA_HIP(attention_thw(pl, p, w, q, q_strides, k, k_strides, v, v_strides, o, o_strides, w.idx_sorted, w.lens, pl.sel_width,
                              lse_out, st, pl.cdf), "attention");
    } else {
        BSA_HIP(launch_fwd(w.qp, w.kp, w.vp, w.idx_sorted, w.lens, padded_k ? w.valid : nullptr, w.op, nullptr, p->B, p->Hn, pl.Sqp, pl.Skp,
                           pl.gq.chunk(), pl.gk.chunk(), pl.sel_width, p->sm_scale, p->dtype, st), "attention");
        BSA_HIP(launch_unpermute(w.op, o, o_strides, p->B, p->Hn, pl.gq, p->D, p->dtype, st), "unpermute");
    }
    const size_t bh = (size_t)p->B * p->Hn;
    if (idx_out && pl.sel_width > 0)
        BSA_HIP(hipMemcpyAsync(idx_out, w.idx, bh * pl.nbq * pl.sel_width * sizeof(int32_t), hipMemcpyDeviceToDevice, st), "copy idx");
    if (walk_out && pl.sel_width > 0)
        BSA_HIP(hipMemcpyAsync(walk_out, w.idx_sorted, bh * pl.nbq * pl.sel_width * sizeof(int32_t), hipMemcpyDeviceToDevice, st), "copy walk order");
    if (lens_out) BSA_HIP(hipMemcpyAsync(lens_out, w.lens, bh * pl.nbq * sizeof(int32_t), hipMemcpyDeviceToDevice, st), "copy lens");
    if (score_out) BSA_HIP(hipMemcpyAsync(score_out, w.score, bh * pl.nbq * (size_t)pl.nbk * pl.es, hipMemcpyDeviceToDevice, st), "copy score");
#undef BSA_HIP
    return BSA_OK;
}

// The scratch memory of bsa_fwd_3d_static: what bsa_fwd_3d carves from its caller's workspace, held in the
// code object instead.  Every GPU the library runs on holds its own copy at its own address until the
// process ends.  In host code the name `scratch` is only a handle for hipGetSymbolAddress, never a device
// address: the address is looked up once per device, with that device current, and kept.
constexpr size_t kStaticScratchBytes = BSA_STATIC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
// Per device: an event recorded behind the last call that used the buffer, and the stream of that call.  A call on
// another stream while that event is pending would race on the buffer and is refused.
struct StaticUse {
    std::mutex mu;
    hipEvent_t done = nullptr;
    hipStream_t stream = nullptr;
    bool pending = false;
};
StaticUse g_static_use[kMaxDevices];

int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "fwd_3d_static: hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return set_error(BSA_ERR_UNSUPPORTED, "fwd_3d_static: device %d beyond the %d supported", dev, kMaxDevices);
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        // set-up, once per device: the buffer's address on this device and the event that later calls record
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) return hip_fail(e, "fwd_3d_static: hipGetSymbolAddress(scratch)");
        StaticUse& use = g_static_use[dev];
        std::lock_guard<std::mutex> lock(use.mu);
        if (use.done == nullptr && (e = hipEventCreateWithFlags(&use.done, hipEventDisableTiming)) != hipSuccess) {
            use.done = nullptr;
            return hip_fail(e, "fwd_3d_static: hipEventCreateWithFlags");
        }
        // two threads racing here look up the same address for the same device
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return BSA_OK;
}
}  // namespace

extern "C" {

int bsa_fwd_3d(const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k,
               const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
               const int64_t o_strides[3], void* workspace, size_t workspace_bytes, int32_t* idx_out,
               int32_t* lens_out, void* score_out, void* stream) {
    Plan pl;
    BSA_TRY(make_plan(p, &pl));
    return fwd_3d_impl(pl, p, q, q_strides, k, k_strides, v, v_strides, o, o_strides, workspace, workspace_bytes, idx_out,
                       lens_out, score_out, stream);
}

int bsa_fwd_3d_lse(const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k,
                   const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
                   const int64_t o_strides[3], float* lse_out, int32_t* walk_out, int32_t* lens_out, void* workspace,
                   size_t workspace_bytes, void* stream) {
    Plan pl;
    BSA_TRY(make_plan(p, &pl));
    if (!pl.direct_qo) return set_error(BSA_ERR_UNSUPPORTED, "fwd_3d_lse: bf16 and fp16 only (the backward is built for them)");
    if (!lse_out || !walk_out || !lens_out) return set_error(BSA_ERR_BAD_ARG, "fwd_3d_lse: lse_out, walk_out and lens_out are required");
    return fwd_3d_impl(pl, p, q, q_strides, k, k_strides, v, v_strides, o, o_strides, workspace, workspace_bytes, nullptr,
                       lens_out, nullptr, stream, nullptr, nullptr, nullptr, lse_out, walk_out);
}

int bsa_fwd_3d_qknorm(const bsa_3d_params* p, const bsa_qk_norm* n, const void* q, const int64_t q_strides[3],
                      void* q_normed, const int64_t qn_strides[3], const void* k, const int64_t k_strides[3], const void* v,
                      const int64_t v_strides[3], void* o, const int64_t o_strides[3], void* workspace, size_t workspace_bytes,
                      int32_t* idx_out, int32_t* lens_out, void* score_out, void* stream) {
    Plan pl;
    BSA_TRY(make_plan(p, &pl));
    if (!n || !n->rope_table || !n->q_weight || !n->k_weight || !q_normed || !qn_strides)
        return set_error(BSA_ERR_BAD_ARG, "fwd_3d_qknorm: null pointer");
    if (!(pl.direct_qo && pl.frag && pl.gq.chunk() == 64 && pl.gk.chunk() == 64) || p->tq > 8 || p->hq > 8 || p->wq > 8 ||
        p->tk > 8 || p->hk > 8 || p->wk > 8)
        return set_error(BSA_ERR_UNSUPPORTED, "fwd_3d_qknorm: bf16 / fp16 with 64-token chunks of at most 8 positions per axis only "
                         "(use bsa_qk_norm_rope and bsa_fwd_3d)");
    if (!(n->eps >= 0.f)) return set_error(BSA_ERR_BAD_ARG, "fwd_3d_qknorm: eps must be non-negative");
    if (n->t_offset_q < 0 || n->t_offset_k < 0 || n->table_T < n->t_offset_q + p->Tq || n->table_T < n->t_offset_k + p->Tk)
        return set_error(BSA_ERR_SHAPE, "fwd_3d_qknorm: the frames of q (%d..) or k (%d..) lie outside a table of %d frames",
                         n->t_offset_q, n->t_offset_k, n->table_T);
    if (p->Hq != p->Hk || p->Wq != p->Wk)
        return set_error(BSA_ERR_SHAPE, "fwd_3d_qknorm: q and k share one rotation table, so their H and W must agree");
    if ((reinterpret_cast<uintptr_t>(n->q_weight) | reinterpret_cast<uintptr_t>(n->k_weight)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "fwd_3d_qknorm: norm weights must be 16-byte aligned");
    BSA_TRY(check_tensor(q_normed, qn_strides, p, "q_normed"));
    return fwd_3d_impl(pl, p, q, q_strides, k, k_strides, v, v_strides, o, o_strides, workspace, workspace_bytes, idx_out,
                       lens_out, score_out, stream, n, q_normed, qn_strides);
}

int bsa_fwd_3d_static(const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k,
                      const int64_t k_strides[3], const void* v, const int64_t v_strides[3], void* o,
                      const int64_t o_strides[3], int32_t* idx_out, int32_t* lens_out, void* score_out, void* stream) {
    Plan pl;
    BSA_TRY(make_plan(p, &pl, true));
    if (pl.total > kStaticScratchBytes)
        return set_error(BSA_ERR_WORKSPACE, "fwd_3d_static: this problem needs %zu bytes of scratch memory, the built-in buffer holds %zu; "
                         "use bsa_fwd_3d with a workspace of bsa_workspace_bytes()", pl.total, kStaticScratchBytes);
    void* ws = nullptr;
    BSA_TRY(static_scratch(&ws));
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return set_error(BSA_ERR_HIP, "fwd_3d_static: hipGetDevice");
    StaticUse& use = g_static_use[dev];
    std::lock_guard<std::mutex> lock(use.mu);          // two host threads enqueue one after the other
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing((hipStream_t)stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
    if (!capturing) {
        if (use.pending && use.stream != (hipStream_t)stream) {
            const hipError_t q_state = hipEventQuery(use.done);
            (void)hipGetLastError();                   // "not ready" is an answer, not a failure to be found later
            if (q_state == hipErrorNotReady)
                return set_error(BSA_ERR_BUSY, "fwd_3d_static: the built-in scratch buffer is in use by a call on another stream; "
                                 "wait for it, or use bsa_fwd_3d with a workspace per stream");
        }
    }
    // Nothing in the buffer has to start at zero: every piece is written by the kernel sequence before it is
    // read (the work counter of the queue schedule is cleared by a fill kernel inside launch_fwd).
    const int rc = fwd_3d_impl(pl, p, q, q_strides, k, k_strides, v, v_strides, o, o_strides, ws, kStaticScratchBytes, idx_out,
                               lens_out, score_out, stream);
    if (!capturing && rc == BSA_OK) {
        if (hipEventRecord(use.done, (hipStream_t)stream) == hipSuccess) {
            use.pending = true;
            use.stream = (hipStream_t)stream;
        } else {
            (void)hipGetLastError();
            use.pending = false;
        }
    }
    return rc;
}

// ---- backward of the operator on token-order tensors ------------------------
namespace {
struct Bwd3dPlan {
    Grid3 gq, gk;
    int64_t Sqp, Skp;
    size_t off_qp, off_vp, off_dop, off_qrows, off_krows, off_valid, off_bwd, total;
};
int make_bwd3d_plan(const bsa_3d_params* p, int idx_stride, Bwd3dPlan* pl) {
    if (!p) return set_error(BSA_ERR_BAD_ARG, "params are null");
    BSA_TRY(check_row(p->D, p->dtype));
    BSA_TRY(check_grid(p->B, p->Hn, p->Tq, p->Hq, p->Wq, p->tq, p->hq, p->wq));
    BSA_TRY(check_grid(p->B, p->Hn, p->Tk, p->Hk, p->Wk, p->tk, p->hk, p->wk));
    pl->gq = make_grid(p->Tq, p->Hq, p->Wq, p->tq, p->hq, p->wq);
    pl->gk = make_grid(p->Tk, p->Hk, p->Wk, p->tk, p->hk, p->wk);
    pl->Sqp = (int64_t)pl->gq.blocks() * pl->gq.chunk();
    pl->Skp = (int64_t)pl->gk.blocks() * pl->gk.chunk();
    BSA_TRY(check_bwd_shape(p->B, p->Hn, pl->Sqp, pl->Skp, p->D, pl->gq.chunk(), pl->gk.chunk(), p->dtype));
    if (idx_stride <= 0 || idx_stride > 4096) return set_error(BSA_ERR_BAD_ARG, "bwd_3d: idx_stride=%d outside [1, 4096]", idx_stride);
    if (!(p->sm_scale > 0.f) || !std::isfinite(p->sm_scale)) return set_error(BSA_ERR_BAD_ARG, "bwd_3d: sm_scale must be positive and finite");
    const size_t bh = (size_t)p->B * p->Hn, row = (size_t)p->D * dtype_size(p->dtype);
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up256(bytes); return o; };
    pl->off_qp = take(bh * pl->Sqp * row);
    pl->off_vp = take(bh * pl->Skp * row);
    pl->off_dop = take(bh * pl->Sqp * row);
    pl->off_qrows = take((size_t)pl->Sqp * sizeof(int32_t));
    pl->off_krows = take((size_t)pl->Skp * sizeof(int32_t));
    pl->off_valid = take((size_t)(pl->Skp / 64) * sizeof(uint64_t));
    pl->off_bwd = take(bwd_workspace_bytes(p->B, p->Hn, pl->Sqp, pl->Skp, pl->gq.chunk(), pl->gk.chunk(), idx_stride));
    pl->total = off;
    return BSA_OK;
}
}  // namespace

size_t bsa_bwd_3d_workspace_bytes(const bsa_3d_params* p, int idx_stride) {
    Bwd3dPlan pl;
    if (make_bwd3d_plan(p, idx_stride, &pl) != BSA_OK) return 0;
    return pl.total;
}

int bsa_bwd_3d(const bsa_3d_params* p, const void* q, const int64_t q_strides[3], const void* k, const int64_t k_strides[3],
               const void* v, const int64_t v_strides[3], const void* o, const int64_t o_strides[3], const void* d_o,
               const int64_t do_strides[3], const float* lse, const int32_t* idx, const int32_t* lens, int idx_stride,
               void* dq, const int64_t dq_strides[3], void* dk, const int64_t dk_strides[3], void* dv,
               const int64_t dv_strides[3], void* workspace, size_t workspace_bytes, void* stream) {
    Bwd3dPlan pl;
    BSA_TRY(make_bwd3d_plan(p, idx_stride, &pl));
    if (!lse || !idx || !lens) return set_error(BSA_ERR_BAD_ARG, "bwd_3d: lse, idx or lens is null");
    BSA_TRY(check_tensor(q, q_strides, p, "q"));
    BSA_TRY(check_tensor(k, k_strides, p, "k"));
    BSA_TRY(check_tensor(v, v_strides, p, "v"));
    BSA_TRY(check_tensor(o, o_strides, p, "o"));
    BSA_TRY(check_tensor(d_o, do_strides, p, "d_o"));
    BSA_TRY(check_tensor(dq, dq_strides, p, "dq"));
    BSA_TRY(check_tensor(dk, dk_strides, p, "dk"));
    BSA_TRY(check_tensor(dv, dv_strides, p, "dv"));
    if (!workspace) return set_error(BSA_ERR_BAD_ARG, "bwd_3d: workspace is null");
    if (workspace_bytes < pl.total) return set_error(BSA_ERR_WORKSPACE, "bwd_3d: workspace of %zu bytes, %zu needed", workspace_bytes, pl.total);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return set_error(BSA_ERR_BAD_ARG, "bwd_3d: workspace must be 256-byte aligned");
    char* ws = static_cast<char*>(workspace);
    hipStream_t st = (hipStream_t)stream;
    int32_t* q_rows = reinterpret_cast<int32_t*>(ws + pl.off_qrows);
    int32_t* k_rows = reinterpret_cast<int32_t*>(ws + pl.off_krows);
    uint64_t* valid = reinterpret_cast<uint64_t*>(ws + pl.off_valid);
    // q and v in blocked order (the kernels stream their tiles as they lie in memory); the passes write the row tables
    // of both grids and the validity words of the keys on the way
    hipError_t e = launch_permute(q, q_strides, ws + pl.off_qp, nullptr, nullptr, p->B, p->Hn, pl.gq, p->D, p->dtype, st, false, q_rows);
    if (e != hipSuccess) return hip_fail(e, "bwd_3d: permute q");
    e = launch_permute(v, v_strides, ws + pl.off_vp, nullptr, valid, p->B, p->Hn, pl.gk, p->D, p->dtype, st, false, k_rows);
    if (e != hipSuccess) return hip_fail(e, "bwd_3d: permute v");
    BwdThw t;
    t.q_rows = q_rows;
    t.k_rows = k_rows;
    t.q_tokens = (int64_t)p->Tq * p->Hq * p->Wq;
    t.k_tokens = (int64_t)p->Tk * p->Hk * p->Wk;
    t.o = o; t.dout = d_o; t.lse = lse; t.k = k;
    t.dout_blocked = ws + pl.off_dop;
    t.dq = dq; t.dk = dk; t.dv = dv;
    for (int i = 0; i < 3; ++i) {
        t.o_st[i] = o_strides[i]; t.do_st[i] = do_strides[i]; t.k_st[i] = k_strides[i];
        t.dq_st[i] = dq_strides[i]; t.dk_st[i] = dk_strides[i]; t.dv_st[i] = dv_strides[i];
    }
    e = launch_bwd(ws + pl.off_qp, nullptr, ws + pl.off_vp, nullptr, nullptr, nullptr, idx, lens, kv_padded(p) ? valid : nullptr, nullptr,
                   nullptr, nullptr, p->B, p->Hn, pl.Sqp, pl.Skp, pl.gq.chunk(), pl.gk.chunk(), idx_stride, p->sm_scale, p->dtype,
                   ws + pl.off_bwd, st, &t);
    return e == hipSuccess ? BSA_OK : hip_fail(e, "bwd_3d launch");
}

}  // extern "C"
