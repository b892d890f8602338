// Glue of the attention module around the block-sparse operator: row RMSNorm,
// fused per-head QK RMSNorm + 3-D RoPE, and bf16 linear layers (hipBLASLt,
// a plain library GEMM with bias / residual epilogue).
#include "bsa_common.h"

#include <hipblaslt/hipblaslt.h>

#include <mutex>

namespace bsa {
namespace {

// ------------------------------------------------------------- row RMSNorm
// out = bf16(x * rsqrt(mean(x^2) + eps)) * w, one wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                           T* __restrict__ out, int64_t rows, int dim, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * dim;
    T* orow = out + row * dim;
    float ss = 0.f;
    for (int d = lane * 8; d < dim; d += 512) {
        const uint4 raw = *reinterpret_cast<const uint4*>(xr + d);
        const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int i = 0; i < 8; ++i) { const float f = (float)e[i]; ss = fmaf(f, f, ss); }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float r = rsqrtf(ss / (float)dim + eps);
    for (int d = lane * 8; d < dim; d += 512) {
        const uint4 raw = *reinterpret_cast<const uint4*>(xr + d);
        const uint4 wraw = *reinterpret_cast<const uint4*>(w + d);
        const T* e = reinterpret_cast<const T*>(&raw);
        const T* we = reinterpret_cast<const T*>(&wraw);
        T res[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) res[i] = (T)((float)(T)((float)e[i] * r) * (float)we[i]);
        *reinterpret_cast<uint4*>(orow + d) = *reinterpret_cast<const uint4*>(res);
    }
}

// ------------------------------------------------- per-head QK RMSNorm + RoPE
// One row = one (token, head) vector of D = 128 elements, handled by 16 lanes
// (8 elements each, i.e. 4 interleaved rotation pairs per lane).
// x -> bf16(x * rsqrt(mean(x^2)+eps)) -> bf16(. * w) -> fp32 x*cos + rot(x)*sin -> bf16
// with rot(x)[2i] = -x[2i+1], rot(x)[2i+1] = x[2i]; the d axis is split
// (t: D - 4*(D/6), h: 2*(D/6), w: 2*(D/6)) and pair i of an axis turns by pos * freq_i.
// tab holds cos_t[T][nt], sin_t[T][nt], cos_h[H][nh], sin_h[H][nh], cos_w[W][nw], sin_w[W][nw] (fp32).
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(T* __restrict__ q, int64_t qsB, int64_t qsH, int64_t qsS,
                                                           T* __restrict__ k, int64_t ksB, int64_t ksH, int64_t ksS,
                                                           const T* __restrict__ qw, const T* __restrict__ kw,
                                                           const float* __restrict__ tab, int B, int Hn, int Tn,
                                                           int Hg, int Wg, float eps) {
    constexpr int D = 128;
    constexpr int nt = (D - 4 * (D / 6)) / 2, nh = (D / 6), nw = (D / 6);   // pairs per axis: 22, 21, 21
    const int sub = threadIdx.x & 15;
    const int64_t S = (int64_t)Tn * Hg * Wg;
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);      // over B*Hn*S rows, and q then k
    const int64_t nrows = (int64_t)B * Hn * S;
    if (row >= 2 * nrows) return;
    const bool is_k = row >= nrows;
    const int64_t r = is_k ? row - nrows : row;
    const int64_t s = r % S;
    const int hd = (int)((r / S) % Hn), b = (int)(r / (S * Hn));
    T* p = is_k ? k + b * ksB + hd * ksH + s * ksS : q + b * qsB + hd * qsH + s * qsS;
    const T* wv = is_k ? kw : qw;
    const int wi = (int)(s % Wg), hi = (int)((s / Wg) % Hg), ti = (int)(s / ((int64_t)Wg * Hg));

    const uint4 raw = *reinterpret_cast<const uint4*>(p + sub * 8);
    const uint4 wraw = *reinterpret_cast<const uint4*>(wv + sub * 8);
    const T* e = reinterpret_cast<const T*>(&raw);
    const T* we = reinterpret_cast<const T*>(&wraw);
    float f[8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) { f[i] = (float)e[i]; ss = fmaf(f[i], f[i], ss); }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float rs = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)(T)((float)(T)(f[i] * rs) * (float)we[i]);

    const float* cos_t = tab;                 const float* sin_t = cos_t + (int64_t)Tn * nt;
    const float* cos_h = sin_t + (int64_t)Tn * nt; const float* sin_h = cos_h + (int64_t)Hg * nh;
    const float* cos_w = sin_h + (int64_t)Hg * nh; const float* sin_w = cos_w + (int64_t)Wg * nw;
    T res[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int pair = sub * 4 + j;          // 0..63
        float c, sn;
        if (pair < nt) { c = cos_t[ti * nt + pair]; sn = sin_t[ti * nt + pair]; }
        else if (pair < nt + nh) { c = cos_h[hi * nh + pair - nt]; sn = sin_h[hi * nh + pair - nt]; }
        else { c = cos_w[wi * nw + pair - nt - nh]; sn = sin_w[wi * nw + pair - nt - nh]; }
        const float x0 = f[2 * j], x1 = f[2 * j + 1];
        // two products, then one add, each rounded: the order of operations of the eager expression
        res[2 * j] = (T)__fadd_rn(__fmul_rn(x0, c), __fmul_rn(-x1, sn));
        res[2 * j + 1] = (T)__fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, sn));
    }
    *reinterpret_cast<uint4*>(p + sub * 8) = *reinterpret_cast<const uint4*>(res);
}

// ------------------------------------------------------------- linear (GEMM)
struct LtState {
    std::mutex mu;
    hipblasLtHandle_t handle = nullptr;
};
LtState& lt_state() { static LtState s; return s; }

}  // namespace
}  // namespace bsa

using namespace bsa;

extern "C" {

int bsa_rmsnorm(const void* x, const void* weight, void* out, int64_t rows, int dim, float eps, int dtype, void* stream) {
    if (!x || !weight || !out) return set_error(BSA_ERR_BAD_ARG, "rmsnorm: null pointer");
    if (rows <= 0 || dim <= 0 || dim % 8 != 0) return set_error(BSA_ERR_BAD_ARG, "rmsnorm: rows=%lld dim=%d (dim must be a positive multiple of 8)", (long long)rows, dim);
    if (!(eps >= 0.f)) return set_error(BSA_ERR_BAD_ARG, "rmsnorm: eps must be non-negative");
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "rmsnorm: pointers must be 16-byte aligned");
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((rmsnorm_rows_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (const __bf16*)x, (const __bf16*)weight, (__bf16*)out, rows, dim, eps);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((rmsnorm_rows_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (const _Float16*)x, (const _Float16*)weight, (_Float16*)out, rows, dim, eps);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "rmsnorm: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "rmsnorm launch: %s", hipGetErrorString(e));
}

int bsa_qk_norm_rope(void* q, const int64_t q_strides[3], void* k, const int64_t k_strides[3], const void* q_weight,
                     const void* k_weight, const float* rope_table, int B, int Hn, int T, int H, int W, int D,
                     float eps, int dtype, void* stream) {
    if (!q || !k || !q_weight || !k_weight || !rope_table || !q_strides || !k_strides)
        return set_error(BSA_ERR_BAD_ARG, "qk_norm_rope: null pointer");
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "qk_norm_rope: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || T <= 0 || H <= 0 || W <= 0) return set_error(BSA_ERR_BAD_ARG, "qk_norm_rope: sizes must be positive");
    for (int i = 0; i < 3; ++i)
        if (q_strides[i] < 0 || k_strides[i] < 0 || (q_strides[i] * 2) % 16 || (k_strides[i] * 2) % 16)
            return set_error(BSA_ERR_BAD_ARG, "qk_norm_rope: strides must keep rows 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(q_weight) |
         reinterpret_cast<uintptr_t>(k_weight)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "qk_norm_rope: pointers must be 16-byte aligned");
    const int64_t rows = 2 * (int64_t)B * Hn * T * H * W;
    if ((rows + 15) / 16 > 0x7fffffffLL) return set_error(BSA_ERR_UNSUPPORTED, "qk_norm_rope: too many rows");
    const dim3 grid((unsigned)((rows + 15) / 16)), block(256);
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((qk_norm_rope_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (__bf16*)q, q_strides[0], q_strides[1], q_strides[2],
                           (__bf16*)k, k_strides[0], k_strides[1], k_strides[2], (const __bf16*)q_weight, (const __bf16*)k_weight, rope_table, B, Hn, T, H, W, eps);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((qk_norm_rope_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (_Float16*)q, q_strides[0], q_strides[1], q_strides[2],
                           (_Float16*)k, k_strides[0], k_strides[1], k_strides[2], (const _Float16*)q_weight, (const _Float16*)k_weight, rope_table, B, Hn, T, H, W, eps);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "qk_norm_rope: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "qk_norm_rope launch: %s", hipGetErrorString(e));
}

int bsa_linear_bf16(const void* x, const void* w, const void* bias, const void* residual, void* out, int64_t M, int N,
                    int K, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !w || !out) return set_error(BSA_ERR_BAD_ARG, "linear: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return set_error(BSA_ERR_BAD_ARG, "linear: sizes must be positive");
    // hipBLASLt has been seen to write through the workspace pointer for large problems even when it was
    // told that there is none, so a workspace is mandatory
    if (!workspace || workspace_bytes < ((size_t)32 << 20))
        return set_error(BSA_ERR_WORKSPACE, "linear: a workspace of at least 32 MiB is required (got %zu bytes)", workspace_bytes);
    LtState& st = lt_state();
    std::lock_guard<std::mutex> lock(st.mu);
    if (!st.handle && hipblasLtCreate(&st.handle) != HIPBLAS_STATUS_SUCCESS)
        return set_error(BSA_ERR_HIP, "linear: hipblasLtCreate failed");
#define BSA_LT(call)                                                                        \
    do {                                                                                    \
        const hipblasStatus_t s_ = (call);                                                  \
        if (s_ != HIPBLAS_STATUS_SUCCESS) { rc = set_error(BSA_ERR_HIP, "linear: %s failed with status %d", #call, (int)s_); goto done; } \
    } while (0)
    int rc = BSA_OK;
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    {
        // row-major out[M,N] = x[M,K] . w[N,K]^T  ==  column-major out'(N x M) = w'(K x N)^T . x'(K x M)
        const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
        const float alpha = 1.f, beta = residual ? 1.f : 0.f;
        BSA_LT(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        BSA_LT(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
        BSA_LT(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
        if (bias) {
            const hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_BIAS;
            const int32_t bt = HIP_R_16BF;
            BSA_LT(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)));
            BSA_LT(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
            BSA_LT(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)));
        }
        BSA_LT(hipblasLtMatrixLayoutCreate(&la, HIP_R_16BF, K, N, K));
        BSA_LT(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16BF, K, M, K));
        BSA_LT(hipblasLtMatrixLayoutCreate(&lc, HIP_R_16BF, N, M, N));
        BSA_LT(hipblasLtMatmulPreferenceCreate(&pref));
        const uint64_t wsb = workspace_bytes;
        BSA_LT(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &wsb, sizeof(wsb)));
        hipblasLtMatmulHeuristicResult_t heur[8];
        int found = 0, pick = -1;
        BSA_LT(hipblasLtMatmulAlgoGetHeuristic(st.handle, desc, la, lb, lc, lc, pref, 8, heur, &found));
        // never hand the library less workspace than the algorithm says it uses
        for (int i = 0; i < found && pick < 0; ++i)
            if (heur[i].state == HIPBLAS_STATUS_SUCCESS && heur[i].workspaceSize <= workspace_bytes) pick = i;
        if (pick < 0) { rc = set_error(BSA_ERR_UNSUPPORTED, "linear: no GEMM algorithm for M=%lld N=%d K=%d within %zu bytes of workspace", (long long)M, N, K, workspace_bytes); goto done; }
        BSA_LT(hipblasLtMatmul(st.handle, desc, &alpha, w, la, x, lb, &beta, residual ? residual : out, lc, out, lc,
                               &heur[pick].algo, workspace, workspace_bytes, (hipStream_t)stream));
    }
done:
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (la) hipblasLtMatrixLayoutDestroy(la);
    if (lb) hipblasLtMatrixLayoutDestroy(lb);
    if (lc) hipblasLtMatrixLayoutDestroy(lc);
    if (desc) hipblasLtMatmulDescDestroy(desc);
#undef BSA_LT
    return rc;
}

}  // extern "C"
