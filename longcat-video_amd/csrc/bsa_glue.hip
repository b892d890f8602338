// Glue of the attention module around the block-sparse operator: row RMSNorm,
// fused per-head QK RMSNorm + 3-D RoPE, and bf16 linear layers (hipBLASLt,
// a plain library GEMM with bias / residual epilogue).
#include "bsa_common.h"
#include "bsa_rope.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <shared_mutex>
#include <tuple>
#include <vector>

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

// --------------------------------------- LayerNorm (no affine) + adaLN modulate
// out = T(((x - mean) * rsqrt(var + eps)) * (scale + 1) + shift), everything in fp32 with one rounding at
// the end; mean and the biased variance over the row (two passes over registers).  shift / scale are fp32
// rows shared by `rows_per_group` consecutive rows (one latent frame).  One wavefront per row, dim <= 8192.
template <typename T>
__global__ __launch_bounds__(256) void layernorm_modulate_kernel(const T* __restrict__ x, const float* __restrict__ shift,
                                                                 const float* __restrict__ scale, T* __restrict__ out,
                                                                 int64_t rows, int rows_per_group, int dim, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * dim;
    const float* sh = shift + (row / rows_per_group) * dim;
    const float* sc = scale + (row / rows_per_group) * dim;
    uint4 raw[16];                     // the row stays in registers in its storage type
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int d = j * 512 + lane * 8;
        if (d < dim) {
            raw[j] = *reinterpret_cast<const uint4*>(xr + d);
            const T* e = reinterpret_cast<const T*>(&raw[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += (float)e[i];
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    const float mean = sum / (float)dim;
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j)
        if (j * 512 + lane * 8 < dim) {
            const T* e = reinterpret_cast<const T*>(&raw[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) { const float c = (float)e[i] - mean; sq = fmaf(c, c, sq); }
        }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
    const float rstd = rsqrtf(sq / (float)dim + eps);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int d = j * 512 + lane * 8;
        if (d < dim) {
            const float4 s0 = *reinterpret_cast<const float4*>(sc + d), s1 = *reinterpret_cast<const float4*>(sc + d + 4);
            const float4 h0 = *reinterpret_cast<const float4*>(sh + d), h1 = *reinterpret_cast<const float4*>(sh + d + 4);
            const float scl[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
            const float sft[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
            const T* e = reinterpret_cast<const T*>(&raw[j]);
            T res[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float n = __fmul_rn((float)e[i] - mean, rstd);
                res[i] = (T)__fadd_rn(__fmul_rn(n, __fadd_rn(scl[i], 1.0f)), sft[i]);     // x * (scale + 1) + shift
            }
            *reinterpret_cast<uint4*>(out + row * dim + d) = *reinterpret_cast<const uint4*>(res);
        }
    }
}

// out = T(float(x) + gate * float(y)), gate fp32 per group of rows (one latent frame).
template <typename T>
__global__ __launch_bounds__(256) void gated_residual_kernel(const T* __restrict__ x, const T* __restrict__ y,
                                                             const float* __restrict__ gate, T* __restrict__ out,
                                                             int64_t rows, int rows_per_group, int dim) {
    // the launch is limited to 2^31 threads: 32-bit divisions (64-bit ones cost more than the 48 bytes moved)
    const uint32_t per_row = (uint32_t)dim / 8;
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= (uint64_t)rows * per_row) return;
    const uint32_t row_u = i / per_row;
    const int64_t row = row_u;
    const int d = (int)(i - row_u * per_row) * 8;
    const uint4 xr = *reinterpret_cast<const uint4*>(x + row * dim + d);
    const uint4 yr = *reinterpret_cast<const uint4*>(y + row * dim + d);
    const float* g = gate + (int64_t)(row_u / (uint32_t)rows_per_group) * dim + d;
    const float4 g0 = *reinterpret_cast<const float4*>(g), g1 = *reinterpret_cast<const float4*>(g + 4);
    const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
    const T* xe = reinterpret_cast<const T*>(&xr);
    const T* ye = reinterpret_cast<const T*>(&yr);
    T res[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) res[k] = (T)__fadd_rn((float)xe[k], __fmul_rn(gv[k], (float)ye[k]));
    *reinterpret_cast<uint4*>(out + row * dim + d) = *reinterpret_cast<const uint4*>(res);
}

// ------------------------------------------------- LoRA side branches
// out = T(org + total) with total = s_0, then T(total + s_i), and s_i = T(T(up_i * multiplier_i) * alpha_i):
// every product and sum of the eager expression is rounded to the tensor dtype, one by one.
constexpr int kMaxLoras = 4;
struct LoraTerms {
    const void* up[kMaxLoras];
    float multiplier[kMaxLoras];
    float alpha[kMaxLoras];
    int n;
};

template <typename T>
__global__ __launch_bounds__(256) void lora_add_kernel(const T* __restrict__ org, LoraTerms terms, T* __restrict__ out,
                                                       int64_t n8) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const uint4 raw = reinterpret_cast<const uint4*>(org)[i];
    const T* oe = reinterpret_cast<const T*>(&raw);
    T total[8];
    for (int j = 0; j < terms.n; ++j) {
        const uint4 ur = reinterpret_cast<const uint4*>(terms.up[j])[i];
        const T* ue = reinterpret_cast<const T*>(&ur);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const T scaled = (T)__fmul_rn((float)(T)__fmul_rn((float)ue[k], terms.multiplier[j]), terms.alpha[j]);
            total[k] = j == 0 ? scaled : (T)__fadd_rn((float)total[k], (float)scaled);
        }
    }
    T res[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) res[k] = (T)__fadd_rn((float)oe[k], (float)total[k]);
    reinterpret_cast<uint4*>(out)[i] = *reinterpret_cast<const uint4*>(res);
}

// ------------------------------------------------- per-head RMSNorm + RoPE
// One row = one (token, head) vector of D = 128 elements, handled by 16 lanes
// (8 elements each, i.e. 4 interleaved rotation pairs per lane).
// x -> bf16(x * rsqrt(mean(x^2)+eps)) -> bf16(. * w) -> fp32 x*cos + rot(x)*sin -> bf16
// with rot(x)[2i] = -x[2i+1], rot(x)[2i+1] = x[2i]; the d axis is split
// (t: D - 4*(D/6), h: 2*(D/6), w: 2*(D/6)) and pair i of an axis turns by pos * freq_i.
// tab holds cos_t[Ttab][nt], sin_t[Ttab][nt], cos_h[H][nh], sin_h[H][nh], cos_w[W][nw], sin_w[W][nw]
// (fp32); the token at grid position (ti, hi, wi) uses row t0 + ti of the t tables.
// Either step can be left out (w == nullptr: no norm; tab == nullptr: no rotation), and the result
// may go to another tensor with other strides, so the same pass also moves q, k, v from the
// token-major layout of the QKV projection into per-head contiguous tensors.
// head_fastest: consecutive rows walk the heads of one token (the order in which a token-major
// source lies in memory); otherwise the tokens of one head.
template <typename T>
__global__ __launch_bounds__(256) void norm_rope_kernel(const T* __restrict__ src, int64_t sB, int64_t sH, int64_t sS,
                                                        T* __restrict__ dst, int64_t dB, int64_t dH, int64_t dS,
                                                        const T* __restrict__ w, const float* __restrict__ tab, int B,
                                                        int Hn, int Tn, int Hg, int Wg, int t0, int Ttab, float eps,
                                                        int head_fastest) {
    constexpr int D = 128;
    constexpr int nt = (D - 4 * (D / 6)) / 2, nh = (D / 6), nw = (D / 6);   // pairs per axis: 22, 21, 21
    const int sub = threadIdx.x & 15;
    // row counts fit 31 bits (checked by the caller): 32-bit divisions, the 64-bit ones cost more than the move
    const uint32_t S = (uint32_t)Tn * Hg * Wg;
    const uint32_t rows = (uint32_t)B * Hn * S;
    // Four rows in flight per 16-lane group.  When the heads of a token lie next to each other in the
    // source (and their count is a multiple of four) the four rows are four heads of one token: they
    // share the token's position and rotation angles, which are then worked out once.
    constexpr int R = 4;
    const bool share = head_fastest && (Hn % R) == 0;
    const uint32_t group = blockIdx.x * 16u + (threadIdx.x >> 4);
    uint32_t s_of[R];
    T* o_of[R];
    uint4 raw_of[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint32_t row = share ? group * R + j : blockIdx.x * (16u * R) + (threadIdx.x >> 4) + 16u * j;
        if (row >= rows) { o_of[j] = nullptr; s_of[j] = 0; continue; }
        uint32_t s, hd, b;
        if (head_fastest) { const uint32_t t = row / Hn; hd = row - t * Hn; b = t / S; s = t - b * S; }
        else { const uint32_t t = row / S; s = row - t * S; b = t / Hn; hd = t - b * Hn; }
        s_of[j] = s;
        o_of[j] = dst + b * dB + hd * dH + s * dS;
        raw_of[j] = *reinterpret_cast<const uint4*>(src + b * sB + hd * sH + s * sS + sub * 8);
    }
    uint4 wraw = make_uint4(0, 0, 0, 0);
    if (w != nullptr) wraw = *reinterpret_cast<const uint4*>(w + sub * 8);
    // cos / sin of this lane's four rotation pairs at token s
    auto angles = [&](uint32_t s, float (&c)[4], float (&sn)[4]) {
        const uint32_t u = s / (uint32_t)Wg, v = u / (uint32_t)Hg;
        rope_angles(tab, Ttab, Hg, Wg, t0 + (int)v, (int)(u - v * Hg), (int)(s - u * Wg), sub, c, sn);
    };
    float c[4] = {1.f, 1.f, 1.f, 1.f}, sn[4] = {0.f, 0.f, 0.f, 0.f};
    if (tab != nullptr && share) angles(s_of[0], c, sn);      // row 0 of a group exists whenever any does
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (o_of[j] == nullptr) continue;
        T* o = o_of[j];
        if (w == nullptr && tab == nullptr) {                 // plain move
            *reinterpret_cast<uint4*>(o + sub * 8) = raw_of[j];
            continue;
        }
        if (tab != nullptr && !share) angles(s_of[j], c, sn);
        *reinterpret_cast<uint4*>(o + sub * 8) = norm_rope_piece<T>(raw_of[j], wraw, w != nullptr, tab != nullptr, c, sn, eps);
    }
}

// ------------------------------------------------------------- linear (GEMM)
// Shape of a linear call on a device -> the algorithm it runs with: the one bsa_linear_bf16_tune measured to be
// the fastest, else hipBLASLt's first proposal that fits the workspace (asked for once per shape, not per call).
struct LinearKey {
    int64_t M, ldx, ldw, ldo;
    int N, K, bias, residual, device;
    bool operator<(const LinearKey& o) const {
        return std::tie(M, ldx, ldw, ldo, N, K, bias, residual, device) <
               std::tie(o.M, o.ldx, o.ldw, o.ldo, o.N, o.K, o.bias, o.residual, o.device);
    }
};
struct TunedAlgo {
    hipblasLtMatmulAlgo_t algo;
    size_t workspace;
};
// Calls from several threads do not serialise: every thread has its own hipBLASLt handle per device, and the
// table of chosen algorithms is read under a shared lock (written once per shape, and by the tuning call).
struct LtState {
    std::shared_mutex mu;
    std::map<LinearKey, TunedAlgo> chosen;
};
LtState& lt_state() { static LtState s; return s; }
constexpr int kMaxLtDevices = 64;
// A thread's handles go back to a per-device pool when the thread ends and are taken from there by the next thread
// that needs one, so the number of handles ever created is bounded by the number of threads alive at one time, not
// by the number of threads that ever called.  Nothing is destroyed: a thread may end while the HIP runtime is
// being torn down, and the pool itself is never freed for the same reason.
struct HandlePool {
    std::mutex mu;
    std::vector<hipblasLtHandle_t> idle[kMaxLtDevices];
};
HandlePool& handle_pool() { static HandlePool* p = new HandlePool; return *p; }
struct ThreadHandles {
    hipblasLtHandle_t h[kMaxLtDevices] = {};
    ~ThreadHandles() {
        HandlePool& pool = handle_pool();
        std::lock_guard<std::mutex> lock(pool.mu);
        for (int d = 0; d < kMaxLtDevices; ++d)
            if (h[d]) pool.idle[d].push_back(h[d]);
    }
};
hipblasLtHandle_t thread_handle(int device) {
    thread_local ThreadHandles mine;
    if (device < 0 || device >= kMaxLtDevices) return nullptr;
    if (!mine.h[device]) {
        HandlePool& pool = handle_pool();
        {
            std::lock_guard<std::mutex> lock(pool.mu);
            if (!pool.idle[device].empty()) {
                mine.h[device] = pool.idle[device].back();
                pool.idle[device].pop_back();
            }
        }
        if (!mine.h[device] && hipblasLtCreate(&mine.h[device]) != HIPBLAS_STATUS_SUCCESS) mine.h[device] = nullptr;
    }
    return mine.h[device];
}

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

int bsa_layernorm_modulate(const void* x, const float* shift, const float* scale, void* out, int64_t rows,
                           int rows_per_group, int dim, float eps, int dtype, void* stream) {
    if (!x || !shift || !scale || !out) return set_error(BSA_ERR_BAD_ARG, "layernorm_modulate: null pointer");
    if (rows <= 0 || rows_per_group <= 0 || rows % rows_per_group != 0)
        return set_error(BSA_ERR_SHAPE, "layernorm_modulate: %lld rows do not split into groups of %d", (long long)rows, rows_per_group);
    if (dim <= 0 || dim % 8 != 0 || dim > 8192) return set_error(BSA_ERR_UNSUPPORTED, "layernorm_modulate: dim %d (multiples of 8 up to 8192)", dim);
    if (!(eps >= 0.f)) return set_error(BSA_ERR_BAD_ARG, "layernorm_modulate: eps must be non-negative");
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(shift) | reinterpret_cast<uintptr_t>(scale) | reinterpret_cast<uintptr_t>(out)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "layernorm_modulate: pointers must be 16-byte aligned");
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((layernorm_modulate_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (const __bf16*)x, shift, scale, (__bf16*)out, rows, rows_per_group, dim, eps);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((layernorm_modulate_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (const _Float16*)x, shift, scale, (_Float16*)out, rows, rows_per_group, dim, eps);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "layernorm_modulate: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "layernorm_modulate launch: %s", hipGetErrorString(e));
}

int bsa_gated_residual(const void* x, const void* y, const float* gate, void* out, int64_t rows, int rows_per_group,
                       int dim, int dtype, void* stream) {
    if (!x || !y || !gate || !out) return set_error(BSA_ERR_BAD_ARG, "gated_residual: null pointer");
    if (rows <= 0 || rows_per_group <= 0 || rows % rows_per_group != 0)
        return set_error(BSA_ERR_SHAPE, "gated_residual: %lld rows do not split into groups of %d", (long long)rows, rows_per_group);
    if (dim <= 0 || dim % 8 != 0) return set_error(BSA_ERR_UNSUPPORTED, "gated_residual: dim %d must be a multiple of 8", dim);
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(out)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "gated_residual: pointers must be 16-byte aligned");
    const int64_t n = rows * (dim / 8);
    if (n > 0x7fffffffLL) return set_error(BSA_ERR_UNSUPPORTED, "gated_residual: too many elements (32-bit thread indices)");
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((gated_residual_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (const __bf16*)x, (const __bf16*)y, gate, (__bf16*)out, rows, rows_per_group, dim);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((gated_residual_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (const _Float16*)x, (const _Float16*)y, gate, (_Float16*)out, rows, rows_per_group, dim);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "gated_residual: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "gated_residual launch: %s", hipGetErrorString(e));
}

int bsa_lora_add(const void* org, const void* const* up, const float* multiplier, const float* alpha_scale, int n_loras,
                 void* out, int64_t n, int dtype, void* stream) {
    if (!org || !up || !multiplier || !alpha_scale || !out) return set_error(BSA_ERR_BAD_ARG, "lora_add: null pointer");
    if (n_loras < 1 || n_loras > kMaxLoras) return set_error(BSA_ERR_UNSUPPORTED, "lora_add: %d side branches (1..%d are built)", n_loras, kMaxLoras);
    if (n <= 0 || n % 8) return set_error(BSA_ERR_BAD_ARG, "lora_add: the element count must be a positive multiple of 8");
    LoraTerms terms{};
    terms.n = n_loras;
    uintptr_t bits = reinterpret_cast<uintptr_t>(org) | reinterpret_cast<uintptr_t>(out);
    for (int j = 0; j < n_loras; ++j) {
        if (!up[j]) return set_error(BSA_ERR_BAD_ARG, "lora_add: null pointer");
        terms.up[j] = up[j];
        terms.multiplier[j] = multiplier[j];
        terms.alpha[j] = alpha_scale[j];
        bits |= reinterpret_cast<uintptr_t>(up[j]);
    }
    if (bits & 15u) return set_error(BSA_ERR_BAD_ARG, "lora_add: pointers must be 16-byte aligned");
    const int64_t n8 = n / 8;
    if ((n8 + 255) / 256 > 0x7fffffffLL) return set_error(BSA_ERR_UNSUPPORTED, "lora_add: too many elements");
    const dim3 grid((unsigned)((n8 + 255) / 256)), block(256);
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((lora_add_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (const __bf16*)org, terms, (__bf16*)out, n8);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((lora_add_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (const _Float16*)org, terms, (_Float16*)out, n8);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "lora_add: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "lora_add launch: %s", hipGetErrorString(e));
}

int bsa_norm_rope(const void* src, const int64_t src_strides[3], void* dst, const int64_t dst_strides[3],
                  const void* weight, const float* rope_table, int B, int Hn, int T, int H, int W, int t_offset,
                  int table_T, int D, float eps, int dtype, void* stream) {
    if (!src || !dst || !src_strides || !dst_strides) return set_error(BSA_ERR_BAD_ARG, "norm_rope: null pointer");
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "norm_rope: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || T <= 0 || H <= 0 || W <= 0) return set_error(BSA_ERR_BAD_ARG, "norm_rope: sizes must be positive");
    if (rope_table && (t_offset < 0 || table_T < t_offset + T))
        return set_error(BSA_ERR_SHAPE, "norm_rope: frames %d..%d lie outside a table of %d frames", t_offset, t_offset + T, table_T);
    for (int i = 0; i < 3; ++i)
        if (src_strides[i] < 0 || dst_strides[i] < 0 || (src_strides[i] * 2) % 16 || (dst_strides[i] * 2) % 16)
            return set_error(BSA_ERR_BAD_ARG, "norm_rope: strides must keep rows 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(weight)) & 15u)
        return set_error(BSA_ERR_BAD_ARG, "norm_rope: pointers must be 16-byte aligned");
    if (!(eps >= 0.f)) return set_error(BSA_ERR_BAD_ARG, "norm_rope: eps must be non-negative");
    const int64_t rows = (int64_t)B * Hn * T * H * W;
    if (rows > 0x7fffffffLL) return set_error(BSA_ERR_UNSUPPORTED, "norm_rope: too many rows (32-bit row indices)");
    const dim3 grid((unsigned)((rows + 63) / 64)), block(256);       // 16 lane groups x 4 rows each
    const int head_fastest = src_strides[1] < src_strides[2] ? 1 : 0;
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((norm_rope_kernel<__bf16>), grid, block, 0, (hipStream_t)stream, (const __bf16*)src, src_strides[0],
                           src_strides[1], src_strides[2], (__bf16*)dst, dst_strides[0], dst_strides[1], dst_strides[2],
                           (const __bf16*)weight, rope_table, B, Hn, T, H, W, t_offset, table_T, eps, head_fastest);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((norm_rope_kernel<_Float16>), grid, block, 0, (hipStream_t)stream, (const _Float16*)src, src_strides[0],
                           src_strides[1], src_strides[2], (_Float16*)dst, dst_strides[0], dst_strides[1], dst_strides[2],
                           (const _Float16*)weight, rope_table, B, Hn, T, H, W, t_offset, table_T, eps, head_fastest);
    else
        return set_error(BSA_ERR_UNSUPPORTED, "norm_rope: dtype %d is not built (bf16, fp16)", dtype);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "norm_rope launch: %s", hipGetErrorString(e));
}

int bsa_qk_norm_rope(void* q, const int64_t q_strides[3], void* k, const int64_t k_strides[3], const void* q_weight,
                     const void* k_weight, const float* rope_table, int B, int Hn, int T, int H, int W, int D,
                     float eps, int dtype, void* stream) {
    if (!q || !k || !q_weight || !k_weight || !rope_table || !q_strides || !k_strides)
        return set_error(BSA_ERR_BAD_ARG, "qk_norm_rope: null pointer");
    const int rc = bsa_norm_rope(q, q_strides, q, q_strides, q_weight, rope_table, B, Hn, T, H, W, 0, T, D, eps, dtype, stream);
    if (rc != BSA_OK) return rc;
    return bsa_norm_rope(k, k_strides, k, k_strides, k_weight, rope_table, B, Hn, T, H, W, 0, T, D, eps, dtype, stream);
}

int bsa_linear_bf16(const void* x, const void* w, const void* bias, const void* residual, void* out, int64_t M, int N,
                    int K, void* workspace, size_t workspace_bytes, void* stream) {
    return bsa_linear_bf16_ld(x, K, w, K, bias, residual, out, N, M, N, K, workspace, workspace_bytes, stream);
}

static int linear_impl(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                       void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                       void* stream, bool tune, float* default_ms, float* best_ms);

int bsa_linear_bf16_ld(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                       void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                       void* stream) {
    return linear_impl(x, ldx, w, ldw, bias, residual, out, ldo, M, N, K, workspace, workspace_bytes, stream, false, nullptr, nullptr);
}

int bsa_linear_bf16_tune(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                         void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                         void* stream, float* default_ms, float* best_ms) {
    return linear_impl(x, ldx, w, ldw, bias, residual, out, ldo, M, N, K, workspace, workspace_bytes, stream, true, default_ms, best_ms);
}

static int linear_impl(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                       void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                       void* stream, bool tune, float* default_ms, float* best_ms) {
    if (!x || !w || !out) return set_error(BSA_ERR_BAD_ARG, "linear: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return set_error(BSA_ERR_BAD_ARG, "linear: sizes must be positive");
    if (ldx < K || ldw < K || ldo < N) return set_error(BSA_ERR_BAD_ARG, "linear: a row stride is shorter than its row");
    // hipBLASLt has been seen to write through the workspace pointer for large problems even when it was
    // told that there is none, so a workspace is mandatory.  Its best algorithms for the 720p projections
    // want just under 64 MiB (1.52 PFLOP/s instead of 1.24 with 32 MiB); more brings nothing.
    if (!workspace || workspace_bytes < ((size_t)64 << 20))
        return set_error(BSA_ERR_WORKSPACE, "linear: a workspace of at least 64 MiB is required (got %zu bytes)", workspace_bytes);
    LtState& st = lt_state();
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return set_error(BSA_ERR_HIP, "linear: hipGetDevice failed");
    const hipblasLtHandle_t handle = thread_handle(device);
    if (!handle) return set_error(BSA_ERR_HIP, "linear: hipblasLtCreate failed");
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
        BSA_LT(hipblasLtMatrixLayoutCreate(&la, HIP_R_16BF, K, N, ldw));
        BSA_LT(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16BF, K, M, ldx));
        BSA_LT(hipblasLtMatrixLayoutCreate(&lc, HIP_R_16BF, N, M, ldo));
        BSA_LT(hipblasLtMatmulPreferenceCreate(&pref));
        const uint64_t wsb = workspace_bytes;
        BSA_LT(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &wsb, sizeof(wsb)));
        const LinearKey key{M, ldx, ldw, ldo, N, K, bias ? 1 : 0, residual ? 1 : 0, device};
        if (!tune) {
            TunedAlgo known;
            bool have = false;
            {
                std::shared_lock<std::shared_mutex> lock(st.mu);
                const auto hit = st.chosen.find(key);
                if (hit != st.chosen.end() && hit->second.workspace <= workspace_bytes) { known = hit->second; have = true; }
            }
            if (have) {
                BSA_LT(hipblasLtMatmul(handle, desc, &alpha, w, la, x, lb, &beta, residual ? residual : out, lc, out, lc,
                                       &known.algo, workspace, workspace_bytes, (hipStream_t)stream));
                goto done;
            }
        }
        constexpr int kMaxAlgos = 32;
        hipblasLtMatmulHeuristicResult_t heur[kMaxAlgos];
        int found = 0, pick = -1;
        BSA_LT(hipblasLtMatmulAlgoGetHeuristic(handle, desc, la, lb, lc, lc, pref, tune ? kMaxAlgos : 8, heur, &found));
        // never hand the library less workspace than the algorithm says it uses
        for (int i = 0; i < found && pick < 0; ++i)
            if (heur[i].state == HIPBLAS_STATUS_SUCCESS && heur[i].workspaceSize <= workspace_bytes) pick = i;
        if (pick < 0) { rc = set_error(BSA_ERR_UNSUPPORTED, "linear: no GEMM algorithm for M=%lld N=%d K=%d within %zu bytes of workspace", (long long)M, N, K, workspace_bytes); goto done; }
        if (tune) {
            // every candidate once to warm up, then three timed runs; the stream is waited for
            hipEvent_t e0 = nullptr, e1 = nullptr;
            if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
                if (e0) (void)hipEventDestroy(e0);
                rc = set_error(BSA_ERR_HIP, "linear tune: hipEventCreate failed");
                goto done;
            }
            float best = 0.f, dflt = 0.f;
            int best_i = -1, tried = 0;
            for (int i = 0; i < found; ++i) {
                if (heur[i].state != HIPBLAS_STATUS_SUCCESS || heur[i].workspaceSize > workspace_bytes) continue;
                bool ok = true;
                for (int r = 0; r < 4 && ok; ++r) {
                    if (r == 1) ok = hipEventRecord(e0, (hipStream_t)stream) == hipSuccess;
                    ok = ok && hipblasLtMatmul(handle, desc, &alpha, w, la, x, lb, &beta, residual ? residual : out, lc, out, lc,
                                               &heur[i].algo, workspace, workspace_bytes, (hipStream_t)stream) == HIPBLAS_STATUS_SUCCESS;
                }
                float ms = 0.f;
                ok = ok && hipEventRecord(e1, (hipStream_t)stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
                     hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
                if (!ok) continue;
                ms /= 3.f;
                if (i == pick) { dflt = ms; if (default_ms) *default_ms = ms; }
                if (best_i < 0 || ms < best) { best = ms; best_i = i; }
                ++tried;
            }
            (void)hipEventDestroy(e0);
            (void)hipEventDestroy(e1);
            if (best_i < 0) { rc = set_error(BSA_ERR_HIP, "linear tune: no candidate ran"); goto done; }
            // three runs each are a noisy measurement: the library's own first choice stays unless it is beaten by 2 %
            if (dflt > 0.f && best > 0.98f * dflt) { best_i = pick; best = dflt; }
            {
                std::unique_lock<std::shared_mutex> lock(st.mu);
                st.chosen[key] = TunedAlgo{heur[best_i].algo, heur[best_i].workspaceSize};
            }
            if (best_ms) *best_ms = best;
            rc = tried;
            goto done;
        }
        {
            std::unique_lock<std::shared_mutex> lock(st.mu);
            st.chosen.emplace(key, TunedAlgo{heur[pick].algo, heur[pick].workspaceSize});      // a measured choice stays
        }
        BSA_LT(hipblasLtMatmul(handle, desc, &alpha, w, la, x, lb, &beta, residual ? residual : out, lc, out, lc,
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
