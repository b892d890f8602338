// Pooled-score GEMM (MFMA) and deterministic per-row top-k selection.
//
// score[bh, m, n] = sum_d q_cmp[bh, m, d] * k_cmp[bh, n, d]   (fp32 accumulate,
// one rounding to the storage type, no softmax scale).
//
// Top-k: each wavefront owns one score row.  Every score is widened to a
// unique, totally ordered integer key (order-preserving image of the score in
// the high bits, inverted column index in the low bits) so that "larger key"
// means "larger score, or equal score and lower index".  The k-th largest key
// is found by a bitwise binary search whose counting step is a wavefront
// ballot + popcount; the winners are compacted into LDS and ranked so that the
// output is in descending score order with ties towards the lowest index.
#include "bsa_common.h"

namespace bsa {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ inline f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ inline f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

template <typename T> struct Vec8;
template <> struct Vec8<__bf16> { typedef bf16x8 type; };
template <> struct Vec8<_Float16> { typedef f16x8 type; };

// ---------------------------------------------------------------- score GEMM
// Workgroup = 4 wavefronts = a 64x64 score tile; each wavefront one 32x32 MFMA
// tile.  Operands come straight from global memory (the pooled tensors are a
// few hundred KB per head and stay in L2): lane l supplies row l%32, and the 8
// consecutive d values 16*s + 8*(l/32) .. +8 of k-step s, for both operands.
template <typename T>
__global__ __launch_bounds__(256) void score_mfma_kernel(const T* __restrict__ qc,
                                                         const T* __restrict__ kc,
                                                         T* __restrict__ score, int nbq, int nbk,
                                                         int D) {
    typedef typename Vec8<T>::type V8;
    const int bh = blockIdx.z;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int m0 = blockIdx.y * 64 + (wave >> 1) * 32;
    const int n0 = blockIdx.x * 64 + (wave & 1) * 32;
    if (m0 >= nbq || n0 >= nbk) return;   // whole wavefront out of range
    const int lr = lane & 31, lh = lane >> 5;
    const int mrow = min(m0 + lr, nbq - 1);   // clamp: rows past the end are computed, not stored
    const int nrow = min(n0 + lr, nbk - 1);
    const T* qa = qc + ((int64_t)bh * nbq + mrow) * D + lh * 8;
    const T* kb = kc + ((int64_t)bh * nbk + nrow) * D + lh * 8;
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int s = 0; s < D / 16; ++s) {
        const V8 a = *reinterpret_cast<const V8*>(qa + s * 16);
        const V8 b = *reinterpret_cast<const V8*>(kb + s * 16);
        acc = mfma32(a, b, acc);
    }
    // accumulator i of lane l: row 8*(i/4) + 4*(l/32) + i%4, column l%32
    const int n = n0 + lr;
    if (n < nbk) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = m0 + 8 * (i / 4) + 4 * lh + (i % 4);
            if (m < nbq) score[((int64_t)bh * nbq + m) * nbk + n] = (T)acc[i];
        }
    }
}

// fp32 storage type: plain fp32 dot products (used by the fp32 plumbing case).
__global__ __launch_bounds__(256) void score_f32_kernel(const float* __restrict__ qc,
                                                        const float* __restrict__ kc,
                                                        float* __restrict__ score, int nbq,
                                                        int nbk, int D) {
    const int bh = blockIdx.z;
    const int n = blockIdx.x * 64 + (threadIdx.x & 63);
    const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (m >= nbq || n >= nbk) return;
    const float* a = qc + ((int64_t)bh * nbq + m) * D;
    const float* b = kc + ((int64_t)bh * nbk + n) * D;
    float s = 0.f;
    for (int d = 0; d < D; ++d) s = fmaf(a[d], b[d], s);
    score[((int64_t)bh * nbq + m) * nbk + n] = s;
}

// ---------------------------------------------------------------- top-k
// Order-preserving maps to unsigned integers (NaN with the sign bit clear sorts
// above +inf, as torch.topk orders NaN).
// -0 is folded onto +0 first: the two compare equal, so they must tie.
__device__ inline uint32_t ord16(uint16_t u) {
    if (u == 0x8000u) u = 0;
    return (u & 0x8000u) ? (uint16_t)~u : (u | 0x8000u);
}
__device__ inline uint32_t ord32(uint32_t u) {
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

template <typename T> struct KeyOf;
template <> struct KeyOf<uint16_t> {   // bf16 / fp16 bit patterns (fp16 orders like its bits too)
    typedef uint32_t type;
    static constexpr int kBits = 32;
    __device__ static uint32_t make(uint16_t s, int idx) { return (ord16(s) << 16) | (0xFFFFu - idx); }
    __device__ static int index(uint32_t k) { return 0xFFFF - (int)(k & 0xFFFFu); }
};
template <> struct KeyOf<uint32_t> {   // fp32 bit patterns
    typedef uint64_t type;
    static constexpr int kBits = 64;
    __device__ static uint64_t make(uint32_t s, int idx) {
        return ((uint64_t)ord32(s) << 32) | (uint64_t)(0xFFFFFFFFu - (uint32_t)idx);
    }
    __device__ static int index(uint64_t k) { return (int)(0xFFFFFFFFu - (uint32_t)k); }
};

constexpr int kMaxSel = 1024;   // keys kept in LDS per wavefront

template <typename S, int NPL>
__global__ __launch_bounds__(256) void topk_kernel(const S* __restrict__ score,
                                                   int32_t* __restrict__ idx_out,
                                                   int32_t* __restrict__ idx_sorted_out,
                                                   int32_t* __restrict__ lens_out, int64_t rows,
                                                   int nbk, int k_sel) {
    typedef typename KeyOf<S>::type K;
    __shared__ K sel[4][kMaxSel];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    if (lane == 0) lens_out[row] = k_sel;
    if (k_sel == 0) return;

    const S* srow = score + row * nbk;
    K key[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int i = j * 64 + lane;
        key[j] = i < nbk ? KeyOf<S>::make(srow[i], i) : (K)0;   // 0 is below every real key
    }
    // largest T with count(key >= T) >= k_sel; keys are unique, so the count ends at k_sel
    K thr = 0;
    for (int bit = KeyOf<S>::kBits - 1; bit >= 0; --bit) {
        const K cand = thr | ((K)1 << bit);
        int cnt = 0;
#pragma unroll
        for (int j = 0; j < NPL; ++j) cnt += __popcll(__ballot(key[j] >= cand));
        if (cnt >= k_sel) {
            thr = cand;
            if (cnt == k_sel) break;
        }
    }
    // compact the winners into LDS (any order), then rank them
    K* mine = sel[wave];
    int base = 0;
    const uint64_t lt = ((uint64_t)1 << lane) - 1;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const bool win = key[j] >= thr;
        const uint64_t m = __ballot(win);
        if (win) mine[base + __popcll(m & lt)] = key[j];
        base += __popcll(m);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): LDS writes of this wavefront landed
    __builtin_amdgcn_wave_barrier();
    // idx_out: descending score, ties towards the lowest index (the order of the keys);
    // idx_sorted_out: the same set in ascending block index
    for (int e = lane; e < k_sel; e += 64) {
        const K me = mine[e];
        const int my_idx = KeyOf<S>::index(me);
        int rank = 0, rank_idx = 0;
        for (int o = 0; o < k_sel; ++o) {
            const K other = mine[o];
            rank += other > me;
            rank_idx += KeyOf<S>::index(other) < my_idx;
        }
        if (idx_out) idx_out[row * k_sel + rank] = my_idx;
        if (idx_sorted_out) idx_sorted_out[row * k_sel + rank_idx] = my_idx;
    }
}

template <typename S>
hipError_t launch_topk_t(const S* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                         int nbk, int k_sel, hipStream_t st) {
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
#define BSA_TOPK(N)                                                                          \
    hipLaunchKernelGGL((topk_kernel<S, N>), grid, block, 0, st, score, idx, idx_sorted, lens, rows, \
                       nbk, k_sel)
    if (nbk <= 4 * 64) BSA_TOPK(4);
    else if (nbk <= 8 * 64) BSA_TOPK(8);
    else if (nbk <= 16 * 64) BSA_TOPK(16);
    else if (nbk <= 24 * 64) BSA_TOPK(24);
    else if (nbk <= 32 * 64) BSA_TOPK(32);
    else BSA_TOPK(64);
#undef BSA_TOPK
    return hipGetLastError();
}

}  // namespace

hipError_t launch_score(const void* q_cmp, const void* k_cmp, void* score, int BH, int nbq, int nbk,
                        int D, int dtype, hipStream_t st) {
    if (dtype == BSA_F32) {
        dim3 grid((nbk + 63) / 64, (nbq + 3) / 4, BH);
        hipLaunchKernelGGL(score_f32_kernel, grid, dim3(256), 0, st, (const float*)q_cmp,
                           (const float*)k_cmp, (float*)score, nbq, nbk, D);
    } else {
        dim3 grid((nbk + 63) / 64, (nbq + 63) / 64, BH);
        if (dtype == BSA_BF16)
            hipLaunchKernelGGL((score_mfma_kernel<__bf16>), grid, dim3(256), 0, st,
                               (const __bf16*)q_cmp, (const __bf16*)k_cmp, (__bf16*)score, nbq,
                               nbk, D);
        else
            hipLaunchKernelGGL((score_mfma_kernel<_Float16>), grid, dim3(256), 0, st,
                               (const _Float16*)q_cmp, (const _Float16*)k_cmp, (_Float16*)score,
                               nbq, nbk, D);
    }
    return hipGetLastError();
}

hipError_t launch_topk(const void* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                       int nbk, int k_sel, int dtype, hipStream_t st) {
    if (dtype == BSA_F32)
        return launch_topk_t<uint32_t>((const uint32_t*)score, idx, idx_sorted, lens, rows, nbk, k_sel, st);
    return launch_topk_t<uint16_t>((const uint16_t*)score, idx, idx_sorted, lens, rows, nbk, k_sel, st);
}

}  // namespace bsa
