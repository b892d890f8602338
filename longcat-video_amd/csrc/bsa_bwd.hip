// Block-sparse flash-attention backward for gfx950 (bf16 / fp16 MFMA).  The kernels work on blocked-order q, k_s, v,
// dO; the caller's tensors are either in blocked order too (launch_bwd without `thw`) or in (T, H, W) token order, in
// which case the two small passes read o, dO, lse and k through row tables and the kernels store every gradient row
// at its token (BwdThw, BwdStore).
//
// Follows the reference's backward (bsa_interface.py:341-461; kernels flash_attn_bsa_varlen_mask.py:288-360
// for dK/dV and :428-462 for dQ, wrappers :630-642 and :943-945) with the same rounding points:
//   M2 = lse * log2(e);  k_s = k * (sm_scale * log2(e)) rounded once to the storage type;
//   delta = rowsum(o * do) in fp32;
//   per (query block, selected KV block): s = q . k_s^T, p = exp2(s - M2), dp = do . v^T (all fp32),
//   ds = p * (dp - delta) rounded to the storage type, p rounded to the storage type for dV;
//   dV = sum p^T do,  dK = sm_scale * sum ds^T q,  dQ = ln 2 * sum ds k_s  (fp32 accumulators, one final rounding).
//
// Data movement: k (pre-scaled) and v, q and dO are read as they lie in memory, in blocked order, through LDS
// (global_load_lds_dwordx4): no fragment-order copies.  Row fragments (A operand whose rows are tokens) come out of
// LDS with ds_read_b128, transposed ones (A operand whose rows are head-dim columns, contraction over 16 tokens in
// accumulator order) with ds_read_b64_tr_b16.
//
// dQ: one wavefront per 64 query rows (two halves of 32, so that every K_s and V fragment feeds two MFMAs).
// S^T = K_s Q^T and dP^T = V dO^T (Q and dO rows in registers as B operands) put one query per lane, so M2 and
// delta are one scalar per lane and dS^T in the accumulator registers is already the B operand of
// dQ^T += K_s^T dS^T.
// dK, dV: one kernel, a workgroup of two wavefronts per 64 keys.  S = Q K_s^T and dP = dO V^T (K_s and V rows in
// registers as B operands) put one key per lane; P and dS in the accumulator registers are the B operands of
// dV^T += dO^T P and dK^T += Q^T dS.  Q and dO are read as they lie in memory, through LDS (see that kernel).
// The query blocks of a KV block come from a bit matrix [KV block][query block] that a small kernel fills from
// the forward's lists (ascending order for free).  Lists are expected to name a block at most once, as a
// selection does; for a repeated block dQ follows the list (as the forward does) and dK / dV the bit matrix, like
// the reference.
#include "bsa_mfma.h"

#include <atomic>

namespace bsa {
namespace {

using namespace mfma;

constexpr float kRcpLn2 = 1.4426950408889634f;
constexpr int kBwdHalfTileBytes = kTileBytes / 2;            // 32 rows of 256 B

// ------------------------------------------------------------------ small passes
// Per query row, both negated because the kernels below add them (as the start value of an MFMA chain):
// delta[row] = -sum_d o * do (fp32), m2[row] = -lse * log2(e), -inf for rows without any key (their p is then 0).
// One 16-lane group per row.
template <typename T>
__global__ __launch_bounds__(256) void bwd_rows_kernel(const T* __restrict__ o, const T* __restrict__ dout,
                                                       const float* __restrict__ lse, float* __restrict__ delta,
                                                       float* __restrict__ m2, int64_t rows) {
    typedef typename Vec8<T>::type V8;
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int c = threadIdx.x & 15;
    float s = 0.f;
    if (row < rows) {
        const V8 a = *reinterpret_cast<const V8*>(o + row * kD + c * 8);
        const V8 b = *reinterpret_cast<const V8*>(dout + row * kD + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)b[e];
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (row < rows && c == 0) {
        delta[row] = -s;
        const float l = lse[row];
        m2[row] = l == -INFINITY ? -INFINITY : -(l * kRcpLn2);
    }
}

// k_s = k * c, rounded once to the storage type (the product is formed in fp32, as torch does for a tensor times
// a Python scalar).
template <typename T>
__global__ __launch_bounds__(256) void bwd_scale_kernel(const T* __restrict__ k, T* __restrict__ ks, float c, int64_t n8) {
    typedef typename Vec8<T>::type V8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    V8 x = *reinterpret_cast<const V8*>(k + i * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * c);
    *reinterpret_cast<V8*>(ks + i * 8) = x;
}

// Where a gradient row goes when the caller's tensors are in token order: the token of every blocked-order slot of one
// (batch, head) (-1: padding, nothing is stored) and the element strides of the destination.  rows null: blocked order.
struct BwdStore {
    const int32_t* rows;
    int64_t sB, sH, sS;
    int Hn;
};
template <typename T>
__device__ __forceinline__ T* store_row(T* blocked, const BwdStore& w, int64_t bh, int64_t rows_per_bh, int64_t slot) {
    if (w.rows == nullptr) return blocked + (bh * rows_per_bh + slot) * kD;
    const int32_t token = w.rows[slot];
    if (token < 0) return nullptr;
    return blocked + (bh / w.Hn) * w.sB + (bh % w.Hn) * w.sH + (int64_t)token * w.sS;
}

// bwd_rows_kernel for o, dO and lse in token order (element strides oS / dS per token, lse [B * Hn][tokens]): the
// same delta and m2 per blocked-order slot, and dO copied into blocked order on the way (padded slots: a zero row,
// delta 0, m2 -inf, so that their p is 0).  One 16-lane group per slot.
template <typename T>
__global__ __launch_bounds__(256) void bwd_rows_thw_kernel(const T* __restrict__ o, int64_t oB, int64_t oH, int64_t oS,
                                                           const T* __restrict__ dout, int64_t dB, int64_t dH, int64_t dS,
                                                           const float* __restrict__ lse, const int32_t* __restrict__ rows,
                                                           int64_t tokens, int Hn, int64_t slots, T* __restrict__ dout_blocked,
                                                           float* __restrict__ delta, float* __restrict__ m2, int64_t total) {
    typedef typename Vec8<T>::type V8;
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int c = threadIdx.x & 15;
    if (row >= total) return;                                    // whole 16-lane groups leave together
    const int64_t bh = row / slots;
    const int32_t token = rows[row - bh * slots];
    float s = 0.f;
    V8 b;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = (T)0.f;
    if (token >= 0) {
        const int64_t at = (bh / Hn), hd = (bh % Hn);
        const V8 a = *reinterpret_cast<const V8*>(o + at * oB + hd * oH + (int64_t)token * oS + c * 8);
        b = *reinterpret_cast<const V8*>(dout + at * dB + hd * dH + (int64_t)token * dS + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)b[e];
    }
    *reinterpret_cast<V8*>(dout_blocked + row * kD + c * 8) = b;
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (c == 0) {
        delta[row] = -s;
        const float l = token >= 0 ? lse[bh * tokens + token] : -INFINITY;
        m2[row] = l == -INFINITY ? -INFINITY : -(l * kRcpLn2);
    }
}

// bwd_scale_kernel for k in token order: k_s in blocked order, padded slots zero.  One 16-lane group per slot.
template <typename T>
__global__ __launch_bounds__(256) void bwd_scale_thw_kernel(const T* __restrict__ k, int64_t kB, int64_t kH, int64_t kS,
                                                            const int32_t* __restrict__ rows, int Hn, int64_t slots,
                                                            T* __restrict__ ks, float c, int64_t total) {
    typedef typename Vec8<T>::type V8;
    const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    if (row >= total) return;
    const int64_t bh = row / slots;
    const int32_t token = rows[row - bh * slots];
    V8 x;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (T)0.f;
    if (token >= 0) {
        x = *reinterpret_cast<const V8*>(k + (bh / Hn) * kB + (bh % Hn) * kH + (int64_t)token * kS + (threadIdx.x & 15) * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * c);
    }
    *reinterpret_cast<V8*>(ks + row * kD + (threadIdx.x & 15) * 8) = x;
}

__global__ void bwd_zero_kernel(uint32_t* p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// bits[bh][kv block][query block / 32] |= 1 << (query block % 32) for every list entry; block indices are clamped
// to the valid range as the forward kernels do.
__global__ __launch_bounds__(256) void bwd_mask_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ lens,
                                                       uint32_t* __restrict__ bits, int nbq, int nbk, int stride,
                                                       int words, int64_t rows) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const int64_t bh = row / nbq;
    const int m = (int)(row % nbq);
    const int n = min(max(lens[row], 0), stride);
    for (int e = lane; e < n; e += 64) {
        const int j = min(max(idx[row * stride + e], 0), nbk - 1);
        atomicOr(bits + (bh * nbk + j) * words + (m >> 5), 1u << (m & 31));
    }
}

// counts[bh * nbk + j] = number of query blocks that selected KV block j (bits set in its row of the bit matrix)
__global__ __launch_bounds__(256) void bwd_count_kernel(const uint32_t* __restrict__ bits, int32_t* __restrict__ counts,
                                                        int words, int64_t rows) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= rows) return;
    int c = 0;
    for (int w = 0; w < words; ++w) c += __popc(bits[row * words + w]);
    counts[row] = c;
}

template <typename T, typename V8>
__device__ __forceinline__ V8 pack8(const f32x16& x, int s) {
    V8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (T)x[8 * s + j];
    return r;
}

// ------------------------------------------------------------------ dQ
// One wavefront per 64 query rows, as two halves of 32 so that every K_s and V fragment feeds two MFMAs.  The K_s and
// V rows of a half tile (32 keys x 256 B each, as they lie in memory - no fragment-order copies) go from global
// memory straight into the wavefront's own LDS (global_load_lds_dwordx4, two stages of 16 KB: one being read, one on
// its way, completion counted by hand), the row fragments come from there with ds_read_b128 and the transposed K_s
// fragments with ds_read_b64_tr_b16 (slot p of row r holds 16-byte unit p ^ f(r), f(r) = ((r & 3) << 2) | ((r >> 2) & 3),
// applied on the global side of the DMA, so that neither kind of read collides on a bank).  That leaves the registers
// for two sets of S^T / dP^T accumulators, so the products of the next half are issued between the exponentials of
// this one: the wavefront has its SIMD to itself and nothing else fills the MFMA pipe while it computes
// exponentials.  S^T and dP^T accumulate in ordinary registers (MFMAs from inline assembly, Q and dO named in the
// accumulation registers they are kept in); the compiler adds no wait states behind such an MFMA and moves no LDS
// read across it, so a set is first read a whole group of MFMAs after it was written and the row fragments are
// requested a group ahead by hand.
// First MFMA of a chain that starts from a block of registers instead of zero (B operand in an accumulation
// register): S^T - M2 comes out of the products, and the exponentials need no subtraction.
__device__ inline void mfma_from(f32x16& acc, bf16x8 a, bf16x8 b, const f32x16& init) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "a"(b), "v"(init));
}
__device__ inline void mfma_from(f32x16& acc, f16x8 a, f16x8 b, const f32x16& init) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "a"(b), "v"(init));
}
// the same with the B operand in an ordinary register
__device__ inline void mfma_from_v(f32x16& acc, bf16x8 a, bf16x8 b, const f32x16& init) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "v"(b), "v"(init));
}
__device__ inline void mfma_from_v(f32x16& acc, f16x8 a, f16x8 b, const f32x16& init) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "v"(b), "v"(init));
}

constexpr int kDqStage = 2 * kBwdHalfTileBytes;              // K_s rows and V rows of 32 keys
constexpr int kDqRingLds = 2 * kDqStage;

// kMasked: the caller has a validity word per KV tile (padding keys exist); they cost nothing per P element (see
// start_block below), only the look-up of the word per half tile.
template <typename T, bool kMasked>
__global__ __launch_bounds__(64) void bwd_dq_lds_kernel(const T* __restrict__ q, const T* __restrict__ dout,
                                                        const T* __restrict__ ks, const T* __restrict__ v,
                                                        const float* __restrict__ m2, const float* __restrict__ delta,
                                                        const int32_t* __restrict__ idx, const int32_t* __restrict__ lens,
                                                        const uint64_t* __restrict__ tile_valid, T* __restrict__ dq,
                                                        int64_t Sq, int64_t Sk, int bs_q, int bs_k, int stride, int item_begin,
                                                        int item_end, int round, BwdStore dq_to) {
    typedef typename Vec8<T>::type V8;
    extern __shared__ __attribute__((aligned(1024))) char dq_ring[];
    const int lane = threadIdx.x, lr = lane & 31, lh = lane >> 5;
    const int64_t groups = Sq / kTile;
    int64_t item;
    {
        const int local = blockIdx.x, r0 = local / round * round;
        const int n = min(round, item_end - item_begin - r0), w = local - r0, x = w & 7;
        item = item_begin + r0 + x * (n >> 3) + min(x, n & 7) + (w >> 3);
    }
    const int64_t bh = item / groups;
    const int64_t qrow0 = (item % groups) * kTile;
    const int nbq = (int)(Sq / bs_q), nbk = (int)(Sk / bs_k), nsub = bs_k / kTile;
    const int64_t lrow = bh * nbq + qrow0 / bs_q;
    const int n = __builtin_amdgcn_readfirstlane(min(max(lens[lrow], 0), stride));
    const int32_t* list = idx + lrow * stride;
    const char* k_src = reinterpret_cast<const char*>(ks) + bh * Sk * (int64_t)(kD * 2);
    const char* v_src = reinterpret_cast<const char*>(v) + bh * Sk * (int64_t)(kD * 2);

    V8 qreg[2][8], doreg[2][8];
    float m_row[2], d_row[2];
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        const int64_t row = bh * Sq + qrow0 + 32 * qq + lr;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            qreg[qq][c] = *reinterpret_cast<const V8*>(q + row * kD + 16 * c + 8 * lh);
            doreg[qq][c] = *reinterpret_cast<const V8*>(dout + row * kD + 16 * c + 8 * lh);
        }
        m_row[qq] = m2[row];
        d_row[qq] = delta[row];
    }
    f32x16 acc[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][qq][i] = 0.f;
    f32x16 neg_m[2];                             // what the S^T accumulators of a query half start from
#pragma unroll
    for (int qq = 0; qq < 2; ++qq)
#pragma unroll
        for (int i = 0; i < 16; ++i) neg_m[qq][i] = m_row[qq];       // m2 and delta come negated

    const int ntiles = n * nsub, nhalves = 2 * ntiles;
    auto tile_at = [&](int tp) -> int64_t {
        const int tc = min(tp, ntiles - 1);
        return (int64_t)min(max(list[tc / nsub], 0), nbk - 1) * nsub + tc % nsub;
    };
    // ---- global -> LDS: 16 loads of 1 KB per half
    const uint32_t lds0 = lds_address(dq_ring);
    uint32_t voff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = 4 * i + (lane >> 4);                                     // + 16 j
        const int f = ((row & 3) << 2) | ((row >> 2) & 3);
        voff[i] = (uint32_t)(row * 256 + (((lane & 15) ^ f) << 4));
    }
    uint32_t hv_ahead = ~0u;                     // validity of the keys of the half tile requested last
    auto issue = [&](int hp) {
        if (hp >= nhalves) return;
        const int64_t tile = (int64_t)__builtin_amdgcn_readfirstlane((int)tile_at(hp >> 1));
        if (kMasked) hv_ahead = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(tile_valid[tile] >> (32 * (hp & 1))));
        const int64_t off = tile * kTileBytes + (hp & 1) * kBwdHalfTileBytes;
        const uint32_t dst = lds0 + (hp & 1) * kDqStage;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                load_to_lds_16(k_src + off + j * 4096, voff[i], dst + j * 4096 + i * 1024);
                load_to_lds_16(v_src + off + j * 4096, voff[i], dst + kBwdHalfTileBytes + j * 4096 + i * 1024);
            }
    };
    // ---- LDS -> fragments
    const uint32_t fl = (uint32_t)(((lr & 3) << 2) | ((lr >> 2) & 3));
    uint32_t roff[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) roff[c] = (uint32_t)(lr * 256) + ((((uint32_t)(2 * c + lh)) ^ fl) << 4);
    const int s16 = lane & 15, g1 = (lane >> 4) & 1, tx = s16 >> 2, ty = (s16 & 3) >> 1, tz = s16 & 1;
    uint32_t toff[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
            toff[t][hi] = (uint32_t)((4 * lh + tx + 8 * hi) * 256) + ((((uint32_t)(4 * t + 2 * g1 + ty)) ^ (uint32_t)((4 * tx) | (lh + 2 * hi))) << 4) +
                          (uint32_t)(tz * 8);
    V8 kt[8];                                    // the transposed K_s fragments of the half whose dQ products come next
    auto take_transposed = [&](int hp) {
        const char* part = dq_ring + (hp & 1) * kDqStage;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const char* base = part + (16 * (x >> 2)) * 256;
            const s16x4 lo = lds_read_tr16(base + toff[x & 3][0]), hi = lds_read_tr16(base + toff[x & 3][1]);
            kt[x] = __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
    };
    // accumulator i <-> key 8 (i / 4) + 4 lh + i % 4 of the half, query lr (+ 32)
    auto exponentials = [&](f32x16 (&s)[2], f32x16 (&dp)[2], int qq, int i0, int count) {
#pragma unroll
        for (int i = i0; i < i0 + count; ++i) {
            const float p = __builtin_amdgcn_exp2f(s[qq][i]);        // s holds S^T - M2, -inf for a padded key
            s[qq][i] = p * (dp[qq][i] + d_row[qq]);
        }
    };
    // Padded keys: the chain of a half tile that holds any starts from -inf in their accumulators instead of -M2, so
    // their p is exp2(-inf) = 0 and the exponentials test nothing.  Such half tiles are the few at the upper edges of
    // the grid; the start block is rebuilt only when the validity of the half in hand differs from all-valid or the
    // one before did.
    bool start_masked = false;
    auto start_block = [&](uint32_t hv) {
        if (!kMasked) return;
        const bool edge = hv != ~0u;
        if (!edge && !start_masked) return;
        start_masked = edge;
        const uint32_t mine = hv >> (4 * lh);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const bool ok = (mine >> (8 * (i / 4) + (i % 4))) & 1u;
            neg_m[0][i] = ok ? m_row[0] : -INFINITY;
            neg_m[1][i] = ok ? m_row[1] : -INFINITY;
        }
    };
    // S^T and dP^T of half hp (both query halves) into (s, dp); between its groups of four MFMAs the exponentials of
    // the half before, on (ps, pdp), eight accumulators per group.
    auto products = [&](int hp, f32x16 (&s)[2], f32x16 (&dp)[2], auto&& behind_requests, auto&& between) {
        const char* kp = dq_ring + (hp & 1) * kDqStage;
        const char* vp = kp + kBwdHalfTileBytes;
        V8 fk[2], fv[2];
        fk[0] = *reinterpret_cast<const V8*>(kp + roff[0]);
        fv[0] = *reinterpret_cast<const V8*>(vp + roff[0]);
        behind_requests();                       // the DMA set-up runs while the first LDS reads are on their way
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int b = c & 1;
            if (c < 7) {
                fk[b ^ 1] = *reinterpret_cast<const V8*>(kp + roff[c + 1]);
                fv[b ^ 1] = *reinterpret_cast<const V8*>(vp + roff[c + 1]);
            }
            if (c == 0) {
                mfma_from(s[0], fk[b], qreg[0][0], neg_m[0]);
                mfma_s<true, true>(dp[0], fv[b], doreg[0][0]);
                mfma_from(s[1], fk[b], qreg[1][0], neg_m[1]);
                mfma_s<true, true>(dp[1], fv[b], doreg[1][0]);
            } else {
                mfma_s<false, true>(s[0], fk[b], qreg[0][c]);
                mfma_s<false, true>(dp[0], fv[b], doreg[0][c]);
                mfma_s<false, true>(s[1], fk[b], qreg[1][c]);
                mfma_s<false, true>(dp[1], fv[b], doreg[1][c]);
            }
            between(c);
        }
    };
    auto gradients = [&](const f32x16 (&s)[2]) {
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            const V8 ds0 = pack8<T, V8>(s[0], st), ds1 = pack8<T, V8>(s[1], st);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[t][0] = mfma32(kt[4 * st + t], ds0, acc[t][0]);
                acc[t][1] = mfma32(kt[4 * st + t], ds1, acc[t][1]);
            }
        }
    };
    // (s, dp): this half, products done; (ns, ndp): the next half
    auto step = [&](int hp, f32x16 (&s)[2], f32x16 (&dp)[2], f32x16 (&ns)[2], f32x16 (&ndp)[2]) {
        start_block(hv_ahead);                   // validity of half hp + 1, looked up when its rows were requested
        // The next half's rows must have landed; the stage that this half was read from (rows and transposed
        // fragments are in registers) takes half hp + 2.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        products(hp + 1, ns, ndp, [&]() { issue(hp + 2); }, [&](int c) { exponentials(s, dp, c >> 2, 4 * (c & 3), 4); });
        __builtin_amdgcn_sched_barrier(0);
        gradients(s);
        __builtin_amdgcn_sched_barrier(0);
        take_transposed(hp + 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // the chains into (ns, ndp) end here, sixteen MFMAs behind their last one
        mfma_chain_end(ns[0]); mfma_chain_end(ns[1]); mfma_chain_end(ndp[0]); mfma_chain_end(ndp[1]);
    };
    if (nhalves > 0) {
        f32x16 sa[2], dpa[2], sb[2], dpb[2];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the Q / dO rows: from here on the DMA loads are counted by hand
        issue(0);
        const uint32_t hv_first = hv_ahead;
        issue(1);
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        start_block(hv_first);
        products(0, sa, dpa, [&]() {}, [&](int) {});
        take_transposed(0);
        asm volatile("s_nop 15\n\ts_nop 7\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
        mfma_chain_end(sa[0]); mfma_chain_end(sa[1]); mfma_chain_end(dpa[0]); mfma_chain_end(dpa[1]);
        for (int hp = 0; hp < nhalves; hp += 2) {                                // halves come in pairs
            step(hp, sa, dpa, sb, dpb);
            step(hp + 1, sb, dpb, sa, dpa);
        }
    }
    // accumulator i of d tile t <-> d = 32 t + 8 (i / 4) + 4 lh + i % 4, query lr (+ 32)
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        T* out = store_row(dq, dq_to, bh, Sq, qrow0 + 32 * qq + lr);
        if (out == nullptr) continue;                            // a padded slot of a token-order destination
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                T x[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) x[j] = (T)(acc[t][qq][4 * g4 + j] * kLn2);
                *reinterpret_cast<uint2*>(out + 32 * t + 8 * g4 + 4 * lh) = *reinterpret_cast<const uint2*>(x);
            }
    }
}

// ------------------------------------------------------------------ dK and dV in one kernel, Q and dO through LDS
// One workgroup of two wavefronts per 64 keys; wavefront w owns keys 32 w .. 32 w + 31 and both of their gradients
// (128 accumulator registers).  The Q and dO tiles of a query tile (64 rows x 256 B each, as they lie in memory)
// go from global memory straight into LDS once per workgroup (global_load_lds_dwordx4; wavefront 0 brings Q and
// the queries' M2 and delta, wavefront 1 brings dO), in halves of 32 queries, four stages deep (two in use, two on
// their way), and both wavefronts take every operand from there: the row fragments (the A operands of S = Q K_s^T and
// dP = dO V^T) with ds_read_b128, the transposed
// ones (the A operands of dV^T += dO^T P and dK^T += Q^T dS) with ds_read_b64_tr_b16.  Per tile pair 32 KB leave
// the caches instead of the 80 KB of fragment-order copies that separate dK and dV kernels stream, S is computed
// once instead of twice (128 MFMAs per tile pair instead of 160), and no fragment-order copy of q or dO is made.
// The LDS side of the DMA is linear in the lane index, so the swizzle that keeps both kinds of read free of bank
// conflicts is applied on the global side: the 16-byte slot p of row r receives unit p ^ f(r),
// f(r) = ((r & 3) << 2) | ((r >> 2) & 3): 16 consecutive rows, and the 4 rows x 4 units of a transposing read's 32 lanes,
// land on different banks.
constexpr int kBwdHalfTile = kTileBytes / 2;                 // 32 query rows of Q or of dO
constexpr int kBwdStats = 1024;                              // M2 (128 B), delta (128 B), the rest filled blindly by the 64-lane DMA
constexpr int kBwdStage = 2 * kBwdHalfTile + kBwdStats;      // one half tile of queries: Q rows, dO rows, M2, delta
constexpr int kBwdStages = 4;                                // two in use (this half, the next half's rows), two on their way

// kMasked: as in the dQ kernel - without validity words no key is padding and the test is compiled out.
template <typename T, bool kMasked>
__global__ __launch_bounds__(128) void bwd_dkdv_kernel(const T* __restrict__ q, const T* __restrict__ dout,
                                                       const T* __restrict__ ks, const T* __restrict__ v,
                                                       const float* __restrict__ m2, const float* __restrict__ delta,
                                                       const uint32_t* __restrict__ bits,
                                                       const uint64_t* __restrict__ tile_valid, T* __restrict__ dk,
                                                       T* __restrict__ dv, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int words,
                                                       float dk_scale, const int32_t* __restrict__ order, int n_items, int round,
                                                       BwdStore dk_to, BwdStore dv_to) {
    typedef typename Vec8<T>::type V8;
    extern __shared__ __attribute__((aligned(1024))) char bwd_lds[];
    const int lane = threadIdx.x & 63, lr = lane & 31, lh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int64_t groups = Sk / kTile;
    // items longest list first, every XCD on a contiguous run of each group of `round` (see launch_bwd)
    int64_t item;
    {
        const int local = blockIdx.x, r0 = local / round * round;
        const int n = min(round, n_items - r0), w = local - r0, x = w & 7;
        item = order[r0 + x * (n >> 3) + min(x, n & 7) + (w >> 3)];
    }
    const int64_t bh = item / groups;
    const int64_t krow0 = (item % groups) * kTile;
    const int nbq = (int)(Sq / bs_q), nbk = (int)(Sk / bs_k), qsub = bs_q / kTile;
    const int kblk = (int)(krow0 / bs_k);
    const uint32_t* mask_row = bits + (bh * nbk + kblk) * words;

    // resident: K_s and V rows of this wavefront's 32 keys, as B operands (lane = key lr, 8 consecutive d)
    V8 kreg[8], vreg[8];
    {
        const int64_t row = bh * Sk + krow0 + 32 * wave + lr;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            kreg[c] = *reinterpret_cast<const V8*>(ks + row * kD + 16 * c + 8 * lh);
            vreg[c] = *reinterpret_cast<const V8*>(v + row * kD + 16 * c + 8 * lh);
        }
    }
    bool key_ok = true;
    if (kMasked) key_ok = (tile_valid[krow0 / kTile] >> (32 * wave + lr)) & 1ull;
    f32x16 acc_dk[4], acc_dv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc_dk[t][i] = 0.f; acc_dv[t][i] = 0.f; }

    // the query blocks of this KV block, ascending, from the bit matrix into LDS (behind the stages)
    int32_t* qlist = reinterpret_cast<int32_t*>(bwd_lds + kBwdStages * kBwdStage);
    int count = 0;
    for (int w0 = 0; w0 < words; w0 += 64) {
        const int w = w0 + lane;
        uint32_t word = w < words ? mask_row[w] : 0u;
        if (w == words - 1 && (nbq & 31)) word &= (1u << (nbq & 31)) - 1u;
        int mine = __popc(word), upto = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(upto, off);
            if (lane >= off) upto += t;
        }
        int pos = count + upto - mine;
        if (wave == 0)
            while (word != 0u) {
                qlist[pos++] = 32 * w + __builtin_ctz(word);
                word &= word - 1u;
            }
        count += __shfl(upto, 63);
    }
    __syncthreads();
    const int ntiles = __builtin_amdgcn_readfirstlane(count) * qsub;          // the same in every lane; the compiler cannot tell
    auto tile_at = [&](int tp) -> int64_t {
        const int tc = min(tp, ntiles - 1);
        return (int64_t)__builtin_amdgcn_readfirstlane(qlist[tc / qsub]) * qsub + tc % qsub;
    };

    // ---- global -> LDS
    const uint32_t lds0 = lds_address(bwd_lds);
    uint32_t voff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = 4 * i + (lane >> 4);                                     // + 16 j
        const int f = ((row & 3) << 2) | ((row >> 2) & 3);
        voff[i] = (uint32_t)(row * 256 + (((lane & 15) ^ f) << 4));
    }
    const uint32_t stat_gap = (uint32_t)(reinterpret_cast<const char*>(m2) - reinterpret_cast<const char*>(delta));
    const uint32_t voff_stats = ((lane & 15) < 8 ? stat_gap : 0u) + (uint32_t)((lane & 7) * 16);
    const char* tile_src = reinterpret_cast<const char*>(wave == 0 ? q : dout) + bh * Sq * (int64_t)(kD * 2);
    const char* stat_src = reinterpret_cast<const char*>(delta) + bh * Sq * 4;
    const int nhalves = 2 * ntiles;
    // half hp = query half hp & 1 of the walk's tile hp / 2, into stage hp % kBwdStages
    auto issue = [&](int hp, int stage) {
        if (hp >= nhalves) return;
        const int64_t tile = (int64_t)__builtin_amdgcn_readfirstlane((int)tile_at(hp >> 1));
        const int h = hp & 1;
        const char* src = tile_src + tile * kTileBytes + h * kBwdHalfTile;
        const uint32_t dst = lds0 + stage * kBwdStage + wave * kBwdHalfTile;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) load_to_lds_16(src + j * 4096, voff[i], dst + j * 4096 + i * 1024);
        if (wave == 0)
            load_to_lds_16(stat_src + tile * (kTile * 4) + h * 128, voff_stats, lds0 + stage * kBwdStage + 2 * kBwdHalfTile);
    };

    // ---- LDS -> fragments
    const uint32_t fl = (uint32_t)(((lr & 3) << 2) | ((lr >> 2) & 3));
    uint32_t roff[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) roff[c] = (uint32_t)(lr * 256) + ((((uint32_t)(2 * c + lh)) ^ fl) << 4);
    const int s16 = lane & 15, g1 = (lane >> 4) & 1, tx = s16 >> 2, ty = (s16 & 3) >> 1, tz = s16 & 1;
    uint32_t toff[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
            toff[t][hi] = (uint32_t)((4 * lh + tx + 8 * hi) * 256) + ((((uint32_t)(4 * t + 2 * g1 + ty)) ^ (uint32_t)((4 * tx) | (lh + 2 * hi))) << 4) +
                          (uint32_t)(tz * 8);
    auto frag_tr_lds = [&](const char* part, int st2, int t) -> V8 {
        const char* base = part + (16 * st2) * 256;
        const s16x4 lo = lds_read_tr16(base + toff[t][0]), hi = lds_read_tr16(base + toff[t][1]);
        return __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    // One half tile of queries (32) against this wavefront's 32 keys is 32 MFMAs in two groups with the exponentials
    // between them.  A wavefront has a SIMD to itself, so it overlaps them on its own: the S and dP products of the
    // NEXT half (into a second pair of accumulators) are issued between the exponentials of this one.  S and dP
    // accumulate in ordinary registers, where the exponentials read them: MFMAs from inline assembly, behind which
    // the compiler adds no wait states - a pair is read a whole group of 16 MFMAs after it was written.
    auto products_and_exponentials = [&](int hp, f32x16& s, f32x16& dp, f32x16& s_next, f32x16& dp_next, auto&& behind_requests) {
        const char* qn = bwd_lds + ((hp + 1) & 3) * kBwdStage;
        const char* dn = qn + kBwdHalfTile;
        // The chains of the next half start from its queries' -M2 and -delta (accumulator i <-> query
        // 8 (i / 4) + 4 lh + i % 4 of the half, key lr), so S - M2 and dP - delta come out of the products and the
        // exponentials need no subtraction.
        const float* st_m2 = reinterpret_cast<const float*>(qn + 2 * kBwdHalfTile);
        const float* st_dl = st_m2 + 32;
        f32x16 from_m, from_d;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 mm = *reinterpret_cast<const float4*>(st_m2 + 8 * g + 4 * lh);
            const float4 dd = *reinterpret_cast<const float4*>(st_dl + 8 * g + 4 * lh);
            from_m[4 * g] = mm.x; from_m[4 * g + 1] = mm.y; from_m[4 * g + 2] = mm.z; from_m[4 * g + 3] = mm.w;
            from_d[4 * g] = dd.x; from_d[4 * g + 1] = dd.y; from_d[4 * g + 2] = dd.z; from_d[4 * g + 3] = dd.w;
        }
        // Volatile assembly keeps the compiler from moving LDS reads across it, so the operands of a group of four
        // MFMAs are requested a group ahead by hand.
        V8 fq[2][2], fd[2][2];
        auto request = [&](int g, int b) {
            fq[b][0] = *reinterpret_cast<const V8*>(qn + roff[2 * g]);
            fd[b][0] = *reinterpret_cast<const V8*>(dn + roff[2 * g]);
            fq[b][1] = *reinterpret_cast<const V8*>(qn + roff[2 * g + 1]);
            fd[b][1] = *reinterpret_cast<const V8*>(dn + roff[2 * g + 1]);
        };
        request(0, 0);
        behind_requests();                       // the DMA set-up runs while the first LDS reads are on their way
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const int c = 2 * g4, b = g4 & 1;
            if (g4 < 3) request(g4 + 1, b ^ 1);
            if (g4 == 0) {
                mfma_from_v(s_next, fq[b][0], kreg[0], from_m);
                mfma_from_v(dp_next, fd[b][0], vreg[0], from_d);
            } else {
                mfma_s<false, false>(s_next, fq[b][0], kreg[c]);
                mfma_s<false, false>(dp_next, fd[b][0], vreg[c]);
            }
            mfma_s<false, false>(s_next, fq[b][1], kreg[c + 1]);
            mfma_s<false, false>(dp_next, fd[b][1], vreg[c + 1]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = 4 * g4 + j;
                float pi = __builtin_amdgcn_exp2f(s[i]);        // s holds S - M2, dp holds dP - delta
                if (kMasked && !key_ok) pi = 0.f;
                s[i] = pi;                                   // P
                dp[i] = pi * dp[i];                          // dS
            }
        }
    };
    auto gradients = [&](int hp, const f32x16& p, const f32x16& ds) {
        const char* qt = bwd_lds + (hp & 3) * kBwdStage;
        const char* dt = qt + kBwdHalfTile;
#pragma unroll
        for (int st2 = 0; st2 < 2; ++st2) {
            const V8 bp = pack8<T, V8>(p, st2), bds = pack8<T, V8>(ds, st2);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc_dv[t] = mfma32(frag_tr_lds(dt, st2, t), bp, acc_dv[t]);
                acc_dk[t] = mfma32(frag_tr_lds(qt, st2, t), bds, acc_dk[t]);
            }
        }
    };
    // During half hp the rows of half hp + 1 are read, so at its end the loads of half hp + 2 must have landed; the
    // half requested after it may still be on its way (wavefront 0 issues 9 loads per half, wavefront 1 issues 8).
    auto step = [&](int hp, f32x16& s, f32x16& dp, f32x16& s_next, f32x16& dp_next) {
        // half hp + 3 takes the stage that half hp - 1 was read from: both wavefronts are past the barrier behind it
        products_and_exponentials(hp, s, dp, s_next, dp_next, [&]() { issue(hp + 3, (hp + 3) & 3); });
        __builtin_amdgcn_sched_barrier(0);
        gradients(hp, s, dp);
        // the chains into (s_next, dp_next) end here, sixteen MFMAs behind their last one
        mfma_chain_end(s_next); mfma_chain_end(dp_next);
        if (hp + 3 < nhalves) {
            if (wave == 0) asm volatile("s_waitcnt vmcnt(9) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();
    };
    if (nhalves > 0) {
        issue(0, 0);
        issue(1, 1);
        issue(2, 2);
        if (nhalves > 2) {
            if (wave == 0) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();
        f32x16 s0, dp0, s1, dp1;
        {
            const char* qn = bwd_lds;
            const char* dn = qn + kBwdHalfTile;
            const float* st_m2 = reinterpret_cast<const float*>(qn + 2 * kBwdHalfTile);
            const float* st_dl = st_m2 + 32;
            f32x16 from_m, from_d;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 mm = *reinterpret_cast<const float4*>(st_m2 + 8 * g + 4 * lh);
                const float4 dd = *reinterpret_cast<const float4*>(st_dl + 8 * g + 4 * lh);
                from_m[4 * g] = mm.x; from_m[4 * g + 1] = mm.y; from_m[4 * g + 2] = mm.z; from_m[4 * g + 3] = mm.w;
                from_d[4 * g] = dd.x; from_d[4 * g + 1] = dd.y; from_d[4 * g + 2] = dd.z; from_d[4 * g + 3] = dd.w;
            }
            mfma_from_v(s0, *reinterpret_cast<const V8*>(qn + roff[0]), kreg[0], from_m);
            mfma_from_v(dp0, *reinterpret_cast<const V8*>(dn + roff[0]), vreg[0], from_d);
#pragma unroll
            for (int c = 1; c < 8; ++c) {
                mfma_s<false, false>(s0, *reinterpret_cast<const V8*>(qn + roff[c]), kreg[c]);
                mfma_s<false, false>(dp0, *reinterpret_cast<const V8*>(dn + roff[c]), vreg[c]);
            }
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
            mfma_chain_end(s0); mfma_chain_end(dp0);
        }
        for (int hp = 0; hp < nhalves; hp += 2) {                                // halves come in pairs
            step(hp, s0, dp0, s1, dp1);
            step(hp + 1, s1, dp1, s0, dp0);
        }
    }
    // accumulator i of d tile t <-> d = 32 t + 8 (i / 4) + 4 lh + i % 4, key lr
    {
        T* out_k = store_row(dk, dk_to, bh, Sk, krow0 + 32 * wave + lr);
        T* out_v = store_row(dv, dv_to, bh, Sk, krow0 + 32 * wave + lr);
        if (out_k != nullptr && out_v != nullptr) {              // both or neither: one row table serves dk and dv
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    T xk[4], xv[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        xk[j] = (T)(acc_dk[t][4 * g4 + j] * dk_scale);
                        xv[j] = (T)acc_dv[t][4 * g4 + j];
                    }
                    *reinterpret_cast<uint2*>(out_k + 32 * t + 8 * g4 + 4 * lh) = *reinterpret_cast<const uint2*>(xk);
                    *reinterpret_cast<uint2*>(out_v + 32 * t + 8 * g4 + 4 * lh) = *reinterpret_cast<const uint2*>(xv);
                }
        }
    }
}

}  // namespace

constexpr size_t kBwdLdsLimit = 160 * 1024;
// LDS of the dK / dV kernel for nbq query blocks: its stages, then the list of a KV block's query blocks
size_t bwd_dkdv_lds_bytes(int nbq) { return (size_t)kBwdStages * kBwdStage + (size_t)nbq * sizeof(int32_t); }
int bwd_max_query_blocks() { return (int)((kBwdLdsLimit - (size_t)kBwdStages * kBwdStage) / sizeof(int32_t)); }

// Workspace of the backward, in bytes: k_s in blocked order, delta and M2, the bit matrix, the lists in the dQ kernel's visiting
// order, per KV block its number of query blocks, the KV tiles of every head by that number.
size_t bwd_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride) {
    const size_t bh = (size_t)B * Hn;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    const size_t words = (size_t)((Sq / bs_q + 31) / 32);
    return up(bh * Sk * kD * 2) + 2 * up(bh * Sq * 4) + up(bh * (Sk / bs_k) * words * 4) +
           up(bh * (Sq / bs_q) * (size_t)idx_stride * 4) + up(bh * (Sk / bs_k) * 4) + up(bh * (Sk / kTile) * 4);
}

hipError_t launch_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                      const int32_t* idx, const int32_t* lens, const uint64_t* tile_valid, void* dq, void* dk, void* dv,
                      int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype,
                      void* workspace, hipStream_t st, const BwdThw* thw) {
    const size_t bh = (size_t)B * Hn;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    char* ws = static_cast<char*>(workspace);
    auto take = [&](size_t n) { char* p = ws; ws += up(n); return p; };
    char* ks = take(bh * Sk * kD * 2);
    float* delta = reinterpret_cast<float*>(take(bh * Sq * 4));
    float* m2 = reinterpret_cast<float*>(take(bh * Sq * 4));
    const int nbq = (int)(Sq / bs_q), nbk = (int)(Sk / bs_k);
    const int words = (nbq + 31) / 32;
    uint32_t* bits = reinterpret_cast<uint32_t*>(take(bh * nbk * (size_t)words * 4));
    int32_t* paced = reinterpret_cast<int32_t*>(take(bh * nbq * (size_t)idx_stride * 4));
    int32_t* counts = reinterpret_cast<int32_t*>(take(bh * nbk * 4));
    int32_t* order = reinterpret_cast<int32_t*>(take(bh * (size_t)(Sk / kTile) * 4));

    const int64_t qrows = (int64_t)bh * Sq, krows = (int64_t)bh * Sk;
    const float c = sm_scale * kRcpLn2;
    BwdStore dq_to = {nullptr, 0, 0, 0, Hn}, dk_to = dq_to, dv_to = dq_to;
    if (thw != nullptr) {
        // o, dO, lse and k in token order: the two passes read them through the row tables, and dO comes out in
        // blocked order for the kernels; q and v are the caller's blocked-order copies
        dq_to = {thw->q_rows, thw->dq_st[0], thw->dq_st[1], thw->dq_st[2], Hn};
        dk_to = {thw->k_rows, thw->dk_st[0], thw->dk_st[1], thw->dk_st[2], Hn};
        dv_to = {thw->k_rows, thw->dv_st[0], thw->dv_st[1], thw->dv_st[2], Hn};
        dq = thw->dq; dk = thw->dk; dv = thw->dv;
        dout = thw->dout_blocked;
        const dim3 gq((unsigned)((qrows + 15) / 16)), gk((unsigned)((krows + 15) / 16)), blk(256);
        if (dtype == BSA_BF16) {
            hipLaunchKernelGGL((bwd_rows_thw_kernel<__bf16>), gq, blk, 0, st, (const __bf16*)thw->o, thw->o_st[0], thw->o_st[1], thw->o_st[2],
                               (const __bf16*)thw->dout, thw->do_st[0], thw->do_st[1], thw->do_st[2], thw->lse, thw->q_rows, thw->q_tokens, Hn,
                               Sq, (__bf16*)thw->dout_blocked, delta, m2, qrows);
            hipLaunchKernelGGL((bwd_scale_thw_kernel<__bf16>), gk, blk, 0, st, (const __bf16*)thw->k, thw->k_st[0], thw->k_st[1], thw->k_st[2],
                               thw->k_rows, Hn, Sk, (__bf16*)ks, c, krows);
        } else {
            hipLaunchKernelGGL((bwd_rows_thw_kernel<_Float16>), gq, blk, 0, st, (const _Float16*)thw->o, thw->o_st[0], thw->o_st[1], thw->o_st[2],
                               (const _Float16*)thw->dout, thw->do_st[0], thw->do_st[1], thw->do_st[2], thw->lse, thw->q_rows, thw->q_tokens, Hn,
                               Sq, (_Float16*)thw->dout_blocked, delta, m2, qrows);
            hipLaunchKernelGGL((bwd_scale_thw_kernel<_Float16>), gk, blk, 0, st, (const _Float16*)thw->k, thw->k_st[0], thw->k_st[1], thw->k_st[2],
                               thw->k_rows, Hn, Sk, (_Float16*)ks, c, krows);
        }
    } else if (dtype == BSA_BF16) {
        hipLaunchKernelGGL((bwd_rows_kernel<__bf16>), dim3((unsigned)((qrows + 15) / 16)), dim3(256), 0, st, (const __bf16*)o,
                           (const __bf16*)dout, lse, delta, m2, qrows);
        hipLaunchKernelGGL((bwd_scale_kernel<__bf16>), dim3((unsigned)((krows * 16 + 255) / 256)), dim3(256), 0, st,
                           (const __bf16*)k, (__bf16*)ks, c, krows * 16);
    } else {
        hipLaunchKernelGGL((bwd_rows_kernel<_Float16>), dim3((unsigned)((qrows + 15) / 16)), dim3(256), 0, st, (const _Float16*)o,
                           (const _Float16*)dout, lse, delta, m2, qrows);
        hipLaunchKernelGGL((bwd_scale_kernel<_Float16>), dim3((unsigned)((krows * 16 + 255) / 256)), dim3(256), 0, st,
                           (const _Float16*)k, (_Float16*)ks, c, krows * 16);
    }
    const int64_t nwords = (int64_t)bh * nbk * words;
    hipLaunchKernelGGL(bwd_zero_kernel, dim3((unsigned)((nwords + 255) / 256)), dim3(256), 0, st, bits, nwords);
    const int64_t lrows = (int64_t)bh * nbq;
    hipLaunchKernelGGL(bwd_mask_kernel, dim3((unsigned)((lrows + 3) / 4)), dim3(256), 0, st, idx, lens, bits, nbq, nbk, idx_stride,
                       words, lrows);
    hipError_t e;
    hipLaunchKernelGGL(bwd_count_kernel, dim3((unsigned)((bh * nbk + 255) / 256)), dim3(256), 0, st, bits, counts, words, (int64_t)(bh * nbk));
    if ((e = launch_order_by_length(counts, order, (int)bh, nbk, bs_k / kTile, nbq, st)) != hipSuccess) return e;
    // dQ walks every list in the forward kernel's visiting order when the list is ascending (a selection in block
    // order); any other order is walked as given.  The order only moves fp32 roundings of the dQ sum.
    if ((e = launch_pace_order(idx, paced, lens, (int64_t)bh * nbq, nbk, idx_stride, st)) != hipSuccess) return e;

    const dim3 block(64);
    // the dK / dV kernel's LDS: four stages of half a Q tile, half a dO tile and the queries' M2 / delta, then a KV block's query blocks
    const size_t lds = bwd_dkdv_lds_bytes(nbq);
    if (lds > kBwdLdsLimit) return hipErrorInvalidValue;          // the C-ABI layer has rejected such a shape already
    const bool masked = tile_valid != nullptr;
    // Per device, once: the four dK / dV instantiations may use all of the LDS, and the number of compute units.
    static std::atomic<int> device_cus[64];
    int dev = 0;
    if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    int cus = device_cus[dev].load(std::memory_order_acquire);
    if (cus == 0) {
        const void* kernels[4] = {reinterpret_cast<const void*>(bwd_dkdv_kernel<__bf16, true>), reinterpret_cast<const void*>(bwd_dkdv_kernel<__bf16, false>),
                                  reinterpret_cast<const void*>(bwd_dkdv_kernel<_Float16, true>), reinterpret_cast<const void*>(bwd_dkdv_kernel<_Float16, false>)};
        for (const void* kf : kernels)
            if ((e = hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBwdLdsLimit)) != hipSuccess) return e;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        device_cus[dev].store(cus, std::memory_order_release);   // threads racing here set the same attributes
    }
    const dim3 grid_k((unsigned)(bh * (Sk / kTile)));
    // dQ: rounds of as many wavefronts as the device runs at once (one per SIMD), two rounds per launch.  The dK / dV
    // kernel runs as one grid, longest list first: its lists (the query blocks of a KV block) differ in length, and
    // rounds that wait for the longest list cost more than they bring.
    const int round = 4 * cus, span = 2 * round;
    const int total_q = (int)(bh * (Sq / kTile)), total_k = (int)(bh * (Sk / kTile));
    if (dtype == BSA_BF16) {
        for (int first = 0; first < total_q; first += span) {
            const int end = first + span < total_q ? first + span : total_q;
            if (tile_valid != nullptr)
                hipLaunchKernelGGL((bwd_dq_lds_kernel<__bf16, true>), dim3(end - first), block, kDqRingLds, st, (const __bf16*)q,
                                   (const __bf16*)dout, (const __bf16*)ks, (const __bf16*)v, m2, delta, paced, lens, tile_valid, (__bf16*)dq, Sq, Sk,
                                   bs_q, bs_k, idx_stride, first, end, round, dq_to);
            else
                hipLaunchKernelGGL((bwd_dq_lds_kernel<__bf16, false>), dim3(end - first), block, kDqRingLds, st, (const __bf16*)q,
                                   (const __bf16*)dout, (const __bf16*)ks, (const __bf16*)v, m2, delta, paced, lens, tile_valid, (__bf16*)dq, Sq, Sk,
                                   bs_q, bs_k, idx_stride, first, end, round, dq_to);
        }
        if (masked)
            hipLaunchKernelGGL((bwd_dkdv_kernel<__bf16, true>), grid_k, dim3(128), lds, st, (const __bf16*)q, (const __bf16*)dout,
                               (const __bf16*)ks, (const __bf16*)v, m2, delta, bits, tile_valid, (__bf16*)dk, (__bf16*)dv, Sq, Sk, bs_q, bs_k, words,
                               sm_scale, order, total_k, round, dk_to, dv_to);
        else
            hipLaunchKernelGGL((bwd_dkdv_kernel<__bf16, false>), grid_k, dim3(128), lds, st, (const __bf16*)q, (const __bf16*)dout,
                               (const __bf16*)ks, (const __bf16*)v, m2, delta, bits, tile_valid, (__bf16*)dk, (__bf16*)dv, Sq, Sk, bs_q, bs_k, words,
                               sm_scale, order, total_k, round, dk_to, dv_to);
    } else {
        for (int first = 0; first < total_q; first += span) {
            const int end = first + span < total_q ? first + span : total_q;
            if (tile_valid != nullptr)
                hipLaunchKernelGGL((bwd_dq_lds_kernel<_Float16, true>), dim3(end - first), block, kDqRingLds, st, (const _Float16*)q,
                                   (const _Float16*)dout, (const _Float16*)ks, (const _Float16*)v, m2, delta, paced, lens, tile_valid, (_Float16*)dq,
                                   Sq, Sk, bs_q, bs_k, idx_stride, first, end, round, dq_to);
            else
                hipLaunchKernelGGL((bwd_dq_lds_kernel<_Float16, false>), dim3(end - first), block, kDqRingLds, st, (const _Float16*)q,
                                   (const _Float16*)dout, (const _Float16*)ks, (const _Float16*)v, m2, delta, paced, lens, tile_valid, (_Float16*)dq,
                                   Sq, Sk, bs_q, bs_k, idx_stride, first, end, round, dq_to);
        }
        if (masked)
            hipLaunchKernelGGL((bwd_dkdv_kernel<_Float16, true>), grid_k, dim3(128), lds, st, (const _Float16*)q, (const _Float16*)dout,
                               (const _Float16*)ks, (const _Float16*)v, m2, delta, bits, tile_valid, (_Float16*)dk, (_Float16*)dv, Sq, Sk, bs_q,
                               bs_k, words, sm_scale, order, total_k, round, dk_to, dv_to);
        else
            hipLaunchKernelGGL((bwd_dkdv_kernel<_Float16, false>), grid_k, dim3(128), lds, st, (const _Float16*)q, (const _Float16*)dout,
                               (const _Float16*)ks, (const _Float16*)v, m2, delta, bits, tile_valid, (_Float16*)dk, (_Float16*)dv, Sq, Sk, bs_q,
                               bs_k, words, sm_scale, order, total_k, round, dk_to, dv_to);
    }
    return hipGetLastError();
}

}  // namespace bsa
