// Block-sparse flash-attention backward for gfx950 (bf16 / fp16 MFMA), blocked-order tensors.
//
// Follows the reference's backward (bsa_interface.py:341-461; kernels flash_attn_bsa_varlen_mask.py:288-360
// for dK/dV and :428-462 for dQ, wrappers :630-642 and :943-945) with the same rounding points:
//   M2 = lse * log2(e);  k_s = k * (sm_scale * log2(e)) rounded once to the storage type;
//   delta = rowsum(o * do) in fp32;
//   per (query block, selected KV block): s = q . k_s^T, p = exp2(s - M2), dp = do . v^T (all fp32),
//   ds = p * (dp - delta) rounded to the storage type, p rounded to the storage type for dV;
//   dV = sum p^T do,  dK = sm_scale * sum ds^T q,  dQ = ln 2 * sum ds k_s  (fp32 accumulators, one final rounding).
//
// Data movement of dQ as in bsa_fwd_frag.hip: k_s and v are first rewritten into fragment order (frag_kernel, "row
// layout" = the K layout of that file: A operand whose rows are tokens), so a wavefront loads a fragment with one
// coalesced 16-byte load per lane.  The transposed K_s fragments (A operand whose rows are head-dim columns,
// contraction over 16 tokens in accumulator order) are made in the kernel from the row fragments, through LDS.
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

namespace bsa {
namespace {

using namespace mfma;

constexpr float kRcpLn2 = 1.4426950408889634f;

// ------------------------------------------------------------------ small passes
// delta[row] = sum_d o * do (fp32), m2[row] = lse * log2(e), +inf for rows without any key (their p is then 0).
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
        delta[row] = s;
        const float l = lse[row];
        m2[row] = l == -INFINITY ? INFINITY : l * kRcpLn2;
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

// ------------------------------------------------------------------ fragment access
// row layout: [tile][half h][d step c][lane][8];  transposed layout: [tile][half h][16-row step s][d tile t][lane][8]
template <typename V8>
__device__ __forceinline__ V8 frag_row(const char* base, int64_t tile, int h, int c, uint32_t lane_off) {
    return *reinterpret_cast<const V8*>(base + tile * kTileBytes + h * (kTileBytes / 2) + c * 1024 + lane_off);
}
template <typename V8>
__device__ __forceinline__ V8 frag_tr(const char* base, int64_t tile, int h, int s, int t, uint32_t lane_off) {
    return *reinterpret_cast<const V8*>(base + tile * kTileBytes + h * (kTileBytes / 2) + (4 * s + t) * 1024 + lane_off);
}

template <typename T, typename V8>
__device__ __forceinline__ V8 pack8(const f32x16& x, int s) {
    V8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (T)x[8 * s + j];
    return r;
}

// ------------------------------------------------------------------ dQ
constexpr int kDqLds = 32 * 256;                             // the K_s rows of a half tile, on their way to being transposed

template <typename T>
__global__ __launch_bounds__(64) void bwd_dq_kernel(const T* __restrict__ q, const T* __restrict__ dout,
                                                    const char* __restrict__ ks_row,
                                                    const char* __restrict__ v_row, const float* __restrict__ m2,
                                                    const float* __restrict__ delta, const int32_t* __restrict__ idx,
                                                    const int32_t* __restrict__ lens,
                                                    const uint64_t* __restrict__ tile_valid, T* __restrict__ dq,
                                                    int64_t Sq, int64_t Sk, int bs_q, int bs_k, int stride, int item_begin,
                                                    int item_end, int round) {
    typedef typename Vec8<T>::type V8;
    const int lane = threadIdx.x, lr = lane & 31, lh = lane >> 5;
    const uint32_t lane_off = (uint32_t)lane * 16u;
    const int64_t groups = Sq / kTile;
    // The launch's items are taken in rounds of `round` (a multiple of 8) in workgroup order; workgroup b runs on
    // XCD b % 8 and within a round every XCD takes a contiguous run of the round's items, as in the forward kernel:
    // the items of a round walk their lists together and share K_s / V tiles in L2.
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
    const int n = min(max(lens[lrow], 0), stride);
    const int32_t* list = idx + lrow * stride;
    const int64_t kv_tiles = Sk / kTile;
    const char* ksr = ks_row + bh * kv_tiles * kTileBytes;
    const char* vr = v_row + bh * kv_tiles * kTileBytes;

    // two query halves of 32 rows: every K_s / V fragment feeds two MFMAs
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

    // The row fragments of a half tile (K_s rows, V rows: 16 KB) are requested one half ahead of their use, into two
    // register buffers that take turns; the transposed K_s fragments at the start of the half that uses them.
    struct Frags { V8 k[8], v[8]; };
    auto load = [&](Frags& f, int64_t tile, int h) {
#pragma unroll
        for (int c = 0; c < 8; ++c) f.k[c] = frag_row<V8>(ksr, tile, h, c, lane_off);
#pragma unroll
        for (int c = 0; c < 8; ++c) f.v[c] = frag_row<V8>(vr, tile, h, c, lane_off);
    };
    // The transposed K_s fragments of a half (the A operands of dQ^T += K_s^T dS^T) are made from its row fragments:
    // every lane parks its 16-byte pieces in the wavefront's 8 KB of LDS and ds_read_b64_tr_b16 hands them back with
    // rows and columns exchanged, which saves a third of the bytes that the wavefront pulls through the L1 path and a
    // fragment-order copy of k_s.  Piece u of key row r lies in slot u ^ f(r), f(r) = ((r << 1) & 14) | ((r >> 3) & 1):
    // neither the writes (16 consecutive rows) nor the 4-row patches of a transposing read collide on a bank.
    extern __shared__ __attribute__((aligned(16))) char dq_lds[];
    V8 kt[8];
    const uint32_t fl = (uint32_t)(((lr << 1) & 14) | ((lr >> 3) & 1));
    uint32_t woff[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) woff[c] = (uint32_t)(lr * 256) + ((((uint32_t)(2 * c + lh)) ^ fl) << 4);
    const int s16 = lane & 15, g1 = (lane >> 4) & 1, tx = s16 >> 2, ty = (s16 & 3) >> 1, tz = s16 & 1;
    uint32_t toff[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
            toff[t][hi] = (uint32_t)((4 * lh + tx + 8 * hi) * 256) + ((((uint32_t)(4 * t + 2 * g1 + ty)) ^ (uint32_t)((8 * lh + 2 * tx) | hi)) << 4) +
                          (uint32_t)(tz * 8);
    auto park_rows = [&](const V8 (&krow)[8]) {
#pragma unroll
        for (int c = 0; c < 8; ++c) *reinterpret_cast<V8*>(dq_lds + woff[c]) = krow[c];
    };
    auto take_transposed = [&]() {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const char* base = dq_lds + (16 * (x >> 2)) * 256;
            const s16x4 lo = lds_read_tr16(base + toff[x & 3][0]), hi = lds_read_tr16(base + toff[x & 3][1]);
            kt[x] = __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
    };
    auto compute = [&](const Frags& f, uint32_t hv) {
        f32x16 s[2], dp[2];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int i = 0; i < 16; ++i) { s[qq][i] = 0.f; dp[qq][i] = 0.f; }
        park_rows(f.k);
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                s[qq] = mfma32(f.k[c], qreg[qq][c], s[qq]);
                dp[qq] = mfma32(f.v[c], doreg[qq][c], dp[qq]);
            }
        // The 16 loads of the next half (requested by the caller just before this step) go out one behind every
        // third MFMA of this step: a load that finds the CU's address unit busy holds up the wavefront's next
        // instructions, and four wavefronts that each ask for 16 KB in one burst keep it busy for most of a step.
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        take_transposed();
        // accumulator i <-> key 8 (i / 4) + 4 lh + i % 4 of the half, query lr (+ 32)
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = 8 * (i / 4) + 4 * lh + (i % 4);
                float p = __builtin_amdgcn_exp2f(s[qq][i] - m_row[qq]);
                if (!((hv >> key) & 1u)) p = 0.f;
                s[qq][i] = p * (dp[qq][i] - d_row[qq]);
            }
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
    const int ntiles = n * nsub;
    auto tile_at = [&](int tp) -> int64_t {
        const int tc = min(tp, ntiles - 1);
        return (int64_t)min(max(list[tc / nsub], 0), nbk - 1) * nsub + tc % nsub;
    };
    if (ntiles > 0) {
        Frags fa, fb;
        int64_t tile = tile_at(0);
        load(fa, tile, 0);
        for (int tp = 0; tp < ntiles; ++tp) {
            const uint64_t valid = tile_valid != nullptr ? tile_valid[tile] : ~0ull;
            load(fb, tile, 1);
            compute(fa, (uint32_t)valid);
            const int64_t next = tile_at(tp + 1);
            load(fa, next, 0);                            // behind the last tile: loaded again, not used
            compute(fb, (uint32_t)(valid >> 32));
            tile = next;
        }
    }
    // accumulator i of d tile t <-> d = 32 t + 8 (i / 4) + 4 lh + i % 4, query lr (+ 32)
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        T* out = dq + (bh * Sq + qrow0 + 32 * qq + lr) * kD;
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
// f(r) = ((r << 1) & 14) | ((r >> 3) & 1): 16 consecutive rows, and the 4 consecutive rows of a transposing read,
// land on different banks.
constexpr int kBwdHalfTile = kTileBytes / 2;                 // 32 query rows of Q or of dO
constexpr int kBwdStats = 1024;                              // M2 (128 B), delta (128 B), the rest filled blindly by the 64-lane DMA
constexpr int kBwdStage = 2 * kBwdHalfTile + kBwdStats;      // one half tile of queries: Q rows, dO rows, M2, delta
constexpr int kBwdStages = 4;                                // two in use (this half, the next half's rows), two on their way

template <typename T>
__global__ __launch_bounds__(128) void bwd_dkdv_kernel(const T* __restrict__ q, const T* __restrict__ dout,
                                                       const T* __restrict__ ks, const T* __restrict__ v,
                                                       const float* __restrict__ m2, const float* __restrict__ delta,
                                                       const uint32_t* __restrict__ bits,
                                                       const uint64_t* __restrict__ tile_valid, T* __restrict__ dk,
                                                       T* __restrict__ dv, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int words,
                                                       float dk_scale, const int32_t* __restrict__ order, int n_items, int round) {
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
    if (tile_valid != nullptr) key_ok = (tile_valid[krow0 / kTile] >> (32 * wave + lr)) & 1ull;
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
        const int f = ((row << 1) & 14) | ((row >> 3) & 1);
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
    const uint32_t fl = (uint32_t)(((lr << 1) & 14) | ((lr >> 3) & 1));
    uint32_t roff[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) roff[c] = (uint32_t)(lr * 256) + ((((uint32_t)(2 * c + lh)) ^ fl) << 4);
    const int s16 = lane & 15, g1 = (lane >> 4) & 1, tx = s16 >> 2, ty = (s16 & 3) >> 1, tz = s16 & 1;
    uint32_t toff[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
            toff[t][hi] = (uint32_t)((4 * lh + tx + 8 * hi) * 256) + ((((uint32_t)(4 * t + 2 * g1 + ty)) ^ (uint32_t)((8 * lh + 2 * tx) | hi)) << 4) +
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
    auto products_and_exponentials = [&](int hp, f32x16& s, f32x16& dp, f32x16& s_next, f32x16& dp_next) {
        const char* qn = bwd_lds + ((hp + 1) & 3) * kBwdStage;
        const char* dn = qn + kBwdHalfTile;
        const float* st_m2 = reinterpret_cast<const float*>(bwd_lds + (hp & 3) * kBwdStage + 2 * kBwdHalfTile);
        const float* st_dl = st_m2 + 32;
        // Volatile assembly keeps the compiler from moving LDS reads across it, so the operands of a group of four
        // MFMAs (and the statistics of four accumulators) are requested a group ahead by hand.
        V8 fq[2][2], fd[2][2];
        float4 mm[2], dd[2];
        auto request = [&](int g, int b) {
            fq[b][0] = *reinterpret_cast<const V8*>(qn + roff[2 * g]);
            fd[b][0] = *reinterpret_cast<const V8*>(dn + roff[2 * g]);
            fq[b][1] = *reinterpret_cast<const V8*>(qn + roff[2 * g + 1]);
            fd[b][1] = *reinterpret_cast<const V8*>(dn + roff[2 * g + 1]);
            mm[b] = *reinterpret_cast<const float4*>(st_m2 + 8 * g + 4 * lh);
            dd[b] = *reinterpret_cast<const float4*>(st_dl + 8 * g + 4 * lh);
        };
        request(0, 0);
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const int c = 2 * g4, b = g4 & 1;
            if (g4 < 3) request(g4 + 1, b ^ 1);
            if (g4 == 0) {
                mfma_s<true, false>(s_next, fq[b][0], kreg[0]);
                mfma_s<true, false>(dp_next, fd[b][0], vreg[0]);
            } else {
                mfma_s<false, false>(s_next, fq[b][0], kreg[c]);
                mfma_s<false, false>(dp_next, fd[b][0], vreg[c]);
            }
            mfma_s<false, false>(s_next, fq[b][1], kreg[c + 1]);
            mfma_s<false, false>(dp_next, fd[b][1], vreg[c + 1]);
            // accumulator i <-> query 8 (i / 4) + 4 lh + i % 4 of the half, key lr
            const float mv[4] = {mm[b].x, mm[b].y, mm[b].z, mm[b].w}, dl[4] = {dd[b].x, dd[b].y, dd[b].z, dd[b].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = 4 * g4 + j;
                float pi = __builtin_amdgcn_exp2f(s[i] - mv[j]);
                if (!key_ok) pi = 0.f;
                s[i] = pi;                                   // P
                dp[i] = pi * (dp[i] - dl[j]);                // dS
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
        issue(hp + 3, (hp + 3) & 3);
        products_and_exponentials(hp, s, dp, s_next, dp_next);
        __builtin_amdgcn_sched_barrier(0);
        gradients(hp, s, dp);
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
            mfma_s<true, false>(s0, *reinterpret_cast<const V8*>(qn + roff[0]), kreg[0]);
            mfma_s<true, false>(dp0, *reinterpret_cast<const V8*>(dn + roff[0]), vreg[0]);
#pragma unroll
            for (int c = 1; c < 8; ++c) {
                mfma_s<false, false>(s0, *reinterpret_cast<const V8*>(qn + roff[c]), kreg[c]);
                mfma_s<false, false>(dp0, *reinterpret_cast<const V8*>(dn + roff[c]), vreg[c]);
            }
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
        }
        for (int hp = 0; hp < nhalves; hp += 2) {                                // halves come in pairs
            step(hp, s0, dp0, s1, dp1);
            step(hp + 1, s1, dp1, s0, dp0);
        }
    }
    // accumulator i of d tile t <-> d = 32 t + 8 (i / 4) + 4 lh + i % 4, key lr
    {
        const int64_t row = bh * Sk + krow0 + 32 * wave + lr;
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
                *reinterpret_cast<uint2*>(dk + row * kD + 32 * t + 8 * g4 + 4 * lh) = *reinterpret_cast<const uint2*>(xk);
                *reinterpret_cast<uint2*>(dv + row * kD + 32 * t + 8 * g4 + 4 * lh) = *reinterpret_cast<const uint2*>(xv);
            }
    }
}

}  // namespace

// Workspace of the backward, in bytes: two fragment-order copies ([B*Hn][Sk/64][16 KB]: k_s and v in row layout),
// k_s in blocked order, delta and M2, the bit matrix, the lists in the dQ kernel's visiting
// order, per KV block its number of query blocks, the KV tiles of every head by that number.
size_t bwd_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride) {
    const size_t bh = (size_t)B * Hn;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    const size_t words = (size_t)((Sq / bs_q + 31) / 32);
    return 3 * up(bh * Sk * kD * 2) + 2 * up(bh * Sq * 4) + up(bh * (Sk / bs_k) * words * 4) +
           up(bh * (Sq / bs_q) * (size_t)idx_stride * 4) + up(bh * (Sk / bs_k) * 4) + up(bh * (Sk / kTile) * 4);
}

hipError_t launch_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                      const int32_t* idx, const int32_t* lens, const uint64_t* tile_valid, void* dq, void* dk, void* dv,
                      int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype,
                      void* workspace, hipStream_t st) {
    const size_t bh = (size_t)B * Hn;
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    char* ws = static_cast<char*>(workspace);
    auto take = [&](size_t n) { char* p = ws; ws += up(n); return p; };
    char* ks_row = take(bh * Sk * kD * 2);
    char* v_row = take(bh * Sk * kD * 2);
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
    if (dtype == BSA_BF16) {
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
    // blocked-order tensors as a grid of 64-token chunks along one axis
    const Grid3 gk = make_grid((int)(Sk / kTile), 1, kTile, 1, 1, kTile);
    const int64_t stk[3] = {(int64_t)Hn * Sk * kD, Sk * kD, kD};
    hipError_t e;
    hipLaunchKernelGGL(bwd_count_kernel, dim3((unsigned)((bh * nbk + 255) / 256)), dim3(256), 0, st, bits, counts, words, (int64_t)(bh * nbk));
    if ((e = launch_order_by_length(counts, order, (int)bh, nbk, bs_k / kTile, nbq, st)) != hipSuccess) return e;
    // dQ walks every list in the forward kernel's visiting order when the list is ascending (a selection in block
    // order); any other order is walked as given.  The order only moves fp32 roundings of the dQ sum.
    if ((e = launch_pace_order(idx, paced, lens, (int64_t)bh * nbq, nbk, idx_stride, st)) != hipSuccess) return e;
    if ((e = launch_frag(ks, stk, ks_row, B, Hn, gk, dtype, false, st)) != hipSuccess) return e;
    if ((e = launch_frag(v, stk, v_row, B, Hn, gk, dtype, false, st)) != hipSuccess) return e;

    const dim3 block(64);
    // the dK / dV kernel's LDS: four stages of half a Q tile, half a dO tile and the queries' M2 / delta, then a KV block's query blocks
    const size_t lds = (size_t)kBwdStages * kBwdStage + (size_t)nbq * sizeof(int32_t);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    if (dtype == BSA_BF16) e = hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_dkdv_kernel<__bf16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    else e = hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_dkdv_kernel<_Float16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    const dim3 grid_k((unsigned)(bh * (Sk / kTile)));
    // dQ: rounds of as many wavefronts as the device runs at once (one per SIMD), two rounds per launch.  The dK / dV
    // kernel runs as one grid, longest list first: its lists (the query blocks of a KV block) differ in length, and
    // rounds that wait for the longest list cost more than they bring.
    int cus = 256, dev = 0;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const int round = 4 * (cus > 0 ? cus : 256), span = 2 * round;
    const int total_q = (int)(bh * (Sq / kTile)), total_k = (int)(bh * (Sk / kTile));
    if (dtype == BSA_BF16) {
        for (int first = 0; first < total_q; first += span) {
            const int end = first + span < total_q ? first + span : total_q;
            hipLaunchKernelGGL((bwd_dq_kernel<__bf16>), dim3(end - first), block, kDqLds, st, (const __bf16*)q, (const __bf16*)dout, ks_row,
                               v_row, m2, delta, paced, lens, tile_valid, (__bf16*)dq, Sq, Sk, bs_q, bs_k, idx_stride, first, end, round);
        }
        hipLaunchKernelGGL((bwd_dkdv_kernel<__bf16>), grid_k, dim3(128), lds, st, (const __bf16*)q, (const __bf16*)dout, (const __bf16*)ks,
                           (const __bf16*)v, m2, delta, bits, tile_valid, (__bf16*)dk, (__bf16*)dv, Sq, Sk, bs_q, bs_k, words, sm_scale, order,
                           total_k, round);
    } else {
        for (int first = 0; first < total_q; first += span) {
            const int end = first + span < total_q ? first + span : total_q;
            hipLaunchKernelGGL((bwd_dq_kernel<_Float16>), dim3(end - first), block, kDqLds, st, (const _Float16*)q, (const _Float16*)dout,
                               ks_row, v_row, m2, delta, paced, lens, tile_valid, (_Float16*)dq, Sq, Sk, bs_q, bs_k, idx_stride, first,
                               end, round);
        }
        hipLaunchKernelGGL((bwd_dkdv_kernel<_Float16>), grid_k, dim3(128), lds, st, (const _Float16*)q, (const _Float16*)dout,
                           (const _Float16*)ks, (const _Float16*)v, m2, delta, bits, tile_valid, (_Float16*)dk, (_Float16*)dv, Sq, Sk, bs_q, bs_k,
                           words, sm_scale, order, total_k, round);
    }
    return hipGetLastError();
}

}  // namespace bsa
