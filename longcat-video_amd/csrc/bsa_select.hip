// Pooled-score GEMM (MFMA) and deterministic per-row top-k selection.
//
// score[bh, m, n] = sum_d q_cmp[bh, m, d] * k_cmp[bh, n, d]   (fp32 accumulate,
// one rounding to the storage type, no softmax scale).
//
// Top-k: each wavefront owns one score row and holds it in registers as
// order-preserving integer images of the scores.  The k-th largest score VALUE
// is found by a bitwise binary search whose counting step is a wavefront
// ballot + popcount; every column above it wins, and of the columns equal to it
// the lowest-indexed ones that are still needed ("larger score, or equal score
// and lower index").  Walking the registers in column order emits the list in
// ascending block order directly; the descending-score list (a total order
// through keys that append the inverted column index to the score image) is
// ranked in LDS only when it is asked for.  The CDF rule counts with the same
// value search over masked sums of softmax weights.
#include "bsa_mfma.h"

namespace bsa {
namespace {

using mfma::f32x16;
using mfma::mfma32;
using mfma::Vec8;

// ---------------------------------------------------------------- score GEMM
// Workgroup = 4 wavefronts = 128 score rows x up to kScoreCols columns.  The pooled key rows of the workgroup's
// columns (64 KB) are staged in LDS once, with fully coalesced loads; each wavefront keeps its 32 pooled query rows
// (all 128 d, the A operand) in registers and walks the 32-column tiles, reading the B fragments from LDS (lane l:
// row l%32 of the tile, the 8 consecutive d values 16*s + 8*(l/32) .. +8 of k-step s).  Read from global memory
// fragment by fragment instead, every load instruction touches 32 rows for 32 bytes each and the four wavefronts
// ask for the same rows again: the L1 path, not the 17 GFLOP of arithmetic, then sets the time (0.107 ms at
// 1440 x 1440 x 32 heads).  A finished 32x32 tile goes through a wavefront-private LDS patch so that it leaves
// as 16-byte stores (half a row per lane) instead of 2-byte ones.
constexpr int kScoreCols = 256;
constexpr int kScorePitch = 128 + 8;     // elements: 272-byte rows keep 16-byte alignment and spread the banks
template <typename T>
__global__ __launch_bounds__(256) void score_mfma_kernel(const T* __restrict__ qc,
                                                         const T* __restrict__ kc,
                                                         T* __restrict__ score, int nbq, int nbk) {
    typedef typename Vec8<T>::type V8;
    constexpr int D = 128;
    __shared__ __attribute__((aligned(16))) T keys[kScoreCols * kScorePitch];
    __shared__ __attribute__((aligned(16))) T patch[4][32][40];      // 80-byte rows: 16-byte aligned, bank-spread
    const int bh = blockIdx.z;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int m0 = blockIdx.y * 128 + wave * 32;
    const int n_begin = blockIdx.x * kScoreCols;
    const int n_end = min(n_begin + kScoreCols, nbk);
    const int lr = lane & 31, lh = lane >> 5;
    // the key rows of this workgroup's columns: 16 pieces of 16 bytes per row, consecutive threads on consecutive pieces
    {
        const T* kb = kc + ((int64_t)bh * nbk) * D;
        uint4 piece[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int e = threadIdx.x + 256 * i, r = e >> 4, c = e & 15;
            piece[i] = *reinterpret_cast<const uint4*>(kb + (int64_t)min(n_begin + r, nbk - 1) * D + c * 8);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int e = threadIdx.x + 256 * i, r = e >> 4, c = e & 15;
            *reinterpret_cast<uint4*>(keys + r * kScorePitch + c * 8) = piece[i];
        }
    }
    const int mrow = min(m0 + lr, nbq - 1);   // clamp: rows past the end are computed, not stored
    const T* qa = qc + ((int64_t)bh * nbq + mrow) * D + lh * 8;
    V8 a[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) a[s] = *reinterpret_cast<const V8*>(qa + s * 16);
    __syncthreads();
    if (m0 >= nbq) return;                    // whole wavefront out of range (no workgroup barrier below)
    T (*mine)[40] = patch[wave];
    const bool vec_ok = (nbk % 8) == 0;       // rows of the score matrix stay 16-byte aligned
    for (int n0 = n_begin; n0 < n_end; n0 += 32) {
        const T* kt = keys + (n0 - n_begin + lr) * kScorePitch + lh * 8;
        V8 b[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) b[s] = *reinterpret_cast<const V8*>(kt + s * 16);
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < 8; ++s) acc = mfma32(a[s], b[s], acc);
        // accumulator i of lane l: row 8*(i/4) + 4*(l/32) + i%4, column l%32
#pragma unroll
        for (int i = 0; i < 16; ++i) mine[8 * (i / 4) + 4 * lh + (i % 4)][lr] = (T)acc[i];
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wavefront's LDS writes have landed
        __builtin_amdgcn_wave_barrier();
        const int r = lane >> 1, c0 = (lane & 1) * 16;
        const int m = m0 + r;
        if (m < nbq) {
            T* dst = score + ((int64_t)bh * nbq + m) * nbk + n0 + c0;
            if (vec_ok && n0 + c0 + 16 <= nbk) {
                *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(&mine[r][c0]);
                *reinterpret_cast<uint4*>(dst + 8) = *reinterpret_cast<const uint4*>(&mine[r][c0 + 8]);
            } else {
                for (int c = 0; c < 16 && n0 + c0 + c < nbk; ++c) dst[c] = mine[r][c0 + c];
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);   // the patch is read before the next tile overwrites it
        __builtin_amdgcn_wave_barrier();
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

constexpr int kMaxSel = 4096;   // longest list: the score-order ranking keeps a row's winners in LDS

// Order-preserving image of a score alone (ties stay ties).
__device__ inline uint32_t ord_of(uint16_t s) { return ord16(s); }
__device__ inline uint32_t ord_of(uint32_t s) { return ord32(s); }

// The k-th largest score value t of a row that a wavefront holds as val[N] per lane (order-preserving images;
// in_range(x): element x of this lane is a column of the row): every column above t wins, and of the columns equal
// to t the first k_sel - cnt_gt in column order.  thr = t, cnt_gt = columns above t, cnt_eq = columns equal to t.
// For 16-bit scores t is first looked for in a histogram of the codes just below the row maximum, otherwise (and for
// rows whose winners reach further down) by a bitwise binary search whose counting step is a ballot + popcount.
// h: 256 words of LDS of this wavefront.
template <int kValueBits, int N, typename InRange>
__device__ inline void kth_value(const uint32_t (&val)[N], InRange in_range, int lane, int k_sel, uint32_t* h,
                                 uint32_t& thr, int& cnt_gt, int& cnt_eq) {
    thr = 0;
    cnt_gt = 0;
    cnt_eq = 0;
    bool found = false;
    if (kValueBits == 16) {
        // 16-bit scores: the winners of a row usually lie within a few hundred codes of the row maximum, so one
        // histogram of (maximum - ord) over 255 bins, built with LDS atomics by the columns that fall into it,
        // and one scan find t.  Rows whose k_sel largest values reach further down take the search below.
        uint32_t mx = 0;
#pragma unroll
        for (int j = 0; j < N; ++j) mx = max(mx, val[j]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o));
        *reinterpret_cast<uint4*>(h + 4 * lane) = make_uint4(0u, 0u, 0u, 0u);
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const uint32_t d = mx - val[j];
            if (in_range(j) && d < 255u) atomicAdd(h + d, 1u);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
        const uint4 c = *reinterpret_cast<const uint4*>(h + 4 * lane);
        const int own = (int)(c.x + c.y + c.z + c.w);
        int upto = own;                                    // columns within bins 0 .. 4 lane + 3
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(upto, o);
            if (lane >= o) upto += t;
        }
        const int before = upto - own;
        const uint64_t holder = __ballot(before < k_sel && k_sel <= upto);
        if (holder != 0) {
            int bin = 4 * lane, run = before, in_bin = (int)c.x;
            if (run + (int)c.x < k_sel) { run += (int)c.x; ++bin; in_bin = (int)c.y;
                if (run + (int)c.y < k_sel) { run += (int)c.y; ++bin; in_bin = (int)c.z;
                    if (run + (int)c.z < k_sel) { run += (int)c.z; ++bin; in_bin = (int)c.w; } } }
            const int src = __builtin_ctzll(holder);
            thr = mx - (uint32_t)__shfl(bin, src);
            cnt_gt = __shfl(run, src);
            cnt_eq = __shfl(in_bin, src);
            found = true;
        }
    }
    if (!found) {
        // Largest t with count(ord >= t) >= k_sel, t = 0 if there is none above, by a bitwise binary search
        // whose counting step is a ballot + popcount.  Every candidate is at least 1, so the zeros past the end
        // of the row never count.  Leaving early with exactly k_sel columns at or above t is fine: the winners
        // are then all columns at or above t.
        for (int bit = kValueBits - 1; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            int cnt = 0;
#pragma unroll
            for (int j = 0; j < N; ++j) cnt += __popcll(__ballot(val[j] >= cand));
            if (cnt >= k_sel) {
                thr = cand;
                if (cnt == k_sel) break;
            }
        }
        cnt_gt = 0;
        cnt_eq = 0;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            cnt_gt += __popcll(__ballot(val[j] > thr));
            cnt_eq += __popcll(__ballot(val[j] == thr && in_range(j)));      // thr may be 0, like the padding of val
        }
    }
}

// Selection of one score row by one wavefront; lane l holds the order-preserving images of columns l, l + 64,
// ... in registers (0 for columns past the end of the row).
//   1. the k-th largest score value t (kth_value);
//   2. every score above t wins, and of the scores equal to t the ones with the lowest column
//      index, as many as are still needed; walking the registers in column order hands out the
//      positions of the ascending-block-order list at the same time (no sort);
//   3. only when the score-order list is wanted: rank the winners by (score desc, index asc).
// raw_at(i): the stored score of column i.  mine: one key of LDS per list entry (SCORE_ORDER only); h: 256 words of LDS.
template <typename S, int NPL, bool SCORE_ORDER, typename RawAt>
__device__ inline void select_row(const uint32_t (&val)[NPL], RawAt raw_at, int lane, int nbk, int k_sel,
                                  int32_t* __restrict__ idx_row, int32_t* __restrict__ idx_sorted_row,
                                  typename KeyOf<S>::type* mine, uint32_t* h) {
    typedef typename KeyOf<S>::type K;
    uint32_t thr;
    int cnt_gt, cnt_eq;
    kth_value<8 * (int)sizeof(S)>(val, [&](int j) { return j * 64 + lane < nbk; }, lane, k_sel, h, thr, cnt_gt, cnt_eq);
    const int need_eq = k_sel - cnt_gt;

    int pos = 0, eq_seen = 0;
    const uint64_t lt = ((uint64_t)1 << lane) - 1;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int i = j * 64 + lane;
        const bool eq = val[j] == thr && i < nbk;          // thr may be 0, like the padding of val
        const uint64_t meq = __ballot(eq);
        const bool win = val[j] > thr || (eq && eq_seen + __popcll(meq & lt) < need_eq);
        const uint64_t m = __ballot(win);
        if (win) {
            const int p = pos + __popcll(m & lt);
            if (idx_sorted_row) idx_sorted_row[p] = i;                        // column order = ascending block order
            if (SCORE_ORDER) mine[p] = KeyOf<S>::make(raw_at(i), i);
        }
        pos += __popcll(m);
        eq_seen += __popcll(meq);
    }
    if (!SCORE_ORDER) return;
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): LDS writes of this wavefront landed
    __builtin_amdgcn_wave_barrier();
    // descending score, ties towards the lowest index: the order of the combined keys
    for (int e = lane; e < k_sel; e += 64) {
        const K me = mine[e];
        int rank = 0;
        for (int o = 0; o < k_sel; ++o) rank += mine[o] > me;
        idx_row[rank] = KeyOf<S>::index(me);
    }
}

// Top-k from a score matrix in memory: one wavefront per score row.
template <typename S, int NPL, bool SCORE_ORDER>
__global__ __launch_bounds__(256) void topk_kernel(const S* __restrict__ score,
                                                   int32_t* __restrict__ idx_out,
                                                   int32_t* __restrict__ idx_sorted_out,
                                                   int32_t* __restrict__ lens_out, int64_t rows,
                                                   int nbk, int k_all, const int32_t* __restrict__ k_rows,
                                                   int stride) {
    typedef typename KeyOf<S>::type K;
    extern __shared__ __attribute__((aligned(16))) unsigned char topk_keys[];    // SCORE_ORDER: 4 x stride keys
    __shared__ __attribute__((aligned(16))) uint32_t hist[4][256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    // the number of columns to keep: the same for every row, or one count per row (k_rows may be lens_out)
    const int k_sel = k_rows != nullptr ? k_rows[row] : k_all;
    if (lane == 0) lens_out[row] = k_sel;
    // unused tail of the row's lists
    for (int e = k_sel + lane; e < stride; e += 64) {
        if (idx_out) idx_out[row * stride + e] = -1;
        if (idx_sorted_out) idx_sorted_out[row * stride + e] = -1;
    }
    if (k_sel == 0) return;

    const S* srow = score + row * nbk;
    uint32_t val[NPL];                      // ord(score); 0 for columns past the end of the row
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int i = j * 64 + lane;
        const S raw = srow[min(i, nbk - 1)];               // unconditional load, masked afterwards
        val[j] = i < nbk ? ord_of(raw) : 0u;
    }
    select_row<S, NPL, SCORE_ORDER>(val, [&](int i) { return srow[i]; }, lane, nbk, k_sel,
                                    idx_out ? idx_out + row * stride : nullptr,
                                    idx_sorted_out ? idx_sorted_out + row * stride : nullptr,
                                    reinterpret_cast<K*>(topk_keys) + (SCORE_ORDER ? (size_t)wave * stride : 0), hist[wave]);
}

// Top-k of 16-bit scores when only the ascending-block-order list is wanted and rows are 16-byte aligned (nbk a
// multiple of 8): the same selection as select_row with another assignment of columns to lanes.  Lane l holds the
// columns 512 j + 8 l .. 8 l + 7 (one 16-byte load per j instead of eight 2-byte loads), so the ascending list
// position of a winner is (winners in earlier j) + (winners in lower lanes: one prefix sum per j) + (winners
// below it in its own lane) - one scan per 512 columns instead of two ballots per 64.
template <int NCH>
__global__ __launch_bounds__(256) void topk_blocked_kernel(const uint16_t* __restrict__ score,
                                                           int32_t* __restrict__ idx_sorted_out,
                                                           int32_t* __restrict__ lens_out, int64_t rows, int nbk, int k_all,
                                                           const int32_t* __restrict__ k_rows, int stride) {
    __shared__ __attribute__((aligned(16))) uint32_t hist[4][256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const int k_sel = k_rows != nullptr ? k_rows[row] : k_all;
    if (lane == 0) lens_out[row] = k_sel;
    int32_t* out = idx_sorted_out + row * stride;
    for (int e = k_sel + lane; e < stride; e += 64) out[e] = -1;          // unused tail of the row's list
    if (k_sel == 0) return;

    const uint16_t* srow = score + row * nbk;
    uint32_t val[NCH * 8];                   // ord(score); 0 for columns past the end of the row
    bool in[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int col0 = 512 * j + 8 * lane;
        in[j] = col0 < nbk;
        const uint4 raw = *reinterpret_cast<const uint4*>(srow + (in[j] ? col0 : 0));   // unconditional load, masked afterwards
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint16_t r = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            val[8 * j + e] = in[j] ? ord16(r) : 0u;
        }
    }
    uint32_t thr;
    int cnt_gt, cnt_eq;
    kth_value<16>(val, [&](int x) { return in[x >> 3]; }, lane, k_sel, hist[wave], thr, cnt_gt, cnt_eq);
    const int need_eq = k_sel - cnt_gt;
    const bool all_equal_win = need_eq >= cnt_eq;            // the same in every lane: no tie is cut

    int pos = 0, eq_seen = 0;                                  // winners / columns equal to t in the chunks before j
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        if (512 * j >= nbk) break;
        uint32_t win = 0;                                      // bit e: column 512 j + 8 lane + e wins
        if (all_equal_win) {
#pragma unroll
            for (int e = 0; e < 8; ++e) win |= (val[8 * j + e] >= thr && in[j]) ? (1u << e) : 0u;
        } else {
            uint32_t gt = 0, eq = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                gt |= (val[8 * j + e] > thr) ? (1u << e) : 0u;
                eq |= (val[8 * j + e] == thr && in[j]) ? (1u << e) : 0u;
            }
            // of the columns equal to t the first need_eq in column order win
            const int n_eq = __popc(eq);
            int upto = n_eq;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int t = __shfl_up(upto, o);
                if (lane >= o) upto += t;
            }
            int take = min(max(need_eq - (eq_seen + upto - n_eq), 0), n_eq);
            eq_seen += __shfl(upto, 63);
            win = gt;
            while (take > 0) {
                const uint32_t low = eq & (0u - eq);
                win |= low;
                eq ^= low;
                --take;
            }
        }
        const int n_win = __popc(win);
        int upto = n_win;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(upto, o);
            if (lane >= o) upto += t;
        }
        int p = pos + upto - n_win;
        pos += __shfl(upto, 63);
        while (win != 0u) {
            out[p++] = 512 * j + 8 * lane + __builtin_ctz(win);
            win &= win - 1u;
        }
    }
}

// ---------------------------------------------------------------- visiting order
// The order in which the attention kernel visits one row's selected KV blocks.  Softmax attention does not
// depend on it beyond rounding, so it is chosen for the L2 cache: the query tiles that run side by side walk
// the KV sequence together when slot s of every list holds a block near s/n of the sequence, and then share
// the K/V tiles they have in common while those are still cached.  A plain ascending list drifts from that
// pace wherever it holds more or fewer blocks than the average in a stretch of the sequence.
//
// One wavefront per row.  in: n = lens[row] blocks in ascending order.  Visit slots are cut into groups of
// kPaceWidth; group g belongs to the blocks b with g == min(b * n / (nbk * kPaceWidth), groups - 1).  A group
// takes its own blocks in ascending order up to its number of slots; the blocks over that number (ascending
// over the whole list) fill the slots left empty (ascending); every group's slots are then put in ascending
// block order.  in == out is allowed.  A malformed list (unsorted, repeated or out-of-range blocks) still
// gives a permutation of the blocks clamped to the valid range.
constexpr int kPaceWidth = 8;
__global__ __launch_bounds__(64) void pace_order_kernel(const int32_t* in, int32_t* out, const int32_t* __restrict__ lens, int nbk, int stride) {
    extern __shared__ int32_t pace_lds[];
    int32_t* const lst = pace_lds;               // [stride] the row, ascending
    int32_t* const slots = lst + stride;         // [stride] block per visit slot, -1 = empty
    int32_t* const spare = slots + stride;       // [stride] blocks over their group's room, ascending
    int32_t* const first = spare + stride;       // [groups] position of a group's first block in lst
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int32_t* src = in + row * stride;
    int32_t* dst = out + row * stride;
    const int n = min(max(lens[row], 0), stride);
    if (src != dst)
        for (int e = n + lane; e < stride; e += 64) dst[e] = src[e];
    if (n <= kPaceWidth) {
        if (src != dst)
            for (int e = lane; e < n; e += 64) dst[e] = src[e];
        return;
    }
    const int groups = (n + kPaceWidth - 1) / kPaceWidth;
    // n <= stride < 2^13 (the LDS that launch_pace_order asks for bounds it) and b < nbk: 32-bit products and quotients
    const uint32_t span = (uint32_t)nbk * kPaceWidth;
    auto group_of = [&](int32_t b) { return (int)min((uint32_t)b * (uint32_t)n / span, (uint32_t)groups - 1u); };
    for (int e = lane; e < n; e += 64) {
        lst[e] = min(max(src[e], 0), nbk - 1);
        slots[e] = -1;
    }
    for (int g = lane; g < groups; g += 64) first[g] = 0;
    __syncthreads();
    for (int e = lane; e < n; e += 64) {
        const int g = group_of(lst[e]);
        if (e == 0 || group_of(lst[e - 1]) != g) first[g] = e;
    }
    __syncthreads();
    const uint64_t below = ((uint64_t)1 << lane) - 1;
    int taken = 0;
    for (int base = 0; base < n; base += 64) {
        const int e = base + lane;
        bool over = false;
        if (e < n) {
            const int g = group_of(lst[e]), rank = e - first[g];
            const int room = min(kPaceWidth, n - g * kPaceWidth);
            if (rank >= 0 && rank < room) slots[g * kPaceWidth + rank] = lst[e];
            else over = true;
        }
        const uint64_t m = __ballot(over);
        if (over) spare[taken + __popcll(m & below)] = lst[e];
        taken += __popcll(m);
    }
    __syncthreads();
    taken = 0;
    for (int base = 0; base < n; base += 64) {
        const int s = base + lane;
        const bool empty = s < n && slots[s] < 0;
        const uint64_t m = __ballot(empty);
        if (empty) slots[s] = spare[taken + __popcll(m & below)];
        taken += __popcll(m);
    }
    __syncthreads();
    for (int s = lane; s < n; s += 64) {
        const int lo = s / kPaceWidth * kPaceWidth, hi = min(lo + kPaceWidth, n);
        const int32_t b = slots[s];
        int rank = 0;
        for (int t = lo; t < hi; ++t) rank += (slots[t] < b || (slots[t] == b && t < s)) ? 1 : 0;
        dst[lo + rank] = b;
    }
}

// ---------------------------------------------------------------- CDF rule
__device__ inline float score_value(uint16_t s, int dtype) {
    if (dtype == BSA_F16) return (float)__builtin_bit_cast(_Float16, s);
    return __uint_as_float((uint32_t)s << 16);
}
__device__ inline float score_value(uint32_t s, int) { return __uint_as_float(s); }
__device__ inline double wave_sum(double x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

// How many columns the CDF rule keeps per row: with the columns sorted by descending score (ties towards
// the lowest index) and weights softmax(score * scale), the number of leading columns whose running sum
// of weights stays at or below `threshold`; never fewer than k_min (the "cdf + top-k" rule) and never
// more than `cap`.  One wavefront per row.  Sums run in double precision on the unnormalised weights
// e_i = exp((s_i - max) * scale): sum_top(e) <= threshold * sum_all(e).  The columns at or above a score
// value t form a prefix of the sorted order, so a bitwise binary search over t finds the value group in
// which the running sum crosses the threshold; inside that group every column weighs the same.
template <typename S, int NPL>
__global__ __launch_bounds__(256) void cdf_count_kernel(const S* __restrict__ score, int32_t* __restrict__ lens_out,
                                                        int64_t rows, int nbk, float threshold, float scale, int k_min,
                                                        int cap, int dtype) {
    constexpr int kValueBits = 8 * (int)sizeof(S);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const S* srow = score + row * nbk;
    uint32_t val[NPL];
    float e[NPL];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int i = j * 64 + lane;
        const S raw = srow[min(i, nbk - 1)];
        val[j] = i < nbk ? ord_of(raw) : 0u;
        e[j] = i < nbk ? score_value(raw, dtype) : -INFINITY;
        mx = fmaxf(mx, e[j]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    double total = 0.0;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        e[j] = j * 64 + lane < nbk ? expf((e[j] - mx) * scale) : 0.f;
        total += (double)e[j];
    }
    total = wave_sum(total);
    const double budget = (double)threshold * total;
    // largest t whose columns at or above t outweigh the budget (t = 0: all columns, if even that holds)
    auto mass_ge = [&](uint32_t t) {
        double m = 0.0;
#pragma unroll
        for (int j = 0; j < NPL; ++j) m += val[j] >= t ? (double)e[j] : 0.0;     // padding has e = 0
        return wave_sum(m);
    };
    int n;
    if (!(total > budget)) {
        n = nbk;                                  // threshold >= 1: everything
    } else {
        uint32_t thr = 0;
        for (int bit = kValueBits - 1; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            if (mass_ge(cand) > budget) thr = cand;
        }
        // columns above thr fit; the group equal to thr crosses: take as many of it as still fit
        double above = 0.0, one = 0.0;
        int cnt_gt = 0, cnt_eq = 0;
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const bool real = j * 64 + lane < nbk;
            above += val[j] > thr ? (double)e[j] : 0.0;
            cnt_gt += __popcll(__ballot(val[j] > thr));
            const bool eq = real && val[j] == thr;
            cnt_eq += __popcll(__ballot(eq));
            if (eq) one = (double)e[j];
        }
        above = wave_sum(above);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) one = fmax(one, __shfl_xor(one, o));
        int fit = one > 0.0 ? (int)floor((budget - above) / one) : cnt_eq;
        fit = max(0, min(fit, cnt_eq));
        n = cnt_gt + fit;
    }
    n = min(max(n, k_min), min(cap, nbk));
    if (lane == 0) lens_out[row] = n;
}

template <typename S>
hipError_t launch_cdf_count_t(const S* score, int32_t* lens, int64_t rows, int nbk, float threshold, float scale,
                              int k_min, int cap, int dtype, hipStream_t st) {
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
#define BSA_CDF(N) hipLaunchKernelGGL((cdf_count_kernel<S, N>), grid, block, 0, st, score, lens, rows, nbk, threshold, scale, k_min, cap, dtype)
    if (nbk <= 4 * 64) BSA_CDF(4);
    else if (nbk <= 8 * 64) BSA_CDF(8);
    else if (nbk <= 16 * 64) BSA_CDF(16);
    else if (nbk <= 24 * 64) BSA_CDF(24);
    else if (nbk <= 32 * 64) BSA_CDF(32);
    else BSA_CDF(64);
#undef BSA_CDF
    return hipGetLastError();
}

template <typename S>
hipError_t launch_topk_t(const S* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                         int nbk, int k_sel, const int32_t* k_rows, int stride, hipStream_t st) {
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (sizeof(S) == 2 && idx == nullptr && idx_sorted != nullptr && nbk % 8 == 0 && (reinterpret_cast<uintptr_t>(score) & 15) == 0) {
        const uint16_t* sc = reinterpret_cast<const uint16_t*>(score);
#define BSA_TOPK_BLOCKED(N) hipLaunchKernelGGL((topk_blocked_kernel<N>), grid, block, 0, st, sc, idx_sorted, lens, rows, nbk, k_sel, k_rows, stride)
        if (nbk <= 512) BSA_TOPK_BLOCKED(1);
        else if (nbk <= 1024) BSA_TOPK_BLOCKED(2);
        else if (nbk <= 1536) BSA_TOPK_BLOCKED(3);
        else if (nbk <= 2048) BSA_TOPK_BLOCKED(4);
        else if (nbk <= 3072) BSA_TOPK_BLOCKED(6);
        else BSA_TOPK_BLOCKED(8);
#undef BSA_TOPK_BLOCKED
        return hipGetLastError();
    }
    // the score-order ranking keeps the winners of the workgroup's four rows in LDS
    const size_t lds = idx != nullptr ? (size_t)4 * stride * sizeof(typename KeyOf<S>::type) : 0;
#define BSA_TOPK(N)                                                                                \
    do {                                                                                           \
        if (idx != nullptr) {                                                                      \
            if (lds > 64 * 1024) {                                                                 \
                const hipError_t ea = hipFuncSetAttribute((const void*)topk_kernel<S, N, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
                if (ea != hipSuccess) return ea;                                                   \
            }                                                                                      \
            hipLaunchKernelGGL((topk_kernel<S, N, true>), grid, block, lds, st, score, idx, idx_sorted, lens, rows, nbk, k_sel, k_rows, stride);  \
        } else {                                                                                   \
            hipLaunchKernelGGL((topk_kernel<S, N, false>), grid, block, 0, st, score, idx, idx_sorted, lens, rows, nbk, k_sel, k_rows, stride); \
        }                                                                                          \
    } while (0)
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
        dim3 grid((nbk + kScoreCols - 1) / kScoreCols, (nbq + 127) / 128, BH);
        if (dtype == BSA_BF16)
            hipLaunchKernelGGL((score_mfma_kernel<__bf16>), grid, dim3(256), 0, st,
                               (const __bf16*)q_cmp, (const __bf16*)k_cmp, (__bf16*)score, nbq, nbk);
        else
            hipLaunchKernelGGL((score_mfma_kernel<_Float16>), grid, dim3(256), 0, st,
                               (const _Float16*)q_cmp, (const _Float16*)k_cmp, (_Float16*)score, nbq, nbk);
    }
    return hipGetLastError();
}

hipError_t launch_topk(const void* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                       int nbk, int k_sel, int dtype, hipStream_t st, const int32_t* k_rows, int stride) {
    if (stride <= 0) stride = k_sel;
    if (dtype == BSA_F32)
        return launch_topk_t<uint32_t>((const uint32_t*)score, idx, idx_sorted, lens, rows, nbk, k_sel, k_rows, stride, st);
    return launch_topk_t<uint16_t>((const uint16_t*)score, idx, idx_sorted, lens, rows, nbk, k_sel, k_rows, stride, st);
}

hipError_t launch_pace_order(const int32_t* in, int32_t* out, const int32_t* lens, int64_t rows, int nbk, int stride,
                             hipStream_t st) {
    if (rows <= 0 || stride <= 0) return hipSuccess;
    const int groups = (stride + kPaceWidth - 1) / kPaceWidth;
    const size_t lds = ((size_t)3 * stride + groups) * sizeof(int32_t);
    if (lds > 64 * 1024 || rows > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(pace_order_kernel, dim3((unsigned)rows), dim3(64), lds, st, in, out, lens, nbk, stride);
    return hipGetLastError();
}

hipError_t launch_cdf_count(const void* score, int32_t* lens, int64_t rows, int nbk, float threshold, float scale,
                            int k_min, int cap, int dtype, hipStream_t st) {
    if (dtype == BSA_F32)
        return launch_cdf_count_t<uint32_t>((const uint32_t*)score, lens, rows, nbk, threshold, scale, k_min, cap, dtype, st);
    return launch_cdf_count_t<uint16_t>((const uint16_t*)score, lens, rows, nbk, threshold, scale, k_min, cap, dtype, st);
}

}  // namespace bsa
