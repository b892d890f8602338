// Block-sparse flash-attention forward for gfx950 (bf16 / fp16 MFMA) on K and V held in
// "fragment order", and the pass that produces that order.
//
// Why another layout.  The kernel of bsa_fwd.hip stages row-major K/V tiles in LDS, where every
// byte is written once and read twice (two wavefronts share each 32-key half): 96 KB of LDS
// traffic per 64 x 64 tile against 512 clocks of MFMA per SIMD, which makes LDS, not the matrix
// unit, its roofline.  Here a wavefront owns all 64 query rows of a work item, so every K and V
// fragment feeds two MFMAs (one per 32 query rows) and is needed by this wavefront alone: it is
// loaded from global memory straight into registers, in exactly the lane order the MFMA operand
// wants, and LDS carries nothing in the tile loop - no staging, no swizzle, no barrier.  That
// needs K and V in a layout whose every 1 KB is one operand fragment (below), written once per
// layer by frag_kernel from the (T, H, W)-ordered tensors (a pass at HBM speed, which also
// replaces the zero-filled copies of the chunks at the padded high edge of the grid).
//
// Fragment order, per 64-key tile (16 KB for K, 16 KB for V; two 8 KB halves of 32 keys):
//   K: [half kh][d step c = 0..7][lane l = 0..63][8 elements]
//        element j of lane l = K[key 32 kh + (l & 31)][d = 16 c + 8 (l >> 5) + j]
//      = the A operand of v_mfma_f32_32x32x16 for S^T (32 keys x 32 queries) += K . Q^T.
//   V: [half kh][key step s = 0..1][d tile t = 0..3][lane l][8 elements]
//        element j of lane l = V[key 32 kh + 16 s + 8 (j >> 2) + 4 (l >> 5) + (j & 3)][d = 32 t + (l & 31)]
//      = the A operand of O^T (32 d x 32 queries) += V^T . P^T, with the 16 keys of a step in the
//        order in which the accumulator registers of S^T hold them, so that P^T needs no shuffle.
//
// Work decomposition.  One wavefront (a workgroup of 64 threads, one per SIMD) = one work item =
// 64 query rows against its list of KV blocks, walked in steps of 32 keys (half a tile).  Per
// step: 16 MFMAs for S^T of the next step interleaved with the exp2 / row sum / rounding of the
// current one, then 16 MFMAs for O^T += V^T P^T interleaved with the row maximum of the next.
// K and V fragments of the following steps are in flight in register rings (kRing steps each).
// The output accumulators (128 registers) and the rings live in the 512-register file that a
// single wavefront per SIMD has to itself.
//
// Softmax: lazy running maximum as in bsa_fwd.hip (raised only when exceeded by 2^8); numerics
// follow flash_attn_bsa_varlen_mask.py:242-285: fp32 logits, scale * log2(e) applied after the
// dot, exp2, P rounded to the storage type for the P V product, fp32 row sum, one final rounding.
#include "bsa_mfma.h"
#include "bsa_rope.h"

#include <type_traits>
#include <utility>

namespace bsa {
namespace {

using namespace mfma;

constexpr int kHalfBytes = 8192;      // 32 keys of a fragment-order K (or V) tile
constexpr int kListEntries = 4096;    // longest list a work item can walk (its staging area in LDS: 17 KB)

template <int kCtrl>
__device__ __forceinline__ float dpp_f32(float x) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), kCtrl, 0xf, 0xf, true));
}

// key_norm[batch * heads + head] = the largest entry of the head's tile norms (see frag_kernel)
__global__ __launch_bounds__(256) void head_norm_kernel(const float* __restrict__ tile_norm, float* __restrict__ key_norm, int tiles) {
    __shared__ float part[4];
    float best = 0.f;
    for (int i = threadIdx.x; i < tiles; i += 256) {
        const float x = tile_norm[(int64_t)blockIdx.x * tiles + i];
        best = x != x ? INFINITY : fmaxf(best, x);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) best = fmaxf(best, __shfl_xor(best, off));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) key_norm[blockIdx.x] = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// ------------------------------------------------------------------ relayout
// One workgroup per 64-slot tile of one (batch, head): the 64 rows are gathered from (T, H, W) order
// (padded slots: zeros) into LDS and written out as 16 fragments of 1 KB.  K (TRANSPOSE = false) moves
// 16-byte pieces; V (TRANSPOSE = true) gathers 8 keys of one d per piece.
// For K of 64-slot chunks the same pass can also produce what the pooling pass of bsa_permute.hip would: the chunk
// mean (pooled, in the storage type given by is_bf16; the summation order of permute_kernel is reproduced, so the
// two routes give the same bits) and the validity word of the tile.
// With a row transform (TRANSPOSE = false only) every row goes through the per-head RMSNorm and / or the 3-D RoPE
// of the attention module on its way (bsa_rope.h: the bits of the stand-alone pass), before the chunk means are
// taken; the transformed rows can also be written out at their token positions (the q of the attention kernel).
template <typename T, bool TRANSPOSE>
__global__ __launch_bounds__(256) void frag_kernel(const T* __restrict__ src, int64_t sB, int64_t sH, int64_t sS,
                                                   char* __restrict__ dst, Grid3 g, int Hn, T* __restrict__ pooled,
                                                   uint64_t* __restrict__ tile_valid, int is_bf16, RowTransform tr,
                                                   float* __restrict__ tile_norm) {
    // rows padded to 264 B for K (16-byte pieces read row by row) and to 288 B for V, whose transposing reads
    // fetch 4 keys x 16 d per 16 lanes: with rows 72 banks apart the four keys of a patch fall on different banks
    constexpr int kPitch = TRANSPOSE ? kD + 16 : kD + 4;
    __shared__ __attribute__((aligned(16))) T tile[kTile * kPitch];
    const int tiles_per_chunk = g.chunk() / kTile;
    // Workgroup -> (tile, batch * head).  For a token-major source (the heads of a token next to each other, as a
    // QKV projection leaves them) the heads of one tile run side by side, so that the 256-byte rows they fetch share
    // DRAM pages and cache lines' neighbourhoods; otherwise the tiles of one head do.
    const int tiles = g.blocks() * tiles_per_chunk;
    int tile_id, bh;
    if (tr.head_fastest) {
        const int per_batch = tiles * Hn, b = blockIdx.x / per_batch, rest = blockIdx.x - b * per_batch;
        tile_id = rest / Hn;
        bh = b * Hn + (rest - tile_id * Hn);
    } else {
        bh = blockIdx.x / tiles;
        tile_id = blockIdx.x - bh * tiles;
    }
    const int blk = tile_id / tiles_per_chunk, sub = tile_id % tiles_per_chunk;
    const int nw = blk % g.Nw, nh = (blk / g.Nw) % g.Nh, nt = blk / (g.Nw * g.Nh);
    const T* sbase = src + (int64_t)(bh / Hn) * sB + (int64_t)(bh % Hn) * sH;
    const int c16 = threadIdx.x & 15, rg = threadIdx.x >> 4;      // 16 pieces of 16 B per row, 16 rows at a time
    // Rotation: a chunk spans at most 8 positions per axis, and a rotation pair turns with one axis only, so the
    // (cos, sin) the 64 rows need are 8 x 64 table entries, fetched once per workgroup instead of per row and head.
    __shared__ float2 cs[8 * 64];
    if (!TRANSPOSE && tr.tab != nullptr) {
        for (int e = threadIdx.x; e < 8 * 64; e += 256) {
            const int a = e >> 6, pr = e & 63;
            int at, dsin;
            if (pr < kRopePairsT) {
                at = min(tr.t0 + nt * g.t + a, tr.Ttab - 1) * kRopePairsT + pr;
                dsin = tr.Ttab * kRopePairsT;
            } else if (pr < kRopePairsT + kRopePairsH) {
                at = 2 * tr.Ttab * kRopePairsT + min(nh * g.h + a, g.H - 1) * kRopePairsH + pr - kRopePairsT;
                dsin = g.H * kRopePairsH;
            } else {
                at = 2 * tr.Ttab * kRopePairsT + 2 * g.H * kRopePairsH + min(nw * g.w + a, g.W - 1) * kRopePairsW + pr - kRopePairsT - kRopePairsH;
                dsin = g.W * kRopePairsW;
            }
            cs[e] = make_float2(tr.tab[at], tr.tab[at + dsin]);
        }
        __syncthreads();
    }
    uint2 val[4][2];
    uint4 xs[4];
    int64_t token_of[4];         // -1: a padded slot
    int loc[4];                  // position inside the chunk, ti | hi << 8 | wi << 16
    // all four loads first, then the arithmetic: a row transformed right behind its own load would wait for it
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = sub * kTile + rg + 16 * i;                   // slot inside the chunk
        const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
        const int tt = nt * g.t + ti, hh = nh * g.h + hi, ww = nw * g.w + wi;
        xs[i] = make_uint4(0, 0, 0, 0);
        token_of[i] = -1;
        loc[i] = ti | (hi << 8) | (wi << 16);
        if (tt < g.T && hh < g.H && ww < g.W) {
            token_of[i] = ((int64_t)tt * g.H + hh) * g.W + ww;
            xs[i] = *reinterpret_cast<const uint4*>(sbase + token_of[i] * sS + c16 * 8);
        }
    }
    if (!TRANSPOSE && (tr.norm_w != nullptr || tr.tab != nullptr)) {
        uint4 wraw = make_uint4(0, 0, 0, 0);
        if (tr.norm_w != nullptr) wraw = *reinterpret_cast<const uint4*>(reinterpret_cast<const T*>(tr.norm_w) + c16 * 8);
        T* rows = tr.rows_out == nullptr ? nullptr
                                         : reinterpret_cast<T*>(tr.rows_out) + (int64_t)(bh / Hn) * tr.rB + (int64_t)(bh % Hn) * tr.rH + c16 * 8;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (token_of[i] < 0) continue;                         // the 16 lanes of a row go together
            float c[4] = {1.f, 1.f, 1.f, 1.f}, sn[4] = {0.f, 0.f, 0.f, 0.f};
            if (tr.tab != nullptr) {
                const int ti = loc[i] & 255, hi = (loc[i] >> 8) & 255, wi = loc[i] >> 16;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int pr = c16 * 4 + jj;
                    const float2 a = cs[(pr < kRopePairsT ? ti : pr < kRopePairsT + kRopePairsH ? hi : wi) * 64 + pr];
                    c[jj] = a.x;
                    sn[jj] = a.y;
                }
            }
            xs[i] = is_bf16 ? norm_rope_piece<__bf16>(xs[i], wraw, tr.norm_w != nullptr, tr.tab != nullptr, c, sn, tr.eps)
                            : norm_rope_piece<_Float16>(xs[i], wraw, tr.norm_w != nullptr, tr.tab != nullptr, c, sn, tr.eps);
            if (rows != nullptr) *reinterpret_cast<uint4*>(rows + token_of[i] * tr.rS) = xs[i];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        val[i][0] = make_uint2(xs[i].x, xs[i].y);
        val[i][1] = make_uint2(xs[i].z, xs[i].w);
    }
    if (!TRANSPOSE && tile_norm != nullptr) {
        // tile_norm[(batch * heads + head) * tiles + tile] = the largest Euclidean norm of a row of this tile as it is
        // stored (after the transform), a little above the exact value: the attention kernel bounds q . k by
        // |q| |k| with the largest of a head.  The sixteen lanes of a row add their squares (butterfly over
        // the row's lanes with DPP moves), then the maximum over the 64 rows.
        float best = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w[4] = {xs[i].x, xs[i].y, xs[i].z, xs[i].w};
            float sq = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo, hi;
                if (is_bf16) { lo = __uint_as_float(w[e] << 16); hi = __uint_as_float(w[e] & 0xffff0000u); }
                else { lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] & 0xffffu)); hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] >> 16)); }
                sq = fmaf(lo, lo, fmaf(hi, hi, sq));
            }
            sq += dpp_f32<0xB1>(sq);         // quad_perm [1, 0, 3, 2]
            sq += dpp_f32<0x4E>(sq);         // quad_perm [2, 3, 0, 1]
            sq += dpp_f32<0x141>(sq);        // row_half_mirror
            sq += dpp_f32<0x140>(sq);        // row_mirror
            best = fmaxf(best, sq);          // NaN squares drop out here; such a row has no bound (below)
            if (sq != sq) best = INFINITY;
        }
#pragma unroll
        for (int off = 32; off >= 16; off >>= 1) best = fmaxf(best, __shfl_xor(best, off));
        __shared__ float wave_best[4];
        if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
        __syncthreads();
        if (threadIdx.x == 0) {
            best = fmaxf(fmaxf(wave_best[0], wave_best[1]), fmaxf(wave_best[2], wave_best[3]));
            tile_norm[(int64_t)bh * tiles + tile_id] = __builtin_sqrtf(best) * 1.001f;
        }
    }
    if (!TRANSPOSE && tile_valid != nullptr && bh == 0 && threadIdx.x < 64) {
        const int r = sub * kTile + threadIdx.x;
        const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
        const uint64_t m = __ballot(nt * g.t + ti < g.T && nh * g.h + hi < g.H && nw * g.w + wi < g.W);
        if (threadIdx.x == 0) tile_valid[tile_id] = m;
    }
    if (!TRANSPOSE && pooled != nullptr) {
        // permute_kernel's order: a thread sums its rows rg, rg + 16, rg + 32, rg + 48 per element, then the 16
        // partial sums of a column are added in ascending rg; mean = sum * (1 / 64), rounded once
        __shared__ float red[16 * kD];
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w[4] = {val[i][0].x, val[i][0].y, val[i][1].x, val[i][1].y};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo, hi;
                if (is_bf16) { lo = __uint_as_float(w[e] << 16); hi = __uint_as_float(w[e] & 0xffff0000u); }
                else { lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] & 0xffffu)); hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] >> 16)); }
                acc[2 * e] += lo;
                acc[2 * e + 1] += hi;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) red[rg * kD + c16 * 8 + e] = acc[e];
        __syncthreads();
        if (threadIdx.x < kD) {
            float sum = 0.f;
            for (int gq = 0; gq < 16; ++gq) sum += red[gq * kD + threadIdx.x];
            sum *= 1.0f / 64.0f;
            uint16_t bits;
            if (is_bf16) bits = __builtin_bit_cast(uint16_t, (__bf16)sum);
            else bits = __builtin_bit_cast(uint16_t, (_Float16)sum);
            reinterpret_cast<uint16_t*>(pooled)[((int64_t)bh * tiles + tile_id) * kD + threadIdx.x] = bits;
        }
    }
    if (dst == nullptr) return;                                    // chunk means (and validity words) only
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        T* row = tile + (rg + 16 * i) * kPitch + c16 * 8;          // 8-byte aligned (pitch 264 B)
        *reinterpret_cast<uint2*>(row) = val[i][0];
        *reinterpret_cast<uint2*>(row + 4) = val[i][1];
    }
    __syncthreads();
    char* out = dst + ((int64_t)bh * tiles + tile_id) * kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = threadIdx.x + 256 * i;                       // 16-byte piece of the output, 0..1023
        const int l = e & 63, f = e >> 6;                          // lane and fragment
        const int lr = l & 31, lh = l >> 5;
        uint16_t piece[8];
        if (!TRANSPOSE) {
            const int kh = f >> 3, c = f & 7;
            const uint16_t* s = reinterpret_cast<const uint16_t*>(tile + (32 * kh + lr) * kPitch + 16 * c + 8 * lh);
#pragma unroll
            for (int j = 0; j < 8; ++j) piece[j] = s[j];
        } else {
            // ds_read_b64_tr_b16: the 16 lanes of a group point at a 4-key x 16-d patch (lane s at key s / 4,
            // d 4 (s % 4) .. + 4) and each receives the 4 keys of one d
            const int kh = f >> 3, s2 = (f >> 2) & 1, t = f & 3;
            const int s16 = l & 15, g1 = (l >> 4) & 1;
            const T* src_lo = tile + (32 * kh + 16 * s2 + 4 * lh + (s16 >> 2)) * kPitch + 32 * t + 16 * g1 + 4 * (s16 & 3);
            const s16x4 lo = lds_read_tr16(src_lo), hi = lds_read_tr16(src_lo + 8 * kPitch);
#pragma unroll
            for (int j = 0; j < 4; ++j) { piece[j] = (uint16_t)lo[j]; piece[4 + j] = (uint16_t)hi[j]; }
        }
        *reinterpret_cast<uint4*>(out + (int64_t)e * 16) = *reinterpret_cast<const uint4*>(piece);
    }
}

// ------------------------------------------------------------------ attention
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
// in every copy of the body (the register arrays of the kernel must never be indexed by a run-time value).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// acc + x[2e]^2 + x[2e+1]^2 for a fragment of eight 16-bit values
__device__ __forceinline__ float dot2_self(bf16x8 x, int e, float acc) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 p = {x[2 * e], x[2 * e + 1]};
    return __builtin_amdgcn_fdot2_f32_bf16(p, p, acc, false);
}
__device__ __forceinline__ float dot2_self(f16x8 x, int e, float acc) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 p = {x[2 * e], x[2 * e + 1]};
    return __builtin_amdgcn_fdot2(p, p, acc, false);
}

struct FragLayout {
    const int32_t* q_rows;        // token row of every blocked-order query slot, -1 = padding; null: q, o in blocked order
    int64_t q_st[3], o_st[3];     // element strides: batch, head, row
};

// Lists of at most this many entries are staged in LDS for the next work item while the current one runs.
constexpr int kPipeList = 256;

// kNsub1: KV blocks of one 64-key tile (bs_k == 64): no division in the walk.
//
// A workgroup (one wavefront) runs the work items b, b + round, b + 2 round, ... of its launch one after the other
// (or draws them from `queue`).  What an item needs before its first MFMA - its list, its Q rows, its first K and
// V fragments - is requested while the item before it still runs, so that an item costs its tile walk and an
// epilogue, not a chain of three dependent memory round trips:
//   * lens and the first list entry of the item after next are scalar loads issued at the start of an item;
//   * the next item's list goes into registers at the start of an item and into its LDS buffer at the end;
//   * the next item's Q rows go from global memory straight into an LDS staging tile (LDS DMA) and from there into
//     the Q registers once the current item's last S^T product has been issued;
//   * the positions of the tile walk behind the end of the list name the next item's first tile, so the fragment
//     rings hold K(0), K(1), V(0), V_A(1) of the next item when the loop ends - what its prologue would load.
// K and V fragments are read through buffer resources (an SGPR base, a 32-bit scalar tile offset, the lane's
// 16 bytes): no 64-bit vector address arithmetic in the loop, and an offset outside the buffer reads zeros.
// kBounded: the kernel for items whose logits are bounded below the level at which the running maximum would move
// (see where the bound is tested): its steps take no row maxima.  An item that fails the test is not computed but
// appended to `fallback` (its count in fallback_count), and the other instantiation, which takes its items from that
// list, runs behind it.
template <typename T, bool kNsub1, bool kBounded>
__global__ __launch_bounds__(64) void fwd_frag_kernel(
    const T* __restrict__ q, const char* __restrict__ kf, const char* __restrict__ vf,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens, const uint64_t* __restrict__ tile_valid,
    T* __restrict__ o, float* __restrict__ lse, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
    float qk_scale, int item_begin, int item_end, int round, int Hn, int64_t lse_S, FragLayout L,
    const int32_t* __restrict__ order, uint32_t* __restrict__ queue, const uint32_t* __restrict__ gate, uint32_t gate_want,
    int bh_first, uint32_t kv_span_bytes, int q_offsets_32, const float* __restrict__ key_norm,
    int32_t* __restrict__ fallback, uint32_t* __restrict__ fallback_count) {
    typedef typename Vec8<T>::type V8;
    // log2 headroom before the running maximum is raised: probabilities reach 2^kTau, which the storage type of P
    // must hold (fp16 ends at 65 504) and the fp32 sums must hold times the number of keys
    constexpr float kTau = std::is_same<T, _Float16>::value ? 14.0f : 30.0f;
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    if (gate != nullptr && *gate != gate_want) return;
    // output staging: 64 rows of 256 B, 272 B apart.  The same memory stages a list that is too long for the small
    // buffers (kListEntries words at most) during the tile loop of an item that was not prepared ahead of time.
    constexpr int kOutPitch = kD + 8;
    __shared__ __attribute__((aligned(16))) T ost[kTile * kOutPitch];
    __shared__ uint32_t lists[2][kPipeList];
    __shared__ int32_t out_rows[2][kTile];       // token rows of this and the next item's 64 query slots (row table given)
    __shared__ __attribute__((aligned(16))) char qstage[kTileBytes];      // Q of the next item, in register order
    uint32_t* const big = reinterpret_cast<uint32_t*>(ost);

    const int lane = threadIdx.x;
    const int lr = lane & 31, lh = lane >> 5;
    const int nbq = (int)(Sq / bs_q);
    const int nqt = (int)(Sq / kTile);
    const int nsub = kNsub1 ? 1 : bs_k / kTile;
    const int nbk = (int)(Sk / bs_k);
    const int tiles_bh = (int)(Sk / kTile);
    const uint32_t lane_off = (uint32_t)lane * 16u;
    // the kernel that runs the fallback list takes as many items as the list holds
    const int n_launch = kBounded ? item_end - item_begin
                                  : (fallback_count != nullptr ? __builtin_amdgcn_readfirstlane((int)min(*fallback_count, (uint32_t)(item_end - item_begin)))
                                                               : item_end - item_begin);

    const int64_t kv_bh_bytes = (int64_t)tiles_bh * kTileBytes;
    const __amdgpu_buffer_rsrc_t krs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(kf) + bh_first * kv_bh_bytes, 0, (int)kv_span_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(vf) + bh_first * kv_bh_bytes, 0, (int)kv_span_bytes, 0x00020000);
    // tile: index of the 64-key tile counted from (batch, head) bh_first; h: its half; c / f: fragment of the half
    auto k_frag = [&](uint32_t tile, int h, int c) -> V8 {
        const uint32_t so = tile * (uint32_t)kTileBytes + (uint32_t)(h * kHalfBytes + (c >> 2) * 4096);
        return __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(krs, lane_off + (uint32_t)((c & 3) * 1024), so, 0));
    };
    auto v_frag = [&](uint32_t tile, int h, int f) -> V8 {          // f = 4 * key step + d tile
        const uint32_t so = tile * (uint32_t)kTileBytes + (uint32_t)(h * kHalfBytes + (f >> 2) * 4096);
        return __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(vrs, lane_off + (uint32_t)((f & 3) * 1024), so, 0));
    };

    // ---- which items this workgroup runs
    // The launch's items are taken in rounds of `round` (a multiple of 8).  Workgroup b runs on XCD b % 8: within
    // a round every XCD takes a contiguous run of the round's items.
    auto round_local = [&](int r) -> int {
        const int64_t r0 = (int64_t)r * round;
        if (r0 >= n_launch) return -1;
        const int n = min(round, n_launch - (int)r0), w = blockIdx.x, x = w & 7;
        if (w >= n) return -1;
        return (int)r0 + x * (n >> 3) + min(x, n & 7) + (w >> 3);
    };
    auto draw = [&]() -> int {
        uint32_t drawn = 0;
        if (lane == 0) drawn = atomicAdd(queue, 1u);
        const uint32_t l = (uint32_t)__builtin_amdgcn_readfirstlane((int)drawn);
        return l < (uint32_t)n_launch ? (int)l : -1;
    };
    int rounds_taken = 0;
    auto next_local = [&]() -> int { return queue != nullptr ? draw() : round_local(rounds_taken++); };
    // what is known of an item ahead of time: its number, the length of its list and its first entry (both as
    // they lie in memory; they are clamped where they are used)
    struct Desc { int item, nent, blk0; float kn; };
    auto fetch = [&](int local) -> Desc {
        Desc d = {-1, 0, 0, INFINITY};
        if (local < 0) return d;
        d.item = item_begin + (order != nullptr ? order[local] : local);
        const int bh = d.item / nqt, qblock = (int)((int64_t)(d.item % nqt) * kTile / bs_q);
        const int64_t row = (int64_t)bh * nbq + qblock;
        d.nent = lens[row];
        if (idx_stride > 0) d.blk0 = idx[row * idx_stride];
        if (key_norm != nullptr) d.kn = key_norm[bh];
        return d;
    };
    // The descriptor's loads are vector loads of one address (behind the stores of an earlier item the compiler
    // does not use the scalar cache): the values are the same in every lane and are made scalars where they are used,
    // not where they are loaded, so that the wait for them stands there.
    auto uni = [](int x) -> int { return __builtin_amdgcn_readfirstlane(x); };
    auto list_length = [&](const Desc& d) -> int { return d.item < 0 ? 0 : min(min(max(uni(d.nent), 0), idx_stride), kListEntries); };
    auto first_tile = [&](const Desc& d) -> uint32_t {              // the tile position 0 of d's walk names
        const int bh = d.item / nqt;
        return (uint32_t)((bh - bh_first) * tiles_bh + min(max(uni(d.blk0), 0), nbk - 1) * nsub);
    };

    // ---- registers that live across items
    V8 qreg[2][8];
    // Register rings: K fragments of two steps, V fragments of two steps (each step: 4 fragments for its
    // first 16 keys, "A", and 4 for its last 16, "B").
    V8 kb[2][8], vb[2][8];
    f32x16 s[2][2];                                            // S^T of the current and of the next step
    V8 pb[2][2];                                               // P^T as B operand: [query half][A | B]
    f32x16 oacc[4][2];
    float m_i[2], l_i[2];
    // Softmax state per query half: running maximum m_i (scaled, log2 units), its negative for the exponent
    // (0 while the maximum is -inf), and the unscaled logit above which the maximum has to be raised.
    float neg_m[2], raise_at[2];
    const float inv_scale = 1.0f / qk_scale;
    // Raising the
    // maximum has two parts.  Here: the new maximum, the exponent offset, the row sum (which already holds
    // every probability of the current step).  The output accumulators are rescaled one quarter of a step later
    // (rescale_out, behind slot 7 of the next step): the product of the current step's P_B, whose
    // probabilities were taken relative to the old maximum, is only issued in slots 0 .. 7 of that step.
    float alpha_p[2];
    bool rescale_pending = false;

    // Q fragments of one query half into their registers, and the lane's part of the rows' squared norms.  Half 1 is
    // read by the assembly MFMAs from accumulation registers.  Its values pass through an assembly statement that
    // ties them to that register class: a value that C++ code also reads (the squares) the compiler would keep in
    // ordinary registers and copy in front of every MFMA that names it, without the wait states such a copy needs.
    float q_sq[2] = {0.f, 0.f};
    auto take_q = [&](int qq, V8 (&rows)[8]) {
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) sq = dot2_self(rows[c], e, sq);
        q_sq[qq] = sq;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (qq == 1) asm volatile("" : "=a"(qreg[1][c]) : "0"(rows[c]));
            else asm volatile("" : "=v"(qreg[0][c]) : "0"(rows[c]));
        }
    };

    // ---- per item
    int ntiles = 0;
    uint32_t tile_base = 0;          // first tile of the item's (batch, head)
    uint32_t beyond_tile = 0;        // what the positions behind the end of the list name
    const uint32_t* ents = big;      // the item's list in LDS
    // window of the walk: positions g, g + 1, g + 2 of loop iteration g (one tile per iteration)
    uint32_t w_tile[3];
    uint64_t w_mask[3];

    // Position tp of the tile walk -> tile and validity word of its 64 keys.  Positions behind the list name
    // `beyond_tile` with every key masked out.  The entry is read from LDS (entry_raw, to be issued early) and
    // decoded later (entry_tile / entry_mask).
    auto entry_raw = [&](int tp) -> uint32_t {
        const int tc = min(tp, ntiles - 1);
        return ents[kNsub1 ? tc : tc / nsub];                   // the same address in every lane
    };
    auto entry_tile = [&](int tp, uint32_t raw) -> uint32_t {
        if (tp >= ntiles) return beyond_tile;
        const int blk = min(max(__builtin_amdgcn_readfirstlane((int)raw), 0), nbk - 1);   // a malformed list: wrong numbers, never a fault
        if (kNsub1) return tile_base + (uint32_t)blk;
        return tile_base + (uint32_t)(blk * nsub + tp % nsub);
    };
    // the validity word of a tile (all keys valid without padding), in two steps so that a caller can ask for several
    // words before it waits for the first
    auto entry_word = [&](int tp, uint32_t tile) -> uint64_t {
        if (tile_valid == nullptr) return ~0ull;
        return tile_valid[tp >= ntiles ? 0u : tile - tile_base];                        // behind the list: another head's tile
    };
    auto mask_of = [&](int tp, uint64_t word) -> uint64_t {
        // the same word in every lane; made a scalar by hand (behind the stores of an earlier item's output the
        // compiler reads it with a vector load)
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)word);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(word >> 32));
        const uint32_t keep = tp >= ntiles ? 0u : ~0u;
        return (uint64_t)(lo & keep) | ((uint64_t)(hi & keep) << 32);
    };
    auto entry_mask = [&](int tp, uint32_t tile) -> uint64_t { return mask_of(tp, entry_word(tp, tile)); };
    // accumulator i <-> key 8 (i / 4) + 4 lh + i % 4 of the step's 32 keys, query lr (+32)
    auto mask_pair = [&](f32x16 (&sv)[2], uint32_t half) {
        if (__builtin_expect(half != ~0u, 0)) {
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");       // the MFMAs into these accumulators have retired
            // the lane's part of the shift first: the tests below then use constants, not sixteen per-lane bit masks
            // that would have to be kept in registers (or spilled) all through the loop for this rare path
            uint32_t mine = half >> (4 * lh);
            asm volatile("" : "+v"(mine));
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (!((mine >> (8 * (i / 4) + (i % 4))) & 1u)) { sv[0][i] = -INFINITY; sv[1][i] = -INFINITY; }
        }
    };
    // combine a lane's maximum with the other key group of the same query (lane ^ 32)
    auto finish_max = [&](float mx) -> float {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
        return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    };
    // mx0, mx1: this lane's unscaled maxima over its 16 accumulators of the step that comes next.  The test
    // needs no exchange between the two key groups of a query: some lane exceeds the limit exactly when the
    // combined maximum does.
    auto raise_max = [&](float mx0, float mx1) {
        if (__builtin_expect(__any(mx0 > raise_at[0] || mx1 > raise_at[1]), 0)) {
            const float mx[2] = {finish_max(mx0) * qk_scale, finish_max(mx1) * qk_scale};
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                const float m_new = fmaxf(m_i[qq], mx[qq]);
                const float alpha = __builtin_amdgcn_exp2f(m_i[qq] - ((m_new == -INFINITY) ? 0.f : m_new));
                m_i[qq] = m_new;
                neg_m[qq] = (m_new == -INFINITY) ? 0.f : -m_new;
                raise_at[qq] = (m_new + kTau) * inv_scale;
                l_i[qq] *= alpha;
                alpha_p[qq] = alpha;
            }
            rescale_pending = true;
        }
    };
    // The output accumulators live in AGPRs, which the VALU cannot multiply in place.  Written out register by
    // register through one temporary, so that this rare path does not make the compiler reserve VGPRs for a copy
    // of the accumulators.
    auto rescale_out = [&]() {
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMA into the accumulators has retired
        static_for<128>([&](auto n_c) {
            constexpr int n = decltype(n_c)::value, qq = n >> 6, t = (n >> 4) & 3, i = n & 15;
            float x = oacc[t][qq][i], tmp;
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1"
                         : "+a"(x), "=&v"(tmp) : "v"(alpha_p[qq]));
            oacc[t][qq][i] = x;
        });
        asm volatile("s_nop 7" ::: "memory");                        // AGPR writes before the next MFMA reads them
        rescale_pending = false;
    };

    // Step u = 2 g + j (j static).  On entry S(u) is complete and the running maximum covers it; P_B(u-1) is
    // complete.  The 32 MFMAs of a step, in issue order ("slots"):
    //    0 ..  7   O^T += V_B(u-1)^T P_B(u-1)^T      the last 16 keys of the previous step
    //    8 .. 23   S(u+1)^T = K(u+1) Q^T
    //   24 .. 31   O^T += V_A(u)^T P_A(u)^T          the first 16 keys of this step
    // The VALU work on S(u) - per pair of accumulators two fma, two exp2, two additions for the row sum and one
    // rounding of the pair to the storage type, 16 pairs - is cut into pieces that go between the MFMAs so that
    // no gap holds more than an MFMA lasts: the first 14 pairs behind slots 0 .. 23 (the eight pairs of P_A
    // first: they are complete well before slot 24), the last two behind slots 24 .. 31 together with the row
    // maximum of S(u+1), which is complete by then.  Fragment registers are reloaded in bursts behind the last
    // MFMA that reads them: V_B(u+1) behind slot 7, K(u+3) behind slot 23, V_A(u+2) behind slot 31, so that every
    // fragment is requested two steps before it is used.  Within a burst the fragment that is used first is
    // requested last: loads return in order, so the wait in front of its first use covers the whole burst and
    // the fragments behind it need none of their own.
    auto step = [&](auto jj) {
        constexpr int j = decltype(jj)::value;
        constexpr int sc = j & 1, sn = sc ^ 1;                 // S(u) and S(u+1) alternate between two register sets
        constexpr int kslot = (j + 1) & 1;                     // ring slot of K(u+1), then of K(u+3)
        constexpr int vprev = (j + 1) & 1, vcur = j & 1;       // ring slots of V(u-1) / V(u+1) and of V(u) / V(u+2)
        // pair n: query half n & 1, accumulators 2 (n >> 1), + 1.  Its arithmetic comes in three pieces of about the
        // same cost - exponential of the first accumulator (h0), of the second (h1), and the use of both: row sum
        // and rounding (t) - in the order h0(0) h1(0) h0(1) t(0) h1(1) h0(2) t(1) h1(2) ...: the result of a
        // transcendental instruction cannot be consumed by the next instruction without a wait state.
        float pa[2][2];
        auto piece = [&](int p) {                               // p = 0 .. 47
            // p = 0: h0(0); p = 1: h1(0); p = 2 + 3 k: h0(k + 1); p = 3 + 3 k: t(k); p = 4 + 3 k: h1(k + 1); p = 47: t(15)
            const int k = p < 2 ? 0 : (p - 2) / 3, r = p < 2 ? 0 : (p - 2) % 3;
            const bool is_t = p == 47 || (p >= 2 && r == 1);
            const int n = p < 2 ? 0 : p == 47 ? 15 : (r == 1 ? k : k + 1);
            const int e = p < 2 ? p : (r == 0 ? 0 : 1);         // which accumulator of the pair (h0 / h1)
            const int qq = n & 1, i = 2 * (n >> 1);
            if (is_t) {
                l_i[qq] += pa[n & 1][0] + pa[n & 1][1];
                pb[qq][i >> 3][i & 7] = (T)pa[n & 1][0];
                pb[qq][i >> 3][(i + 1) & 7] = (T)pa[n & 1][1];
                asm volatile("" : "+v"(l_i[qq]), "+v"(pb[qq][i >> 3]));
            } else {
                pa[n & 1][e] = __builtin_amdgcn_exp2f(fmaf(s[sc][qq][i + e], qk_scale, neg_m[qq]));
                asm volatile("" : "+v"(pa[n & 1][e]));
            }
        };
        float mx[2];
        __builtin_amdgcn_sched_barrier(0);
        static_for<32>([&](auto slot_c) {
            constexpr int slot = decltype(slot_c)::value;
            // ---- the MFMA of this slot
            if constexpr (slot < 8) {
                constexpr int t = slot >> 1, qq = slot & 1;
                oacc[t][qq] = mfma32(vb[vprev][4 + t], pb[qq][1], oacc[t][qq]);
            } else if constexpr (slot < 24) {
                constexpr int c = (slot - 8) >> 1, qq = slot & 1;
                if constexpr (qq == 0) {
                    if constexpr (c == 0) mfma_s<true, false>(s[sn][0], kb[kslot][0], qreg[0][0]);
                    else mfma_s<false, false>(s[sn][0], kb[kslot][c], qreg[0][c]);
                } else {
                    if constexpr (c == 0) mfma_s<true, true>(s[sn][1], kb[kslot][0], qreg[1][0]);
                    else mfma_s<false, true>(s[sn][1], kb[kslot][c], qreg[1][c]);
                }
            } else {
                constexpr int t = (slot - 24) >> 1, qq = slot & 1;
                oacc[t][qq] = mfma32(vb[vcur][t], pb[qq][0], oacc[t][qq]);
            }
            // ---- reloads, in bursts behind the last MFMA that reads the fragments (single loads between the
            // arithmetic cost more issue time than they take): V_B(u+1), K(u+3), V_A(u+2)
            if constexpr (slot == 7) {
#pragma unroll
                for (int tt = 1; tt <= 4; ++tt) vb[vprev][4 + (tt & 3)] = v_frag(w_tile[(j + 1) >> 1], (j + 1) & 1, 4 + (tt & 3));
            }
            if constexpr (slot == 23) {
#pragma unroll
                for (int cc = 1; cc <= 8; ++cc) kb[kslot][cc & 7] = k_frag(w_tile[(j + 3) >> 1], (j + 1) & 1, cc & 7);
            }
            if constexpr (slot == 31) {
#pragma unroll
                for (int tt = 1; tt <= 4; ++tt) vb[vcur][tt & 3] = v_frag(w_tile[(j + 2) >> 1], j & 1, tt & 3);
            }
            if constexpr (slot == 7) {
                if (__builtin_expect(rescale_pending, 0)) rescale_out();
            }
            // ---- VALU pieces: 42 of the 48 (14 pairs) behind slots 0 .. 23, one or two per slot; the other 6 behind
            // slots 24 .. 31 next to the row maximum of S(u+1).  S(u+1) is first read behind slot 25: its last MFMA
            // (slot 23) has retired by the time the MFMA of slot 25 has been issued, which the compiler cannot
            // check for the assembly MFMAs.
            if constexpr (slot < 24) {
                constexpr int lo = (slot * 42) / 24, hi = ((slot + 1) * 42) / 24;      // one or two pieces
                piece(lo);
                if constexpr (hi - lo > 1) piece(lo + 1);
            } else {
                constexpr int r = slot - 24;                    // 0 .. 7
                if constexpr (r == 0) { piece(42); piece(43); }
                if constexpr (r == 1) {
                    mfma_chain_end(s[sn][0]);
                    mfma_chain_end(s[sn][1]);
                    // validity of the keys of step u + 1: tile window slot (j + 1) / 2, half (j + 1) & 1
                    mask_pair(s[sn], (uint32_t)(w_mask[(j + 1) >> 1] >> (32 * ((j + 1) & 1))));
                    if constexpr (!kBounded) {
                        mx[0] = fmaxf(fmaxf(s[sn][0][0], s[sn][0][1]), s[sn][0][2]);
                        mx[1] = fmaxf(fmaxf(s[sn][1][0], s[sn][1][1]), s[sn][1][2]);
                        mx[0] = fmaxf(fmaxf(mx[0], s[sn][0][3]), s[sn][0][15]);
                        mx[1] = fmaxf(fmaxf(mx[1], s[sn][1][3]), s[sn][1][15]);
                    }
                }
                if constexpr (!kBounded && r >= 2 && r < 7) {   // accumulators 4 .. 13, two per slot and query half
                    mx[0] = fmaxf(fmaxf(mx[0], s[sn][0][2 * r]), s[sn][0][2 * r + 1]);
                    mx[1] = fmaxf(fmaxf(mx[1], s[sn][1][2 * r]), s[sn][1][2 * r + 1]);
                }
                if constexpr (!kBounded && r == 7) {
                    mx[0] = fmaxf(mx[0], s[sn][0][14]);
                    mx[1] = fmaxf(mx[1], s[sn][1][14]);
                }
                if constexpr (r == 2) piece(44);
                if constexpr (r == 4) piece(45);
                if constexpr (r == 6) piece(46);
                if constexpr (r == 7) piece(47);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (!kBounded) raise_max(mx[0], mx[1]);
    };

    // ---- the workgroup's items
    Desc cur = fetch(next_local());
    Desc nxt = fetch(next_local());
    bool prepared = false;           // the current item's list, Q rows and first fragments were requested by the item before it
    int list_buf = 0;                // which of the small list buffers holds the current item's list, if prepared
    while (uni(cur.item) >= 0) {
        cur.item = uni(cur.item);
        const Desc nx2 = fetch(next_local());                    // in flight while this item runs
        const int bh = cur.item / nqt;
        const int qtile = cur.item % nqt;
        const int64_t qrow0 = (int64_t)qtile * kTile;
        const int qblock = (int)(qrow0 / bs_q);
        const int64_t o_bh = (int64_t)(bh / Hn) * L.o_st[0] + (int64_t)(bh % Hn) * L.o_st[1];
        const int nent = list_length(cur);
        ntiles = uni(nent * nsub);
        tile_base = (uint32_t)uni((bh - bh_first) * tiles_bh);
        // the next item can be prepared while this one runs if this one has a loop to hide it behind, the next one
        // has a first tile to point the walk at, a list that fits a small buffer, and Q rows the LDS DMA can address
        const int next_nent = list_length(nxt);
        const bool prepare_next = nxt.item >= 0 && ntiles > 0 && next_nent > 0 && next_nent <= kPipeList && q_offsets_32 != 0;
        beyond_tile = (uint32_t)uni((int)(prepare_next ? first_tile(nxt) : tile_base));
        const int nbh = prepare_next ? nxt.item / nqt : 0;
        const int64_t nqrow0 = prepare_next ? (int64_t)(nxt.item % nqt) * kTile : 0;
        const int32_t* nlist = idx + ((int64_t)nbh * nbq + nqrow0 / bs_q) * idx_stride;

        if (!prepared) {
            // Q as the B operand of S^T: lane holds rows lr and 32 + lr, d = 16 c + 8 lh .. +8.  Requested before the
            // list is staged, so that the two chains of dependent loads (row table -> Q rows, list -> LDS) run side by side.
            const int64_t q_bh = (int64_t)(bh / Hn) * L.q_st[0] + (int64_t)(bh % Hn) * L.q_st[1];
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                int64_t row = qrow0 + 32 * qq + lr;
                if (L.q_rows != nullptr) row = max(L.q_rows[row], 0);          // padded slots read token 0, never stored
                const T* qp = q + q_bh + row * L.q_st[2] + 8 * lh;
                V8 rows[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) rows[c] = *reinterpret_cast<const V8*>(qp + 16 * c);
                take_q(qq, rows);
            }
            const int32_t* list = idx + ((int64_t)bh * nbq + qblock) * idx_stride;
            int lane_now = lane;                                     // see the epilogue
            asm volatile("" : "+v"(lane_now));
            if (L.q_rows != nullptr) out_rows[list_buf][lane_now] = L.q_rows[qrow0 + lane_now];
            for (int e = lane_now; e < nent; e += 64) big[e] = (uint32_t)list[e];
            ents = big;
            __syncthreads();
        } else {
            ents = lists[list_buf];
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                V8 rows[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) rows[c] = *reinterpret_cast<const V8*>(qstage + (qq * 8 + c) * 1024 + lane_off);
                take_q(qq, rows);
            }
        }
        m_i[0] = m_i[1] = -INFINITY;
        l_i[0] = l_i[1] = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int qq = 0; qq < 2; ++qq)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[t][qq][i] = 0.f;

        bool run = true;                     // this kernel computes the item (see the bound on q . k below)
        if (ntiles > 0) {
            {
                // the three entries, then the three words, each kind in one sweep: one wait per kind instead of three
                uint32_t raw3[3];
                uint64_t word3[3];
#pragma unroll
                for (int r = 0; r < 3; ++r) raw3[r] = entry_raw(r);
#pragma unroll
                for (int r = 0; r < 3; ++r) w_tile[r] = entry_tile(r, raw3[r]);
#pragma unroll
                for (int r = 0; r < 3; ++r) word3[r] = entry_word(r, w_tile[r]);
#pragma unroll
                for (int r = 0; r < 3; ++r) w_mask[r] = mask_of(r, word3[r]);
            }
            // ---- prologue.  In flight when the loop starts: K(1), K(2), V_A(0), V_B(0), V_A(1); the ring slot of
            // V_B(1) holds zeros, which the first step multiplies with P = 0 (there is no step -1).  A prepared item
            // finds all of them but K(2) requested already (K(0) sits where K(2) belongs until S(0) has been issued).
            if (!prepared) {
#pragma unroll
                for (int c = 0; c < 8; ++c) kb[0][c] = k_frag(w_tile[0], 0, c);             // K(0)
#pragma unroll
                for (int c = 0; c < 8; ++c) kb[1][c] = k_frag(w_tile[0], 1, c);             // K(1)
#pragma unroll
                for (int f = 0; f < 8; ++f) vb[0][f] = v_frag(w_tile[0], 0, f);             // V_A(0), V_B(0)
#pragma unroll
                for (int f = 0; f < 4; ++f) vb[1][f] = v_frag(w_tile[0], 1, f);             // V_A(1)
            }
#pragma unroll
            for (int f = 4; f < 8; ++f)
#pragma unroll
                for (int e = 0; e < 8; ++e) vb[1][f][e] = (T)0.f;
#pragma unroll
            for (int qq = 0; qq < 2; ++qq)
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[qq][1][e] = (T)0.f;
            neg_m[0] = neg_m[1] = 0.f;
            raise_at[0] = raise_at[1] = -INFINITY;
            alpha_p[0] = alpha_p[1] = 1.f;
            // the token rows of the next item's queries are looked up now; its list and its Q rows are asked for once
            // it is known that this item runs here
            int32_t next_rows[2] = {0, 0};
            if (prepare_next) {
#pragma unroll
                for (int qq = 0; qq < 2; ++qq) {
                    const int64_t row = nqrow0 + 32 * qq + lr;
                    next_rows[qq] = L.q_rows != nullptr ? L.q_rows[row] : (int32_t)row;      // used (and clamped) behind S(0): no wait here
                }
            }
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                if (c == 0) { mfma_s<true, false>(s[0][0], kb[0][0], qreg[0][0]); mfma_s<true, true>(s[0][1], kb[0][0], qreg[1][0]); }
                else { mfma_s<false, false>(s[0][0], kb[0][c], qreg[0][c]); mfma_s<false, true>(s[0][1], kb[0][c], qreg[1][c]); }
            }
#pragma unroll
            for (int c = 0; c < 8; ++c) kb[0][c] = k_frag(w_tile[1], 0, c);                 // K(2), behind the last reader of K(0)
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");           // MFMA results before the VALU reads them
            mfma_chain_end(s[0][0]);
            mfma_chain_end(s[0][1]);
            mask_pair(s[0], (uint32_t)w_mask[0]);
            float mx[2];
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                mx[qq] = fmaxf(s[0][qq][0], s[0][qq][1]);
#pragma unroll
                for (int i = 2; i < 16; i += 2) mx[qq] = fmaxf(fmaxf(mx[qq], s[0][qq][i]), s[0][qq][i + 1]);
            }
            raise_max(mx[0], mx[1]);
            rescale_pending = false;                                     // nothing accumulated yet

            // Cauchy-Schwarz: no logit of this item exceeds |q| times the largest key norm of the head.  If that bound
            // lies below the level at which the running maximum would be raised - for every query of the item, with
            // the maximum the first 32 keys have set - no later step can raise it, and the steps of this kernel, which
            // do not look at the row maxima (a fifth of the softmax instructions), give the same result.  An item
            // without such a bound (a first half tile of padding, norms far above the logits) is left to the kernel
            // that does look: it is put on the fallback list, nothing of it is stored, and the item after it
            // starts from scratch.
            if constexpr (kBounded) {
                float qn[2];
#pragma unroll
                for (int qq = 0; qq < 2; ++qq) qn[qq] = __builtin_sqrtf(q_sq[qq] + __shfl_xor(q_sq[qq], 32)) * 1.001f;   // both halves of the row's d
                const float kn = __uint_as_float((uint32_t)uni((int)__float_as_uint(cur.kn)));
                run = __all(qn[0] * kn <= raise_at[0] && qn[1] * kn <= raise_at[1]);
                if (!run && lane == 0) fallback[atomicAdd(fallback_count, 1u)] = cur.item;
            }
            if (run) {
            if (prepare_next) {
                // What the next item needs and what takes long to arrive is asked for now.  Its list goes from global
                // memory straight into the list buffer that is not in use (LDS DMA, 64 entries per instruction; the
                // lanes behind the end of the list repeat its last entry); its Q rows go into the staging tile,
                // fragment (qq, c) as 1 KB in lane order.  These loads are invisible to the compiler's count of
                // outstanding loads, which can only make its waits for the fragment loads stricter than they need
                // be while the DMA is under way.
#pragma unroll
                for (int e = 0; e < kPipeList / 64; ++e)
                    if (64 * e < next_nent)
                        load_to_lds_4(nlist, (uint32_t)min(lane + 64 * e, next_nent - 1) * 4u, (uint32_t)uni((int)lds_address(&lists[list_buf ^ 1][64 * e])));
                // and the token rows of its 64 query slots, which its epilogue stores through
                if (L.q_rows != nullptr)
                    load_to_lds_4(L.q_rows + nqrow0, (uint32_t)lane * 4u, (uint32_t)uni((int)lds_address(&out_rows[list_buf ^ 1][0])));
                const int64_t nq_bh = (int64_t)(nbh / Hn) * L.q_st[0] + (int64_t)(nbh % Hn) * L.q_st[1];
                const char* qsrc = reinterpret_cast<const char*>(q + nq_bh);
#pragma unroll
                for (int qq = 0; qq < 2; ++qq) {
                    const uint32_t voff = (uint32_t)max(next_rows[qq], 0) * (uint32_t)(L.q_st[2] * 2) + (uint32_t)(16 * lh);   // padded slots read token 0
#pragma unroll
                    for (int c = 0; c < 8; ++c) load_to_lds_16(qsrc + 32 * c, voff, lds_address(qstage + (qq * 8 + c) * 1024));
                }
            }
            // The entry that comes into the window is decoded one iteration before it enters (its validity word may
            // be a load) and read from LDS one iteration before that.
            uint32_t p_tile = entry_tile(3, entry_raw(3));
            uint64_t p_mask = entry_mask(3, p_tile);
            uint32_t raw = entry_raw(4);
            for (int g = 0; g < ntiles; ++g) {
                step(std::integral_constant<int, 0>{});
                step(std::integral_constant<int, 1>{});
                w_tile[0] = w_tile[1]; w_mask[0] = w_mask[1];
                w_tile[1] = w_tile[2]; w_mask[1] = w_mask[2];
                w_tile[2] = p_tile;
                w_mask[2] = p_mask;
                asm volatile("" : "+s"(w_tile[0]), "+s"(w_tile[1]), "+s"(w_tile[2]));
                asm volatile("" : "+s"(w_mask[0]), "+s"(w_mask[1]), "+s"(w_mask[2]));
                p_tile = entry_tile(g + 4, raw);
                p_mask = entry_mask(g + 4, p_tile);
                __builtin_amdgcn_sched_barrier(0);
                raw = entry_raw(g + 5);
                __builtin_amdgcn_sched_barrier(0);
            }
            __syncthreads();                          // the list in LDS has been read: the memory may become the staging tile
            if (prepare_next) {
                // The DMA of the next item's list and Q rows was issued in front of the loop and every iteration has
                // issued 32 loads since; loads complete in order, so all but the newest 24 done (the next item's first
                // fragments, which may still be on their way) means that the DMA has landed.  The wait stands here, in
                // front of the epilogue's stores, whose number depends on the data; Q moves into its registers when
                // the next item starts and the output accumulators are free.
                asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
            }
            // the last 16 keys of the last step (V_B of an odd step sits in ring slot 1)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int qq = 0; qq < 2; ++qq) oacc[t][qq] = mfma32(vb[1][4 + t], pb[qq][1], oacc[t][qq]);
            if (rescale_pending) rescale_out();
            }   // run
        }   // ntiles > 0

        if (run) {
        // ---- epilogue: combine the two key groups of every query, normalise, store through LDS ----
        float inv[2];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            const float l = l_i[qq] + __shfl_xor(l_i[qq], 32);
            inv[qq] = l > 0.f ? 1.0f / l : 0.f;
            if (lse != nullptr && lh == 0) {
                int64_t row = qrow0 + 32 * qq + lr;
                if (L.q_rows != nullptr) row = out_rows[list_buf][32 * qq + lr];
                if (row >= 0) lse[(int64_t)bh * lse_S + row] = l > 0.f ? (m_i[qq] + __builtin_log2f(l)) * kLn2 : -INFINITY;
            }
        }
        // accumulator i of d tile t <-> d = 32 t + 8 (i / 4) + 4 lh + i % 4, query 32 qq + lr
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            T* orow = ost + (32 * qq + lr) * kOutPitch;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    T out4[4];
#pragma unroll
                    for (int jx = 0; jx < 4; ++jx) out4[jx] = (T)(oacc[t][qq][4 * gq + jx] * inv[qq]);
                    *reinterpret_cast<uint2*>(orow + 32 * t + 8 * gq + 4 * lh) = *reinterpret_cast<uint2*>(out4);
                }
        }
        __syncthreads();                          // one wavefront: orders its LDS writes before the reads below
        {
            // The lane index goes through an opaque statement: what is derived from it here (sixteen row numbers and
            // their addresses) would otherwise be computed once in front of the item loop and held in registers, or
            // in scratch memory, all through the tile loop.
            int lane_now = lane;
            asm volatile("" : "+v"(lane_now));
            const int kc = lane_now & 15, kr = lane_now >> 4;
            // in three sweeps - the sixteen token rows, the sixteen pieces, the stores - so that the LDS reads are all
            // on their way before the first is waited for (row by row, every store sat behind two LDS round trips)
            int32_t rows[16];                         // relative to qrow0 without a row table
            u32x4 pieces[16];
            if (L.q_rows != nullptr) {
#pragma unroll
                for (int i = 0; i < 16; ++i) rows[i] = out_rows[list_buf][kr + 4 * i];
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) rows[i] = kr + 4 * i;
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(rows[i]));
            const int64_t row_base = L.q_rows != nullptr ? 0 : qrow0;
#pragma unroll
            for (int i = 0; i < 16; ++i) pieces[i] = *reinterpret_cast<const u32x4*>(ost + (kr + 4 * i) * kOutPitch + kc * 8);
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(pieces[i]));      // read here, not inside the branches below
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (rows[i] >= 0) *reinterpret_cast<u32x4*>(o + o_bh + (row_base + rows[i]) * L.o_st[2] + kc * 8) = pieces[i];
        }
        }   // run
        // ---- on to the next item
        prepared = prepare_next && run;
        if (prepared) list_buf ^= 1;
        __syncthreads();                          // the staging tile is free again
        cur = nxt;
        nxt = nx2;
    }   // work items
}

}  // namespace

// Rounds per launch: five (four to six measure the same at 90 tiles per list and 1.5 % better than two, now that an
// item that was prepared by the one before it starts 7 us sooner than a launch's first; from eight on the items drift
// apart and the L2 hit rate falls); eight for short lists (six to ten measure the same, twenty lose 3 %).
constexpr int kRoundsPerLaunch = 5;
constexpr int kRoundsPerLaunchShort = 8;     // lists of at most kShortList tiles
constexpr int kShortList = 64;

// Workgroups (of one wavefront) the device runs at once with this kernel: one per SIMD.
static int resident_wavefronts() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 1024;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = 4 * cus;
    }
    return cached[dev];
}

// kf / vf: fragment-order K and V, [B * Hn][Sk / 64][16 KB].  q, o in blocked order (q_rows null) or in
// (T, H, W) order through the row table.  Scheduling: rounds of as many work items as the device runs at once,
// across (batch, head) boundaries, kRoundsPerLaunch rounds per launch, every workgroup running one item of each round;
// with `order` and `queue` also the schedule that draws items longest list first, the choice between the two being
// made on the device.
__global__ void frag_zero_kernel(uint32_t* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// int32 entries launch_fwd_frag's `fallback` argument must hold for `items` work items (64-row query tiles)
size_t frag_fallback_ints(int64_t items) { return 64 + (size_t)items; }

hipError_t launch_fwd_frag(const void* q, const void* kf, const void* vf, const int32_t* idx, const int32_t* lens,
                           const uint64_t* tile_valid, void* o, float* lse, int B, int Hn, int64_t Sq, int64_t Sk,
                           int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype, hipStream_t st,
                           const int32_t* q_rows, const int64_t q_st[3], const int64_t o_st[3], int64_t lse_rows,
                           const int32_t* order, uint32_t* queue, const float* key_norm, int32_t* fallback) {
    if (idx_stride > kListEntries) return hipErrorInvalidValue;   // the C-ABI layer keeps lists within this limit
    const float qk_scale = sm_scale * kLog2e;
    FragLayout L;
    L.q_rows = q_rows;
    for (int i = 0; i < 3; ++i) { L.q_st[i] = q_st[i]; L.o_st[i] = o_st[i]; }
    const int per_head = (int)(Sq / kTile);
    const int total = B * Hn * per_head;
    const int resident = resident_wavefronts();
    const dim3 block(64);
    const uint32_t* gate = nullptr;
    // The kernel addresses K and V through a buffer of less than 4 GB that starts at the first (batch, head) of a
    // launch: a launch covers as many heads as fit.  One head always does (fewer than 2^24 keys of 256 B).
    const int64_t kv_bh_bytes = (Sk / kTile) * (int64_t)kTileBytes;
    const int64_t span_limit = ((int64_t)1 << 32) - 1;
    if (kv_bh_bytes > span_limit) return hipErrorInvalidValue;
    const int heads_per_span = (int)(span_limit / kv_bh_bytes);
    const bool one_span = (int64_t)B * Hn <= heads_per_span;
    const uint32_t whole_span = one_span ? (uint32_t)((int64_t)B * Hn * kv_bh_bytes) : 0u;
    // the LDS DMA that brings the next item's Q rows forms its addresses from 32-bit row offsets
    const int64_t q_rows_max = q_rows != nullptr ? lse_rows : Sq;
    const int q_offsets_32 = q_rows_max * q_st[2] * 2 + 512 < ((int64_t)1 << 32) ? 1 : 0;
    // The rounds run the kernel whose steps take no row maxima when the key norms are known, a place for the list of
    // the items it has to leave to the other kernel is given, and that kernel can reach every head from one buffer.
    const bool bounded = key_norm != nullptr && fallback != nullptr && one_span;
    uint32_t* fb_count = bounded ? reinterpret_cast<uint32_t*>(fallback) : nullptr;
    int32_t* fb_list = bounded ? fallback + 64 : nullptr;
#define BSA_FRAG_LAUNCH_T(T, N1, BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc)                           \
    hipLaunchKernelGGL((fwd_frag_kernel<T, N1, BD>), grid, block, 0, st, (const T*)q, (const char*)kf, (const char*)vf, idx, \
                       lens, tile_valid, (T*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, begin, end, resident, Hn, lse_rows, \
                       L, ord, que, gate, want, bh0, span, q_offsets_32, key_norm, fbl, fbc)
#define BSA_FRAG_LAUNCH(BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc)                                     \
    do {                                                                                                               \
        if (dtype == BSA_BF16) {                                                                                       \
            if (bs_k == kTile) BSA_FRAG_LAUNCH_T(__bf16, true, BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc);   \
            else BSA_FRAG_LAUNCH_T(__bf16, false, BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc);          \
        } else {                                                                                                       \
            if (bs_k == kTile) BSA_FRAG_LAUNCH_T(_Float16, true, BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc); \
            else BSA_FRAG_LAUNCH_T(_Float16, false, BD, grid, begin, end, ord, que, want, bh0, span, fbl, fbc);        \
        }                                                                                                              \
    } while (0)
    if (queue != nullptr && one_span) {
        launch_schedule_choice(lens, (int)(Sq / bs_q), bs_q / kTile, total, resident, resident, idx_stride, queue, st);
        gate = queue + 1;
        const dim3 grid((unsigned)(total < resident ? total : resident));
        BSA_FRAG_LAUNCH(false, grid, 0, total, order, queue, 1u, 0, whole_span, (int32_t*)nullptr, (uint32_t*)nullptr);
    }
    if (bounded) hipLaunchKernelGGL(frag_zero_kernel, dim3(1), dim3(64), 0, st, fb_count, 1);
    // kRoundsPerLaunch rounds per launch, every workgroup running one item of each: the items of a round start
    // together and keep in step (with many more rounds per launch they drift apart and the L2 hit rate falls).
    const int span = (idx_stride * (bs_k / kTile) <= kShortList ? kRoundsPerLaunchShort : kRoundsPerLaunch) * resident;
    for (int first = 0; first < total;) {
        int end = first + span < total ? first + span : total;
        const int bh0 = first / per_head;
        if ((end - 1) / per_head - bh0 + 1 > heads_per_span) end = (bh0 + heads_per_span) * per_head;
        const int heads = (end - 1) / per_head - bh0 + 1;
        const int n = end - first;
        const dim3 grid((unsigned)(n < resident ? n : resident));
        if (bounded)
            BSA_FRAG_LAUNCH(true, grid, first, end, (const int32_t*)nullptr, (uint32_t*)nullptr, 0u, bh0, (uint32_t)(heads * kv_bh_bytes), fb_list, fb_count);
        else
            BSA_FRAG_LAUNCH(false, grid, first, end, (const int32_t*)nullptr, (uint32_t*)nullptr, 0u, bh0, (uint32_t)(heads * kv_bh_bytes),
                            (int32_t*)nullptr, (uint32_t*)nullptr);
        first = end;
    }
    if (bounded) {
        // what the rounds left over: as many items as the list holds, found out on the device
        const dim3 grid((unsigned)(total < resident ? total : resident));
        BSA_FRAG_LAUNCH(false, grid, 0, total, (const int32_t*)fb_list, (uint32_t*)nullptr, 0u, 0, whole_span, (int32_t*)nullptr, fb_count);
    }
#undef BSA_FRAG_LAUNCH
#undef BSA_FRAG_LAUNCH_T
    return hipGetLastError();
}

// floats launch_frag's key_norm argument must hold: one per (batch, head), then (from a 256-byte boundary) one per tile
size_t frag_key_norm_floats(int B, int Hn, int64_t tiles) {
    return (((size_t)B * Hn + 63) & ~(size_t)63) + (size_t)B * Hn * (size_t)tiles;
}

hipError_t launch_frag(const void* src, const int64_t st3[3], void* dst, int B, int Hn, const Grid3& g, int dtype,
                       bool transpose, hipStream_t st, void* pooled, uint64_t* tile_valid, const RowTransform* tr,
                       float* key_norm) {
    RowTransform t = tr ? *tr : RowTransform{};
    t.head_fastest = st3[1] < st3[2] ? 1 : 0;
    const dim3 grid((unsigned)((int64_t)g.blocks() * (g.chunk() / kTile) * B * Hn)), block(256);
    // 16-bit types move as raw bits
    if (transpose)
        hipLaunchKernelGGL((frag_kernel<uint16_t, true>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn, (uint16_t*)nullptr, (uint64_t*)nullptr, 0, t, (float*)nullptr);
    else {
        // key_norm: [B * Hn] floats followed by [B * Hn][tiles] floats of the tiles' norms they are taken from
        const int tiles = g.blocks() * (g.chunk() / kTile);
        float* tile_norm = key_norm != nullptr ? key_norm + (((size_t)B * Hn + 63) & ~(size_t)63) : nullptr;
        hipLaunchKernelGGL((frag_kernel<uint16_t, false>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn, (uint16_t*)pooled, tile_valid, dtype == BSA_BF16 ? 1 : 0, t, tile_norm);
        if (key_norm != nullptr)
            hipLaunchKernelGGL(head_norm_kernel, dim3((unsigned)(B * Hn)), dim3(256), 0, st, tile_norm, key_norm, tiles);
    }
    return hipGetLastError();
}

}  // namespace bsa
