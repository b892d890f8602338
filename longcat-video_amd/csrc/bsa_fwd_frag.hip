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

#include <utility>

namespace bsa {
namespace {

using namespace mfma;

constexpr int kHalfBytes = 8192;      // 32 keys of a fragment-order K (or V) tile
constexpr int kListEntries = 4096;    // longest list a work item can walk (its staging area in LDS: 17 KB)

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
                                                   uint64_t* __restrict__ tile_valid, int is_bf16, RowTransform tr) {
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

struct FragLayout {
    const int32_t* q_rows;        // token row of every blocked-order query slot, -1 = padding; null: q, o in blocked order
    int64_t q_st[3], o_st[3];     // element strides: batch, head, row
};

// kNsub1: KV blocks of one 64-key tile (bs_k == 64): no division in the walk.
template <typename T, bool kNsub1>
__global__ __launch_bounds__(64) void fwd_frag_kernel(
    const T* __restrict__ q, const char* __restrict__ kf, const char* __restrict__ vf,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens, const uint64_t* __restrict__ tile_valid,
    T* __restrict__ o, float* __restrict__ lse, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
    float qk_scale, int item_begin, int item_end, int round, int Hn, int64_t lse_S, FragLayout L,
    const int32_t* __restrict__ order, uint32_t* __restrict__ queue, const uint32_t* __restrict__ gate, uint32_t gate_want) {
    typedef typename Vec8<T>::type V8;
    if (gate != nullptr && *gate != gate_want) return;
    // output staging: 64 rows of 256 B, 272 B apart.  During the tile loop the same memory holds the work item's
    // list of KV blocks (kListEntries words at most), bit 31 of an entry flagging a block with padded keys.
    constexpr int kOutPitch = kD + 8;
    __shared__ __attribute__((aligned(16))) T ost[kTile * kOutPitch];
    uint32_t* const ents = reinterpret_cast<uint32_t*>(ost);

    const int lane = threadIdx.x;
    const int lr = lane & 31, lh = lane >> 5;
    const int nbq = (int)(Sq / bs_q);
    const int nqt = (int)(Sq / kTile);
    const int nsub = kNsub1 ? 1 : bs_k / kTile;
    const int nbk = (int)(Sk / bs_k);
    const int64_t kv_bh_bytes = (Sk / kTile) * (int64_t)kTileBytes;
    const uint32_t lane_off = (uint32_t)lane * 16u;

    int local = blockIdx.x;
    {
        // The launch's items are taken in rounds of `round` (a multiple of 8) in workgroup order.  Workgroup b
        // runs on XCD b % 8: within a round every XCD takes a contiguous run of the round's items.
        const int r0 = local / round * round;
        const int n = min(round, item_end - item_begin - r0), w = local - r0, x = w & 7;
        local = r0 + x * (n >> 3) + min(x, n & 7) + (w >> 3);
    }
    for (;;) {
    if (queue != nullptr) {
        uint32_t drawn = 0;
        if (lane == 0) drawn = atomicAdd(queue, 1u);
        local = (int)__builtin_amdgcn_readfirstlane(drawn);
    }
    if (local >= item_end - item_begin) break;
    const int item = item_begin + (order != nullptr ? order[local] : local);
    const int bh = item / nqt;
    const int qtile = item % nqt;
    const int64_t qrow0 = (int64_t)qtile * kTile;
    const int qblock = (int)(qrow0 / bs_q);
    const int64_t q_bh = (int64_t)(bh / Hn) * L.q_st[0] + (int64_t)(bh % Hn) * L.q_st[1];
    const int64_t o_bh = (int64_t)(bh / Hn) * L.o_st[0] + (int64_t)(bh % Hn) * L.o_st[1];
    const int32_t* list = idx + ((int64_t)bh * nbq + qblock) * idx_stride;
    const int nent = min(min(max(lens[(int64_t)bh * nbq + qblock], 0), idx_stride), kListEntries);
    const int ntiles = nent * nsub;
    const int nsteps = 2 * ntiles;
    // Q as the B operand of S^T: lane holds rows lr and 32 + lr, d = 16 c + 8 lh .. +8.  Requested before the list
    // is staged, so that the two chains of dependent loads (row table -> Q rows, list length -> list -> LDS) run
    // side by side.
    V8 qreg[2][8];
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        int64_t row = qrow0 + 32 * qq + lr;
        if (L.q_rows != nullptr) row = max(L.q_rows[row], 0);          // padded slots read token 0, never stored
        const T* qp = q + q_bh + row * L.q_st[2] + 8 * lh;
#pragma unroll
        for (int c = 0; c < 8; ++c) qreg[qq][c] = *reinterpret_cast<const V8*>(qp + 16 * c);
    }
    // the list goes to LDS: clamped block index (a malformed list gives wrong numbers, never a fault) and the flag
    for (int e = lane; e < nent; e += 64) {
        const int blk = min(max(list[e], 0), nbk - 1);
        uint32_t flag = 0;
        if (tile_valid != nullptr)
            for (int sub = 0; sub < nsub; ++sub) flag |= tile_valid[blk * nsub + sub] != ~0ull ? 1u : 0u;
        ents[e] = (uint32_t)blk | (flag << 31);
    }
    __syncthreads();
    const char* kbase = kf + (int64_t)bh * kv_bh_bytes;
    const char* vbase = vf + (int64_t)bh * kv_bh_bytes;

    f32x16 oacc[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[t][qq][i] = 0.f;
    float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.f, 0.f};

    if (nsteps > 0) {
    // Position tp of the tile walk -> tile inside this (batch, head) and validity word of its 64 keys.  Positions
    // behind the list repeat the last tile with every key masked out.  The entry is read from LDS (entry_raw, to
    // be issued early) and decoded later (entry_tile / entry_mask).
    auto entry_raw = [&](int tp) -> uint32_t {
        const int tc = min(tp, ntiles - 1);
        return ents[kNsub1 ? tc : tc / nsub];                   // the same address in every lane
    };
    auto entry_tile = [&](int tp, uint32_t raw) -> uint32_t {
        const uint32_t blk = (uint32_t)__builtin_amdgcn_readfirstlane((int)raw) & 0x7fffffffu;
        if (kNsub1) return blk;
        return blk * (uint32_t)nsub + (uint32_t)(min(tp, ntiles - 1) % nsub);
    };
    auto entry_mask = [&](int tp, uint32_t raw, uint32_t tile) -> uint64_t {
        if (tp >= ntiles) return 0ull;
        if (__builtin_expect(__builtin_amdgcn_readfirstlane((int)raw) < 0, 0)) return tile_valid[tile];
        return ~0ull;
    };
    // window of the walk: positions g, g + 1, g + 2 of loop iteration g (one tile per iteration)
    uint32_t w_tile[3];
    uint64_t w_mask[3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const uint32_t raw = entry_raw(r);
        w_tile[r] = entry_tile(r, raw);
        w_mask[r] = entry_mask(r, raw, w_tile[r]);
    }

    // Register rings: K fragments of two steps, V fragments of two steps (each step: 4 fragments for its
    // first 16 keys, "A", and 4 for its last 16, "B").
    V8 kb[2][8], vb[2][8];
    f32x16 s[2][2];                                            // S^T of the current and of the next step
    V8 pb[2][2];                                               // P^T as B operand: [query half][A | B]
    auto k_frag = [&](int r, int h, int c) -> V8 {          // window slot r, half h, d step c
        return *reinterpret_cast<const V8*>(kbase + (uint64_t)w_tile[r] * kTileBytes + h * kHalfBytes + lane_off + c * 1024);
    };
    auto v_frag = [&](int r, int h, int f) -> V8 {          // f = 4 * key step + d tile
        return *reinterpret_cast<const V8*>(vbase + (uint64_t)w_tile[r] * kTileBytes + h * kHalfBytes + lane_off + f * 1024);
    };
    // accumulator i <-> key 8 (i / 4) + 4 lh + i % 4 of the step's 32 keys, query lr (+32)
    auto mask_pair = [&](f32x16 (&sv)[2], uint32_t half) {
        if (__builtin_expect(half != ~0u, 0)) {
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");       // the MFMAs into these accumulators have retired
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (!((half >> (8 * (i / 4) + 4 * lh + (i % 4))) & 1u)) { sv[0][i] = -INFINITY; sv[1][i] = -INFINITY; }
        }
    };
    // Softmax state per query half: running maximum m_i (scaled, log2 units), its negative for the exponent
    // (0 while the maximum is -inf), and the unscaled logit above which the maximum has to be raised.
    float neg_m[2] = {0.f, 0.f}, raise_at[2] = {-INFINITY, -INFINITY};
    const float inv_scale = 1.0f / qk_scale;
    // Raising the
    // maximum has two parts.  Here: the new maximum, the exponent offset, the row sum (which already holds
    // every probability of the current step).  The output accumulators are rescaled one quarter of a step later
    // (rescale_out, behind slot 7 of the next step): the product of the current step's P_B, whose
    // probabilities were taken relative to the old maximum, is only issued in slots 0 .. 7 of that step.
    float alpha_p[2] = {1.f, 1.f};
    bool rescale_pending = false;
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
                raise_at[qq] = (m_new + kLazyTau) * inv_scale;
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

    // ---- prologue.  In flight when the loop starts: K(1), K(2), V_A(0), V_B(0), V_A(1); the ring slot of
    // V_B(1) holds zeros, which the first step multiplies with P = 0 (there is no step -1).
    {
        V8 k0[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) k0[c] = k_frag(0, 0, c);
#pragma unroll
        for (int c = 0; c < 8; ++c) kb[1][c] = k_frag(0, 1, c);                 // K(1)
#pragma unroll
        for (int f = 0; f < 8; ++f) vb[0][f] = v_frag(0, 0, f);                 // V_A(0), V_B(0)
#pragma unroll
        for (int c = 0; c < 8; ++c) kb[0][c] = k_frag(1, 0, c);                 // K(2)
#pragma unroll
        for (int f = 0; f < 4; ++f) vb[1][f] = v_frag(0, 1, f);                 // V_A(1)
#pragma unroll
        for (int f = 4; f < 8; ++f)
#pragma unroll
            for (int e = 0; e < 8; ++e) vb[1][f][e] = (T)0.f;
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int e = 0; e < 8; ++e) pb[qq][1][e] = (T)0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c == 0) { mfma_s<true, false>(s[0][0], k0[0], qreg[0][0]); mfma_s<true, true>(s[0][1], k0[0], qreg[1][0]); }
            else { mfma_s<false, false>(s[0][0], k0[c], qreg[0][c]); mfma_s<false, true>(s[0][1], k0[c], qreg[1][c]); }
        }
        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");           // MFMA results before the VALU reads them
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
    }

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
    // fragment is requested two steps before it is used.
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
                for (int t = 0; t < 4; ++t) vb[vprev][4 + t] = v_frag((j + 1) >> 1, (j + 1) & 1, 4 + t);
            }
            if constexpr (slot == 23) {
#pragma unroll
                for (int c = 0; c < 8; ++c) kb[kslot][c] = k_frag((j + 3) >> 1, (j + 1) & 1, c);
            }
            if constexpr (slot == 31) {
#pragma unroll
                for (int t = 0; t < 4; ++t) vb[vcur][t] = v_frag((j + 2) >> 1, j & 1, t);
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
                    // validity of the keys of step u + 1: tile window slot (j + 1) / 2, half (j + 1) & 1
                    mask_pair(s[sn], (uint32_t)(w_mask[(j + 1) >> 1] >> (32 * ((j + 1) & 1))));
                    mx[0] = fmaxf(fmaxf(s[sn][0][0], s[sn][0][1]), s[sn][0][2]);
                    mx[1] = fmaxf(fmaxf(s[sn][1][0], s[sn][1][1]), s[sn][1][2]);
                    mx[0] = fmaxf(fmaxf(mx[0], s[sn][0][3]), s[sn][0][15]);
                    mx[1] = fmaxf(fmaxf(mx[1], s[sn][1][3]), s[sn][1][15]);
                }
                if constexpr (r >= 2 && r < 7) {                // accumulators 4 .. 13, two per slot and query half
                    mx[0] = fmaxf(fmaxf(mx[0], s[sn][0][2 * r]), s[sn][0][2 * r + 1]);
                    mx[1] = fmaxf(fmaxf(mx[1], s[sn][1][2 * r]), s[sn][1][2 * r + 1]);
                }
                if constexpr (r == 7) {
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
        raise_max(mx[0], mx[1]);
    };

    // The entry that comes into the window is read from LDS one iteration before it is decoded.  The read is
    // issued behind everything else of an iteration that waits on the scalar / LDS counter (the rare validity
    // word), so that no wait for it lands in front of the MFMAs.
    uint32_t raw = entry_raw(3);
    for (int g = 0; g < ntiles; ++g) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        w_tile[0] = w_tile[1]; w_mask[0] = w_mask[1];
        w_tile[1] = w_tile[2]; w_mask[1] = w_mask[2];
        w_tile[2] = entry_tile(g + 3, raw);
        w_mask[2] = entry_mask(g + 3, raw, w_tile[2]);
        asm volatile("" : "+s"(w_tile[0]), "+s"(w_tile[1]), "+s"(w_tile[2]));
        asm volatile("" : "+s"(w_mask[0]), "+s"(w_mask[1]), "+s"(w_mask[2]));
        __builtin_amdgcn_sched_barrier(0);
        raw = entry_raw(g + 4);
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();                          // the list in LDS has been read: the memory becomes the staging tile
    // the last 16 keys of the last step (V_B of an odd step sits in ring slot 1)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) oacc[t][qq] = mfma32(vb[1][4 + t], pb[qq][1], oacc[t][qq]);
    if (rescale_pending) rescale_out();
    }   // nsteps > 0

    // ---- epilogue: combine the two key groups of every query, normalise, store through LDS ----
    float inv[2];
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        const float l = l_i[qq] + __shfl_xor(l_i[qq], 32);
        inv[qq] = l > 0.f ? 1.0f / l : 0.f;
        if (lse != nullptr && lh == 0) {
            int64_t row = qrow0 + 32 * qq + lr;
            if (L.q_rows != nullptr) row = L.q_rows[row];
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
        const int kc = lane & 15, kr = lane >> 4;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int r = kr + 4 * i;
            int64_t row = qrow0 + r;
            if (L.q_rows != nullptr) row = L.q_rows[row];
            if (row >= 0)
                *reinterpret_cast<uint4*>(o + o_bh + row * L.o_st[2] + kc * 8) =
                    *reinterpret_cast<const uint4*>(ost + r * kOutPitch + kc * 8);
        }
    }
    if (queue == nullptr) break;
    __syncthreads();                          // the staging tile is free again
    }   // work items
}

}  // namespace

constexpr int kRoundsPerLaunch = 2;

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
// (T, H, W) order through the row table.  Scheduling as in launch_fwd: rounds of as many work items as
// the device runs at once, across (batch, head) boundaries; with `order` and `queue` also the schedule that
// draws items longest list first, the choice between the two being made on the device.
hipError_t launch_fwd_frag(const void* q, const void* kf, const void* vf, const int32_t* idx, const int32_t* lens,
                           const uint64_t* tile_valid, void* o, float* lse, int B, int Hn, int64_t Sq, int64_t Sk,
                           int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype, hipStream_t st,
                           const int32_t* q_rows, const int64_t q_st[3], const int64_t o_st[3], int64_t lse_rows,
                           const int32_t* order, uint32_t* queue) {
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
#define BSA_FRAG_LAUNCH_T(T, N1, grid, begin, end, ord, que, want)                                                   \
    hipLaunchKernelGGL((fwd_frag_kernel<T, N1>), grid, block, 0, st, (const T*)q, (const char*)kf, (const char*)vf, idx, \
                       lens, tile_valid, (T*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, begin, end, resident, Hn, lse_rows, \
                       L, ord, que, gate, want)
#define BSA_FRAG_LAUNCH(grid, begin, end, ord, que, want)                                                             \
    do {                                                                                                               \
        if (dtype == BSA_BF16) {                                                                                       \
            if (bs_k == kTile) BSA_FRAG_LAUNCH_T(__bf16, true, grid, begin, end, ord, que, want);                      \
            else BSA_FRAG_LAUNCH_T(__bf16, false, grid, begin, end, ord, que, want);                                   \
        } else {                                                                                                       \
            if (bs_k == kTile) BSA_FRAG_LAUNCH_T(_Float16, true, grid, begin, end, ord, que, want);                    \
            else BSA_FRAG_LAUNCH_T(_Float16, false, grid, begin, end, ord, que, want);                                 \
        }                                                                                                              \
    } while (0)
    if (queue != nullptr) {
        launch_schedule_choice(lens, (int)(Sq / bs_q), bs_q / kTile, total, resident, resident, idx_stride, queue, st);
        gate = queue + 1;
        const dim3 grid((unsigned)(total < resident ? total : resident));
        BSA_FRAG_LAUNCH(grid, 0, total, order, queue, 1u);
    }
    // Two rounds per launch: the wavefronts of the second round start as those of the first finish, which takes
    // half of the launch boundaries away and still keeps the items in step (with three or four rounds the gain is
    // the same, from six on the items drift apart and the L2 hit rate falls).
    const int span = kRoundsPerLaunch * resident;
    for (int first = 0; first < total; first += span) {
        const int end = first + span < total ? first + span : total;
        const dim3 grid((unsigned)(end - first));
        BSA_FRAG_LAUNCH(grid, first, end, (const int32_t*)nullptr, (uint32_t*)nullptr, 0u);
    }
#undef BSA_FRAG_LAUNCH
#undef BSA_FRAG_LAUNCH_T
    return hipGetLastError();
}

hipError_t launch_frag(const void* src, const int64_t st3[3], void* dst, int B, int Hn, const Grid3& g, int dtype,
                       bool transpose, hipStream_t st, void* pooled, uint64_t* tile_valid, const RowTransform* tr) {
    RowTransform t = tr ? *tr : RowTransform{};
    t.head_fastest = st3[1] < st3[2] ? 1 : 0;
    const dim3 grid((unsigned)((int64_t)g.blocks() * (g.chunk() / kTile) * B * Hn)), block(256);
    // 16-bit types move as raw bits
    if (transpose)
        hipLaunchKernelGGL((frag_kernel<uint16_t, true>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn, (uint16_t*)nullptr, (uint64_t*)nullptr, 0, t);
    else
        hipLaunchKernelGGL((frag_kernel<uint16_t, false>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn, (uint16_t*)pooled, tile_valid, dtype == BSA_BF16 ? 1 : 0, t);
    return hipGetLastError();
}

}  // namespace bsa
