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

namespace bsa {
namespace {

using namespace mfma;

constexpr int kHalfBytes = 8192;      // 32 keys of a fragment-order K (or V) tile
constexpr int kRing = 2;              // steps of K fragments and of V fragments in flight
constexpr int kUnroll = 2;            // steps per loop body: one tile (two halves), which is also one turn of the rings

// ------------------------------------------------------------------ relayout
// One workgroup per 64-slot tile of one (batch, head): the 64 rows are gathered from (T, H, W) order
// (padded slots: zeros) into LDS and written out as 16 fragments of 1 KB.  K (TRANSPOSE = false) moves
// 16-byte pieces; V (TRANSPOSE = true) gathers 8 keys of one d per piece.
template <typename T, bool TRANSPOSE>
__global__ __launch_bounds__(256) void frag_kernel(const T* __restrict__ src, int64_t sB, int64_t sH, int64_t sS,
                                                   char* __restrict__ dst, Grid3 g, int Hn) {
    // rows padded to 264 B: the transposing reads below walk down a column
    constexpr int kPitch = kD + 4;
    __shared__ __attribute__((aligned(16))) T tile[kTile * kPitch];
    const int tiles_per_chunk = g.chunk() / kTile;
    const int blk = blockIdx.x / tiles_per_chunk, sub = blockIdx.x % tiles_per_chunk;
    const int bh = blockIdx.y;
    const int nw = blk % g.Nw, nh = (blk / g.Nw) % g.Nh, nt = blk / (g.Nw * g.Nh);
    const T* sbase = src + (int64_t)(bh / Hn) * sB + (int64_t)(bh % Hn) * sH;
    const int c16 = threadIdx.x & 15, rg = threadIdx.x >> 4;      // 16 pieces of 16 B per row, 16 rows at a time
    uint2 val[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = sub * kTile + rg + 16 * i;                   // slot inside the chunk
        const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
        const int tt = nt * g.t + ti, hh = nh * g.h + hi, ww = nw * g.w + wi;
        uint4 x = make_uint4(0, 0, 0, 0);
        if (tt < g.T && hh < g.H && ww < g.W)
            x = *reinterpret_cast<const uint4*>(sbase + (((int64_t)tt * g.H + hh) * g.W + ww) * sS + c16 * 8);
        val[i][0] = make_uint2(x.x, x.y);
        val[i][1] = make_uint2(x.z, x.w);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        T* row = tile + (rg + 16 * i) * kPitch + c16 * 8;          // 8-byte aligned (pitch 264 B)
        *reinterpret_cast<uint2*>(row) = val[i][0];
        *reinterpret_cast<uint2*>(row + 4) = val[i][1];
    }
    __syncthreads();
    char* out = dst + ((int64_t)bh * gridDim.x + blockIdx.x) * kTileBytes;
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
            const int kh = f >> 3, s2 = (f >> 2) & 1, t = f & 3;
            const uint16_t* s = reinterpret_cast<const uint16_t*>(tile) + 32 * t + lr;
#pragma unroll
            for (int j = 0; j < 8; ++j) piece[j] = s[(32 * kh + 16 * s2 + 8 * (j >> 2) + 4 * lh + (j & 3)) * kPitch];
        }
        *reinterpret_cast<uint4*>(out + (int64_t)e * 16) = *reinterpret_cast<const uint4*>(piece);
    }
}

// ------------------------------------------------------------------ attention
// S^T accumulators must sit in ordinary VGPRs, where the softmax reads them, while the (four times larger)
// output accumulators belong in AGPRs.  For a kernel that may use more than 256 registers the compiler puts
// the result of every builtin MFMA into AGPRs, so the S^T MFMAs are written as inline assembly with VGPR
// operands.  The compiler does not see that such a statement is an MFMA and adds no wait states behind it:
// the code keeps every VALU access to these accumulators at least eight MFMAs (256 clocks) behind the MFMA
// that writes them, or puts explicit s_nop there.
// kAgprB: the B operand (the Q fragment) lives in an AGPR.  The queries 32 .. 63 of a work item are kept there,
// the queries 0 .. 31 in VGPRs, which balances the two register files (VGPR: S^T, P^T, the K ring, half of Q;
// AGPR: the output accumulators, the V ring, the other half of Q).
template <bool kFirst, bool kAgprB>
__device__ inline void mfma_s(f32x16& acc, bf16x8 a, bf16x8 b) {
    if (kFirst) {
        if (kAgprB) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
    } else {
        if (kAgprB) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
    }
}
template <bool kFirst, bool kAgprB>
__device__ inline void mfma_s(f32x16& acc, f16x8 a, f16x8 b) {
    if (kFirst) {
        if (kAgprB) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
        else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
    } else {
        if (kAgprB) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
        else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
    }
}

struct FragLayout {
    const int32_t* q_rows;        // token row of every blocked-order query slot, -1 = padding; null: q, o in blocked order
    int64_t q_st[3], o_st[3];     // element strides: batch, head, row
};

template <typename T>
__global__ __launch_bounds__(64) void fwd_frag_kernel(
    const T* __restrict__ q, const char* __restrict__ kf, const char* __restrict__ vf,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens, const uint64_t* __restrict__ tile_valid,
    T* __restrict__ o, float* __restrict__ lse, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
    float qk_scale, int item_begin, int item_end, int Hn, int64_t lse_S, FragLayout L,
    const int32_t* __restrict__ order, uint32_t* __restrict__ queue, const uint32_t* __restrict__ gate, uint32_t gate_want) {
    typedef typename Vec8<T>::type V8;
    if (gate != nullptr && *gate != gate_want) return;
    // output staging: 64 rows of 256 B, 272 B apart
    constexpr int kOutPitch = kD + 8;
    __shared__ __attribute__((aligned(16))) T ost[kTile * kOutPitch];

    const int lane = threadIdx.x;
    const int lr = lane & 31, lh = lane >> 5;
    const int nbq = (int)(Sq / bs_q);
    const int nqt = (int)(Sq / kTile);
    const int nsub = bs_k / kTile;
    const int nbk = (int)(Sk / bs_k);
    const int64_t kv_bh_bytes = (Sk / kTile) * (int64_t)kTileBytes;
    const uint32_t lane_off = (uint32_t)lane * 16u;

    int local = blockIdx.x;
    {
        // workgroup b of a launch runs on XCD b % 8: every XCD takes a contiguous run of the launch's items
        const int n = item_end - item_begin, x = local & 7;
        local = x * (n >> 3) + min(x, n & 7) + (local >> 3);
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
    const int ntiles = min(max(lens[(int64_t)bh * nbq + qblock], 0), idx_stride) * nsub;
    const int nsteps = 2 * ntiles;
    const char* kbase = kf + (int64_t)bh * kv_bh_bytes;
    const char* vbase = vf + (int64_t)bh * kv_bh_bytes;

    // Q as the B operand of S^T: lane holds rows lr and 32 + lr, d = 16 c + 8 lh .. +8
    V8 qreg[2][8];
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
        int64_t row = qrow0 + 32 * qq + lr;
        if (L.q_rows != nullptr) row = max(L.q_rows[row], 0);          // padded slots read token 0, never stored
        const T* qp = q + q_bh + row * L.q_st[2] + 8 * lh;
#pragma unroll
        for (int c = 0; c < 8; ++c) qreg[qq][c] = *reinterpret_cast<const V8*>(qp + 16 * c);
    }

    f32x16 oacc[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int qq = 0; qq < 2; ++qq)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[t][qq][i] = 0.f;
    float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.f, 0.f};

    if (nsteps > 0) {
    // Position tp of the tile walk -> byte offset of the tile inside this (batch, head) and its validity
    // word.  Positions behind the list repeat the last tile with every key masked out, so that the loop
    // body can run in whole groups of kUnroll steps.  A block index outside [0, nbk) is clamped.
    auto tile_of = [&](int tp) -> uint32_t {
        const int tc = min(tp, ntiles - 1);
        const int blk = min(max(list[tc / nsub], 0), nbk - 1);
        return (uint32_t)(blk * nsub + tc % nsub);
    };
    auto mask_of = [&](int tp, uint32_t tile) -> uint64_t {
        if (tp >= ntiles) return 0ull;
        return tile_valid != nullptr ? tile_valid[tile] : ~0ull;
    };
    // window of the walk: entries for positions g .. g+3 of loop iteration g (one tile per iteration)
    uint32_t w_tile[4];
    uint64_t w_mask[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) { w_tile[r] = tile_of(r); w_mask[r] = mask_of(r, w_tile[r]); }

    V8 kb[kRing][8], vb[kRing][8];
    // fragments of step (tile window slot r, half h) into ring slot `slot`
    auto load_k = [&](auto slot, int r, int h) {
        constexpr int sl = decltype(slot)::value;
        const char* p = kbase + (uint64_t)w_tile[r] * kTileBytes + h * kHalfBytes + lane_off;
#pragma unroll
        for (int c = 0; c < 8; ++c) kb[sl][c] = *reinterpret_cast<const V8*>(p + c * 1024);
    };
    auto load_v = [&](auto slot, int r, int h) {
        constexpr int sl = decltype(slot)::value;
        const char* p = vbase + (uint64_t)w_tile[r] * kTileBytes + h * kHalfBytes + lane_off;
#pragma unroll
        for (int c = 0; c < 8; ++c) vb[sl][c] = *reinterpret_cast<const V8*>(p + c * 1024);
    };
    // accumulator i <-> key 8 (i / 4) + 4 lh + i % 4 of the step's 32 keys, query lr (+32)
    auto mask_pair = [&](f32x16 (&s)[2], uint32_t half) {
        if (__builtin_expect(half != ~0u, 0)) {
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (!((half >> (8 * (i / 4) + 4 * lh + (i % 4))) & 1u)) { s[0][i] = -INFINITY; s[1][i] = -INFINITY; }
        }
    };
    auto raise_max = [&](float mx0, float mx1) {
        if (__builtin_expect(__any(mx0 > m_i[0] + kLazyTau || mx1 > m_i[1] + kLazyTau), 0)) {
            const float mx[2] = {mx0, mx1};
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");       // the last MFMA into the accumulators has retired
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                const float m_new = fmaxf(m_i[qq], mx[qq]);
                const float alpha = __builtin_amdgcn_exp2f(m_i[qq] - ((m_new == -INFINITY) ? 0.f : m_new));
                m_i[qq] = m_new;
                l_i[qq] *= alpha;
                // The output accumulators live in AGPRs, which the VALU cannot multiply in place.  Written out
                // register by register through one temporary, so that this rare path does not make the compiler
                // reserve VGPRs for a copy of the accumulators.
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        float x = oacc[t][qq][i], tmp;
                        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1"
                                     : "+a"(x), "=&v"(tmp) : "v"(alpha));
                        oacc[t][qq][i] = x;
                    }
            }
            asm volatile("s_nop 7" ::: "memory");                    // AGPR writes before the next MFMA reads them
        }
    };
    // combine a lane's maximum with the other key group of the same query (lane ^ 32) and scale it
    auto finish_max = [&](float mx) -> float {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
        return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * qk_scale;
    };

    // ---- prologue: K(0), V(0), K(1), V(1) in flight; S(0) with nothing to overlap; then K(2)
    load_k(std::integral_constant<int, 0>{}, 0, 0);
    load_v(std::integral_constant<int, 0>{}, 0, 0);
    load_k(std::integral_constant<int, 1>{}, 0, 1);
    load_v(std::integral_constant<int, 1>{}, 0, 1);
    f32x16 s[2][2];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        if (c == 0) { mfma_s<true, false>(s[0][0], kb[0][0], qreg[0][0]); mfma_s<true, true>(s[0][1], kb[0][0], qreg[1][0]); }
        else { mfma_s<false, false>(s[0][0], kb[0][c], qreg[0][c]); mfma_s<false, true>(s[0][1], kb[0][c], qreg[1][c]); }
    }
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");               // MFMA results before the VALU reads them
    load_k(std::integral_constant<int, 0>{}, 1, 0);                  // K(2)
    mask_pair(s[0], (uint32_t)w_mask[0]);
    {
        float mx[2];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            mx[qq] = fmaxf(s[0][qq][0], s[0][qq][1]);
#pragma unroll
            for (int i = 2; i < 16; i += 2) mx[qq] = fmaxf(fmaxf(mx[qq], s[0][qq][i]), s[0][qq][i + 1]);
        }
        raise_max(finish_max(mx[0]), finish_max(mx[1]));
    }

    // Step u = 2 g + j (j static).  S(u) is finished and the running maximum covers it.
    //   X: S(u+1) = K(u+1) . Q^T from ring slot (j+1) % 2, under the exp2 of the first part of S(u);
    //      then K(u+3) is requested into that slot.
    //   Y: O^T += V(u)^T P(u)^T from ring slot j % 2: the MFMAs of the first 16 keys under the exp2 of
    //      the rest of S(u), those of the last 16 keys under the row maximum of S(u+1);
    //      then V(u+2) is requested into that slot.
    auto step = [&](auto jj) {
        constexpr int j = decltype(jj)::value;
        constexpr int sc = j & 1, sn = sc ^ 1;                 // S(u) and S(u+1) alternate between two register sets
        constexpr int kslot = (j + 1) % kRing, vslot = j % kRing;
        float neg_m[2];
        V8 pb[2][2];                                            // P^T as B operand: [query half][key step]
        float psum[2];
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) neg_m[qq] = (m_i[qq] == -INFINITY) ? 0.f : -m_i[qq];
        // The exp2 of a pair of accumulators and the use of its results sit in different slots between the
        // MFMAs: a transcendental result cannot be consumed by the next instruction without a wait state.
        float pa0, pa1;
        auto exp_pair = [&](int n) {                            // pair n: query half n & 1, accumulators 2 (n >> 1), + 1
            const int qq = n & 1, i = 2 * (n >> 1);
            pa0 = __builtin_amdgcn_exp2f(fmaf(s[sc][qq][i], qk_scale, neg_m[qq]));
            pa1 = __builtin_amdgcn_exp2f(fmaf(s[sc][qq][i + 1], qk_scale, neg_m[qq]));
        };
        auto use_pair = [&](int n) {
            const int qq = n & 1, i = 2 * (n >> 1);
            if (n < 2) psum[qq] = pa0 + pa1;
            else psum[qq] += pa0 + pa1;
            pb[qq][i >> 3][i & 7] = (T)pa0;
            pb[qq][i >> 3][(i + 1) & 7] = (T)pa1;
            asm volatile("" : "+v"(psum[qq]), "+v"(pb[qq][i >> 3]));
        };
        constexpr int kPairsX = 12;                             // pairs handled under the MFMAs of X; the other 4 under Y
        __builtin_amdgcn_sched_barrier(0);
        // X: 16 MFMAs
#pragma unroll
        for (int c = 0; c < 8; ++c) {
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                if (qq == 0) {
                    if (c == 0) mfma_s<true, false>(s[sn][0], kb[kslot][0], qreg[0][0]);
                    else mfma_s<false, false>(s[sn][0], kb[kslot][c], qreg[0][c]);
                } else {
                    if (c == 0) mfma_s<true, true>(s[sn][1], kb[kslot][0], qreg[1][0]);
                    else mfma_s<false, true>(s[sn][1], kb[kslot][c], qreg[1][c]);
                }
                const int n = 2 * c + qq;                       // 0 .. 15
                if (n >= 1 && n <= kPairsX) use_pair(n - 1);
                if (n < kPairsX) exp_pair(n);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // K(u+3): tile window slot (j + 3) / 2, half (j + 1) & 1
        load_k(std::integral_constant<int, kslot>{}, (j + 3) >> 1, (j + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
        // Y, first 16 keys: 8 MFMAs under the remaining pairs
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                oacc[t][qq] = mfma32(vb[vslot][t], pb[qq][0], oacc[t][qq]);
                const int n = kPairsX + 2 * t + qq;             // 12 .. 19
                if (n > kPairsX && n <= 16) use_pair(n - 1);
                if (n < 16) exp_pair(n);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        l_i[0] += psum[0];
        l_i[1] += psum[1];
        // validity of the keys of step u + 1: tile window slot (j + 1) / 2, half (j + 1) & 1
        mask_pair(s[sn], (uint32_t)(w_mask[(j + 1) >> 1] >> (32 * ((j + 1) & 1))));
        // Y, last 16 keys: 8 MFMAs under the row maximum of S(u+1)
        float mx[2] = {fmaxf(s[sn][0][0], s[sn][0][1]), fmaxf(s[sn][1][0], s[sn][1][1])};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int qq = 0; qq < 2; ++qq) {
                oacc[t][qq] = mfma32(vb[vslot][4 + t], pb[qq][1], oacc[t][qq]);
                const int n = 2 * t + qq;                       // 0 .. 7: two of the 14 remaining accumulators each
                if (n < 7) {
                    mx[0] = fmaxf(fmaxf(mx[0], s[sn][0][2 * n + 2]), s[sn][0][2 * n + 3]);
                    mx[1] = fmaxf(fmaxf(mx[1], s[sn][1][2 * n + 2]), s[sn][1][2 * n + 3]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // V(u+2): tile window slot (j + 2) / 2, half j & 1
        load_v(std::integral_constant<int, vslot>{}, (j + 2) >> 1, j & 1);
        raise_max(finish_max(mx[0]), finish_max(mx[1]));
    };

    for (int g = 0; g < ntiles; ++g) {
        // entry of the window position that comes in (g + 4), read ahead
        const uint32_t n_tile = tile_of(g + 4);
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            w_tile[r] = w_tile[r + 1];
            w_mask[r] = w_mask[r + 1];
        }
        w_tile[3] = n_tile;
        w_mask[3] = mask_of(g + 4, n_tile);
    }
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
    const float qk_scale = sm_scale * kLog2e;
    FragLayout L;
    L.q_rows = q_rows;
    for (int i = 0; i < 3; ++i) { L.q_st[i] = q_st[i]; L.o_st[i] = o_st[i]; }
    const int per_head = (int)(Sq / kTile);
    const int total = B * Hn * per_head;
    const int resident = resident_wavefronts();
    const dim3 block(64);
    const uint32_t* gate = nullptr;
#define BSA_FRAG_LAUNCH(grid, begin, end, ord, que, want)                                                             \
    do {                                                                                                               \
        if (dtype == BSA_BF16)                                                                                         \
            hipLaunchKernelGGL((fwd_frag_kernel<__bf16>), grid, block, 0, st, (const __bf16*)q, (const char*)kf,       \
                               (const char*)vf, idx, lens, tile_valid, (__bf16*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, \
                               qk_scale, begin, end, Hn, lse_rows, L, ord, que, gate, want);                           \
        else                                                                                                           \
            hipLaunchKernelGGL((fwd_frag_kernel<_Float16>), grid, block, 0, st, (const _Float16*)q, (const char*)kf,   \
                               (const char*)vf, idx, lens, tile_valid, (_Float16*)o, lse, Sq, Sk, bs_q, bs_k,          \
                               idx_stride, qk_scale, begin, end, Hn, lse_rows, L, ord, que, gate, want);               \
    } while (0)
    if (queue != nullptr) {
        launch_schedule_choice(lens, (int)(Sq / bs_q), bs_q / kTile, total, resident, resident, idx_stride, queue, st);
        gate = queue + 1;
        const dim3 grid((unsigned)(total < resident ? total : resident));
        BSA_FRAG_LAUNCH(grid, 0, total, order, queue, 1u);
    }
    for (int first = 0; first < total; first += resident) {
        const int end = first + resident < total ? first + resident : total;
        const dim3 grid((unsigned)(end - first));
        BSA_FRAG_LAUNCH(grid, first, end, (const int32_t*)nullptr, (uint32_t*)nullptr, 0u);
    }
#undef BSA_FRAG_LAUNCH
    return hipGetLastError();
}

hipError_t launch_frag(const void* src, const int64_t st3[3], void* dst, int B, int Hn, const Grid3& g, int dtype,
                       bool transpose, hipStream_t st) {
    const dim3 grid((unsigned)(g.blocks() * (g.chunk() / kTile)), (unsigned)(B * Hn)), block(256);
    // 16-bit types move as raw bits
    if (transpose)
        hipLaunchKernelGGL((frag_kernel<uint16_t, true>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn);
    else
        hipLaunchKernelGGL((frag_kernel<uint16_t, false>), grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2],
                           (char*)dst, g, Hn);
    (void)dtype;
    return hipGetLastError();
}

}  // namespace bsa
