// Block-sparse flash-attention forward for gfx950 (bf16 / fp16 MFMA), plus a
// plain fp32 kernel for fp32 inputs.
//
// Work decomposition (MFMA kernel).  One workgroup = 256 threads = 4
// wavefronts processes one work item at a time: 64 query rows against the
// list of selected KV blocks, walked in 64-key tiles.  Wavefront (qh, kh) owns
// query rows 32*qh..+32 and keys 32*kh..+32 of every tile and runs an
// independent online softmax over its key half; the two halves are merged once
// per work item, in the epilogue, with the usual log-sum-exp rescale.
//
// Per tile and wavefront: S^T (32 keys x 32 queries) = K_half . Q^T as 8
// v_mfma_f32_32x32x16 over d = 128 (A = K rows from LDS, B = Q held in
// registers), so every lane ends up with one query column and 16 keys: the
// softmax state (running max, running sum) is one scalar per lane, and P^T in
// the accumulator registers already has the layout the B operand of the second
// product needs.  O^T (128 d x 32 queries) += V^T . P^T is 8 more MFMAs whose A
// operand (d along lanes, keys along the k slots) is read from the row-major V
// tile with the transposing LDS read ds_read_b64_tr_b16: 16 lanes fetch a
// 4-key x 16-d patch and each lane receives the 4 keys of one d.
//
// Data movement.  K and V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4, no staging registers): every wavefront issues
// 4 + 4 loads of 1 KB per tile.  The LDS side of such a load is linear in the
// lane index, so the XOR swizzle that keeps the later LDS reads free of bank
// conflicts is applied on the global side: lane l of a load fetches the
// 16-byte chunk (l%16) ^ f(row) of its row.  Two stages of (K 16 KB + V 16 KB)
// per workgroup, two workgroups per CU, one barrier per tile.
//
// Software pipeline.  An MFMA keeps the matrix pipe busy for 32 clocks, during
// which the SIMD goes on issuing VALU instructions, of the same wavefront or of
// its neighbour (measured: an MFMA followed by 7 independent VALU instructions
// takes about 40 clocks, not 60); a wavefront that waits on an MFMA result leaves
// the SIMD to its neighbour.  In iteration i the 8 MFMAs of S(i+1) are therefore
// interleaved with the exp2 of tile i, and the 8 MFMAs of O += P(i) V(i) with
// the row maximum of S(i+1).
//
// Softmax.  The running maximum is only raised when a row's new maximum
// exceeds it by more than 2^8 (lazy rescale): probabilities are then at most
// 2^8 instead of 1, which bf16/fp32 hold without loss, and the 64-register
// rescale of the output accumulator drops out of almost every iteration.  The
// result is the same softmax up to fp32 rounding.
//
// Scheduling.  The work items are launched in rounds of as many workgroups as
// the device runs at once (2 per CU), head after head.  The workgroups of a
// round start together and, because every item of a top-k selection has the
// same number of tiles, stay roughly in step.  With KV lists in ascending block
// order the workgroups of an XCD then sweep the K/V of a head in the same
// direction at the same time, which turns a large part of the tile fetches into
// L2 hits (the 4 MB L2 of an XCD cannot hold the 47 MB of K/V of one 720p head,
// and L2 misses are served at only ~8 TB/s for 16 KB tiles).  One launch of the
// whole grid loses this: workgroups then start whenever a slot frees up.
// Within a round every XCD takes a contiguous run of the query blocks (workgroup b
// runs on XCD b % 8): spatial neighbours select largely the same KV blocks on real
// inputs, and only the workgroups of one XCD share an L2.  The second, MFMA-only
// half of a step runs at raised wave priority, which puts the two wavefronts that
// share a SIMD (one of each resident workgroup) into alternating phases.
// Lists of unequal length (the CDF rule) have a second schedule: one launch
// whose workgroups draw the items, longest list first, from a counter.
#include "bsa_mfma.h"

namespace bsa {
namespace {

using namespace mfma;

template <typename T>
__global__ __launch_bounds__(256, 2) void fwd_mfma_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens,
    const uint64_t* __restrict__ tile_valid, T* __restrict__ o, float* __restrict__ lse,
    int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float qk_scale, int item_begin, int item_end,
    int Hn, int64_t lse_S, int64_t edge_bh_bytes, FwdLayout L, const int32_t* __restrict__ order,
    uint32_t* __restrict__ queue, const uint32_t* __restrict__ gate, uint32_t gate_want) {
    typedef typename Vec8<T>::type V8;
    // both schedules are enqueued when the lists may be of unequal length; a word written on the device
    // says which of them runs
    if (gate != nullptr && *gate != gate_want) return;
    __shared__ int next_sm;                   // queue mode: the rank this workgroup drew
    // [stage][0 = K tile | 1 = V tile][64 rows x 128], rows swizzled in 16-byte chunks
    __shared__ __attribute__((aligned(1024))) T smem[2][2][kTile * kD];
    // the tile list of the current work item: first key row and validity word per tile
    __shared__ int32_t tile_row_sm[kListCap];
    __shared__ uint64_t tile_mask_sm[kListCap];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int qh = wave & 1, kh = wave >> 1;
    const int lr = lane & 31, lh = lane >> 5;
    const int nbq = (int)(Sq / bs_q);
    const int nqt = (int)(Sq / kTile);
    const int nsub = bs_k / kTile;

    // ---- global -> LDS: load i of this wavefront fills LDS rows 4*(4*i + wave) .. +4 ----
    // lane: physical row 16*i + 4*wave + lane/16, physical chunk lane%16,
    // fetches logical chunk (lane%16) ^ f(row);  f_K(row) = row & 15, f_V(row) = (row & 3) << 2
    // The four rows of such a load are a run of 4 consecutive slots of the tile, which are 4
    // consecutive tokens along w in THW order as well: the lane part of the address (row in the
    // run, chunk in the row) is the same for every load and the position of the run goes into the
    // scalar base.  In blocked order the runs simply follow each other.
    const int drow = 4 * wave + (lane >> 4);
    const uint32_t kv_sb = (uint32_t)(L.k_st[2] * (int64_t)sizeof(T));        // token stride in bytes
    const uint32_t koff = (uint32_t)(lane >> 4) * kv_sb + (uint32_t)(((lane & 15) ^ (drow & 15)) << 4);
    const uint32_t voff = (uint32_t)(lane >> 4) * kv_sb + (uint32_t)(((lane & 15) ^ ((drow & 3) << 2)) << 4);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_address(&smem[0][0][0]) + wave * 1024);
    uint32_t run_off[4];     // load i of this wavefront fetches run 4*i + wave of the tile
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int slot = 16 * i + 4 * wave;
        const uint32_t rows = (uint32_t)(((slot / (L.kw * L.kh)) * L.kH + (slot / L.kw) % L.kh) * L.kW + slot % L.kw);
        run_off[i] = __builtin_amdgcn_readfirstlane(rows * kv_sb);
    }

    // ---- LDS read addresses (element offsets inside a tile) ----
    // K, A operand of S^T: row 32*kh + lr, logical chunk 2*c + lh
    const int krow = 32 * kh + lr;
    int kaddr[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) kaddr[c] = krow * kD + (((2 * c + lh) ^ (krow & 15)) << 3);
    // V, transposing read for (d tile t, key step c, half r):
    //   source lane s = lane%16 points at key 32*kh + 8*(2c + r) + 4*lh + s/4, d = 32*t + 16*g1 + 4*(s%4)
    const int s16 = lane & 15, g1 = (lane >> 4) & 1;
    const int vkey0 = 32 * kh + 4 * lh + (s16 >> 2);          // + 8*(2c + r)
    const int vsw = (vkey0 & 3) << 2;                          // key & 3 does not depend on c, r
    int vaddr[4];                                              // per d tile t, for key offset 0
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int chunk = 4 * t + 2 * g1 + ((s16 & 3) >> 1);
        vaddr[t] = vkey0 * kD + ((chunk ^ vsw) << 3) + (s16 & 1) * 4;
    }

    // Workgroup b of a launch runs on XCD b % 8 (round-robin dispatch).  Each XCD gets a contiguous run of
    // the launch's work items: neighbouring query blocks tend to select the same KV blocks, and only
    // workgroups of one XCD share an L2.
    int local = blockIdx.x;
    {
        const int n = item_end - item_begin, x = local & 7;
        local = x * (n >> 3) + min(x, n & 7) + (local >> 3);
    }
    // Two ways to hand out work items.  Rounds (queue == nullptr): the launch covers exactly one item
    // per workgroup.  Queue: the resident workgroups of one launch draw ranks from a counter until it
    // runs past the last item, and `order` (longest lists first) turns a rank into an item - for lists
    // of unequal length, where a round would wait for its longest one.
    for (;;) {
    if (queue != nullptr) {
        __syncthreads();                      // everybody has read the previous draw
        if (tid == 0) next_sm = (int)atomicAdd(queue, 1u);
        __syncthreads();
        local = next_sm;
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
    const int len_raw = lens[(int64_t)bh * nbq + qblock];
    const char* kbase = reinterpret_cast<const char*>(k + (int64_t)(bh / Hn) * L.k_st[0] + (int64_t)(bh % Hn) * L.k_st[1]);
    const char* vbase = reinterpret_cast<const char*>(v + (int64_t)(bh / Hn) * L.v_st[0] + (int64_t)(bh % Hn) * L.v_st[1]);

    // Q as the B operand: lane holds row 32*qh + lr, d = 16*s + 8*lh .. +8
    V8 qreg[8];
    {
        // padded query slots read token 0 (always there); their rows are never stored
        int64_t row = qrow0 + 32 * qh + lr;
        if (L.q_rows != nullptr) row = max(L.q_rows[row], 0);
        const T* qp = q + q_bh + row * L.q_st[2] + 8 * lh;
#pragma unroll
        for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const V8*>(qp + 16 * s);
    }
    // `entry` < 2^24: first token row of the tile, fetched run by run from where it lies.
    // Otherwise: 2^24 + index of a 64-slot tile in the blocked-order copies of the edge chunks.
    auto issue_tile = [&](const char* base, const char* edge, uint32_t entry, uint32_t lds, uint32_t off, int vswz) {
        if (__builtin_expect(entry < (1u << 24), 1)) {
            const char* tile = base + (uint64_t)entry * kv_sb;
#pragma unroll
            for (int i = 0; i < 4; ++i) load_to_lds_16(tile + run_off[i], off, lds + i * 4096);
        } else {
            // rare: the lane part for 256-byte rows is rebuilt from the thread index, which costs
            // nothing while the common path runs
            int t2 = tid;
            asm volatile("" : "+v"(t2));
            const int l2 = t2 & 63, d2 = 4 * (t2 >> 6) + (l2 >> 4);
            const uint32_t off2 = (uint32_t)(d2 * 256 + (((l2 & 15) ^ (vswz ? (d2 & 3) << 2 : d2 & 15)) << 4));
            const char* tile = edge + (uint64_t)(entry & 0xffffffu) * kTileBytes;
#pragma unroll
            for (int i = 0; i < 4; ++i) load_to_lds_16(tile + i * 4096, off2, lds + i * 4096);
        }
    };
    const char* kedge = reinterpret_cast<const char*>(L.k_edge) + (int64_t)bh * edge_bh_bytes;
    const char* vedge = reinterpret_cast<const char*>(L.v_edge) + (int64_t)bh * edge_bh_bytes;
    auto issue_k = [&](uint32_t entry, int st) { issue_tile(kbase, kedge, entry, lds0 + st * (2 * kTileBytes), koff, 0); };
    auto issue_v = [&](uint32_t entry, int st) {
        issue_tile(vbase, vedge, entry, lds0 + st * (2 * kTileBytes) + kTileBytes, voff, 1);
    };

    f32x16 oacc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[t][i] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;

    // A list row of at most 256 tiles is staged whole before the length of the list has arrived (one
    // dependent load less before the first tile can be fetched): what lies behind the length is
    // clamped like any entry and never walked.  Longer rows wait for the length and go in chunks.
    const bool early = idx_stride * nsub <= 256;
    int ntiles = early ? idx_stride * nsub : min(max(len_raw, 0), idx_stride) * nsub;   // never past the list row
    for (int chunk0 = 0; chunk0 < ntiles; chunk0 += kListCap) {
    int nloc = min(ntiles - chunk0, kListCap);
    __syncthreads();                          // previous chunk / previous item fully consumed
    for (int j = tid; j < nloc; j += 256) {
        const int it = chunk0 + j;
        // a block index outside [0, Sk / bs_k) is clamped: a malformed list gives wrong numbers, never a fault
        const int blk = min(max(list[it / nsub], 0), (int)(Sk / bs_k) - 1);
        const int tile = blk * nsub + it % nsub;
        const uint32_t entry = L.k_tiles != nullptr ? L.k_tiles[tile] : (uint32_t)tile * kTile;
        tile_row_sm[j] = (int)entry;
        tile_mask_sm[j] = tile_valid ? tile_valid[tile] : ~0ull;
    }
    if (early) {
        ntiles = nloc = min(max(len_raw, 0), idx_stride) * nsub;
        if (ntiles == 0) break;
    }
    // consume the Q loads here: otherwise their vmcnt waits land inside the tile loop,
    // where they would also wait for the LDS loads of the next tile
#pragma unroll
    for (int s = 0; s < 8; ++s) asm volatile("" :: "v"(qreg[s]));
    __syncthreads();

    // Padded keys of tile j get -inf (accumulator i <-> key 32*kh + 8*(i/4) + 4*lh + i%4, query lr).
    auto mask_tile = [&](f32x16& s, uint64_t vmask) {
        if (__builtin_expect(vmask != ~0ull, 0)) {
            const uint32_t half = (uint32_t)(vmask >> (32 * kh));
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (!((half >> (8 * (i / 4) + 4 * lh + (i % 4))) & 1u)) s[i] = -INFINITY;
        }
    };
    // Raises the running maximum (and rescales the accumulators) only when some row's new maximum
    // `mx` (already combined over the tile and scaled) exceeds it by more than 2^kLazyTau.
    auto raise_max = [&](float mx) {
        if (__builtin_expect(__any(mx > m_i + kLazyTau), 0)) {
            const float m_new = fmaxf(m_i, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_i - ((m_new == -INFINITY) ? 0.f : m_new));
            m_i = m_new;
            l_i *= alpha;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[t][i] *= alpha;
        }
    };
    // combine a lane's maximum with the other key group of the same query (lane ^ 32) and scale it
    auto finish_max = [&](float mx) -> float {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
        return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * qk_scale;
    };
    auto update_max = [&](const f32x16& s) {
        float mx = fmaxf(s[0], s[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
        raise_max(finish_max(mx));
    };
    auto qk_plain = [&](auto stage) -> f32x16 {      // S^T from K stage st, nothing interleaved
        constexpr int st = decltype(stage)::value;
        const T* ks = smem[st][0];
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) s = mfma32(*reinterpret_cast<const V8*>(ks + kaddr[c]), qreg[c], s);
        return s;
    };

    // K(i) and V(i) live in stage i&1.  Iteration i, with S(i) finished and the running maximum
    // already raised for it:
    //   X: the 8 MFMAs of S(i+1), each followed by the exp2 of two probabilities of tile i;
    //   Y: the 8 MFMAs of O += P(i) V(i), interleaved with the row sum of P(i);
    //   then the maximum of S(i+1) (its rare rescale waits for Y by data dependence).
    // At the top of iteration i the loads issued one iteration earlier (V(i), K(i+1)) are awaited,
    // then V(i+1) and K(i+2) are issued.
    issue_k(__builtin_amdgcn_readfirstlane(tile_row_sm[0]), 0);
    issue_v(__builtin_amdgcn_readfirstlane(tile_row_sm[0]), 0);
    if (nloc > 1) issue_k(__builtin_amdgcn_readfirstlane(tile_row_sm[1]), 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // S^T of the current and of the next tile alternate between two register sets
    f32x16 s_a = qk_plain(std::integral_constant<int, 0>{}), s_b;
    mask_tile(s_a, tile_mask_sm[0]);
    update_max(s_a);
    int row_v = nloc > 1 ? __builtin_amdgcn_readfirstlane(tile_row_sm[1]) : 0;   // first key row of tile it+1
    int row_pref = tile_row_sm[nloc > 2 ? 2 : 0];                                     // ... of tile it+2, read ahead

    // An LDS read takes about as long as four MFMAs, so every fragment is requested four MFMAs
    // before the one that consumes it; sched_barrier pins that order.
    // full_step: tile `it` is not the last one of the list.  S(it+1) runs on the MFMA unit while the
    // VALU turns S(it) into P(it); then O += P(it) V(it).
    auto full_step = [&](int it, auto stage, f32x16& s_cur, f32x16& s_next) {
        constexpr int st = decltype(stage)::value;
        const T* ks = smem[st ^ 1][0];
        const T* vs = smem[st][1];
        auto read_v = [&](int u) -> V8 {             // u = 2*t + c
            const int t = u >> 1, c = u & 1;
            const s16x4 lo = lds_read_tr16(vs + vaddr[t] + (8 * (2 * c)) * kD);
            const s16x4 hi = lds_read_tr16(vs + vaddr[t] + (8 * (2 * c + 1)) * kD);
            return __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        };
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's share of V(it), K(it+1) is in LDS
        __syncthreads();                                     // ... and everybody else's; K(it), V(it-1) are consumed
        V8 kf[8], vf[8];
#pragma unroll
        for (int c = 0; c < 4; ++c) kf[c] = *reinterpret_cast<const V8*>(ks + kaddr[c]);
        const uint64_t mask_next = tile_mask_sm[it + 1];     // needed only after the 8 MFMAs below
        __builtin_amdgcn_sched_barrier(0);
        issue_v(row_v, st ^ 1);
        row_v = __builtin_amdgcn_readfirstlane(row_pref);    // tile it+2: K now, V in the next step
        if (it + 2 < nloc) issue_k(row_v, st);
        const float neg_m = (m_i == -INFINITY) ? 0.f : -m_i;
        V8 pb[2];      // P^T as B operand: k-slot (lh, j) of step c <-> accumulator 8*c + j
        float psum = 0.f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (c + 4 < 8) kf[c + 4] = *reinterpret_cast<const V8*>(ks + kaddr[c + 4]);
            else vf[c - 4] = read_v(c - 4);
            if (c == 0) {
                f32x16 zero;
#pragma unroll
                for (int i = 0; i < 16; ++i) zero[i] = 0.f;
                s_next = mfma32(kf[0], qreg[0], zero);
            } else {
                s_next = mfma32(kf[c], qreg[c], s_next);
            }
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s_cur[2 * c], qk_scale, neg_m));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s_cur[2 * c + 1], qk_scale, neg_m));
            psum += p0 + p1;
            pb[c >> 2][(2 * c) & 7] = (T)p0;
            pb[c >> 2][(2 * c + 1) & 7] = (T)p1;
            // keep this VALU work here, between the MFMAs: without a use in this block the compiler
            // sinks it below the branch that follows the loop
            asm volatile("" : "+v"(psum), "+v"(pb[c >> 2]));
            __builtin_amdgcn_sched_barrier(0);
        }
        l_i += psum;
        mask_tile(s_next, mask_next);
        row_pref = tile_row_sm[it + 3 < nloc ? it + 3 : 0];  // consumed at the top of the next step
        // O += P(it) V(it); the row maximum of S(it+1) fills the VALU slots between the MFMAs.
        // This stretch runs at a raised wave priority: of the two wavefronts that share a SIMD (one of
        // each resident workgroup) the one in its MFMA-only phase goes first, reaches the top of its next
        // step - where the tile loads are issued - sooner, and the two fall into alternating phases.
        __builtin_amdgcn_s_setprio(1);
        float mx = fmaxf(s_next[0], s_next[1]);
#pragma unroll
        for (int u = 0; u < 8; ++u) {        // u = 2*t + c
            if (u + 4 < 8) vf[u + 4] = read_v(u + 4);
            oacc[u >> 1] = mfma32(vf[u], pb[u & 1], oacc[u >> 1]);
            if (u < 7) mx = fmaxf(fmaxf(mx, s_next[2 * u + 2]), s_next[2 * u + 3]);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
        raise_max(finish_max(mx));
    };
    // last_step: the final tile of the list, nothing left to prefetch or to overlap with.
    auto last_step = [&](int it, auto stage, f32x16& s_cur) {
        constexpr int st = decltype(stage)::value;
        const T* vs = smem[st][1];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const float neg_m = (m_i == -INFINITY) ? 0.f : -m_i;
        V8 pb[2];
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s_cur[i], qk_scale, neg_m));
            psum += p;
            pb[i >> 3][i & 7] = (T)p;
        }
        l_i += psum;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = u >> 1, c = u & 1;
            const s16x4 lo = lds_read_tr16(vs + vaddr[t] + (8 * (2 * c)) * kD);
            const s16x4 hi = lds_read_tr16(vs + vaddr[t] + (8 * (2 * c + 1)) * kD);
            const s16x8 av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            oacc[t] = mfma32(__builtin_bit_cast(V8, av), pb[c], oacc[t]);
        }
    };
    int it = 0;
    for (; it + 2 < nloc; it += 2) {
        full_step(it, std::integral_constant<int, 0>{}, s_a, s_b);
        full_step(it + 1, std::integral_constant<int, 1>{}, s_b, s_a);
    }
    if (nloc - it == 2) {
        full_step(it, std::integral_constant<int, 0>{}, s_a, s_b);
        last_step(it + 1, std::integral_constant<int, 1>{}, s_b);
    } else {
        last_step(it, std::integral_constant<int, 0>{}, s_a);
    }
    }
    __syncthreads();

    // ---- epilogue: merge the two key halves, normalise, store coalesced ----
    const int kc = tid & 15, kr = tid >> 4;
    float* xch = reinterpret_cast<float*>(&smem[0][0][0]);                  // [qh][66][64] fp32
    constexpr int kOutPitch = kD + 8;
    T* ost = reinterpret_cast<T*>(reinterpret_cast<char*>(xch) + 2 * 66 * 64 * 4);   // [64][kOutPitch]
    if (kh == 1) {
        float* dst = xch + qh * 66 * 64 + lane;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[(t * 16 + i) * 64] = oacc[t][i];
        dst[64 * 64] = m_i;
        dst[65 * 64] = l_i;
    }
    __syncthreads();
    if (kh == 0) {
        const float* src = xch + qh * 66 * 64 + lane;
        const float m1 = src[64 * 64];
        float l1 = src[65 * 64];
        float l0 = l_i + __shfl_xor(l_i, 32);
        l1 = l1 + __shfl_xor(l1, 32);
        const float m = fmaxf(m_i, m1);
        const float m_safe = (m == -INFINITY) ? 0.f : m;
        const float a0 = __builtin_amdgcn_exp2f(m_i - m_safe);
        const float a1 = __builtin_amdgcn_exp2f(m1 - m_safe);
        const float l = a0 * l0 + a1 * l1;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        // rows of the staging tile are 272 B apart: at 256 B the 32 rows that one store instruction touches
        // would all lie in the same banks
        T* orow = ost + (32 * qh + lr) * kOutPitch;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                T out4[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = 4 * g + j;
                    out4[j] = (T)((oacc[t][i] * a0 + src[(t * 16 + i) * 64] * a1) * inv);
                }
                *reinterpret_cast<uint2*>(orow + 32 * t + 8 * g + 4 * lh) = *reinterpret_cast<uint2*>(out4);
            }
        if (lse != nullptr && lh == 0) {
            int64_t row = qrow0 + 32 * qh + lr;
            if (L.q_rows != nullptr) row = L.q_rows[row];
            if (row >= 0) lse[(int64_t)bh * lse_S + row] = l > 0.f ? (m + __builtin_log2f(l)) * kLn2 : -INFINITY;
        }
    }
    __syncthreads();
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = kr + 16 * i;
            int64_t row = qrow0 + r;
            if (L.q_rows != nullptr) row = L.q_rows[row];
            if (row >= 0)
                *reinterpret_cast<uint4*>(o + o_bh + row * L.o_st[2] + kc * 8) =
                    *reinterpret_cast<const uint4*>(ost + r * kOutPitch + kc * 8);
        }
    }
    if (queue == nullptr) break;
    }   // work items
}

// ------------------------------------------------------------------ fp32
// 4 lanes per query row, each owning the d values 4*p + 16*j .. +4 (j = 0..7);
// K and V tiles staged in LDS as fp32; one online-softmax step per key.
__global__ __launch_bounds__(256) void fwd_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens,
    const uint64_t* __restrict__ tile_valid, float* __restrict__ o, float* __restrict__ lse,
    int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float qk_scale) {
    __shared__ __attribute__((aligned(16))) float ks[kTile * kD];
    __shared__ __attribute__((aligned(16))) float vs[kTile * kD];
    const int tid = threadIdx.x;
    const int r = tid >> 2, p = tid & 3;
    const int bh = blockIdx.y;
    const int64_t qrow0 = (int64_t)blockIdx.x * kTile;
    const int nbq = (int)(Sq / bs_q);
    const int qblock = (int)(qrow0 / bs_q);
    const int nsub = bs_k / kTile;
    const int32_t* list = idx + ((int64_t)bh * nbq + qblock) * idx_stride;
    const int ntiles = min(max(lens[(int64_t)bh * nbq + qblock], 0), idx_stride) * nsub;   // never past the list row
    const float* kbase = k + (int64_t)bh * Sk * kD;
    const float* vbase = v + (int64_t)bh * Sk * kD;

    float4 qv[8], acc[8];
    const float* qp = q + ((int64_t)bh * Sq + qrow0 + r) * kD + 4 * p;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        qv[j] = *reinterpret_cast<const float4*>(qp + 16 * j);
        acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float m_i = -INFINITY, l_i = 0.f;
    for (int it = 0; it < ntiles; ++it) {
        const int64_t row0 = (int64_t)min(max(list[it / nsub], 0), (int)(Sk / bs_k) - 1) * bs_k + (int64_t)(it % nsub) * kTile;
        const uint64_t vmask = tile_valid ? tile_valid[row0 / kTile] : ~0ull;
        __syncthreads();
        for (int i = tid; i < kTile * kD / 4; i += 256) {
            reinterpret_cast<float4*>(ks)[i] = reinterpret_cast<const float4*>(kbase + row0 * kD)[i];
            reinterpret_cast<float4*>(vs)[i] = reinterpret_cast<const float4*>(vbase + row0 * kD)[i];
        }
        __syncthreads();
        for (int key = 0; key < kTile; ++key) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float4 kk = *reinterpret_cast<const float4*>(ks + key * kD + 16 * j + 4 * p);
                s = fmaf(qv[j].x, kk.x, s); s = fmaf(qv[j].y, kk.y, s);
                s = fmaf(qv[j].z, kk.z, s); s = fmaf(qv[j].w, kk.w, s);
            }
            s += __shfl_xor(s, 1);
            s += __shfl_xor(s, 2);
            if (!((vmask >> key) & 1ull)) continue;
            s *= qk_scale;
            const float m_new = fmaxf(m_i, s);
            const float alpha = exp2f(m_i - m_new);
            const float pe = exp2f(s - m_new);
            l_i = l_i * alpha + pe;
            m_i = m_new;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float4 vv = *reinterpret_cast<const float4*>(vs + key * kD + 16 * j + 4 * p);
                acc[j].x = fmaf(pe, vv.x, acc[j].x * alpha); acc[j].y = fmaf(pe, vv.y, acc[j].y * alpha);
                acc[j].z = fmaf(pe, vv.z, acc[j].z * alpha); acc[j].w = fmaf(pe, vv.w, acc[j].w * alpha);
            }
        }
    }
    const float inv = l_i > 0.f ? 1.0f / l_i : 0.f;
    float* op = o + ((int64_t)bh * Sq + qrow0 + r) * kD + 4 * p;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        *reinterpret_cast<float4*>(op + 16 * j) =
            make_float4(acc[j].x * inv, acc[j].y * inv, acc[j].z * inv, acc[j].w * inv);
    if (lse != nullptr && p == 0)
        lse[(int64_t)bh * Sq + qrow0 + r] = l_i > 0.f ? (m_i + log2f(l_i)) * kLn2 : -INFINITY;
}

}  // namespace

__global__ void zero_words_kernel(uint32_t* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// order[bh * per_head + r] = the work item (64-row query tile) of (batch, head) bh with the r-th longest
// list: a counting sort on the list lengths, one workgroup per (batch, head).  Items of equal length
// keep no particular order (the result of an item does not depend on when it runs).
__global__ __launch_bounds__(256) void order_by_length_kernel(const int32_t* __restrict__ lens, int32_t* __restrict__ order,
                                                              int nbq, int tiles_per_block, int max_len) {
    extern __shared__ int bins[];             // [max_len + 1] counts, then running offsets
    const int bh = blockIdx.x, per_head = nbq * tiles_per_block;
    for (int i = threadIdx.x; i <= max_len; i += 256) bins[i] = 0;
    __syncthreads();
    for (int t = threadIdx.x; t < per_head; t += 256)
        atomicAdd(&bins[min(max(lens[(int64_t)bh * nbq + t / tiles_per_block], 0), max_len)], 1);
    __syncthreads();
    if (threadIdx.x == 0) {                   // offsets in descending length
        int run = 0;
        for (int l = max_len; l >= 0; --l) { const int c = bins[l]; bins[l] = run; run += c; }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < per_head; t += 256) {
        const int l = min(max(lens[(int64_t)bh * nbq + t / tiles_per_block], 0), max_len);
        order[(int64_t)bh * per_head + atomicAdd(&bins[l], 1)] = bh * per_head + t;
    }
}

// Rounds or queue?  A round lasts as long as its longest list, the queue keeps every workgroup busy but
// gives up the lock-step walk (measured on equal lists: 1.55 x the time).  *choice = 1 (queue) when
// 1.55 * (sum of lengths / resident workgroups) + longest < sum over rounds of the longest list of each round.
__global__ __launch_bounds__(256) void choose_schedule_kernel(const int32_t* __restrict__ lens, int nbq, int tiles_per_block,
                                                              int total, int round, int resident, int max_len,
                                                              uint32_t* __restrict__ choice) {
    constexpr int kMaxRounds = 8192;
    __shared__ int round_max[kMaxRounds];
    __shared__ unsigned long long sum_sm;
    __shared__ int longest_sm;
    const int n_rounds = (total + round - 1) / round;
    if (n_rounds > kMaxRounds) { if (threadIdx.x == 0) *choice = 0u; return; }
    for (int r = threadIdx.x; r < n_rounds; r += 256) round_max[r] = 0;
    if (threadIdx.x == 0) { sum_sm = 0ull; longest_sm = 0; }
    __syncthreads();
    unsigned long long sum = 0ull;
    int longest = 0;
    for (int item = threadIdx.x; item < total; item += 256) {
        const int per_head = nbq * tiles_per_block;
        const int bh = item / per_head, t = item % per_head;
        const int l = min(max(lens[(int64_t)bh * nbq + t / tiles_per_block], 0), max_len);
        sum += (unsigned long long)l;
        longest = max(longest, l);
        atomicMax(&round_max[item / round], l);
    }
    atomicAdd(&sum_sm, sum);
    atomicMax(&longest_sm, longest);
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long rounds_cost = 0ull;
        for (int r = 0; r < n_rounds; ++r) rounds_cost += (unsigned long long)round_max[r] * (unsigned long long)(round / resident);
        // rounds of `round` items run as round / resident waves of workgroups, each as long as its longest list:
        // an upper bound for the rounds, which only makes the comparison cautious
        const double queue_cost = 1.55 * (double)sum_sm / (double)resident + (double)longest_sm;
        *choice = queue_cost < (double)rounds_cost ? 1u : 0u;
    }
}

void launch_schedule_choice(const int32_t* lens, int nbq, int tiles_per_block, int total, int round, int resident,
                            int max_len, uint32_t* queue, hipStream_t st) {
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, st, queue, 1);
    hipLaunchKernelGGL(choose_schedule_kernel, dim3(1), dim3(256), 0, st, lens, nbq, tiles_per_block, total, round, resident,
                       max_len, queue + 1);
}

hipError_t launch_order_by_length(const int32_t* lens, int32_t* order, int BH, int nbq, int tiles_per_block, int max_len,
                                  hipStream_t st) {
    hipLaunchKernelGGL(order_by_length_kernel, dim3((unsigned)BH), dim3(256), (size_t)(max_len + 1) * sizeof(int), st, lens, order,
                       nbq, tiles_per_block, max_len);
    return hipGetLastError();
}

// Workgroups the device runs at once with this kernel (2 per CU), cached per device.
static int resident_workgroups() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 512;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = 2 * cus;
    }
    return cached[dev];
}

hipError_t launch_fwd(const void* q, const void* k, const void* v, const int32_t* idx,
                      const int32_t* lens, const uint64_t* tile_valid, void* o, float* lse, int B,
                      int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
                      float sm_scale, int dtype, hipStream_t st, const FwdLayout* layout, int64_t layout_lse_rows,
                      int64_t layout_edge_bytes, const int32_t* order, uint32_t* queue) {
    const float qk_scale = sm_scale * kLog2e;
    FwdLayout L;
    int64_t lse_S = Sq, edge_bh_bytes = 0;
    if (layout != nullptr) {
        L = *layout;
        lse_S = layout_lse_rows;
        edge_bh_bytes = layout_edge_bytes;
    } else {
        L.q_rows = nullptr;
        L.k_tiles = nullptr;
        L.k_edge = L.v_edge = nullptr;
        L.q_st[0] = L.o_st[0] = (int64_t)Hn * Sq * kD;
        L.q_st[1] = L.o_st[1] = Sq * kD;
        L.k_st[0] = L.v_st[0] = (int64_t)Hn * Sk * kD;
        L.k_st[1] = L.v_st[1] = Sk * kD;
        L.q_st[2] = L.o_st[2] = L.k_st[2] = L.v_st[2] = kD;
        L.kw = 4; L.kh = 16; L.kH = 16; L.kW = 4;     // 16 runs of 4 rows, one after the other
    }
    const dim3 block(256);
    if (dtype == BSA_F32) {
        const dim3 grid((unsigned)(Sq / kTile), (unsigned)(B * Hn));
        hipLaunchKernelGGL(fwd_f32_kernel, grid, block, 0, st, (const float*)q, (const float*)k,
                           (const float*)v, idx, lens, tile_valid, (float*)o, lse, Sq, Sk, bs_q,
                           bs_k, idx_stride, qk_scale);
        return hipGetLastError();
    }
    // One launch per round of as many work items as the device runs at once: the workgroups of a
    // launch start together and walk their (ascending) KV lists in step, so that a tile fetched
    // by one of them is still in L2 when its neighbours ask for it.  When the query tiles of a head
    // fill whole rounds, every round works on one head's K/V; otherwise the rounds run on across
    // the (batch, head) boundaries rather than leave the last round of every head partly empty:
    // an XCD takes a contiguous run of a round's items, so even in a round that holds two heads
    // almost every XCD still works on one.
    const int per_head = (int)(Sq / kTile);
    // short lists: three (at most 64 tiles) or two (at most 128) items per resident workgroup and launch, so
    // that the gap between launches and the wait for a round's slowest workgroup weigh less (39 tiles: -4 %,
    // 90 tiles: -1.5 %, nothing at 156 tiles)
    const int resident = resident_workgroups();
    const int list_tiles = idx_stride * (bs_k / kTile);
    const int round = resident * (list_tiles <= 64 ? 3 : list_tiles <= 128 ? 2 : 1);
    const uint32_t* gate = nullptr;
    if (queue != nullptr) {
        // Lists of possibly unequal length.  queue[0] is the counter the items are drawn with, queue[1] the
        // choice between the two schedules, made on the device from the lengths; both are enqueued.
        const int total = B * Hn * per_head;
        launch_schedule_choice(lens, (int)(Sq / bs_q), bs_q / kTile, total, round, resident, idx_stride, queue, st);
        gate = queue + 1;
        const dim3 grid((unsigned)(total < resident ? total : resident));
        if (dtype == BSA_BF16)
            hipLaunchKernelGGL((fwd_mfma_kernel<__bf16>), grid, block, 0, st, (const __bf16*)q,
                               (const __bf16*)k, (const __bf16*)v, idx, lens, tile_valid, (__bf16*)o,
                               lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, 0, total, Hn, lse_S, edge_bh_bytes, L, order, queue, gate, 1u);
        else
            hipLaunchKernelGGL((fwd_mfma_kernel<_Float16>), grid, block, 0, st, (const _Float16*)q,
                               (const _Float16*)k, (const _Float16*)v, idx, lens, tile_valid,
                               (_Float16*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, 0, total, Hn, lse_S, edge_bh_bytes, L, order, queue, gate, 1u);
    }
    const int tail = per_head % round;
    const bool across = tail != 0;
    const int n_outer = across ? 1 : B * Hn;
    const int n_inner = across ? B * Hn * per_head : per_head;
    for (int bh = 0; bh < n_outer; ++bh) {
        for (int first = 0; first < n_inner; first += round) {
            const int begin = bh * per_head + first;
            const int end = bh * per_head + (first + round < n_inner ? first + round : n_inner);
            const dim3 grid((unsigned)(end - begin));
            if (dtype == BSA_BF16)
                hipLaunchKernelGGL((fwd_mfma_kernel<__bf16>), grid, block, 0, st, (const __bf16*)q,
                                   (const __bf16*)k, (const __bf16*)v, idx, lens, tile_valid, (__bf16*)o,
                                   lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, begin, end, Hn, lse_S, edge_bh_bytes, L, nullptr, nullptr, gate, 0u);
            else
                hipLaunchKernelGGL((fwd_mfma_kernel<_Float16>), grid, block, 0, st, (const _Float16*)q,
                                   (const _Float16*)k, (const _Float16*)v, idx, lens, tile_valid,
                                   (_Float16*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale, begin, end, Hn, lse_S, edge_bh_bytes, L, nullptr, nullptr, gate, 0u);
        }
    }
    return hipGetLastError();
}

}  // namespace bsa
