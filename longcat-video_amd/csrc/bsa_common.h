// Shared declarations of the gfx950 block-sparse attention engine.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "bsa_mi355x.h"

namespace bsa {

// Geometry of a (T,H,W) token grid cut into (t,h,w) chunks, padded high.
struct Grid3 {
    int T, H, W;      // real grid
    int t, h, w;      // chunk shape
    int Nt, Nh, Nw;   // chunks per axis (ceil)
    __host__ __device__ int chunk() const { return t * h * w; }
    __host__ __device__ int blocks() const { return Nt * Nh * Nw; }
};

inline Grid3 make_grid(int T, int H, int W, int t, int h, int w) {
    Grid3 g;
    g.T = T; g.H = H; g.W = W; g.t = t; g.h = h; g.w = w;
    g.Nt = (T + t - 1) / t; g.Nh = (H + h - 1) / h; g.Nw = (W + w - 1) / w;
    return g;
}

// Where the rows of the attention operands live.  Blocked order: tile i of a (batch, head) is rows
// 64*i .. 64*i+63 of a contiguous [B, Hn, S, D] tensor.  THW order: tile i is (a 64-slot part of)
// chunk i of the grid and its slots are gathered from / scattered to token positions, so the
// separate permute and unpermute passes over that tensor disappear.  Strides are in elements:
// batch, head, token.
struct FwdLayout {
    // token row of every blocked-order query slot, -1 for padding ([Sq]); null: q and o are in
    // blocked order themselves
    const int32_t* q_rows;
    // per 64-slot kv tile: token row of its first slot (< 2^24) when the tile is read where it
    // lies, or 2^24 + index of the tile in the edge copies ([Sk / 64]); null: k and v are in
    // blocked order themselves
    const uint32_t* k_tiles;
    int64_t q_st[3], o_st[3], k_st[3], v_st[3];   // k_st[2] == v_st[2]
    // blocked-order, zero-padded copies of the chunks that touch the padded high edge of the kv
    // grid, [B*Hn][edge_count][chunk][D]; every other chunk is read where it lies
    const void* k_edge;
    const void* v_edge;
    int kw, kh, kH, kW;        // kv tile geometry: runs of kw slots, kh runs per plane, grid H and W
};

// Chunks with padded slots ("edge chunks") are numbered densely: first the whole last t layer if
// T is ragged, then the last h row of the remaining layers if H is ragged, then the last w column
// of what is left if W is ragged.  Returns -1 for a chunk without padding.
__host__ __device__ inline int edge_index(const Grid3& g, int blk) {
    const int nw = blk % g.Nw, nh = (blk / g.Nw) % g.Nh, nt = blk / (g.Nw * g.Nh);
    const bool rt = g.T % g.t != 0, rh = g.H % g.h != 0, rw = g.W % g.w != 0;
    const int Nt1 = g.Nt - (rt ? 1 : 0), Nh1 = g.Nh - (rh ? 1 : 0);
    int base = 0;
    if (rt) {
        if (nt == g.Nt - 1) return nh * g.Nw + nw;
        base += g.Nh * g.Nw;
    }
    if (rh) {
        if (nh == g.Nh - 1) return base + nt * g.Nw + nw;
        base += Nt1 * g.Nw;
    }
    if (rw && nw == g.Nw - 1) return base + nt * Nh1 + nh;
    return -1;
}
inline int edge_count(const Grid3& g) {
    const bool rt = g.T % g.t != 0, rh = g.H % g.h != 0, rw = g.W % g.w != 0;
    const int Nt1 = g.Nt - (rt ? 1 : 0), Nh1 = g.Nh - (rh ? 1 : 0);
    return (rt ? g.Nh * g.Nw : 0) + (rh ? Nt1 * g.Nw : 0) + (rw ? Nt1 * Nh1 : 0);
}

// k and v tiles can be gathered from THW order when a 64-slot tile is a whole number of (h, w)
// planes of its chunk, built from runs of at least 4 tokens along w, and when all offsets inside
// a tile fit 32 bits.
inline bool kv_direct_ok(const Grid3& g, int64_t token_stride_bytes) {
    auto pow2 = [](int x) { return x > 0 && (x & (x - 1)) == 0; };
    if (!pow2(g.w) || !pow2(g.h) || g.w < 4 || g.w > 64) return false;
    if ((64 / g.w) % g.h != 0) return false;
    if ((int64_t)g.T * g.H * g.W >= (1 << 24)) return false;
    const int64_t planes = 64 / (g.w * g.h);
    return token_stride_bytes > 0 && planes * g.H * g.W * token_stride_bytes < ((int64_t)1 << 32);
}

inline int dtype_size(int dtype) {
    switch (dtype) {
        case BSA_BF16: case BSA_F16: return 2;
        case BSA_F32: return 4;
        default: return 0;
    }
}

// Records the message returned by bsa_last_error() and passes `code` through.
int set_error(int code, const char* fmt, ...);

// Kernel launchers (one per source file); all validate nothing and assume the
// C-ABI layer has checked shapes.  Each returns a hipError_t from the launch.
// edge_only: dst is [B*Hn][edge_count(g)][chunk][D] and only chunks with padded slots are copied
// row_table ([S_padded] int32): token row of every blocked-order slot, -1 for padding.
// tile_table ([S_padded/64] uint32): FwdLayout::k_tiles.  Both optional.
// src2 / dst2 (edge_only): a second tensor on the same grid whose edge chunks are copied as well.
hipError_t launch_permute(const void* src, const int64_t strides[3], void* dst, void* pooled,
                          uint64_t* tile_valid, int B, int Hn, const Grid3& g, int D, int dtype,
                          hipStream_t st, bool edge_only = false, int32_t* row_table = nullptr,
                          uint32_t* tile_table = nullptr, const void* src2 = nullptr,
                          const int64_t* strides2 = nullptr, void* dst2 = nullptr);
// Chunk means of a 16-bit tensor with 64-slot chunks and D = 128, nothing else: the bits of launch_permute's pooling
// from a read-only pass.  row_table: the token of every slot of one (batch, head), -1 for padding, as launch_permute
// writes it.
hipError_t launch_pool_tiles(const void* src, const int64_t strides[3], const int32_t* row_table, void* pooled, int B, int Hn,
                             const Grid3& g, int dtype, hipStream_t st);
hipError_t launch_unpermute(const void* src, void* dst, const int64_t strides[3], int B, int Hn,
                            const Grid3& g, int D, int dtype, hipStream_t st);
hipError_t launch_mean_pool(const void* x, void* out, int B, int Hn, int64_t S, int block, int D,
                            int dtype, hipStream_t st);
hipError_t launch_score(const void* q_cmp, const void* k_cmp, void* score, int BH, int nbq, int nbk,
                        int D, int dtype, hipStream_t st);
// idx: descending score order; idx_sorted: ascending block index; either may be null
// k_rows: one count per row instead of k_sel (may alias lens); stride: row pitch of idx / idx_sorted
// (default k_sel), entries past a row's count are set to -1
hipError_t launch_topk(const void* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                       int nbk, int k_sel, int dtype, hipStream_t st, const int32_t* k_rows = nullptr,
                       int stride = 0);
// lens[row] = number of columns the CDF rule keeps, clamped to [k_min, cap]
hipError_t launch_cdf_count(const void* score, int32_t* lens, int64_t rows, int nbk, float threshold,
                            float scale, int k_min, int cap, int dtype, hipStream_t st);
hipError_t launch_fwd(const void* q, const void* k, const void* v, const int32_t* idx,
                      const int32_t* lens, const uint64_t* tile_valid, void* o, float* lse,
                      int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
                      float sm_scale, int dtype, hipStream_t st, const FwdLayout* layout = nullptr,
                      int64_t layout_lse_rows = 0, int64_t layout_edge_bytes = 0, const int32_t* order = nullptr,
                      uint32_t* queue = nullptr);
// Rewrites every row's ascending list of KV blocks into the order the attention kernel visits them in (see
// pace_order_kernel).  rows of `stride` entries, lens[row] of them in use; in == out allowed; stride <= 5000.
hipError_t launch_pace_order(const int32_t* in, int32_t* out, const int32_t* lens, int64_t rows, int nbk, int stride,
                             hipStream_t st);
// order: for every (batch, head) its 64-row query tiles by descending list length (lens is per query
// block of tiles_per_block tiles, clamped to [0, max_len]); with `order` and a two-word `queue`
// launch_fwd enqueues the 16-bit kernel both as rounds and as one launch whose workgroups draw items
// from a counter, and a kernel that compares the list lengths decides on the device which of them runs
hipError_t launch_order_by_length(const int32_t* lens, int32_t* order, int BH, int nbq, int tiles_per_block, int max_len,
                                  hipStream_t st);

// queue[0] = 0 (the counter work items are drawn with) and queue[1] = the choice between rounds (0) and the
// longest-first queue (1), made on the device from the list lengths (see choose_schedule_kernel)
void launch_schedule_choice(const int32_t* lens, int nbq, int tiles_per_block, int total, int round, int resident,
                            int max_len, uint32_t* queue, hipStream_t st);

// K or V of a (T, H, W)-ordered tensor in fragment order (bsa_fwd_frag.hip): dst [B*Hn][padded slots / 64][16 KB],
// padded slots zero; transpose = false for K, true for V.  bf16 / fp16.
// For K (transpose = false) of 64-slot chunks the pass can also write the chunk means (pooled, [B*Hn][blocks][128],
// the bits launch_permute's pooling gives) and the tile validity words; both optional.  dst may be null: the pass
// then only reads (chunk means of q).
// tr (optional, transpose = false only): per-head RMSNorm and / or 3-D RoPE of every row on its way through the pass.
// key_norm (optional, transpose = false only, frag_key_norm_floats() floats): its first B*Hn entries receive the largest
// Euclidean norm of a row of every (batch, head) as the pass writes it (a part in a thousand above), the rest is
// the per-tile norms they are reduced from; launch_fwd_frag takes the first part to bound q . k.
size_t frag_key_norm_floats(int B, int Hn, int64_t tiles);
struct RowTransform {
    const void* norm_w;      // 128 norm weights in the storage type; null: no norm
    const float* tab;        // rotation table (the layout bsa_norm_rope reads); null: no rotation
    int t0, Ttab;            // frame offset of the grid inside the table, frames of the table
    float eps;
    void* rows_out;          // optional: the transformed rows at their token positions
    int64_t rB, rH, rS;      // ... element strides {batch, head, token}
    int head_fastest;        // set by launch_frag: the order in which workgroups take (tile, head)
};
hipError_t launch_frag(const void* src, const int64_t strides[3], void* dst, int B, int Hn, const Grid3& g, int dtype,
                       bool transpose, hipStream_t st, void* pooled = nullptr, uint64_t* tile_valid = nullptr,
                       const RowTransform* tr = nullptr, float* key_norm = nullptr);
// The attention kernel on fragment-order K and V.  q_rows (optional): token row of every blocked-order query
// slot, -1 for padding; q_st / o_st: element strides {batch, head, row}; lse_rows: rows per (batch, head) of lse.
hipError_t launch_fwd_frag(const void* q, const void* kf, const void* vf, const int32_t* idx, const int32_t* lens,
                           const uint64_t* tile_valid, void* o, float* lse, int B, int Hn, int64_t Sq, int64_t Sk,
                           int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype, hipStream_t st,
                           const int32_t* q_rows, const int64_t q_st[3], const int64_t o_st[3], int64_t lse_rows,
                           const int32_t* order = nullptr, uint32_t* queue = nullptr, const float* key_norm = nullptr,
                           int32_t* fallback = nullptr);
// fallback (optional, frag_fallback_ints(B * Hn * Sq / 64) int32): with it and key_norm the rounds run the kernel that
// takes no row maxima and list here the items whose logits it cannot bound; a last launch computes those.
size_t frag_fallback_ints(int64_t items);


// Backward of the blocked-order attention (bsa_bwd.hip), bf16 / fp16.  workspace: bwd_workspace_bytes() bytes.
size_t bwd_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride);
int bwd_max_query_blocks();      // the dK / dV kernel stages a KV block's query blocks in LDS: Sq / bs_q may not exceed this
// With `thw` the caller's o, dO, lse, k and the three gradients are in token order: the passes that take delta and k_s
// read them through the row tables (token of every blocked-order slot of one (batch, head), -1 = padding) and the
// kernels store the gradient rows at their tokens.  q and v are then blocked-order copies (launch_permute), and the
// arguments k, o, dout, lse, dq, dk, dv of launch_bwd are not used.  Strides count elements.
struct BwdThw {
    const int32_t* q_rows;
    const int32_t* k_rows;
    int64_t q_tokens, k_tokens;       // real tokens per (batch, head)
    const void* o; int64_t o_st[3];
    const void* dout; int64_t do_st[3];
    const float* lse;                 // [B * Hn][q_tokens]
    const void* k; int64_t k_st[3];
    void* dout_blocked;               // B * Hn * Sq rows of 128 elements
    void* dq; int64_t dq_st[3];
    void* dk; int64_t dk_st[3];
    void* dv; int64_t dv_st[3];
};
hipError_t launch_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                      const int32_t* idx, const int32_t* lens, const uint64_t* tile_valid, void* dq, void* dk, void* dv,
                      int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype,
                      void* workspace, hipStream_t st, const BwdThw* thw = nullptr);

}  // namespace bsa
