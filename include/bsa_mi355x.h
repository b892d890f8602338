/*
 * bsa_mi355x.h - C ABI of the MI355X (gfx950) block-sparse attention engine.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*, 0 = the null stream).  Nothing here allocates device
 * memory, synchronises with the host or keeps mutable global state besides a
 * thread-local error string; callers own every buffer.  All functions return
 * BSA_OK (0) or a negative bsa_status; bsa_last_error() describes the last
 * failure on the calling thread.  Arguments are validated on the host before
 * anything is launched, so a bad call never reaches the GPU.
 *
 * Layouts.  "THW order" is the reference's token order, S = (T, H, W)
 * row-major.  "Blocked order" is (Nt, Nh, Nw, t, h, w): consecutive runs of
 * t*h*w slots form one 3-D chunk.  When a grid axis is not a multiple of its
 * chunk axis it is padded at the high end; padded slots hold zeros and are
 * flagged invalid in a per-64-slot bit mask ("tile validity", bit s of word i
 * covers slot 64*i+s).
 *
 * Reference interfaces replaced (paths relative to the reference checkout,
 * bsa = longcat_video/block_sparse_attention/bsa_interface.py,
 * vmask = longcat_video/block_sparse_attention/flash_attn_bsa_varlen_mask.py):
 * cited per function below.
 */
#ifndef BSA_MI355X_H
#define BSA_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum bsa_status {
    BSA_OK = 0,
    BSA_ERR_BAD_ARG = -1,        /* null pointer, non-positive size, misalignment */
    BSA_ERR_UNSUPPORTED = -2,    /* dtype / head_dim / chunk size not built */
    BSA_ERR_SHAPE = -3,          /* sizes inconsistent with each other */
    BSA_ERR_WORKSPACE = -4,      /* workspace smaller than bsa_workspace_bytes() */
    BSA_ERR_HIP = -5,            /* a HIP call failed; text in bsa_last_error() */
    BSA_ERR_BUSY = -6            /* bsa_fwd_3d_static: the built-in scratch buffer is still in use by a call on another stream */
} bsa_status;

typedef enum bsa_dtype {
    BSA_BF16 = 0,
    BSA_F16 = 1,
    BSA_F32 = 2
} bsa_dtype;

/* Library version, major*10000 + minor*100 + patch. */
int bsa_version(void);

/* Text of the last error raised on this thread ("" if none). */
const char* bsa_last_error(void);

/* Number of KV blocks kept per query block: int((1 - sparsity) * n_kv_blocks)
 * in IEEE doubles with truncation.  Replaces bsa:214. */
int bsa_num_selected(double sparsity, int n_kv_blocks);

/* Padded slot count of a (T,H,W) grid cut into (t,h,w) chunks. */
int64_t bsa_padded_tokens(int T, int H, int W, int t, int h, int w);

/*
 * R1.  THW order -> blocked order, zero-filling padded slots.
 * Replaces rearrange_THW_to_3d_block, bsa:600-604 (called bsa:650-652).
 *   src          [B, Hn, T*H*W, D], element strides src_strides = {B, Hn, S};
 *                the D axis must be contiguous and every row 16-byte aligned
 *   dst          [B, Hn, S_padded, D] contiguous
 *   pooled       optional [B, Hn, n_blocks, D] in `dtype`: per-chunk mean over
 *                all t*h*w slots (zeros included), fp32 sum, one rounding;
 *                the same result as bsa_mean_pool on dst (bsa:168-178)
 *   tile_valid   optional [S_padded/64] uint64 tile validity (needs t*h*w % 64 == 0)
 */
int bsa_permute_thw_to_blocks(const void* src, const int64_t src_strides[3], void* dst,
                              void* pooled, uint64_t* tile_valid,
                              int B, int Hn, int T, int H, int W, int t, int h, int w,
                              int D, int dtype, void* stream);

/*
 * R7.  Blocked order -> THW order, dropping padded slots.
 * Replaces rearrange_3d_block_to_THW, bsa:606-610 (called bsa:659).
 *   src [B, Hn, S_padded, D] contiguous; dst [B, Hn, T*H*W, D] with element
 *   strides dst_strides = {B, Hn, S} (so the caller may point it at a
 *   [B, S, Hn, D] buffer and skip the transpose of attention.py:140-141).
 */
int bsa_unpermute_blocks_to_thw(const void* src, void* dst, const int64_t dst_strides[3],
                                int B, int Hn, int T, int H, int W, int t, int h, int w,
                                int D, int dtype, void* stream);

/*
 * R2.  Block mean pooling.  Replaces mean_pooling_compression, bsa:168-178.
 *   x [B, Hn, S, D] contiguous; out [B, Hn, ceil(S/block), D] in `dtype`.
 *   A ragged last block is summed over its real rows and still divided by
 *   `block` (the reference zero-pads first, bsa:175-177).
 */
int bsa_mean_pool(const void* x, void* out, int B, int Hn, int64_t S, int block, int D,
                  int dtype, void* stream);

/*
 * R3 + R4.  Pooled scores and top-k selection.
 * Replaces cal_score (bsa:180-184) and get_select_indices_topk_from_score
 * (bsa:212-224).
 *   q_cmp [B, Hn, nbq, D], k_cmp [B, Hn, nbk, D] contiguous, `dtype`
 *   score = q_cmp . k_cmp^T, fp32 accumulate, rounded once to `dtype`, unscaled
 *   idx_out   int32 [B, Hn, nbq, k_sel]: the k_sel best blocks of every row in
 *             descending score order, ties broken towards the lowest index
 *   idx_sorted_out  the same set in ascending block index (the order in which
 *             the attention kernel is most cache friendly); at least one of
 *             idx_out / idx_sorted_out must be given
 *   lens_out  int32 [B, Hn, nbq], every entry k_sel (bsa:217-222)
 *   score_out optional [B, Hn, nbq, nbk] in `dtype`
 * Limits: D == 128, 0 <= k_sel <= nbk <= 4096.
 * NaN scores order above +inf, as torch.topk orders them.
 */
int bsa_score_topk(const void* q_cmp, const void* k_cmp, int32_t* idx_out, int32_t* idx_sorted_out,
                   int32_t* lens_out, void* score_out, int B, int Hn, int nbq, int nbk, int D,
                   int k_sel, int dtype, void* stream);

/*
 * Selection by cumulative attention mass.  Replaces get_select_indices_cdf_from_score (bsa:233-243) and, with
 * k_min > 0, get_select_indices_cdf_topk_from_score (bsa:252-266).
 *   weights = softmax(score * sm_scale) per row; the columns are ordered by descending score, ties towards
 *   the lowest index; a row keeps the leading columns whose running sum of weights is <= cdf_threshold
 *   (torch.searchsorted(cdf, threshold, right=True), bsa:241), at least k_min and at most idx_stride of them.
 *   idx_out / idx_sorted_out  int32 [B, Hn, nbq, idx_stride], row m filled up to lens_out[m], -1 behind
 *   (the reference returns all nbk sorted columns, of which the attention kernel reads the first lens).
 * The weights are fp32 for every storage type and the running sum is kept in double precision: a row may
 * differ from an fp32 running sum only where that sum comes within rounding of the threshold.
 * Limits as for bsa_score_topk; idx_stride <= nbk.
 */
int bsa_score_cdf(const void* q_cmp, const void* k_cmp, int32_t* idx_out, int32_t* idx_sorted_out,
                  int32_t* lens_out, void* score_out, int B, int Hn, int nbq, int nbk, int D,
                  float cdf_threshold, float sm_scale, int k_min, int idx_stride, int dtype, void* stream);
int bsa_cdf_from_score(const void* score, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out,
                       int B, int Hn, int nbq, int nbk, float cdf_threshold, float sm_scale, int k_min,
                       int idx_stride, int dtype, void* stream);

/* R4 alone, from a caller-supplied score tensor [B, Hn, nbq, nbk] in `dtype`. */
int bsa_topk_from_score(const void* score, int32_t* idx_out, int32_t* idx_sorted_out, int32_t* lens_out,
                        int B, int Hn, int nbq, int nbk, int k_sel, int dtype, void* stream);

/*
 * The order in which bsa_fwd_3d's attention kernel visits each query block's selected KV blocks.  No
 * counterpart in the reference: its kernel visits the blocks in list order (vmask:249-285), and softmax
 * attention depends on that order only through floating-point rounding, so the engine chooses the order that
 * keeps the query tiles running side by side at the same place of the KV sequence (they then share K/V tiles
 * in the L2 cache).  The attention entry points (bsa_fwd, bsa_fwd_thw) visit a caller's list in the order it
 * is given; this entry point gives callers that build their own lists the operator's order.
 *
 *   idx_sorted [rows, idx_stride] i32, lens[row] blocks in ascending order per row; idx_out the same shape
 *   (may be idx_sorted itself); nbk KV blocks in the sequence.  Slot groups of 8: group g takes the blocks b
 *   with g == min(b*n/(nbk*8), groups-1), n = lens[row], up to its number of slots; the blocks over that
 *   number fill the slots left empty, both in ascending order; every group's slots end in ascending block
 *   order.  Rows of at most 8 blocks stay as they are.  idx_stride <= 4096.
 */
int bsa_visit_order(const int32_t* idx_sorted, const int32_t* lens, int32_t* idx_out, int64_t rows, int nbk,
                    int idx_stride, void* stream);

/*
 * R5 + R6.  Block-sparse flash-attention forward over blocked-order tensors.
 * Replaces attn_fwd_bsa_varlen_triton (bsa:290-341) and the kernel
 * _attn_fwd_bsa_varlen_align (vmask:172-285).
 *   q [B, Hn, Sq, D], k/v [B, Hn, Sk, D], o [B, Hn, Sq, D] contiguous
 *   idx  int32 [B, Hn, Sq/bs_q, idx_stride]; lens int32 [B, Hn, Sq/bs_q];
 *        row m attends to KV blocks idx[..., m, 0 .. lens[..., m])
 *   tile_valid optional [Sk/64] uint64: keys whose bit is 0 get -inf logits
 *   lse  optional fp32 [B, Hn, Sq], natural-log sum-exp (bsa:338-339)
 *   o = softmax(q k^T * sm_scale) v restricted to the listed blocks; logits are
 *   fp32, the scale is applied after the dot as sm_scale*log2(e), probabilities
 *   are rounded to `dtype` for the P V product while the row sum stays fp32.
 *   An empty list gives o = 0, lse = -inf.  The kernels clamp every block index
 *   to [0, Sk/bs_k) and every length to [0, idx_stride]: a malformed list gives
 *   wrong numbers for its query block, never an access outside k and v (the
 *   reference's kernel reads wherever such an index points).
 * Limits: D == 128; bs_q, bs_k multiples of 64; Sq % bs_q == 0, Sk % bs_k == 0.
 */
int bsa_fwd(const void* q, const void* k, const void* v, const int32_t* idx, const int32_t* lens,
            const uint64_t* tile_valid, void* o, float* lse,
            int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride,
            float sm_scale, int dtype, void* stream);

/*
 * bsa_fwd for bf16 / fp16 on the engine's faster attention kernel (one wavefront per 64 query rows, K and V
 * rewritten once per call into the order its matrix instructions consume them): the same boundary -
 * attn_fwd_bsa_varlen_triton (bsa:290-341), kernel vmask:172-285 - the same arguments, results within the
 * rounding of another summation order, plus a workspace of bsa_fwd_fragment_workspace_bytes() bytes
 * (two copies of k's size and two small tables), 256-byte aligned.  Padded key slots may hold anything finite: they are masked
 * by tile_valid.  idx_stride <= 4096.
 */
size_t bsa_fwd_fragment_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int D, int dtype);
int bsa_fwd_fragment(const void* q, const void* k, const void* v, const int32_t* idx, const int32_t* lens,
                     const uint64_t* tile_valid, void* o, float* lse,
                     int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride,
                     float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * R9.  The whole operator on THW-order tensors: permute q,k,v (+pool), score,
 * top-k, attention, unpermute.  Replaces flash_attn_bsa_3d, bsa:612-660, and
 * _attention_bsa.forward, bsa:535-568 (cdf_threshold = None).
 *   q [B, Hn, Tq*Hq*Wq, D] with element strides q_strides = {B, Hn, S}; same
 *   for k, v; o likewise with o_strides.  k_sel from bsa_num_selected() on the
 *   padded KV block count.  With p->cdf_threshold > 0 the selection follows
 *   bsa_score_cdf instead (bsa:268-277 dispatch), at most nbk blocks per
 *   row, and idx_out has that many columns.  workspace: bsa_workspace_bytes() bytes, 256-byte
 *   aligned.  idx_out/lens_out/score_out are optional copies for inspection
 *   (shapes as in bsa_score_topk).  With cdf_threshold the lists differ in length: the work is then also
 *   enqueued as one launch whose workgroups draw the query tiles longest list first, and a kernel decides
 *   from the lengths, on the device, whether that or the usual rounds of equal tiles run (bf16 / fp16).
 * For bf16 / fp16 no permuted copy of q, k, v or o is made: one pass over q and k
 * produces the pooled means (and the tables of bsa_thw_prepare), and the attention
 * kernel reads and writes THW order directly; k and v must then share one token
 * stride (BSA_ERR_UNSUPPORTED otherwise).  fp32 goes through blocked copies.
 */
typedef struct bsa_3d_params {
    int B, Hn, D, dtype;
    int Tq, Hq, Wq, Tk, Hk, Wk;      /* latent grids */
    int tq, hq, wq, tk, hk, wk;      /* chunk shapes */
    int k_sel;                       /* top-k count; with cdf_threshold > 0: the minimum per row (0 = none) */
    float sm_scale;
    float cdf_threshold;             /* > 0 selects by cumulative attention mass (bsa_score_cdf), else top-k */
} bsa_3d_params;

size_t bsa_workspace_bytes(const bsa_3d_params* p);

int bsa_fwd_3d(const bsa_3d_params* p,
               const void* q, const int64_t q_strides[3],
               const void* k, const int64_t k_strides[3],
               const void* v, const int64_t v_strides[3],
               void* o, const int64_t o_strides[3],
               void* workspace, size_t workspace_bytes,
               int32_t* idx_out, int32_t* lens_out, void* score_out, void* stream);

/*
 * bsa_fwd_3d for a caller that will ask for gradients: the same kernels and the same output bit for bit
 * (_attention_bsa.forward runs one kernel with and without grad and keeps lse, bsa:538-568), plus what the
 * backward needs: lse_out [B, Hn, Tq*Hq*Wq] fp32 in token order (natural log; -inf for a query without keys),
 * walk_out int32 [B, Hn, nbq, width] - every query block's selected KV blocks in the order the kernel visited them,
 * block numbers counted in the padded chunk grid (width as idx_out of bsa_fwd_3d) - and lens_out int32 [B, Hn, nbq].
 * bf16 / fp16.
 */
int bsa_fwd_3d_lse(const bsa_3d_params* p,
                   const void* q, const int64_t q_strides[3],
                   const void* k, const int64_t k_strides[3],
                   const void* v, const int64_t v_strides[3],
                   void* o, const int64_t o_strides[3],
                   float* lse_out, int32_t* walk_out, int32_t* lens_out,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward of bsa_fwd: gradients of the block-sparse attention with respect to q, k and v.
 * Replaces attn_bwd_bsa_varlen_triton (bsa:341-461) and the kernels _attn_bwd_preprocess (common.py:94-111),
 * _attn_bwd_dkdv_bsa_varlen_wrapper (vmask:505-642) and _attn_bwd_dq_bsa_varlen(_align)_wrapper (vmask:665-945),
 * including create_indices_k_from_indices_q_varlen (bsa:152-165), with their rounding points: k pre-scaled by
 * sm_scale*log2(e) and rounded once to the storage type, p = exp2(q.k_s - lse*log2(e)) in fp32, p and
 * dS = p*(dP - delta) rounded to the storage type for the products, fp32 accumulators, dK scaled by sm_scale and dQ
 * by ln 2 before the final rounding.
 *   q, o, d_o, dq [B, Hn, Sq, D]; k, v, dk, dv [B, Hn, Sk, D]: contiguous, blocked order, bf16 / fp16, D == 128.
 *   lse [B, Hn, Sq] fp32 (natural log) and idx / lens as bsa_fwd took and returned them (a row names a block at
 *   most once); tile_valid as in bsa_fwd (padded keys get no gradient and give none).
 *   workspace: bsa_bwd_workspace_bytes() bytes, 256-byte aligned (the scaled k, two fp32 vectors per query row, a
 *   bit matrix [kv block][query block], a copy of the lists, two small per-block tables).  Ascending lists are
 *   walked in bsa_visit_order's order by the dQ kernel (fp32 roundings only).
 */
size_t bsa_bwd_workspace_bytes(int B, int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride, int dtype);
int bsa_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
            const int32_t* idx, const int32_t* lens, const uint64_t* tile_valid, void* dq, void* dk, void* dv, int B,
            int Hn, int64_t Sq, int64_t Sk, int D, int bs_q, int bs_k, int idx_stride, float sm_scale, int dtype,
            void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward of bsa_fwd_3d_lse on the operator's own tensors: what _attention_bsa.backward (bsa:570-596) computes
 * for the q, k, v that flash_attn_bsa_3d rearranged (bsa:650-652, whose gradient is the inverse rearrangement), with
 * every tensor left in (T, H, W) token order.  Same arithmetic and rounding points as bsa_bwd.
 *   q, o, d_o, dq [B, Hn, Tq*Hq*Wq, D] and k, v, dk, dv [B, Hn, Tk*Hk*Wk, D]: element strides as in bsa_fwd_3d,
 *   bf16 / fp16, D == 128, 16-byte aligned; lse [B, Hn, Tq*Hq*Wq] fp32 contiguous and idx [B, Hn, nbq, idx_stride],
 *   lens [B, Hn, nbq] as bsa_fwd_3d_lse returned them (blocks counted in the padded chunk grids).  p->k_sel and
 *   p->cdf_threshold are not read.  Padded keys give and get no gradient; dq, dk, dv are written at every token.
 *   workspace: bsa_bwd_3d_workspace_bytes() bytes, 256-byte aligned: blocked-order copies of q, v and d_o (the kernels
 *   stream their tiles as they lie in memory), the row tables of both grids, and bsa_bwd's workspace.  o, d_o, lse
 *   and k are read through the row tables by the passes that take delta and the scaled k, and the kernels store the
 *   gradient rows at their tokens: five of the eight rearrangements a caller of bsa_bwd would run are not made.
 */
size_t bsa_bwd_3d_workspace_bytes(const bsa_3d_params* p, int idx_stride);
int bsa_bwd_3d(const bsa_3d_params* p,
               const void* q, const int64_t q_strides[3],
               const void* k, const int64_t k_strides[3],
               const void* v, const int64_t v_strides[3],
               const void* o, const int64_t o_strides[3],
               const void* d_o, const int64_t do_strides[3],
               const float* lse, const int32_t* idx, const int32_t* lens, int idx_stride,
               void* dq, const int64_t dq_strides[3],
               void* dk, const int64_t dk_strides[3],
               void* dv, const int64_t dv_strides[3],
               void* workspace, size_t workspace_bytes, void* stream);

/*
 * bsa_fwd_3d without a workspace argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  What bsa_fwd_3d carves from its workspace
 * lives in a buffer of BSA_STATIC_SCRATCH_BYTES that is part of the library's code object, so every GPU the
 * library is used on holds that much memory from the first call on it until the process ends.
 *   - Arguments and results are those of bsa_fwd_3d: the same selection bit for bit.  To fit the buffer it
 *     makes no fragment-order copies of k and v; its attention kernel reads them where they lie (the
 *     LDS-tiled kernel), so the output agrees with bsa_fwd_3d's within the rounding of a different
 *     summation order (bf16 / fp16: max-abs 1.6e-2, mean-abs 1e-3 on unit-variance inputs; fp32: equal).
 *   - A problem that needs more scratch than BSA_STATIC_SCRATCH_BYTES - pooled means, scores, lists, tables and
 *     the zero-filled copies of the KV chunks at the padded edge of the grid, i.e. bsa_workspace_bytes() less
 *     the two fragment-order copies - is rejected with BSA_ERR_WORKSPACE before anything is launched (64 MiB
 *     covers, in bf16 with 4x4x4 chunks, the 720p grid at up to 6 heads or the 480p grid at up to 17 heads:
 *     one GPU's share of a head-sharded layer).
 *   - The call itself makes no hipMalloc / hipFree and calls no allocating library routine.  The first call
 *     on a device is also the set-up for that device: it looks up the buffer's address (hipGetSymbolAddress) and
 *     creates the one event that later calls record; make that call outside graph capture.
 *   - All calls on one GPU share the one buffer, which keeps the previous call's contents; nothing in it
 *     needs to start at zero.  Calls that overlap in time on one GPU would race on it: serialise them, or use
 *     bsa_fwd_3d with one workspace per stream.  A call made while the previous call on the same GPU, enqueued
 *     on ANOTHER stream, has not finished is refused with BSA_ERR_BUSY and launches nothing (an event recorded
 *     behind every call is queried; calls on one stream run in order and are never refused).  Under stream
 *     capture nothing is recorded or queried: replays of graphs that hold such calls are the caller's to order.
 */
#define BSA_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int bsa_fwd_3d_static(const bsa_3d_params* p,
                      const void* q, const int64_t q_strides[3],
                      const void* k, const int64_t k_strides[3],
                      const void* v, const int64_t v_strides[3],
                      void* o, const int64_t o_strides[3],
                      int32_t* idx_out, int32_t* lens_out, void* score_out, void* stream);

/*
 * R1 + R5 + R6 + R7 with a caller-supplied selection, bf16 / fp16: attention over THW-order
 * tensors without permuted copies.  Replaces the sequence rearrange_THW_to_3d_block x3 (bsa:650-652),
 * attn_fwd_bsa_varlen_triton (bsa:290-341), rearrange_3d_block_to_THW (bsa:659) for callers that
 * select KV blocks themselves.  Two steps on one workspace of bsa_workspace_bytes(p) bytes:
 *
 * bsa_thw_prepare: builds what depends on the grids and on k, v only: the token row of every
 *   blocked-order query slot, the position of every 64-slot kv tile, the tile validity words, and
 *   blocked-order copies of the kv chunks that touch the padded high edge of the grid (all kv
 *   chunks when the chunk shape does not allow gathering: w a power of two >= 4, h a power of two,
 *   64-slot tiles made of whole (h, w) planes).  Call again whenever k or v change.
 * bsa_fwd_thw: the attention kernel alone.  idx / lens / idx_stride / lse as in bsa_fwd, block
 *   indices counted in the padded chunk grids; lse is [B, Hn, Tq*Hq*Wq] in THW order.
 *   p->k_sel is not used.  k and v must share one token stride.  p->cdf_threshold > 0 (any positive
 *   value, in both calls) declares that the lists may differ in length: the kernel is then enqueued in
 *   both schedules described at bsa_fwd_3d and the choice is made on the device.
 */
int bsa_thw_prepare(const bsa_3d_params* p, const void* k, const int64_t k_strides[3],
                    const void* v, const int64_t v_strides[3],
                    void* workspace, size_t workspace_bytes, void* stream);

int bsa_fwd_thw(const bsa_3d_params* p,
                const void* q, const int64_t q_strides[3],
                const void* k, const int64_t k_strides[3],
                const void* v, const int64_t v_strides[3],
                void* o, const int64_t o_strides[3],
                const int32_t* idx, const int32_t* lens, int idx_stride, float* lse,
                void* workspace, size_t workspace_bytes, void* stream);

/*
 * R11 glue of the attention module (longcat_video/modules/attention.py:107-147).
 */

/* Row RMSNorm: out = cast(x * rsqrt(mean(x^2) + eps)) * weight, rows of `dim` elements (dim % 8 == 0),
 * fp32 statistics, result rounded to `dtype` before and after the weight multiply.
 * Replaces RMSNorm_FP32.forward, longcat_video/modules/blocks.py:42-53.  bf16 / fp16. */
int bsa_rmsnorm(const void* x, const void* weight, void* out, int64_t rows, int dim, float eps,
                int dtype, void* stream);

/* The adaLN wrapper of the self-attention branch of a DiT block (longcat_video/modules/longcat_video_dit.py:
 * 82-103), bf16 / fp16, rows of `dim` elements, `rows_per_group` consecutive rows (the tokens of one latent
 * frame) sharing one fp32 row of shift / scale / gate:
 *   bsa_layernorm_modulate: out = cast(layer_norm(float(x)) * (scale + 1) + shift), LayerNorm without affine
 *     parameters, biased variance, everything in fp32, one rounding.  Replaces modulate_fp32(mod_norm_attn, ...)
 *     (blocks.py:56-69, 126-134; longcat_video_dit.py:88).  dim <= 8192.
 *   bsa_gated_residual: out = cast(float(x) + gate * float(y)).  Replaces longcat_video_dit.py:101-103. */
int bsa_layernorm_modulate(const void* x, const float* shift, const float* scale, void* out, int64_t rows,
                           int rows_per_group, int dim, float eps, int dtype, void* stream);
int bsa_gated_residual(const void* x, const void* y, const float* gate, void* out, int64_t rows,
                       int rows_per_group, int dim, int dtype, void* stream);

/* In-place per-head RMSNorm (blocks.py:42-53, called attention.py:116) followed by 3-D RoPE
 * (longcat_video/modules/rope_3d.py:99-120, called attention.py:121) on q and k.
 *   q, k  [B, Hn, T*H*W, 128] with element strides {B, Hn, S} (views of the QKV projection are fine)
 *   q_weight, k_weight  [128] in `dtype`
 *   rope_table  fp32, concatenation of cos_t[T][22], sin_t[T][22], cos_h[H][21], sin_h[H][21],
 *               cos_w[W][21], sin_w[W][21]: cos/sin of position * frequency per rotation pair
 *               (rope_3d.py:70-87; the d axis is split 44/42/42 between t, h, w) */
int bsa_qk_norm_rope(void* q, const int64_t q_strides[3], void* k, const int64_t k_strides[3],
                     const void* q_weight, const void* k_weight, const float* rope_table,
                     int B, int Hn, int T, int H, int W, int D, float eps, int dtype, void* stream);

/* One tensor of the same chain, with every step optional and an optional move to another layout:
 *   dst = rope(norm(src)).  weight == NULL skips the RMSNorm, rope_table == NULL skips the rotation, both
 *   NULL copies.  src / dst [B, Hn, T*H*W, 128] with element strides {B, Hn, S}; src == dst with equal
 *   strides works in place.  The token at grid position (t, h, w) is rotated by frame t_offset + t of a
 *   table built for table_T frames (layout as in bsa_qk_norm_rope with T = table_T).
 * Serves the plain forward (q, k, v moved from the token-major projection output into per-head contiguous
 * tensors while q and k are normalised and rotated), return_kv (attention.py:118-119: k after the norm,
 * before the rotation) and forward_with_kv_cache (attention.py:166-171: cached keys and new queries are
 * rotated on a grid of T + num_cond_latents frames, the queries starting at frame num_cond_latents). */
int bsa_norm_rope(const void* src, const int64_t src_strides[3], void* dst, const int64_t dst_strides[3],
                  const void* weight, const float* rope_table, int B, int Hn, int T, int H, int W,
                  int t_offset, int table_T, int D, float eps, int dtype, void* stream);

/* out[M,N] = x[M,K] . w[N,K]^T (+ bias[N]) (+ residual[M,N]), bf16 in/out, fp32 accumulate, on MFMA
 * through hipBLASLt.  Replaces the nn.Linear calls attention.py:111 and :142.  `workspace`: at least
 * 64 MiB of device memory (BSA_ERR_WORKSPACE otherwise); its contents do not matter.  Every calling thread
 * uses a hipBLASLt handle of its own per device; a thread that ends hands its handles to the next thread that
 * needs one, so their number stays at the largest number of threads that called at one time. */
int bsa_linear_bf16(const void* x, const void* w, const void* bias, const void* residual, void* out,
                    int64_t M, int N, int K, void* workspace, size_t workspace_bytes, void* stream);

/* The same product with row strides (in elements): x rows ldx apart, w rows ldw apart, out (and residual)
 * rows ldo apart.  Lets one output block of a LoRA up-projection that is split over the output features
 * (lora_utils.py:12-21: chunk the rank axis, one Linear per chunk, concatenate) read its slice of the
 * rank axis and write its slice of the output columns in place. */
int bsa_linear_bf16_ld(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                       void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                       void* stream);

/* One-time tuning of a linear shape (no counterpart in the reference, whose nn.Linear leaves the choice to the
 * BLAS library): runs every algorithm hipBLASLt proposes for this call (up to 32, each four times on the given
 * buffers; `out` is overwritten), and remembers the fastest for later bsa_linear_bf16 / _ld calls with the same
 * M, N, K, row strides, bias / residual presence in this process.  Unlike every other entry point it WAITS for
 * the stream, so call it at set-up, outside graph capture.  Returns the number of algorithms timed (> 0) or a
 * negative status; default_ms / best_ms (optional) receive the time of the algorithm an untuned call uses and
 * of the one chosen.  Algorithms differ in summation order, so results can differ in the last bit. */
int bsa_linear_bf16_tune(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                         void* out, int64_t ldo, int64_t M, int N, int K, void* workspace, size_t workspace_bytes,
                         void* stream, float* default_ms, float* best_ms);

/* LoRA side branches of a Linear (longcat_video_dit.py:234-249): out = org + total, where total sums
 * up_i * multiplier_i * alpha_scale_i over the active branches, up_i = lora_up(lora_down(x)) already
 * computed (bsa_linear_bf16 / _ld).  Every product and every sum is rounded to `dtype` as the eager
 * expression does: s_i = T(T(up_i * multiplier_i) * alpha_scale_i); total = s_0, then T(total + s_i);
 * out = T(org + total).  up, multiplier, alpha_scale are HOST arrays of n_loras entries (1..4); the
 * up[i] are device pointers to n elements each; out may alias org.  The caller passes alpha_scale as the
 * reference holds it (a buffer cast to the model dtype, longcat_video_dit.py:221). */
int bsa_lora_add(const void* org, const void* const* up, const float* multiplier, const float* alpha_scale, int n_loras,
                 void* out, int64_t n, int dtype, void* stream);

/* bsa_fwd_3d for the attention module (attention.py:116-137): q and k arrive as the QKV projection left them
 * (strided views into its output are fine) and go through the per-head RMSNorm (RMSNorm_FP32, blocks.py:42-53) and
 * the 3-D RoPE (rope_3d.py:100-120) inside the operator's own passes over them, at the rounding points of
 * bsa_norm_rope: the pass that takes q's chunk means writes the transformed rows to q_normed ([B, Hn, Tq*Hq*Wq, 128]
 * through qn_strides; the attention kernel reads q from there), the pass that rewrites k into the attention
 * kernel's operand order transforms it on the way, so the stand-alone norm / rotation passes over q and k and one
 * read of q drop out.  rope_table as for bsa_norm_rope with the H and W of the grids (Hq = Hk, Wq = Wk); q sits at
 * frames t_offset_q.. and k at frames t_offset_k.. of its table_T frames.  bf16 / fp16, 64-token chunks for q and
 * k with at most 8 positions per axis (BSA_ERR_UNSUPPORTED otherwise: use bsa_qk_norm_rope + bsa_fwd_3d).  Everything else as bsa_fwd_3d; idx_out /
 * lens_out / score_out refer to the transformed q and k. */
typedef struct bsa_qk_norm {
    const void* q_weight;      /* 128 elements of the tensors' type, 16-byte aligned */
    const void* k_weight;
    const float* rope_table;
    int table_T, t_offset_q, t_offset_k;
    float eps;
} bsa_qk_norm;
int bsa_fwd_3d_qknorm(const bsa_3d_params* p, const bsa_qk_norm* n, const void* q, const int64_t q_strides[3],
                      void* q_normed, const int64_t qn_strides[3], const void* k, const int64_t k_strides[3], const void* v,
                      const int64_t v_strides[3], void* o, const int64_t o_strides[3], void* workspace, size_t workspace_bytes,
                      int32_t* idx_out, int32_t* lens_out, void* score_out, void* stream);

/* The engine's own GEMM for the two projections of the attention module (attention.py:111 and :142):
 * out[M,N] = x[M,K] . w[N,K]^T (+ bias[N]) (+ residual[M,N]), bf16 in/out, fp32 accumulation on MFMA, one
 * rounding at the end.  Row strides in elements (ldx, ldw >= K; ldo, ldr >= N; multiples of 8).  N must be a
 * multiple of 128 and K of 64; x, w, out, residual 16-byte aligned.  Needs no workspace and allocates nothing. */
int bsa_gemm_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                  int64_t ldr, void* out, int64_t ldo, int64_t M, int N, int K, void* stream);

/* attention.py:111-121 in one kernel: qkv = Linear(x) with w [3*Hn*128, K] (rows: q heads, k heads, v heads, as
 * the view/permute of attention.py:112-113 splits them), the projection output rounded to bf16 as the reference's
 * tensor is, q and k normalised per head (RMSNorm_FP32, blocks.py:42-53, weights q_weight / k_weight of 128
 * elements) and rotated (rope_3d.py:100-120; rope_table as for bsa_norm_rope, frames t_offset.. of table_T), v
 * as projected.  x holds M = B*T*H*W token rows.  q, k, v receive [B, Hn, T*H*W, 128] through
 * dst_strides = {batch, head, token} (elements, multiples of 8): per-head contiguous tensors, or any other
 * layout bsa_fwd_3d accepts.  Rounding points are those of bsa_norm_rope fed with the bf16 projection. */
int bsa_qkv_projection(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* q_weight,
                       const void* k_weight, const float* rope_table, void* q, void* k, void* v,
                       const int64_t dst_strides[3], int B, int Hn, int T, int H, int W, int t_offset, int table_T,
                       int D, int K, float eps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BSA_MI355X_H */
