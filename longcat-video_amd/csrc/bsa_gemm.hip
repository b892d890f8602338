// The two projections of the attention module as one hand-written gfx950 GEMM:
//   out[M, N] = x[M, K] . w[N, K]^T (+ bias) (+ residual)            (plain epilogue)
//   q, k, v   = split(x . w^T + bias) per head, q and k normalised per head (RMSNorm over the 128
//               features of a head) and rotated (3-D RoPE), every head written as a contiguous
//               [tokens, 128] tensor                                    (QKV epilogue)
// bf16 operands, fp32 accumulation in v_mfma_f32_32x32x16_bf16.
//
// Shape of the computation.  Both operands have k as their fastest axis, which is the layout both MFMA
// operands want: lane l of a 32x32x16 product holds 8 consecutive k of row l % 32, starting at k = 8 (l / 32).
// The weight rows are the A operand and the token rows the B operand, so an accumulator register holds
// C^T: lane l has token l % 32 and, in its 16 registers, features 8 (r / 4) + 4 (l / 32) + r % 4 of the
// 32x32 block.  A lane therefore owns whole rotation pairs (features 2i, 2i + 1) and half of the features of
// its tokens: the per-head sum of squares is an in-lane sum plus one exchange between lane l and l ^ 32.
//
// A workgroup of four wavefronts (one per SIMD, 512 registers each) computes a tile of 256 tokens x 256
// features; every wavefront owns 128 x 128 of it (16 accumulator blocks = 256 registers), which for the QKV
// projection is exactly one head of 128 tokens.  Per k block of 64 the workgroup brings 256 rows x 128 bytes of
// either operand (a half-slab of 32 KB, whole cache lines) from global memory straight into LDS
// (global_load_lds_dwordx4, no staging registers); five half-slab stages fill the 160 KB of LDS: two in use, up to
// three on their way.  The LDS side of such a load is linear in the lane index, so the XOR swizzle that keeps the
// fragment reads (ds_read_b128, rows 128 bytes apart; measured: bank-conflict cycles 4 % of the LDS-active ones)
// free of bank conflicts is applied on the global side: the 16-byte slot p of row r receives k unit
// p ^ ((r >> 1) & 7).
//
// One barrier per k block, after the third of its four k sub-steps: the fragments of a sub-step are read during
// the MFMAs of the one before.  At the barrier every wavefront has awaited its own share of the next block's two
// half-slabs and holds the last fragments of this one; the two stages so drained take the half-slabs five further
// on, requested one load per four MFMAs over the k block that follows.
//
// Tiles are handed out so that the workgroups resident on one XCD (32 CUs, one shared L2; workgroup b runs
// on XCD b % 8) form a block of 8 token tiles x 4 feature tiles: they run in step, so each slab fetched from
// HBM serves 4 (token slab) or 8 (weight slab) workgroups out of L2 (measured at the 720p QKV shape: 15 GB leave
// L2 per call for 65 GB that enter LDS).
//
// What bounds it (measured at [86400, 4096] x [4096, 12288]^T on random data): the board's power limit.  Under this
// kernel the clock settles near 1.83 GHz instead of 2.4 (under hipBLASLt's kernel for the same product near
// 1.72 GHz), so a gain in work per clock is partly paid back in clock.  Per clock the k loop reaches about 0.61 of
// the MFMA rate.  Variants measured on the way: all sixteen loads of a k block in one burst after the barrier
// 8.5 ms (the wavefronts then wait for the address unit, not for data: with a software barrier instead of
// s_barrier no better, without any barrier 5.3 ms but wrong); two stages of a whole k block 8.0 ms; ten 16 KB
// stages with paired loads of the two halves of a cache line 8.4 ms; register prefetch two blocks ahead with
// compiler-placed waits 9.1 ms (the waits it places allow only one block in flight).
#include "bsa_mfma.h"

namespace bsa {
namespace {

using namespace mfma;

constexpr int kTileM = 256;              // tokens per workgroup
constexpr int kTileN = 256;              // features per workgroup
constexpr int kBK = 64;                  // k per pipeline step
constexpr int kPart = 256 * kBK * 2;     // bytes of one operand's slab
constexpr int kStages = 5;               // half-slabs resident in LDS: 160 KB
constexpr int kEpiPitch = 272;           // bytes per token row of the output staging area (256 + 16)
constexpr int kEpiBytes = 64 * kEpiPitch;
constexpr int kSuperM = 8, kSuperN = 4;  // tiles of one XCD's block

typedef bf16x8 V8;
template <int N> using IC = std::integral_constant<int, N>;

struct GemmArgs {
    const __bf16* x; int64_t ldx;
    const __bf16* w; int64_t ldw;
    const __bf16* bias;
    const __bf16* residual; int64_t ldr;
    __bf16* out; int64_t ldo;
    int M, N, K;
    int tiles_m, tiles_n, super_m, super_total;
    // QKV epilogue
    __bf16* dst[3];
    int64_t dB, dH, dS;
    const __bf16* norm_w[2];
    const float* tab;
    int Hn, S, Hg, Wg, t0, Ttab;
    float eps;
};

template <bool QKV>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const GemmArgs a) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;      // this wavefront's feature half and token half

    // tile of this workgroup
    const int b = blockIdx.x;
    const int super = (b >> 8) * 8 + (b & 7), pos = (b >> 3) & 31;
    if (super >= a.super_total) return;
    const int sf = super / a.super_m, sm = super - sf * a.super_m;
    const int tile_f = sf * kSuperN + (pos & 3), tile_m = sm * kSuperM + (pos >> 2);
    if (tile_f >= a.tiles_n || tile_m >= a.tiles_m) return;
    const int f_tile0 = tile_f * kTileN, m_tile0 = tile_m * kTileM;

    // ---- global -> LDS: this wavefront brings rows [64 wave, 64 wave + 64) of a half-slab, 8 rows (of 128 bytes:
    // one cache line each) per load
    uint32_t voff_w[8], voff_x[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int row = wave * 64 + r * 8 + (lane >> 3);
        const int unit = (lane & 7) ^ ((row >> 1) & 7);
        const int frow = min(row, a.N - 1 - f_tile0), mrow = min(row, a.M - 1 - m_tile0);   // edge tiles repeat their last row
        voff_w[r] = (uint32_t)((int64_t)frow * a.ldw * 2 + unit * 16);
        voff_x[r] = (uint32_t)((int64_t)mrow * a.ldx * 2 + unit * 16);
    }
    const char* wbase = reinterpret_cast<const char*>(a.w + (int64_t)f_tile0 * a.ldw);
    const char* xbase = reinterpret_cast<const char*>(a.x + (int64_t)m_tile0 * a.ldx);
    // Half-slab h (even: weight rows, odd: token rows, of k block h / 2) lives in stage h % kStages.
    const uint32_t lds0 = lds_address(smem) + wave * 8192;
    const int nblocks = a.K / kBK, nhalf = 2 * nblocks;
    // load r (of eight) of half-slab h; `odd` = h & 1, known at compile time
    auto issue_one = [&](int h, int stage, auto odd_c, int r) __attribute__((always_inline)) {
        constexpr int odd = decltype(odd_c)::value;
        if (h >= nhalf) return;
        const char* base = (odd ? xbase : wbase) + (int64_t)(h >> 1) * (kBK * 2);
        load_to_lds_16(base, odd ? voff_x[r] : voff_w[r], lds0 + stage * kPart + r * 1024);
    };

    // ---- LDS -> fragments
    const uint32_t swz = ((lane & 31) >> 1) & 7, g = lane >> 5;
    const uint32_t a_lane = (wm * 128 + (lane & 31)) * 128, b_lane = (wn * 128 + (lane & 31)) * 128;
    uint32_t unit_of[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) unit_of[ks] = ((2 * ks + g) ^ swz) * 16;
    V8 af[2][4], bf[2][4];
    auto read_frags = [&](int stage_w, int stage_x, int ks) __attribute__((always_inline)) {
        const char* sw = smem + stage_w * kPart + unit_of[ks] + a_lane;
        const char* sx = smem + stage_x * kPart + unit_of[ks] + b_lane;
#pragma unroll
        for (int i = 0; i < 4; ++i) af[ks & 1][i] = *reinterpret_cast<const V8*>(sw + i * 4096);
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[ks & 1][j] = *reinterpret_cast<const V8*>(sx + j * 4096);
    };
    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    // The sixteen MFMAs of k sub-step ks, and between them four of the sixteen loads requested at the last barrier
    // (token half-slab pend_h first, then weight half-slab pend_h + 1): one load per four MFMAs.  Issued in one
    // burst right after the barrier, the four wavefronts' loads queue up in the CU's one address unit and the
    // wavefronts, which issue in order, cannot start their MFMAs until their last load is taken.
    int pend_h = nhalf, pend_sw = 0, pend_sx = 0;
    auto products = [&](auto ks_c) __attribute__((always_inline)) {
        constexpr int ks = decltype(ks_c)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma32(af[ks & 1][i], bf[ks & 1][j], acc[i][j]);
            constexpr int quarter = (ks + 1) & 3;            // sub-step 3 is the first after the barrier
            const int n = 4 * quarter + i;
            __builtin_amdgcn_sched_barrier(0);
            if (n < 8) issue_one(pend_h, pend_sx, IC<1>{}, n); else issue_one(pend_h + 1, pend_sw, IC<0>{}, n - 8);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- pipeline
#pragma unroll
    for (int r = 0; r < 8; ++r) issue_one(0, 0, IC<0>{}, r);
#pragma unroll
    for (int r = 0; r < 8; ++r) issue_one(1, 1, IC<1>{}, r);
#pragma unroll
    for (int r = 0; r < 8; ++r) issue_one(2, 2, IC<0>{}, r);
#pragma unroll
    for (int r = 0; r < 8; ++r) issue_one(3, 3, IC<1>{}, r);
#pragma unroll
    for (int r = 0; r < 8; ++r) issue_one(4, 4, IC<0>{}, r);
    if (nhalf >= kStages) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");    // half-slabs 0 and 1 of five
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    read_frags(0, 1, 0);
    // k block kb, with c = kb % kStages known at compile time
    auto block = [&](int kb, auto c_) __attribute__((always_inline)) {
        constexpr int c = decltype(c_)::value;
        constexpr int sw = (2 * c) % kStages, sx = (2 * c + 1) % kStages;              // stages of this block
        constexpr int nw = (2 * c + 2) % kStages, nx = (2 * c + 3) % kStages;          // ... of the next one
        read_frags(sw, sx, 1);
        products(IC<0>{});
        read_frags(sw, sx, 2);
        products(IC<1>{});
        read_frags(sw, sx, 3);
        products(IC<2>{});
        // The next block's two half-slabs: this wavefront's share has landed (the one requested after them may still
        // be on its way), then (barrier) everybody's; and everybody holds the last fragments of this block in
        // registers, so its two stages can take the half-slabs five further on (tokens of block kb + 2, needed at
        // the next barrier, then weights of block kb + 3), requested piecemeal by products().
        if (2 * kb + 4 < nhalf) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        pend_h = 2 * kb + kStages;
        pend_sx = sw;                    // half-slab 2 kb + 5 (tokens) takes the stage of half-slab 2 kb (weights)
        pend_sw = sx;                    // half-slab 2 kb + 6 (weights) the stage of half-slab 2 kb + 1 (tokens)
        if (kb + 1 < nblocks) read_frags(nw, nx, 0);
        products(IC<3>{});
    };
    int kb = 0;
    for (; kb + kStages <= nblocks; kb += kStages) {
        block(kb, IC<0>{});
        block(kb + 1, IC<1>{});
        block(kb + 2, IC<2>{});
        block(kb + 3, IC<3>{});
        block(kb + 4, IC<4>{});
    }
    if (kb < nblocks) { block(kb, IC<0>{}); ++kb; }
    if (kb < nblocks) { block(kb, IC<1>{}); ++kb; }
    if (kb < nblocks) { block(kb, IC<2>{}); ++kb; }
    if (kb < nblocks) { block(kb, IC<3>{}); ++kb; }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();        // every wavefront is done with the slabs: the staging area may overwrite them

    // ---- epilogue.  Feature of register r of block i: f0 + 32 i + 8 (r / 4) + 4 g + r % 4; token of block j: m0 + 32 j + lane % 32.
    const int f0 = f_tile0 + wm * 128;                    // first feature of this wavefront
    const int m0 = m_tile0 + wn * 128;                    // first token
    if (f0 >= a.N) return;
    char* stage_area = smem + wave * kEpiBytes;
    // bias, four consecutive features at a time
    if (a.bias != nullptr) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint2 raw = *reinterpret_cast<const uint2*>(a.bias + f0 + 32 * i + 8 * q + 4 * g);
                const __bf16* bv = reinterpret_cast<const __bf16*>(&raw);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += (float)bv[e];
            }
    }
    if constexpr (!QKV) {
        if (a.residual != nullptr) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int tok = min(m0 + 32 * j + (lane & 31), a.M - 1);
                const __bf16* rrow = a.residual + (int64_t)tok * a.ldr + f0 + 4 * g;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint2 raw = *reinterpret_cast<const uint2*>(rrow + 32 * i + 8 * q);
                        const __bf16* rv = reinterpret_cast<const __bf16*>(&raw);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += (float)rv[e];
                    }
            }
        }
    }
    int section = 0, head = 0;
    if constexpr (QKV) {
        const int per_section = a.Hn * 128;
        section = f0 / per_section;
        head = (f0 - section * per_section) >> 7;
        if (section < 2) {
#pragma clang fp contract(off)       // every product and sum below is rounded on its own, as in the eager expressions
            constexpr int D = 128;
            constexpr int nt = (D - 4 * (D / 6)) / 2, nh = D / 6, nw = D / 6;    // rotation pairs per axis: 22, 21, 21
            const __bf16* nwgt = a.norm_w[section];
            // the projection output is a bf16 tensor in the module this replaces: round before normalising
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float v = (float)(__bf16)acc[i][j][r];
                        acc[i][j][r] = v;
                        ss = fmaf(v, v, ss);
                    }
                ss += __shfl_xor(ss, 32);
                const float rs = __builtin_amdgcn_rsqf(ss * (1.0f / (float)D) + a.eps);    // as bsa_rope.h
                // position of this lane's token of block j
                const uint32_t tok = (uint32_t)min(m0 + 32 * j + (lane & 31), a.M - 1);
                const uint32_t s = tok % (uint32_t)a.S;
                const uint32_t u = s / (uint32_t)a.Wg, v2 = u / (uint32_t)a.Hg;
                const int wi = (int)(s - u * a.Wg), hi = (int)(u - v2 * a.Hg), ti = a.t0 + (int)v2;
                const int sin_t = a.Ttab * nt, cos_h = 2 * a.Ttab * nt, sin_h = a.Hg * nh, cos_w = cos_h + 2 * a.Hg * nh,
                          sin_w = a.Wg * nw;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint2 raw = *reinterpret_cast<const uint2*>(nwgt + 32 * i + 8 * q + 4 * g);
                        const __bf16* wv = reinterpret_cast<const __bf16*>(&raw);
                        float f[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            f[e] = (float)(__bf16)((float)(__bf16)(acc[i][j][4 * q + e] * rs) * (float)wv[e]);
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            const int pair = 16 * i + 4 * q + 2 * (int)g + e;
                            int at, dsin;
                            if (pair < nt) { at = ti * nt + pair; dsin = sin_t; }
                            else if (pair < nt + nh) { at = cos_h + hi * nh + pair - nt; dsin = sin_h; }
                            else { at = cos_w + wi * nw + pair - nt - nh; dsin = sin_w; }
                            const float c = a.tab[at], sn = a.tab[at + dsin];
                            const float x0 = f[2 * e], x1 = f[2 * e + 1];
                            // two products, then one add, each rounded: the order of operations of the eager expression
                            acc[i][j][4 * q + 2 * e] = x0 * c + (-x1) * sn;
                            acc[i][j][4 * q + 2 * e + 1] = x1 * c + x0 * sn;
                        }
                    }
            }
        }
    }
    // through LDS into token rows, 64 tokens at a time, then 16 bytes per lane to global memory
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = 2 * half + jj;
            char* row = stage_area + (32 * jj + (lane & 31)) * kEpiPitch + 8 * g;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    __bf16 v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (__bf16)acc[i][j][4 * q + e];
                    *reinterpret_cast<uint2*>(row + (32 * i + 8 * q) * 2) = *reinterpret_cast<const uint2*>(v);
                }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wavefront's LDS writes have landed
#pragma unroll 4
        for (int it = 0; it < 16; ++it) {
            const int lrow = 4 * it + (lane >> 4);
            const int tok = m0 + 64 * half + lrow;
            const uint4 val = *reinterpret_cast<const uint4*>(stage_area + lrow * kEpiPitch + (lane & 15) * 16);
            if (tok < a.M) {
                __bf16* o;
                if constexpr (QKV) {
                    const uint32_t bb = (uint32_t)tok / (uint32_t)a.S, s = (uint32_t)tok - bb * (uint32_t)a.S;
                    o = a.dst[section] + bb * a.dB + head * a.dH + s * a.dS;
                } else {
                    o = a.out + (int64_t)tok * a.ldo + f0;
                }
                *reinterpret_cast<uint4*>(o + (lane & 15) * 8) = val;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);   // the rows are read before the next half overwrites them
    }
}


template <bool QKV>
int launch_gemm(GemmArgs& a, hipStream_t stream) {
    a.tiles_m = (a.M + kTileM - 1) / kTileM;
    a.tiles_n = (a.N + kTileN - 1) / kTileN;
    a.super_m = (a.tiles_m + kSuperM - 1) / kSuperM;
    a.super_total = a.super_m * ((a.tiles_n + kSuperN - 1) / kSuperN);
    const unsigned grid = (unsigned)((a.super_total + 7) / 8) * 256u;
    const size_t lds = (size_t)kStages * kPart;
    static_assert(kStages * kPart >= 4 * kEpiBytes, "the staging area reuses the slabs");
    auto kernel = gemm_nt_kernel<QKV>;
    // more than the 64 KB a kernel gets without asking; the attribute is per device, so it is set on every call
    const hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (ea != hipSuccess) return set_error(BSA_ERR_HIP, "gemm: LDS size: %s", hipGetErrorString(ea));
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, stream, a);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? BSA_OK : set_error(BSA_ERR_HIP, "gemm launch: %s", hipGetErrorString(e));
}

int check_gemm_operands(const char* what, const void* x, int64_t ldx, const void* w, int64_t ldw, int64_t M, int N, int K) {
    if (!x || !w) return set_error(BSA_ERR_BAD_ARG, "%s: null pointer", what);
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffffLL) return set_error(BSA_ERR_BAD_ARG, "%s: M=%lld N=%d K=%d", what, (long long)M, N, K);
    if (K % kBK != 0) return set_error(BSA_ERR_UNSUPPORTED, "%s: K=%d must be a multiple of %d", what, K, kBK);
    if (N % 128 != 0) return set_error(BSA_ERR_UNSUPPORTED, "%s: N=%d must be a multiple of 128", what, N);
    if (ldx < K || ldw < K || ldx % 8 || ldw % 8) return set_error(BSA_ERR_BAD_ARG, "%s: row strides %lld, %lld (at least K, multiples of 8)", what, (long long)ldx, (long long)ldw);
    if (ldx >= (1 << 22) || ldw >= (1 << 22)) return set_error(BSA_ERR_UNSUPPORTED, "%s: row strides above 4M elements are not built", what);
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15u) return set_error(BSA_ERR_BAD_ARG, "%s: pointers must be 16-byte aligned", what);
    return BSA_OK;
}

}  // namespace
}  // namespace bsa

using namespace bsa;

extern "C" {

int bsa_gemm_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* residual,
                  int64_t ldr, void* out, int64_t ldo, int64_t M, int N, int K, void* stream) {
    const int rc = check_gemm_operands("gemm_bf16", x, ldx, w, ldw, M, N, K);
    if (rc != BSA_OK) return rc;
    if (!out) return set_error(BSA_ERR_BAD_ARG, "gemm_bf16: null pointer");
    if (ldo < N || ldo % 8 || (residual && (ldr < N || ldr % 8)))
        return set_error(BSA_ERR_BAD_ARG, "gemm_bf16: output / residual row strides (at least N, multiples of 8)");
    if ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(residual)) & 15u || reinterpret_cast<uintptr_t>(bias) & 7u)
        return set_error(BSA_ERR_BAD_ARG, "gemm_bf16: out and residual must be 16-byte aligned, bias 8-byte aligned");
    GemmArgs a = {};
    a.x = (const __bf16*)x; a.ldx = ldx; a.w = (const __bf16*)w; a.ldw = ldw; a.bias = (const __bf16*)bias;
    a.residual = (const __bf16*)residual; a.ldr = ldr; a.out = (__bf16*)out; a.ldo = ldo;
    a.M = (int)M; a.N = N; a.K = K;
    return launch_gemm<false>(a, (hipStream_t)stream);
}

int bsa_qkv_projection(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, const void* q_weight,
                       const void* k_weight, const float* rope_table, void* q, void* k, void* v,
                       const int64_t dst_strides[3], int B, int Hn, int T, int H, int W, int t_offset, int table_T,
                       int D, int K, float eps, void* stream) {
    if (D != 128) return set_error(BSA_ERR_UNSUPPORTED, "qkv_projection: head dim %d is not built (only 128)", D);
    if (B <= 0 || Hn <= 0 || T <= 0 || H <= 0 || W <= 0) return set_error(BSA_ERR_BAD_ARG, "qkv_projection: sizes must be positive");
    const int64_t S = (int64_t)T * H * W, M = (int64_t)B * S;
    if (S > 0x7fffffffLL || (int64_t)3 * Hn * D > 0x7fffffffLL) return set_error(BSA_ERR_UNSUPPORTED, "qkv_projection: too many tokens or features");
    const int rc = check_gemm_operands("qkv_projection", x, ldx, w, ldw, M, 3 * Hn * D, K);
    if (rc != BSA_OK) return rc;
    if (!q || !k || !v || !q_weight || !k_weight || !rope_table || !dst_strides)
        return set_error(BSA_ERR_BAD_ARG, "qkv_projection: null pointer");
    if (t_offset < 0 || table_T < t_offset + T)
        return set_error(BSA_ERR_SHAPE, "qkv_projection: frames %d..%d lie outside a table of %d frames", t_offset, t_offset + T, table_T);
    for (int i = 0; i < 3; ++i)
        if (dst_strides[i] < 0 || dst_strides[i] % 8) return set_error(BSA_ERR_BAD_ARG, "qkv_projection: strides must keep rows 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15u ||
        (reinterpret_cast<uintptr_t>(bias) | reinterpret_cast<uintptr_t>(q_weight) | reinterpret_cast<uintptr_t>(k_weight)) & 7u)
        return set_error(BSA_ERR_BAD_ARG, "qkv_projection: q, k, v must be 16-byte aligned, bias and norm weights 8-byte aligned");
    if (!(eps >= 0.f)) return set_error(BSA_ERR_BAD_ARG, "qkv_projection: eps must be non-negative");
    GemmArgs a = {};
    a.x = (const __bf16*)x; a.ldx = ldx; a.w = (const __bf16*)w; a.ldw = ldw; a.bias = (const __bf16*)bias;
    a.M = (int)M; a.N = 3 * Hn * D; a.K = K;
    a.dst[0] = (__bf16*)q; a.dst[1] = (__bf16*)k; a.dst[2] = (__bf16*)v;
    a.dB = dst_strides[0]; a.dH = dst_strides[1]; a.dS = dst_strides[2];
    a.norm_w[0] = (const __bf16*)q_weight; a.norm_w[1] = (const __bf16*)k_weight;
    a.tab = rope_table; a.Hn = Hn; a.S = (int)S; a.Hg = H; a.Wg = W; a.t0 = t_offset; a.Ttab = table_T; a.eps = eps;
    return launch_gemm<true>(a, (hipStream_t)stream);
}

}  // extern "C"
