// Per-head RMSNorm and 3-D RoPE of one (token, head) row of 128 elements held by 16 consecutive lanes, 8
// elements (4 interleaved rotation pairs) per lane.  Shared by the stand-alone pass (bsa_glue.hip) and by the
// passes that apply the same steps while they move q and k (bsa_fwd_frag.hip), so that every route rounds at the
// same points:
//   x -> T(x * rsqrt(mean(x^2) + eps)) -> T(. * w) -> fp32 x*cos + rot(x)*sin -> T
// with rot(x)[2i] = -x[2i+1], rot(x)[2i+1] = x[2i] (blocks.py:42-53, rope_3d.py:34-38, 112-120).  Every product
// and sum is rounded on its own: the function body switches floating-point contraction off for the plain operators
// written in it (__fmul_rn / __fadd_rn would not do: they are inline functions whose bodies take the file's setting
// with them).  A file that includes this header must be compiled with -ffp-contract=off or fast-honor-pragmas.
#pragma once
#include "bsa_common.h"

namespace bsa {

constexpr int kRopeD = 128;
constexpr int kRopePairsT = (kRopeD - 4 * (kRopeD / 6)) / 2, kRopePairsH = kRopeD / 6, kRopePairsW = kRopeD / 6;   // 22, 21, 21

// cos / sin of lane `sub`'s four rotation pairs (pairs 4 sub .. 4 sub + 3) of the token at grid position
// (ti, hi, wi).  tab holds cos_t[Ttab][22], sin_t[Ttab][22], cos_h[Hg][21], sin_h[Hg][21], cos_w[Wg][21],
// sin_w[Wg][21] (fp32); ti already includes the frame offset.
__device__ inline void rope_angles(const float* __restrict__ tab, int Ttab, int Hg, int Wg, int ti, int hi, int wi, int sub,
                                   float (&c)[4], float (&sn)[4]) {
    constexpr int nt = kRopePairsT, nh = kRopePairsH, nw = kRopePairsW;
    const float* cos_t = tab;                        const float* sin_t = cos_t + (int64_t)Ttab * nt;
    const float* cos_h = sin_t + (int64_t)Ttab * nt; const float* sin_h = cos_h + (int64_t)Hg * nh;
    const float* cos_w = sin_h + (int64_t)Hg * nh;   const float* sin_w = cos_w + (int64_t)Wg * nw;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        const int pair = sub * 4 + jj;         // 0..63
        if (pair < nt) { c[jj] = cos_t[ti * nt + pair]; sn[jj] = sin_t[ti * nt + pair]; }
        else if (pair < nt + nh) { c[jj] = cos_h[hi * nh + pair - nt]; sn[jj] = sin_h[hi * nh + pair - nt]; }
        else { c[jj] = cos_w[wi * nw + pair - nt - nh]; sn[jj] = sin_w[wi * nw + pair - nt - nh]; }
    }
}

// x of the lane N positions further on in its row of 16 lanes (cyclic)
template <int N>
__device__ inline float row_ror(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x120 + N, 0xf, 0xf, false));
}

// The row piece of this lane through the norm (wraw: the lane's 8 weights; skipped when !do_norm) and the rotation
// (skipped when !do_rope).  The 16 lanes of the row must all be active: the sum of squares crosses them.
template <typename T>
__device__ inline uint4 norm_rope_piece(uint4 raw, uint4 wraw, bool do_norm, bool do_rope, const float (&c)[4],
                                        const float (&sn)[4], float eps) {
#pragma clang fp contract(off)
    const T* e = reinterpret_cast<const T*>(&raw);
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)e[i];
    if (do_norm) {
        const T* we = reinterpret_cast<const T*>(&wraw);
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(f[i], f[i], ss);
        // sum over the 16 lanes of the row, which are one DPP row: four rotations within the row (8, 4, 2, 1) leave the
        // total in every lane, without a trip through the LDS crossbar that a lane shuffle by 4 or 8 would take
        ss = ss + row_ror<8>(ss);
        ss = ss + row_ror<4>(ss);
        ss = ss + row_ror<2>(ss);
        ss = ss + row_ror<1>(ss);
        // the hardware's reciprocal square root (1 ulp) named directly: rsqrtf() expands differently under different
        // floating-point flags, and the files that share this function are compiled with different ones
        const float rs = __builtin_amdgcn_rsqf(ss * (1.0f / (float)kRopeD) + eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)(T)((float)(T)(f[i] * rs) * (float)we[i]);
    }
    T res[8];
    if (do_rope) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const float x0 = f[2 * jj], x1 = f[2 * jj + 1];
            // two products, then one add, each rounded: the order of operations of the eager expression
            res[2 * jj] = (T)(x0 * c[jj] + (-x1) * sn[jj]);
            res[2 * jj + 1] = (T)(x1 * c[jj] + x0 * sn[jj]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) res[i] = (T)f[i];
    }
    return *reinterpret_cast<const uint4*>(res);
}

}  // namespace bsa
