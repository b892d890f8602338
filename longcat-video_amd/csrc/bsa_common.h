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
hipError_t launch_permute(const void* src, const int64_t strides[3], void* dst, void* pooled,
                          uint64_t* tile_valid, int B, int Hn, const Grid3& g, int D, int dtype,
                          hipStream_t st);
hipError_t launch_unpermute(const void* src, void* dst, const int64_t strides[3], int B, int Hn,
                            const Grid3& g, int D, int dtype, hipStream_t st);
hipError_t launch_mean_pool(const void* x, void* out, int B, int Hn, int64_t S, int block, int D,
                            int dtype, hipStream_t st);
hipError_t launch_score(const void* q_cmp, const void* k_cmp, void* score, int BH, int nbq, int nbk,
                        int D, int dtype, hipStream_t st);
// idx: descending score order; idx_sorted: ascending block index; either may be null
hipError_t launch_topk(const void* score, int32_t* idx, int32_t* idx_sorted, int32_t* lens, int64_t rows,
                       int nbk, int k_sel, int dtype, hipStream_t st);
hipError_t launch_fwd(const void* q, const void* k, const void* v, const int32_t* idx,
                      const int32_t* lens, const uint64_t* tile_valid, void* o, float* lse,
                      int B, int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
                      float sm_scale, int dtype, hipStream_t st);

}  // namespace bsa
