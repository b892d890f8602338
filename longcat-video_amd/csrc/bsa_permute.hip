// 3-D chunk permute / unpermute and block mean pooling (HBM-bound kernels).
//
// One workgroup moves one chunk (t*h*w slots of D elements).  Rows are moved
// as 16-byte pieces: the D/EPV lanes that share a row read one contiguous row
// (256 B for D=128 bf16) and consecutive row groups walk the w-run, so both
// the gather from THW order and the store to blocked order are coalesced.
// The pooled mean is accumulated on the fly from the registers that already
// hold the row, so q and k are read from HBM once for permute + pool.
#include "bsa_common.h"

namespace bsa {
namespace {

constexpr int kThreads = 256;

template <typename T> struct Piece { static constexpr int EPV = 16 / sizeof(T); };

template <typename T>
__device__ inline void accumulate(float* acc, const uint4& v) {
    constexpr int EPV = Piece<T>::EPV;
    const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
    for (int i = 0; i < EPV; ++i) acc[i] += (float)e[i];
}

// Sum the per-row-group partials in a fixed order (row group ascending) and
// store mean = sum * (1/bs) rounded once to T.
template <typename T>
__device__ inline void finish_pool(float* acc, float* red, T* out_row, int cpr, int c, int rg,
                                   int RG, float inv_bs) {
    constexpr int EPV = Piece<T>::EPV;
    const int D = cpr * EPV;
#pragma unroll
    for (int i = 0; i < EPV; ++i) red[rg * D + c * EPV + i] = acc[i];
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += kThreads) {
        float s = 0.f;
        for (int g = 0; g < RG; ++g) s += red[g * D + d];
        out_row[d] = (T)(s * inv_bs);
    }
}

template <typename T, bool POOL>
__global__ __launch_bounds__(kThreads) void permute_kernel(
    const T* __restrict__ src, int64_t sB, int64_t sH, int64_t sS, T* __restrict__ dst,
    T* __restrict__ pooled, uint64_t* __restrict__ tile_valid, Grid3 g, int Hn, int D, int edge_only, int n_edge,
    int32_t* __restrict__ row_table, uint32_t* __restrict__ tile_table,
    const T* __restrict__ src2, int64_t s2B, int64_t s2H, int64_t s2S, T* __restrict__ dst2) {
    extern __shared__ float red[];
    constexpr int EPV = Piece<T>::EPV;
    const int blk = blockIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / Hn, hd = bh % Hn;
    const int nw = blk % g.Nw, nh = (blk / g.Nw) % g.Nh, nt = blk / (g.Nw * g.Nh);
    const int bs = g.chunk();
    const int nb = g.blocks();
    const int cpr = D / EPV;
    const int c = threadIdx.x % cpr, rg = threadIdx.x / cpr, RG = kThreads / cpr;
    const T* sbase = src + (int64_t)b * sB + (int64_t)hd * sH;
    T* dbase = dst + ((int64_t)bh * nb + blk) * bs * D;
    if (bh == 0 && row_table != nullptr) {
        for (int r = threadIdx.x; r < bs; r += kThreads) {
            const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
            const int tt = nt * g.t + ti, hh = nh * g.h + hi, ww = nw * g.w + wi;
            row_table[(int64_t)blk * bs + r] = (tt < g.T && hh < g.H && ww < g.W) ? (tt * g.H + hh) * g.W + ww : -1;
        }
    }
    if (bh == 0 && tile_table != nullptr && threadIdx.x < bs / 64) {
        const int sub = threadIdx.x, nsub = bs / 64, e = edge_index(g, blk);
        const int planes = 64 / (g.w * g.h);          // a tile is a whole number of (h, w) planes here
        tile_table[(int64_t)blk * nsub + sub] =
            e < 0 ? (uint32_t)(((nt * g.t + sub * planes) * g.H + nh * g.h) * g.W + nw * g.w)
                  : (1u << 24) + (uint32_t)(e * nsub + sub);
    }
    if (edge_only) {
        const int e = edge_index(g, blk);
        dbase = e < 0 ? nullptr : dst + ((int64_t)bh * n_edge + e) * bs * D;
    }
    if (dst == nullptr) dbase = nullptr;
    float acc[EPV];
#pragma unroll
    for (int i = 0; i < EPV; ++i) acc[i] = 0.f;

    // The rows are only read when they are copied or pooled.  Four rows per thread are requested
    // before the first one is used, so that a workgroup has its whole 64-slot chunk in flight.
    auto fetch = [&](const T* base, int64_t stride_s, int r) -> uint4 {
        const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
        const int tt = nt * g.t + ti, hh = nh * g.h + hi, ww = nw * g.w + wi;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (r < bs && tt < g.T && hh < g.H && ww < g.W) {
            const int64_t s = ((int64_t)tt * g.H + hh) * g.W + ww;
            val = *reinterpret_cast<const uint4*>(base + s * stride_s + c * EPV);
        }
        return val;
    };
    for (int r0 = (POOL || dbase != nullptr) ? rg : bs; r0 < bs; r0 += 4 * RG) {
        uint4 val[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) val[j] = fetch(sbase, sS, r0 + j * RG);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = r0 + j * RG;
            if (r < bs) {
                if (dbase != nullptr) *reinterpret_cast<uint4*>(dbase + (int64_t)r * D + c * EPV) = val[j];
                if (POOL) accumulate<T>(acc, val[j]);
            }
        }
    }
    // a second tensor on the same grid (v next to k): edge chunks only
    if (src2 != nullptr && edge_only && dbase != nullptr) {
        const T* sbase2 = src2 + (int64_t)b * s2B + (int64_t)hd * s2H;
        T* dbase2 = dst2 + (dbase - dst);
        for (int r0 = rg; r0 < bs; r0 += 4 * RG) {
            uint4 val[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) val[j] = fetch(sbase2, s2S, r0 + j * RG);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = r0 + j * RG;
                if (r < bs) *reinterpret_cast<uint4*>(dbase2 + (int64_t)r * D + c * EPV) = val[j];
            }
        }
    }
    if (tile_valid != nullptr && bh == 0) {
        // bit s of word i <=> slot 64*i+s of the blocked order holds a real token
        for (int r0 = (threadIdx.x / 64) * 64; r0 < bs; r0 += kThreads) {
            const int r = r0 + (threadIdx.x & 63);
            const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
            const bool ok = nt * g.t + ti < g.T && nh * g.h + hi < g.H && nw * g.w + wi < g.W;
            const uint64_t m = __ballot(ok);
            if ((threadIdx.x & 63) == 0) tile_valid[((int64_t)blk * bs + r0) / 64] = m;
        }
    }
    if (POOL)
        finish_pool<T>(acc, red, pooled + ((int64_t)bh * nb + blk) * D, cpr, c, rg, RG, 1.0f / bs);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void unpermute_kernel(
    const T* __restrict__ src, T* __restrict__ dst, int64_t sB, int64_t sH, int64_t sS, Grid3 g,
    int Hn, int D) {
    constexpr int EPV = Piece<T>::EPV;
    const int blk = blockIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / Hn, hd = bh % Hn;
    const int nw = blk % g.Nw, nh = (blk / g.Nw) % g.Nh, nt = blk / (g.Nw * g.Nh);
    const int bs = g.chunk();
    const int nb = g.blocks();
    const int cpr = D / EPV;
    const int c = threadIdx.x % cpr, rg = threadIdx.x / cpr, RG = kThreads / cpr;
    const T* sbase = src + ((int64_t)bh * nb + blk) * bs * D;
    T* dbase = dst + (int64_t)b * sB + (int64_t)hd * sH;
    for (int r = rg; r < bs; r += RG) {
        const int wi = r % g.w, hi = (r / g.w) % g.h, ti = r / (g.w * g.h);
        const int tt = nt * g.t + ti, hh = nh * g.h + hi, ww = nw * g.w + wi;
        if (tt < g.T && hh < g.H && ww < g.W) {
            const int64_t s = ((int64_t)tt * g.H + hh) * g.W + ww;
            *reinterpret_cast<uint4*>(dbase + s * sS + c * EPV) =
                *reinterpret_cast<const uint4*>(sbase + (int64_t)r * D + c * EPV);
        }
    }
}

// Mean over consecutive `block`-row groups of a contiguous [BH, S, D] tensor.
template <typename T>
__global__ __launch_bounds__(kThreads) void mean_pool_kernel(const T* __restrict__ x,
                                                            T* __restrict__ out, int64_t S,
                                                            int block, int nb, int D) {
    extern __shared__ float red[];
    constexpr int EPV = Piece<T>::EPV;
    const int blk = blockIdx.x;
    const int bh = blockIdx.y;
    const int cpr = D / EPV;
    const int c = threadIdx.x % cpr, rg = threadIdx.x / cpr, RG = kThreads / cpr;
    const T* base = x + (int64_t)bh * S * D;
    float acc[EPV];
#pragma unroll
    for (int i = 0; i < EPV; ++i) acc[i] = 0.f;
    for (int r = rg; r < block; r += RG) {
        const int64_t s = (int64_t)blk * block + r;
        if (s < S) accumulate<T>(acc, *reinterpret_cast<const uint4*>(base + s * D + c * EPV));
    }
    finish_pool<T>(acc, red, out + ((int64_t)bh * nb + blk) * D, cpr, c, rg, RG, 1.0f / block);
}

// Chunk means only, for 64-slot chunks of 16-bit rows of 128 elements: one wavefront per chunk, no LDS, no
// barrier, all of a lane's sixteen 16-byte loads in flight at once (the read-only pass over q of the operator).
// Rows come through the row table (token of every slot, -1 = padding: a zero row).  The sums are taken in
// permute_kernel's order - a thread's rows rg, rg + 16, rg + 32, rg + 48 first, then the sixteen partial sums
// of a column in ascending rg, starting from zero - so the means carry the same bits.  Lane = (c16, r4): 16-byte
// piece c16 of the rows rg = 4 r4 .. 4 r4 + 3.
template <bool kBf16>
__global__ __launch_bounds__(256) void pool_tiles_kernel(const uint16_t* __restrict__ src, int64_t sB, int64_t sH, int64_t sS,
                                                         const int32_t* __restrict__ row_table, uint16_t* __restrict__ pooled,
                                                         int tiles, int Hn, int64_t total, int head_fastest) {
    const int lane = threadIdx.x & 63;
    const int64_t id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (id >= total) return;
    int tile_id, bh;
    if (head_fastest) {
        const int64_t per_batch = (int64_t)tiles * Hn;
        const int b = (int)(id / per_batch), rest = (int)(id - b * per_batch);
        tile_id = rest / Hn;
        bh = b * Hn + (rest - tile_id * Hn);
    } else {
        bh = (int)(id / tiles);
        tile_id = (int)(id - (int64_t)bh * tiles);
    }
    const uint16_t* sbase = src + (int64_t)(bh / Hn) * sB + (int64_t)(bh % Hn) * sH;
    const int c16 = lane & 15, r4 = lane >> 4;
    // the table entries first, then every row unconditionally (a padded slot reads token 0 and is cleared afterwards):
    // sixteen independent loads per lane, no branch between them
    int32_t token[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) token[u][i] = row_table[tile_id * 64 + 4 * r4 + u + 16 * i];
    uint4 xs[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            xs[u][i] = *reinterpret_cast<const uint4*>(sbase + (int64_t)max(token[u][i], 0) * sS + c16 * 8);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (token[u][i] < 0) xs[u][i] = make_uint4(0, 0, 0, 0);
    float part[4][8];                       // this lane's rows rg = 4 r4 + u: rg, rg + 16, rg + 32, rg + 48 in that order
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int e = 0; e < 8; ++e) part[u][e] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w[4] = {xs[u][i].x, xs[u][i].y, xs[u][i].z, xs[u][i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo, hi;
                if (kBf16) { lo = __uint_as_float(w[e] << 16); hi = __uint_as_float(w[e] & 0xffff0000u); }
                else { lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] & 0xffffu)); hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] >> 16)); }
                part[u][2 * e] += lo;
                part[u][2 * e + 1] += hi;
            }
        }
    }
    // the sixteen partial sums of a column in ascending rg: four per lane, handed from r4 to r4 + 1
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.f;
#pragma unroll
    for (int stage = 0; stage < 4; ++stage) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float below = stage == 0 ? 0.f : __shfl_up(sum[e], 16);
            if (r4 == stage) sum[e] = (((below + part[0][e]) + part[1][e]) + part[2][e]) + part[3][e];
        }
    }
    if (r4 == 3) {
        uint16_t out[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float mean = sum[e] * (1.0f / 64.0f);
            out[e] = kBf16 ? __builtin_bit_cast(uint16_t, (__bf16)mean) : __builtin_bit_cast(uint16_t, (_Float16)mean);
        }
        *reinterpret_cast<uint4*>(pooled + ((int64_t)bh * tiles + tile_id) * 128 + c16 * 8) = *reinterpret_cast<const uint4*>(out);
    }
}

inline size_t red_bytes(int D, int esize) {
    const int cpr = D / (16 / esize);
    return (size_t)(kThreads / cpr) * D * sizeof(float);
}

}  // namespace

hipError_t launch_permute(const void* src, const int64_t st3[3], void* dst, void* pooled,
                          uint64_t* tile_valid, int B, int Hn, const Grid3& g, int D, int dtype,
                          hipStream_t st, bool edge_only, int32_t* row_table, uint32_t* tile_table,
                          const void* src2, const int64_t* st3_2, void* dst2) {
    const int64_t zero3[3] = {0, 0, 0};
    const int64_t* s2 = st3_2 ? st3_2 : zero3;
    dim3 grid(g.blocks(), B * Hn), block(kThreads);
    const size_t smem = pooled ? red_bytes(D, dtype_size(dtype)) : 0;
    const int eo = edge_only ? 1 : 0, ne = edge_only ? edge_count(g) : 0;
#define BSA_LAUNCH(T)                                                                          \
    if (pooled)                                                                                \
        hipLaunchKernelGGL((permute_kernel<T, true>), grid, block, smem, st, (const T*)src,     \
                           st3[0], st3[1], st3[2], (T*)dst, (T*)pooled, tile_valid, g, Hn, D, eo, ne, row_table, tile_table, \
                           (const T*)src2, s2[0], s2[1], s2[2], (T*)dst2); \
    else                                                                                       \
        hipLaunchKernelGGL((permute_kernel<T, false>), grid, block, smem, st, (const T*)src,    \
                           st3[0], st3[1], st3[2], (T*)dst, (T*)pooled, tile_valid, g, Hn, D, eo, ne, row_table, tile_table, \
                           (const T*)src2, s2[0], s2[1], s2[2], (T*)dst2);
    if (dtype == BSA_BF16) { BSA_LAUNCH(__bf16) }
    else if (dtype == BSA_F16) { BSA_LAUNCH(_Float16) }
    else { BSA_LAUNCH(float) }
#undef BSA_LAUNCH
    return hipGetLastError();
}

hipError_t launch_pool_tiles(const void* src, const int64_t st3[3], const int32_t* row_table, void* pooled, int B, int Hn,
                             const Grid3& g, int dtype, hipStream_t st) {
    if (g.chunk() != 64 || (dtype != BSA_BF16 && dtype != BSA_F16) || row_table == nullptr) return hipErrorInvalidValue;
    const int64_t total = (int64_t)g.blocks() * B * Hn;
    const dim3 grid((unsigned)((total + 3) / 4)), block(256);
    const int head_fastest = st3[1] < st3[2] ? 1 : 0;
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL(pool_tiles_kernel<true>, grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2], row_table,
                           (uint16_t*)pooled, g.blocks(), Hn, total, head_fastest);
    else
        hipLaunchKernelGGL(pool_tiles_kernel<false>, grid, block, 0, st, (const uint16_t*)src, st3[0], st3[1], st3[2], row_table,
                           (uint16_t*)pooled, g.blocks(), Hn, total, head_fastest);
    return hipGetLastError();
}

hipError_t launch_unpermute(const void* src, void* dst, const int64_t st3[3], int B, int Hn,
                            const Grid3& g, int D, int dtype, hipStream_t st) {
    dim3 grid(g.blocks(), B * Hn), block(kThreads);
    if (dtype == BSA_F32)
        hipLaunchKernelGGL((unpermute_kernel<float>), grid, block, 0, st, (const float*)src,
                           (float*)dst, st3[0], st3[1], st3[2], g, Hn, D);
    else  // 16-bit types move as raw bits
        hipLaunchKernelGGL((unpermute_kernel<uint16_t>), grid, block, 0, st, (const uint16_t*)src,
                           (uint16_t*)dst, st3[0], st3[1], st3[2], g, Hn, D);
    return hipGetLastError();
}

hipError_t launch_mean_pool(const void* x, void* out, int B, int Hn, int64_t S, int block, int D,
                            int dtype, hipStream_t st) {
    const int nb = (int)((S + block - 1) / block);
    dim3 grid(nb, B * Hn), blk(kThreads);
    const size_t smem = red_bytes(D, dtype_size(dtype));
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((mean_pool_kernel<__bf16>), grid, blk, smem, st, (const __bf16*)x,
                           (__bf16*)out, S, block, nb, D);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((mean_pool_kernel<_Float16>), grid, blk, smem, st, (const _Float16*)x,
                           (_Float16*)out, S, block, nb, D);
    else
        hipLaunchKernelGGL((mean_pool_kernel<float>), grid, blk, smem, st, (const float*)x,
                           (float*)out, S, block, nb, D);
    return hipGetLastError();
}

}  // namespace bsa
