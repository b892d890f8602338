// Block-sparse flash-attention forward for gfx950 (bf16 / fp16 MFMA), plus a
// plain fp32 kernel for fp32 inputs.
//
// Work decomposition (MFMA kernel).  One workgroup = 256 threads = 4
// wavefronts owns 64 query rows and walks the list of selected KV blocks in
// 64-key tiles.  Wavefront (qh, kh) owns query rows 32*qh..+32 and keys
// 32*kh..+32 of every tile and runs an independent online softmax over its
// key half; the two halves are merged once, in the epilogue, with the usual
// log-sum-exp rescale.  No per-tile exchange between wavefronts is needed.
//
// Per tile and wavefront: S^T (32 keys x 32 queries) = K_half . Q^T as 8
// v_mfma_f32_32x32x16 over d = 128 (A = K rows from LDS, B = Q held in
// registers for the whole kernel), so every lane ends up with one query column
// and 16 keys: the softmax state (running max, running sum) is one scalar per
// lane, and P^T in the accumulator registers already has the layout the B
// operand of the second product needs.  O^T (128 d x 32 queries) += V^T . P^T
// is 8 more MFMAs whose A operand is read from a transposed copy of the V
// tile.  The transpose happens while staging: each thread loads 4 key rows x
// 8 d of V, transposes in registers and writes 8-byte key quads.
//
// LDS: 2 stages x (K tile 16 KB + V^T tile 16 KB) = 64 KB per workgroup, two
// workgroups per CU.  Both tiles use XOR-swizzled 16-byte chunks so that the
// ds_read_b128 of 16 consecutive lanes fall on distinct banks.
#include "bsa_common.h"

namespace bsa {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ inline f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ inline f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
template <typename T> struct Vec8;
template <> struct Vec8<__bf16> { typedef bf16x8 type; };
template <> struct Vec8<_Float16> { typedef f16x8 type; };

constexpr int kD = 128;          // head dim
constexpr int kTile = 64;        // query rows per workgroup, keys per tile
constexpr float kLog2e = 1.44269504f;
constexpr float kLn2 = 0.6931471824645996f;

// (x.lo16, y.lo16) and (x.hi16, y.hi16) packed into one dword
__device__ inline uint32_t pack_lo(uint32_t x, uint32_t y) { return __builtin_amdgcn_perm(y, x, 0x05040100u); }
__device__ inline uint32_t pack_hi(uint32_t x, uint32_t y) { return __builtin_amdgcn_perm(y, x, 0x07060302u); }

__device__ inline int vt_swizzle(int d) { return (d & 7) ^ ((d >> 3) & 7); }

template <typename T>
__global__ __launch_bounds__(256, 2) void fwd_mfma_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const int32_t* __restrict__ idx, const int32_t* __restrict__ lens,
    const uint64_t* __restrict__ tile_valid, T* __restrict__ o, float* __restrict__ lse,
    int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride, float qk_scale) {
    typedef typename Vec8<T>::type V8;
    // [stage][0 = K tile, row-major | 1 = V tile, transposed][64*128]
    __shared__ __attribute__((aligned(16))) T smem[2][2][kTile * kD];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int qh = wave & 1, kh = wave >> 1;
    const int lr = lane & 31, lh = lane >> 5;
    const int bh = blockIdx.y;
    const int64_t qrow0 = (int64_t)blockIdx.x * kTile;
    const int nbq = (int)(Sq / bs_q);
    const int qblock = (int)(qrow0 / bs_q);
    const int nsub = bs_k / kTile;
    const int32_t* list = idx + ((int64_t)bh * nbq + qblock) * idx_stride;
    const int ntiles = lens[(int64_t)bh * nbq + qblock] * nsub;

    const T* kbase = k + (int64_t)bh * Sk * kD;
    const T* vbase = v + (int64_t)bh * Sk * kD;

    // Q as the B operand: lane holds row 32*qh + lr, d = 16*s + 8*lh .. +8
    V8 qreg[8];
    {
        const T* qp = q + ((int64_t)bh * Sq + qrow0 + 32 * qh + lr) * kD + 8 * lh;
#pragma unroll
        for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const V8*>(qp + 16 * s);
    }

    // staging roles
    const int kc = tid & 15, kr = tid >> 4;   // K: 16-byte chunk kc of rows kr + 16*i
    const int vd = tid & 15, vq = tid >> 4;   // V: d-octet vd of key rows 4*vq + i
    const int v_chunk = ((vq >> 3) << 2) | (((vq >> 2) & 1) << 1) | (vq & 1);
    const int v_half = (vq >> 1) & 1;

    uint4 kreg[4], vreg[4];
    auto tile_row0 = [&](int it) -> int64_t {
        return (int64_t)list[it / nsub] * bs_k + (int64_t)(it % nsub) * kTile;
    };
    auto load_tile = [&](int64_t row0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            kreg[i] = *reinterpret_cast<const uint4*>(kbase + (row0 + kr + 16 * i) * kD + kc * 8);
            vreg[i] = *reinterpret_cast<const uint4*>(vbase + (row0 + 4 * vq + i) * kD + vd * 8);
        }
    };
    auto store_tile = [&](int st) {
        T* ks = smem[st][0];
        T* vt = smem[st][1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = kr + 16 * i;
            *reinterpret_cast<uint4*>(ks + r * kD + ((kc ^ (r & 15)) << 3)) = kreg[i];
        }
        const uint32_t* r0 = reinterpret_cast<const uint32_t*>(&vreg[0]);
        const uint32_t* r1 = reinterpret_cast<const uint32_t*>(&vreg[1]);
        const uint32_t* r2 = reinterpret_cast<const uint32_t*>(&vreg[2]);
        const uint32_t* r3 = reinterpret_cast<const uint32_t*>(&vreg[3]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int d = 8 * vd + e;
            uint2 w;
            if (e & 1) {
                w.x = pack_hi(r0[e >> 1], r1[e >> 1]);
                w.y = pack_hi(r2[e >> 1], r3[e >> 1]);
            } else {
                w.x = pack_lo(r0[e >> 1], r1[e >> 1]);
                w.y = pack_lo(r2[e >> 1], r3[e >> 1]);
            }
            *reinterpret_cast<uint2*>(vt + d * kTile + ((v_chunk ^ vt_swizzle(d)) << 3) + v_half * 4) = w;
        }
    };

    f32x16 oacc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[t][i] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;

    uint64_t vmask_next = ~0ull;
    if (ntiles > 0) {
        const int64_t row0 = tile_row0(0);
        if (tile_valid) vmask_next = tile_valid[row0 / kTile];
        load_tile(row0);
        store_tile(0);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
        const int st = it & 1;
        const uint64_t vmask = vmask_next;
        if (it + 1 < ntiles) {
            const int64_t row0 = tile_row0(it + 1);
            if (tile_valid) vmask_next = tile_valid[row0 / kTile];
            load_tile(row0);
        }
        const T* ks = smem[st][0];
        const T* vt = smem[st][1];

        // S^T = K_half . Q^T
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
        {
            const int row = 32 * kh + lr;
            const T* kp = ks + row * kD;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const V8 a = *reinterpret_cast<const V8*>(kp + (((2 * c + lh) ^ (row & 15)) << 3));
                s = mfma32(a, qreg[c], s);
            }
        }
        // accumulator i <-> key 32*kh + 8*(i/4) + 4*lh + i%4, query lr
        if (vmask != ~0ull) {
            const uint32_t half = (uint32_t)(vmask >> (32 * kh));
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (!((half >> (8 * (i / 4) + 4 * lh + (i % 4))) & 1u)) s[i] = -INFINITY;
        }
        float mx = s[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_i, mx * qk_scale);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_safe);
        float psum = 0.f;
        float p[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            p[i] = __builtin_amdgcn_exp2f(fmaf(s[i], qk_scale, -m_safe));
            psum += p[i];
        }
        l_i = fmaf(l_i, alpha, psum);
        m_i = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[t][i] *= alpha;
        }
        // P^T as B operand: k-slot (lh, j) of step c <-> accumulator 8*c + j
        V8 pb[2];
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) pb[c][j] = (T)p[8 * c + j];
        // O^T += V^T . P^T
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int d = 32 * t + lr;
            const T* vp = vt + d * kTile;
            const int sw = vt_swizzle(d);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const V8 a = *reinterpret_cast<const V8*>(vp + (((kh * 4 + 2 * c + lh) ^ sw) << 3));
                oacc[t] = mfma32(a, pb[c], oacc[t]);
            }
        }
        if (it + 1 < ntiles) store_tile(st ^ 1);
        __syncthreads();
    }

    // ---- epilogue: merge the two key halves, normalise, store coalesced ----
    float* xch = reinterpret_cast<float*>(&smem[0][0][0]);                  // [qh][66][64] fp32
    T* ost = reinterpret_cast<T*>(reinterpret_cast<char*>(xch) + 2 * 66 * 64 * 4);   // [64][128]
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
        T* orow = ost + (32 * qh + lr) * kD;
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
        if (lse != nullptr && lh == 0)
            lse[(int64_t)bh * Sq + qrow0 + 32 * qh + lr] = l > 0.f ? (m + __builtin_log2f(l)) * kLn2 : -INFINITY;
    }
    __syncthreads();
    {
        T* ob = o + ((int64_t)bh * Sq + qrow0) * kD;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = kr + 16 * i;
            *reinterpret_cast<uint4*>(ob + (int64_t)r * kD + kc * 8) =
                *reinterpret_cast<const uint4*>(ost + r * kD + kc * 8);
        }
    }
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
    const int ntiles = lens[(int64_t)bh * nbq + qblock] * nsub;
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
        const int64_t row0 = (int64_t)list[it / nsub] * bs_k + (int64_t)(it % nsub) * kTile;
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

hipError_t launch_fwd(const void* q, const void* k, const void* v, const int32_t* idx,
                      const int32_t* lens, const uint64_t* tile_valid, void* o, float* lse, int B,
                      int Hn, int64_t Sq, int64_t Sk, int bs_q, int bs_k, int idx_stride,
                      float sm_scale, int dtype, hipStream_t st) {
    dim3 grid((unsigned)(Sq / kTile), (unsigned)(B * Hn)), block(256);
    const float qk_scale = sm_scale * kLog2e;
    if (dtype == BSA_BF16)
        hipLaunchKernelGGL((fwd_mfma_kernel<__bf16>), grid, block, 0, st, (const __bf16*)q,
                           (const __bf16*)k, (const __bf16*)v, idx, lens, tile_valid, (__bf16*)o,
                           lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale);
    else if (dtype == BSA_F16)
        hipLaunchKernelGGL((fwd_mfma_kernel<_Float16>), grid, block, 0, st, (const _Float16*)q,
                           (const _Float16*)k, (const _Float16*)v, idx, lens, tile_valid,
                           (_Float16*)o, lse, Sq, Sk, bs_q, bs_k, idx_stride, qk_scale);
    else
        hipLaunchKernelGGL(fwd_f32_kernel, grid, block, 0, st, (const float*)q, (const float*)k,
                           (const float*)v, idx, lens, tile_valid, (float*)o, lse, Sq, Sk, bs_q,
                           bs_k, idx_stride, qk_scale);
    return hipGetLastError();
}

}  // namespace bsa
