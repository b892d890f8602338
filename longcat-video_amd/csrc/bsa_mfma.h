// Pieces shared by the MFMA attention kernels: vector types, the MFMA wrappers, the LDS DMA and the
// transposing LDS read.
#pragma once
#include "bsa_common.h"

#include <type_traits>

namespace bsa {
namespace mfma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

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
constexpr int kTile = 64;        // query rows per work item, keys per tile
constexpr int kTileBytes = kTile * kD * 2;
constexpr float kLog2e = 1.44269504f;
constexpr float kLn2 = 0.6931471824645996f;
constexpr float kLazyTau = 8.0f; // log2 headroom before the running max is raised
constexpr int kListCap = 1024;   // tiles whose addresses are staged in LDS at a time

// 16 bytes per lane from global memory straight into LDS.  The LDS address is
// m0 + 16*lane; the global address is sbase + voff.  Issued from inline assembly
// so that the compiler does not order later LDS reads of other stages behind it;
// completion is awaited explicitly (s_waitcnt vmcnt) before the stage is read.
// m0 is not on the clobber list: it is a reserved register for this target (the compiler rejects it there
// as undefined behaviour) and every compiler-generated use of m0 on gfx9 (movrel, readlane selectors, LDS DMA
// builtins) writes m0 itself immediately before the instruction that reads it, so nothing is assumed to
// survive this statement.  The kernels that use this helper index no register array dynamically.
__device__ inline void load_to_lds_16(const void* sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
// The same with 4 bytes per lane: the LDS address is m0 + 4*lane.
__device__ inline void load_to_lds_4(const void* sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ inline uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
// 4 keys x 16 d patch -> this lane's d, 4 keys (see the header comment)
__device__ inline s16x4 lds_read_tr16(const void* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

// S^T accumulators must sit in ordinary VGPRs, where the softmax reads them, while the (four times larger)
// output accumulators belong in AGPRs.  For a kernel that may use more than 256 registers the compiler puts
// the result of every builtin MFMA into AGPRs, so the S^T MFMAs are written as inline assembly with VGPR
// operands.  The compiler does not see that such a statement is an MFMA and adds no wait states behind it:
// the code keeps every VALU access to these accumulators at least eight MFMAs (256 clocks) behind the MFMA
// that writes them, or puts explicit s_nop there.
// The register allocator sees such a statement as an ordinary instruction that is complete when issued.  If the
// result were dead behind the last statement of a chain (a timing build that compiles the consumer out, say), the
// allocator could hand the registers to something else - an address, a loaded value - while the MFMA, whose
// passes run for another 32 clocks and more, still writes them: the new value is overwritten, and an overwritten
// address is a memory fault.  mfma_chain_end() (below) costs no instruction and ties the accumulators as live up
// to the place where it stands; every chain is closed with one, placed where the distance rule above holds.
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

// Marks the end of a chain of assembly MFMAs into `acc`: from here on the accumulators may be read, written or
// reused.  Emits nothing; it only keeps `acc` allocated, and unchanged, between the chain's last MFMA and this
// point, which the caller places at least eight MFMAs (or the equivalent s_nop) behind that MFMA.
__device__ __forceinline__ void mfma_chain_end(f32x16& acc) { asm volatile("" : "+v"(acc)); }

}  // namespace mfma
}  // namespace bsa
