// Global -> LDS copies without a register stage (buffer_load ... lds) and the explicit waits that go with them.
//
// One wave instruction copies 64 x 16 bytes (or 64 x 4): lane l lands at LDS address M0 + 16 * l (4 * l); lanes whose
// offset is outside the buffer write zeros.  The copies are issued from inline assembly, which the compiler's own
// wait-count insertion does not see: callers wait for them with wait_vmcnt<N>().  Vector-memory loads complete in
// order, so a compiler-issued load or store between two copies can only make such a wait stricter, never too weak.
#pragma once
#include "igemm_shared.h"

namespace mi355 {

__device__ __forceinline__ void lds_copy64x16(uint32_t lds_addr, int voff, const v4i& rsrc) {
    // M0 needs one wait state before an LDS-direct load reads it
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, 0 offen lds"
        :
        : "s"(lds_addr), "v"(voff), "s"(rsrc)
        : "memory", "m0");
}

// 64 x 4 bytes: lane l lands at M0 + 4 * l (4-packed activations: one pixel's channel block per lane)
__device__ __forceinline__ void lds_copy64x4(uint32_t lds_addr, int voff, const v4i& rsrc) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dword %1, %2, 0 offen lds"
        :
        : "s"(lds_addr), "v"(voff), "s"(rsrc)
        : "memory", "m0");
}

// the same with a wave-uniform part of the address in the scalar offset (lanes that are masked off write nothing)
__device__ __forceinline__ void lds_copy_row64x4(uint32_t lds_addr, int voff, int soff, const v4i& rsrc) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dword %1, %2, %3 offen lds"
        :
        : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
        : "memory", "m0");
}

__device__ __forceinline__ void lds_copy_row64x16(uint32_t lds_addr, int voff, int soff, const v4i& rsrc) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen lds"
        :
        : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
        : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// a buffer descriptor held in scalar registers (the inline assembly takes it as an "s" operand)
__device__ __forceinline__ v4i uniform_rsrc(const void* p, uint32_t bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)p;
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = 0x00020000;
    return r;
}

}  // namespace mi355
