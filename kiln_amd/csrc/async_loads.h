// Loads whose completion a kernel tracks itself (gfx950 only): inline-asm requests that the
// compiler neither reorders nor waits for, explicit s_waitcnt, then pin() on the registers.
// Vector memory loads of a wavefront complete in issue order, so "at most n outstanding" names
// the request that has landed.  Rules for the caller: a register filled by a request must stay
// where it is until it has been waited for and pinned, and request, wait and use must sit in
// one basic block (straight-line code), or the compiler may copy the register in between.
#pragma once
#include <type_traits>

#include "device_common.h"

namespace kiln {

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// f(integral_constant<int, I>) for I = first ... last - 1, unrolled at compile time
template <int I, int N, class F>
__device__ __forceinline__ void unrolled(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        unrolled<I + 1, N>(f);
    }
}

// 16 bytes per lane from global memory straight into LDS at lds_addr + 16 * lane (lds_addr is
// the same for the whole wavefront).  Counts as a vector memory load for s_waitcnt.
__device__ __forceinline__ void load_to_lds_b128(const void *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// The same with the address as wavefront-uniform base (scalar registers) + per-lane byte offset.
__device__ __forceinline__ void load_to_lds_b128(const void *base, uint32_t lane_off, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_off), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
}

// A zero the compiler cannot see through, defined where it is called: arithmetic that depends on
// it stays behind the preceding asm statements instead of being hoisted to the top of a long
// straight-line kernel (where it would hold registers for its whole length).
__device__ __forceinline__ uint32_t opaque_zero() {
    uint32_t z;
    asm volatile("v_mov_b32 %0, 0" : "=v"(z));
    return z;
}

// Address = wavefront-uniform base (scalar registers) + per-lane byte offset.
__device__ __forceinline__ void load_b128_streaming(u32x4 &dst, const void *base, uint32_t lane_off) {
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(dst) : "v"(lane_off), "s"(base) : "memory");
}
__device__ __forceinline__ void load_u16(uint32_t &dst, const void *base, uint32_t lane_off) {
    asm volatile("global_load_ushort %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(base) : "memory");
}

// Device-scope (coherent across the dies) 128-bit accesses: one instruction where four 32-bit
// atomic accesses would be four.  The load is a request like the ones above: wait, then pin.
// A store of more than 64 bits reads the upper part of its data registers after it has issued: a
// vector ALU instruction in the next two issue slots that overwrites them changes what is stored.
// The compiler pads that for its own stores and cannot see into this one, hence the s_nop.
__device__ __forceinline__ void store_b128_device_scope(void *ptr, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ void load_b128_device_scope(u32x4 &dst, const void *ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(dst) : "v"(ptr) : "memory");
}

// Orders every later use of v after this point (and hence after the preceding wait).
__device__ __forceinline__ void pin_loaded(u32x4 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin_loaded(uint32_t &v) { asm volatile("" : "+v"(v)); }

// Waits as inline asm with a memory clobber: unlike the s_waitcnt builtin, the compiler keeps
// ordinary loads and stores (LDS reads of data that an LDS-direct load delivered, stores that
// must be acknowledged before a barrier) on their side of it.
template <int N>
__device__ __forceinline__ void wait_vector_loads() {
    static_assert(N >= 0 && N <= 63, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }

}  // namespace kiln
