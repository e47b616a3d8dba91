// LDS primitives shared by the kernels that stream operand tiles from global memory straight into
// LDS (global_load_lds) and read MFMA fragments back with explicit waits.
//
// Fragment reads are inline assembly so that the compiler neither guesses at aliasing between them
// and the in-flight global->LDS transfers (it would wait for *all* transfers before a transpose
// read) nor places the waits: the kernels wait explicitly on the lgkmcnt / vmcnt counters.
//
// The price: the compiler takes a read's destination registers to be written when the instruction issues, not when
// the data arrives. Every value returned by lds_read_* must therefore be consumed, after a wait that covers it, on
// every path that issued the read. A result left unused has no live range, its registers go to the next value the
// compiler needs (a global address, say), and the LDS data lands on top of that value later. The readers are
// [[nodiscard]] and the library is built with -Werror=unused-result, so a call whose value is dropped does not compile;
// tests/test_isa_hazards.py checks the compiled kernels for values that are assigned and then never read.
#pragma once

#include "common.h"

namespace dml {

typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// 16 bytes per lane, global -> LDS without staging registers. The LDS destination of lane l is
// lds_dst + 16*l; lds_dst must be wavefront-uniform.
__device__ __forceinline__ void lds_dma16(const _Float16* gptr, char* lds_dst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                     (__attribute__((address_space(3))) void*)lds_dst, 16, 0, 0);
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)p;
}

template <int OFFSET>
[[nodiscard]] __device__ __forceinline__ half8 lds_read_b128(uint32_t addr) {
    half8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}

// LDS transpose read: within each group of 16 lanes, lane s points at four consecutive 16-bit
// elements of row s/4 (columns 4*(s%4)..+3 of the group's 16 columns); lane j receives column j of
// the four rows. A lane thus gets four consecutive K values of "its" column, the MFMA operand layout.
template <int OFFSET>
[[nodiscard]] __device__ __forceinline__ half4v lds_read_tr16_b64(uint32_t addr) {
    half4v v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}

// 16 bytes per lane to global memory at agent scope (sc1): the line goes through the L2 to the memory side as it is
// written instead of staying dirty in the XCD's L2 until the kernel ends. For a result that a kernel writes in one burst
// at its end (a GEMM tile), the write-back of up to 32 MB of dirty lines between this kernel and the next one goes
// away. A store of more than 64 bits reads its data registers up to two wait states after it issues, and the compiler's
// hazard recognizer, which keeps vector writes to those registers away for that long, does not look into inline assembly:
// the two wait states are part of the statement.
__device__ __forceinline__ void global_store_b128_through(void* p, half8 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_lgkm() {
    static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit counter");
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}

template <int VM>
__device__ __forceinline__ void wait_vm_lgkm0() {
    static_assert(VM >= 0 && VM <= 63, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(VM) : "memory");
}

}  // namespace dml
