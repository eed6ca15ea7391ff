// Copies from global memory straight into LDS (global_load_lds_dwordx4), for kernels that
// keep several tiles in flight.
//
// A wave's copy instruction writes 64 pieces of 16 bytes to consecutive LDS addresses, from
// one address per lane.  The copies are written as inline assembly: the compiler then does
// not count them, so it neither makes every LDS read wait for all of them nor drains them at
// each barrier; a kernel waits for exactly the tile it is about to use (s_waitcnt vmcnt) and
// meets the other waves at a bare s_barrier.  A lane whose piece does not exist reads from a
// block of zeros instead, so every tile issues the same number of copies and one counter
// value tells when a tile has landed.
#pragma once

#include "common.h"

static __device__ uint4 xr_zero_chunk[4];      // zero-initialised

__device__ inline void lds_dma16(const void* src, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(src), "s"(lds_byte_addr) : "memory");
}
// the same with the source as a base that all lanes share (in scalar registers) and a 32-bit
// byte offset per lane: no 64-bit arithmetic per lane and copy
__device__ inline void lds_dma16_base(const void* base, uint32_t byte_offset, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(byte_offset), "s"(base), "s"(lds_byte_addr) : "memory");
}
template <int N> __device__ inline void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "the counter holds 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
