// Inline-asm memory operations shared by the 128x256-tile GEMM kernels: the direct global->LDS load and a store with a
// wave-uniform base.  The compiler cannot see inside an asm statement, so each statement carries its own wait states.
#pragma once
#include "common.h"

namespace tbik {

// One 16-byte-per-lane direct global->LDS load: lane l's 16 bytes land at lds_addr + 16*l.
// The compiler cannot see inside the statement, so the statement takes care of its own hazards without idle wait
// states: the load must not follow the write of m0 directly, and a vector-memory instruction must not read a scalar
// register less than five states after a VECTOR instruction wrote it (which is how a spilled scalar comes back:
// v_readlane_b32).  The scalar copy of the base address between the write of m0 and the load settles both: it is the
// one state behind m0, and the load then reads a register that a scalar instruction has written.  m0 is declared
// clobbered so that the compiler never keeps a value of its own there.
__device__ __forceinline__ void dma16(uint32_t lds_addr, uint32_t voff, const void* base) {
  const void* base_copy;
  asm volatile("s_mov_b32 m0, %1\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0"
               : "=&s"(base_copy)
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}

// The same load to lds_base + offset, the offset a compile-time constant: the sum is formed in m0 itself (one scalar
// instruction instead of an add and a move; the scalar condition code is clobbered).
__device__ __forceinline__ void dma16_at(uint32_t lds_base, int offset, uint32_t voff, const void* base) {
  const void* base_copy;
  asm volatile("s_add_u32 m0, %1, %4\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0"
               : "=&s"(base_copy)
               : "s"(lds_base), "v"(voff), "s"(base), "n"(offset)
               : "memory", "m0", "scc");
}

// 16-byte-per-lane store to (wave-uniform base) + voff, scalar-base addressing: no per-lane 64-bit pointer.
__device__ __forceinline__ void store16_sbase(void* base, uint32_t voff, u32x4 v) {
  // the wait states behind the store keep the next instruction from overwriting the data registers while the store
  // still reads them, the ones in front of it cover a scalar base that a vector instruction has just written
  // (hazards the compiler handles for its own instructions, but cannot see inside an asm statement)
  asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2\n\ts_nop 1" : : "v"(voff), "v"(v), "s"(base) : "memory");
}

}  // namespace tbik
