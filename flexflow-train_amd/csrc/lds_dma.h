// Direct global -> LDS loads (no VGPR staging, no LDS write instructions) and
// what goes with them: scalar buffer descriptors, scalar LDS addresses, and
// explicit waits on the vector-memory counter.
#pragma once
#include "ffk_common.h"

namespace ffk {

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Waits for every vector-memory load of the wave, as an instruction the compiler sees.  The
// compiler counts only the loads it issued itself; after loads that it issued before a loop
// (operand fragments fetched once) it repeats its waits for them at their uses in every
// iteration, where the counter meanwhile holds the loop's direct loads: the wave then waits for
// the tile it has just asked for.  This wait, placed before the loop, tells it that nothing of
// its own is pending any more.  (simm16: vmcnt 0, expcnt 7, lgkmcnt 15.)
__device__ __forceinline__ void wait_all_vmem_known_to_compiler() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// One direct global->LDS load: lane l's 16 bytes at `g` land at LDS address
// lds_base + 16 l (M0 carries the wave-uniform base).  Issued as inline
// assembly on purpose: the compiler then does not know that LDS is being
// written asynchronously, and therefore does not put a full `vmcnt(0)` wait in
// front of later LDS reads it cannot prove disjoint (it did so in front of
// every transposing read, which serialised load and compute).  The kernel
// orders these loads against its LDS reads itself, with wait_vmcnt and the
// barrier.  Loads the compiler does know about stay correct: its vmcnt waits
// count these extra, younger loads too, which only makes them stricter.
// The load is the buffer form (a scalar resource descriptor for the operand
// panel, a scalar byte offset for what is uniform, one 32-bit byte offset per
// lane that never changes) rather than the flat-global form with a 64-bit
// address per lane: no vector address arithmetic remains in the k-loop, and
// the instruction issues through the vector-memory port alone.
typedef int i32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_dma16(i32x4 rsrc, unsigned lane_byte_off, unsigned uniform_byte_off,
                                          unsigned lds_byte_addr) {
  // lds_byte_addr is wave-uniform and held in a scalar register by the caller
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_byte_addr), "v"(lane_byte_off), "s"(rsrc), "s"(uniform_byte_off)
               : "memory");  // M0 is not in the clobber list (the compiler rejects
                             // reserved registers there).  The invariant every
                             // kernel that includes this header keeps: no register
                             // array is indexed by a run-time value (all such loops
                             // are fully unrolled), so the compiler emits no
                             // relative-move or GDS/message instruction and holds
                             // nothing live in M0 across these blocks.  Guarded by
                             // the bit-equality tests against the kernels without
                             // direct loads (tests/test_gpu_linear.py: GEMM variants)
                             // and by the attention kernels' tests against the oracle.
}
// The same for 4 bytes per lane: lane l's dword lands at lds_base + 4 l.
__device__ __forceinline__ void lds_dma4(i32x4 rsrc, unsigned lane_byte_off, unsigned uniform_byte_off,
                                         unsigned lds_byte_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(lds_byte_addr), "v"(lane_byte_off), "s"(rsrc), "s"(uniform_byte_off)
               : "memory");
}
// Raw buffer descriptor over num_bytes bytes from `base` on (by default no bound: stride 0,
// the offsets are then checked on the host), 32-bit data format.
__device__ __forceinline__ i32x4 buffer_resource(void const *base, unsigned num_bytes = 0xffffffffu) {
  uint64_t const a = reinterpret_cast<uint64_t>(base);
  i32x4 r;
  r[0] = (int)__builtin_amdgcn_readfirstlane((unsigned)a);
  r[1] = (int)(__builtin_amdgcn_readfirstlane((unsigned)(a >> 32)) & 0xffffu);
  // a load whose bytes do not all lie below num_bytes delivers zeros
  r[2] = (int)__builtin_amdgcn_readfirstlane(num_bytes);
  r[3] = 0x00020000;
  return r;
}
// The LDS byte address of a __shared__ object, as a scalar.
__device__ __forceinline__ unsigned lds_address_of(void *p) {
  return __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)p);
}

}  // namespace ffk
