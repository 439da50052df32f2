// Direct-to-LDS buffer loads, hand-placed vector-memory waits, a fence-less workgroup barrier and a
// wave-wide OR: the pieces shared by the kernels that stream gathered rows through LDS rings.
#pragma once
#include "common.h"

namespace cummhip {

#define CUMM_LDS_PTR(x) ((__attribute__((address_space(3))) void *)(x))

// s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = simm16[15:14,3:0])
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// OR over the 64 lanes of a wave with row shifts and row broadcasts (no LDS round trips)
__device__ __forceinline__ uint32_t wave_or_dpp(uint32_t v) {
  int t = (int)v;
  t |= __builtin_amdgcn_update_dpp(0, t, 0x111, 0xf, 0xf, true);   // row_shr:1
  t |= __builtin_amdgcn_update_dpp(0, t, 0x112, 0xf, 0xf, true);   // row_shr:2
  t |= __builtin_amdgcn_update_dpp(0, t, 0x114, 0xf, 0xf, true);   // row_shr:4
  t |= __builtin_amdgcn_update_dpp(0, t, 0x118, 0xf, 0xf, true);   // row_shr:8 -> lane 15 of a row
  t |= __builtin_amdgcn_update_dpp(0, t, 0x142, 0xa, 0xf, true);   // row_bcast:15 into rows 1, 3
  t |= __builtin_amdgcn_update_dpp(0, t, 0x143, 0xc, 0xf, true);   // row_bcast:31 into rows 2, 3
  return (uint32_t)__builtin_amdgcn_readlane(t, 63);
}

// Direct-to-LDS buffer loads, written as asm so that the compiler's wait-count pass does not see
// them: it guards LDS reads that may alias an outstanding direct-to-LDS load with waits of its
// own, and at a loop header it assumes the worst (waits for all of them), which would drain the
// ring once per trip.  Every wait for these loads is placed by hand (wait_vmcnt).  Hidden loads
// cannot make a wait of the compiler too weak: loads complete in order, so more outstanding loads
// than it counted only make its waits stricter than needed.
// rsrc: buffer descriptor words; lds: byte address of the destination of lane 0 (lane l lands at
// lds + l*size); voff: per-lane byte offset; soff: wave-uniform byte offset.
__device__ __forceinline__ v4i rsrc_words(const void *ptr, uint32_t bytes) {
  const uint64_t a = (uint64_t)ptr;
  return v4i{(int)(uint32_t)a, (int)((uint32_t)(a >> 32) & 0xffffu), (int)bytes, 0x00020000};
}
template <class P>
__device__ __forceinline__ uint32_t lds_addr(P *ptr) {
  return (uint32_t)(uintptr_t)CUMM_LDS_PTR(ptr);
}
__device__ __forceinline__ void dma_b128(v4i rsrc, uint32_t lds, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
__device__ __forceinline__ void dma_b32(v4i rsrc, uint32_t lds, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :: "s"(lds), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}

// The compiler's hazard recognizer does not look into asm statements.  A vector-memory instruction
// that reads a scalar register within four instructions of the vector instruction that wrote it
// (v_readlane restoring a spilled descriptor, v_readfirstlane, a compare into a register pair)
// gets the old value: a descriptor restored just before a hidden load made that load return
// zeros.  The register loads below therefore start with five wait states of their own; the
// direct-to-LDS loads above, which sit in the step loops, have two (s_mov m0 + s_nop 0) and are
// covered by the check of the generated code in cumm_amd/build.py (check_asm_hazards).
// A 4-byte buffer load into a register that the compiler does not see as a load: it cannot sink it
// into a branch (a plain load that feeds only a select is moved behind the select's condition and
// then waited for there, one round trip per conditional value).  To the compiler the result exists
// at once: the caller waits by hand (wait_vmcnt) and names the register in keep_after_wait() before
// the first use, which also keeps the register allocated while the load is in flight.
__device__ __forceinline__ int load_b32_hidden(v4i rsrc, uint32_t voff) {
  int r;
  asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2, 0 offen" : "=&v"(r) : "v"(voff), "s"(rsrc) : "memory");
  return r;
}
__device__ __forceinline__ void keep_after_wait(int &r) { asm volatile("" : "+v"(r)); }
// The same for 8 and 16 bytes.
typedef int v2i_hidden __attribute__((ext_vector_type(2)));
__device__ __forceinline__ v2i_hidden load_b64_hidden(v4i rsrc, uint32_t voff) {
  v2i_hidden r;
  asm volatile("s_nop 4\n\tbuffer_load_dwordx2 %0, %1, %2, 0 offen" : "=&v"(r) : "v"(voff), "s"(rsrc) : "memory");
  return r;
}
__device__ __forceinline__ v4i load_b128_hidden(v4i rsrc, uint32_t voff) {
  v4i r;
  asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, 0 offen" : "=&v"(r) : "v"(voff), "s"(rsrc) : "memory");
  return r;
}
__device__ __forceinline__ void keep_after_wait(v2i_hidden &r) { asm volatile("" : "+v"(r)); }
__device__ __forceinline__ void keep_after_wait(v4i &r) { asm volatile("" : "+v"(r)); }
template <int W>
__device__ __forceinline__ auto load_hidden_words(v4i rsrc, uint32_t voff) {
  static_assert(W == 2 || W == 4, "8 or 16 bytes");
  if constexpr (W == 2) return load_b64_hidden(rsrc, voff);
  else return load_b128_hidden(rsrc, voff);
}
// The same into a variable that already has a value (a conditional load: the variable keeps its
// value on the other path).  The register is read-write to the compiler, so both paths end in
// the same register and no copy - which would copy too early - is needed where they meet.
__device__ __forceinline__ void load_hidden_into(v2i_hidden &r, v4i rsrc, uint32_t voff) {
  asm volatile("s_nop 4\n\tbuffer_load_dwordx2 %0, %1, %2, 0 offen" : "+v"(r) : "v"(voff), "s"(rsrc) : "memory");
}
__device__ __forceinline__ void load_hidden_into(v4i &r, v4i rsrc, uint32_t voff) {
  asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, 0 offen" : "+v"(r) : "v"(voff), "s"(rsrc) : "memory");
}

// Workgroup barrier without the fence of __syncthreads(): the fence would wait for every
// outstanding direct-to-LDS load, i.e. also for the stages that are being prefetched.  The empty
// asm statements keep the compiler from moving LDS accesses across the barrier; the caller waits
// for the loads that the other waves are going to read before calling this.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

}  // namespace cummhip
