// Global -> LDS loader primitives shared by every LDS-staged kernel of this library (gfx950 only).
//
// One direct-to-LDS load (`dma16`): every lane fetches 16 bytes at rsrc.base + voff + soff and the hardware writes them
// at LDS address lds_base + 16 * lane, so an LDS image is produced by choosing which global bytes each lane fetches
// (the idea of the reference's swizzled global offsets, include/ops/warp/memory/tile/global_to_shared.cuh:46-72).  The
// loads are issued from inline assembly so that the VMEM counter is managed by hand (`wait_vmcnt<N>`): the kernels keep
// several batches in flight across barriers and loop back-edges, which the compiler's own waits would drain.  No load
// issued through here has a register destination, so nothing can read a register before its load has landed.  M0 is
// used by nothing else in these kernels.
#pragma once
#include "common.hpp"

namespace mxfp6 {

__device__ __forceinline__ void dma16(const __amdgpu_buffer_rsrc_t& rsrc, uint32_t lds_base, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}
// at most N of this wave's loads (and stores) may still be in flight; they retire in order
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// every LDS read (and LDS atomic) of this wave has returned
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// workgroup barrier the compiler schedules nothing across
__device__ __forceinline__ void barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
// make_rsrc for a base and a length that are the same in every lane but that the compiler cannot prove so (inside a branch on
// the wave's number, say): the resource must live in scalar registers
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc_uniform(const void* base, uint32_t bytes) {
  const uint64_t b = (uint64_t)(uintptr_t)base;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  return make_rsrc(reinterpret_cast<const void*>((uintptr_t)((uint64_t)hi << 32 | lo)), __builtin_amdgcn_readfirstlane(bytes));
}
// LDS address (as the hardware counts it) of a __shared__ object
__device__ __forceinline__ uint32_t lds_address(const void* p) { return (uint32_t)(uintptr_t)(const MXFP6_LDS uint8_t*)p; }

// Flags in LDS for waves of one workgroup that hand each other ring slots without a workgroup-wide barrier
// (the reference's ready / done counters, kernels/gemm/bf16fp32/micros/producer_consumer/32x16/micro_09_async.cpp:129-186).
// All lanes of the calling wave see the same value.
__device__ __forceinline__ int lds_flag_load(uint32_t addr) {
  int v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return __builtin_amdgcn_readfirstlane(v);
}
// one lane stores / adds; LDS operations of a wave execute in order, so whatever the wave read or waited for before is done
__device__ __forceinline__ void lds_flag_store(uint32_t addr, int value) {
  if ((threadIdx.x & 63) == 0) asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(value) : "memory");
}
__device__ __forceinline__ void lds_flag_add(uint32_t addr, int value) {
  if ((threadIdx.x & 63) == 0) asm volatile("ds_add_u32 %0, %1" ::"v"(addr), "v"(value) : "memory");
}

}  // namespace mxfp6
