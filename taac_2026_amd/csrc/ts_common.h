// Pieces shared by the token-stationary kernels (ffn.hip, fp8_ts.hip) and the attention kernels: direct global->LDS
// staging and hand-issued, hand-awaited LDS / global operations.
#pragma once

#include <type_traits>
#include <utility>

#include "common.h"

namespace taac {

// The low 32 bits of a generic pointer into LDS are the LDS byte offset.
__device__ __forceinline__ uint32_t lds_offset(const void* lds_ptr) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_ptr));
}

// 16 bytes per lane from global memory straight into LDS; lane l lands at lds_wave_base + 16 * l (lds_wave_base is
// wavefront-uniform). Issued by hand rather than through the compiler's builtin: the compiler models the builtin as
// a "flat" access and, while one is in flight, turns every wait it inserts into a wait for ALL outstanding memory
// operations (vmcnt(0) and lgkmcnt(0)), which would serialise the weight stream with the loads and stores around it.
// Consequences: the compiler does not know about these transfers at all, so (1) completion is awaited by hand with
// vm_wait<N>() - the operations of the vector-memory counter complete in issue order, N = number of vector-memory
// instructions this wavefront issued after the transfer, and a count that is too small only waits longer - and
// (2) the LDS bytes they write must only be read through the hand-issued lds_read_* below, after such a wait and a
// workgroup barrier.
__device__ __forceinline__ void lds_dma16(const void* gsrc, void* lds_wave_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_offset(lds_wave_base));
  asm volatile(
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, off"
      :
      : "v"(gsrc), "s"(base)
      : "memory", "m0");
}

// lds_dma16 with the source given as a wavefront-uniform base (scalar registers) + a 32-bit per-lane byte offset.
__device__ __forceinline__ void lds_dma16_offset(const void* base, uint32_t lane_offset, void* lds_wave_base) {
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(lds_offset(lds_wave_base));
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(lane_offset), "s"(base), "s"(lds_base)
      : "memory", "m0");
}

// Transposed 64-bit read: element e of lane j of a 16-lane group receives element j % 4 of the 8-byte row whose address
// lane 4 * e + j / 4 of that group supplies.
template <int OFFSET>
__device__ __forceinline__ void lds_read_tr16(u32x2& dst, uint32_t addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}

// Hand-issued LDS reads and hand-written waits: fragment reads run several MFMAs ahead of their use with exact
// lgkmcnt counts (LDS operations complete in issue order; a count that is too small only waits longer).
template <int OFFSET>
__device__ __forceinline__ void lds_read_frag(bf16x8& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}

// Waits until at most N of this wavefront's LDS operations are outstanding; the two fragments are tied to the wait so
// that their consumers cannot be scheduled above it.
template <int N>
__device__ __forceinline__ void lds_wait_pair(bf16x8& a, bf16x8& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

template <int N>
__device__ __forceinline__ void vm_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int OFFSET>
__device__ __forceinline__ void lds_read_u16(uint32_t& dst, uint32_t addr) {
  asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}

// Same for a single fragment, optionally tying one more value (read earlier than the fragment) to the wait.
template <int N>
__device__ __forceinline__ void lds_wait_frag(bf16x8& a) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_frag(bf16x8& a, uint32_t& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

// Calls f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}) in order.
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// Copies n bf16 values (or zeros when src is null) into LDS with the whole workgroup; n is a multiple of 8.
__device__ __forceinline__ void stage_bias(const bf16_t* src, bf16_t* dst, int n, int tid, int nthreads) {
  for (int i = tid * 8; i < n; i += nthreads * 8) {
    bf16x8 v;
    if (src != nullptr) {
      v = *reinterpret_cast<const bf16x8*>(src + i);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(0.f);
    }
    *reinterpret_cast<bf16x8*>(dst + i) = v;
  }
}

}  // namespace taac
