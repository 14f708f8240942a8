// Buffer-addressed loads, asynchronous global -> LDS copies and the waits that go with them (gfx950).
#pragma once
#include "kmoe_common.h"

namespace kmoe {

typedef int v4i_raw __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over [base, base + 4 GiB): loads take a 32-bit per-lane offset
// plus a scalar offset, so no 64-bit address arithmetic sits in the MFMA loop.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
__device__ inline v4i_raw buffer_load16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t wave_off) {
  return (v4i_raw)__builtin_amdgcn_raw_buffer_load_b128(r, lane_off, wave_off, 0);
}

// Asynchronous copy global -> LDS, 16 bytes per lane: lane l's bytes land at lds + 16 l (the
// destination is one contiguous KB per instruction; which global bytes a lane fetches is free).
// No register holds the data; the wave's VMEM counter covers completion.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
__device__ inline void buffer_load16_to_lds(__amdgpu_buffer_rsrc_t r, lds_ptr_t lds, uint32_t lane_off,
                                            uint32_t wave_off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, lds, 16, lane_off, wave_off, 0, 0);
}
// LDS reads the compiler does not see: it would otherwise drain every asynchronous copy in
// flight before each of them. OFF: immediate byte offset. The wait that makes the value usable
// is lds_wait<N> on the same variable (LDS operations of a wave complete in order).
template <int OFF>
__device__ inline v4i_raw lds_read16_raw(uint32_t addr) {
  v4i_raw v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
  return v;
}
template <int N>
__device__ inline void lds_wait(v4i_raw& v) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(N));
}
// s_waitcnt with only the vector-memory counter set: at most N loads of this wave in flight
template <int N>
__device__ inline void vmem_wait() {
  static_assert(N >= 0 && N < 64, "6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}


}  // namespace kmoe
