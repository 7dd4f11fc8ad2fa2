// Loads that go from global memory straight into LDS (buffer_load ... lds) and the barrier that
// goes with them, shared by the kernels that stage their operands this way.
#pragma once
#include "ahl_device.h"

namespace ahl {

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// s_waitcnt immediate (gfx9 encoding): vmcnt(n), lgkmcnt(0), expcnt unconstrained
static constexpr int vm_wait(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0070; }

// Workgroup barrier that orders LDS accesses and waits until at most `flying` of this wave's
// vector memory operations are outstanding. __syncthreads() would wait for all of them, i.e.
// drain the direct-to-LDS loads of the chunks ahead at every barrier.
template <int FLYING>
AHL_DEV void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(vm_wait(FLYING));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// 16 bytes per lane from global memory straight into LDS: lane L's data lands at lds_base + 16 L
// (a device-only wrapper: the builtin inside a kernel body keeps the host pass from emitting the
// kernel's launch stub)
AHL_DEV void load_to_lds16(__amdgpu_buffer_rsrc_t rsrc, char* lds_base, int voffset, int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)lds_base, 16, voffset, soffset, 0, 0);
}

// Buffer descriptor over `bytes` bytes from `base` (raw addressing; reads beyond return zero).
AHL_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint64_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0,
                                           (int)(bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes),
                                           0x00020000);
}

}  // namespace ahl
