// 16-byte accesses at agent scope and vector-memory waits, shared by the kernels that hand partial results from
// one workgroup to another.  Stores and loads at agent scope are served on the memory side of the XCDs' L2s,
// where every CU of the device sees them; a load's result may be used only after wait_vmcnt<0>().
#pragma once
#include <hip/hip_runtime.h>

namespace a81w41 {

typedef float v4f __attribute__((ext_vector_type(4)));

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0070);  // and lgkmcnt = 0
}
__device__ __forceinline__ void store16_agent(float* p, v4f v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ v4f load16_agent(const float* p) {
    v4f v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}

}  // namespace a81w41
