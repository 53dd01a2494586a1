// Chains of dependent launches that overlap: launch j+1 of a chain is enqueued on another stream than launch j,
// starts while j is still running, requests what does not depend on j (its first weight blocks), and then waits
// inside the kernel until every workgroup of j has signalled.  What a kernel boundary would have done is done
// explicitly:
//   * the producer writes its outputs with agent-scope stores (served on the memory side of the XCDs' L2s), waits
//     until they are acknowledged, passes a workgroup barrier, and one thread bumps the launch's counter;
//   * the consumer's thread 0 polls that counter with agent-scope loads, a workgroup barrier releases the other
//     waves, and the rows the producer wrote are read with agent-scope loads, which miss in this XCD's L2.
// Counters are zero at rest.  Every consumer workgroup acknowledges on the producer's counter once it has seen
// it complete; the acknowledgement that brings it to producers + consumers resets it, so a captured chain can be
// replayed without any clearing launch in between (the last launch's own counter is cleared by whoever closes
// the chain).
// Every wait is bounded: after spin_limit polls (or as soon as the chain's status word is already set) the
// workgroup sets the status word and goes on with whatever is in memory, so that every kernel of a broken chain
// still exits; the host reads the status word at its next synchronisation and reports the failure.
// Launches of a chain may be co-resident two at a time (j and j+1; j+2 shares j's stream), so each must leave room
// for the other: at most half of a CU's waves, registers and LDS per workgroup pair, at most one workgroup per CU.
//
// Measured on MI355X (36 x 7 one-row linears of Qwen3-8B + lm_head, replayed from a HIP graph): the plain launches
// on one stream take 1.76 ms, the same launches as a chain 5.3 ms; the chained kernels on one stream (every wait
// satisfied at once) 3.2 ms; on two streams without waits and signals 1.41 ms.  The cost is the hand-over itself:
// operations on one line served on the memory side (the counter's atomics, the polls of 256 waiting workgroups) are
// served one at a time, about 25 ns each, so a launch of 256 workgroups pays 6 us and more for what a kernel
// boundary does in 3.  Flags per workgroup and values that carry their own tag (one store trip, one load trip, no
// counter) were measured too and lose for the same reason: 256 workgroups that each read the producer's row from
// the memory side, instead of once per L2, ask for every line 256 times (7.4 -> 10.4 us per link on a dependent
// chain of 4096-wide layers).  Chains are therefore an option for experiments, not the default path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace a81w41 {

struct ChainLink {
    unsigned* wait = nullptr;    // the counter of the launch this one depends on (null: nothing to wait for)
    unsigned wait_for = 0;       // workgroups of that launch
    unsigned* signal = nullptr;  // this launch's counter (null: nobody waits for it)
    unsigned* status = nullptr;  // set to 1 by a wait that gave up
    unsigned spin_limit = 0;     // polls before a wait gives up
};

#if defined(__HIPCC__)
template <typename T>
__device__ __forceinline__ T load_agent(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ void store_agent(T* p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes as two 8-byte agent-scope accesses (the widest the memory model offers)
__device__ __forceinline__ uint4 load16_agent_u4(const void* p) {
    const unsigned long long* q = static_cast<const unsigned long long*>(p);
    const unsigned long long a = load_agent(q), b = load_agent(q + 1);
    return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
}
__device__ __forceinline__ float4 load16_agent_f4(const void* p) {
    const uint4 u = load16_agent_u4(p);
    return make_float4(__uint_as_float(u.x), __uint_as_float(u.y), __uint_as_float(u.z), __uint_as_float(u.w));
}
__device__ __forceinline__ void store16_agent_f4(void* p, float4 v) {
    unsigned long long* q = static_cast<unsigned long long*>(p);
    store_agent(q, (unsigned long long)__float_as_uint(v.x) | ((unsigned long long)__float_as_uint(v.y) << 32));
    store_agent(q + 1, (unsigned long long)__float_as_uint(v.z) | ((unsigned long long)__float_as_uint(v.w) << 32));
}

// Called by every thread of the workgroup, after the loads that do not depend on the producer have been issued
// (they stay in flight: the barrier here does not wait for vector memory).  On return the producer's outputs may
// be read with agent-scope loads.
__device__ __forceinline__ void chain_wait(const ChainLink& c) {
    if (c.wait == nullptr) return;
    if (threadIdx.x == 0) {
        unsigned polls = 0;
        while (load_agent(c.wait) < c.wait_for) {
            if (++polls > c.spin_limit || load_agent(c.status) != 0u) {
                store_agent(c.status, 1u);
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // no load of the producer's rows is moved above the barrier
}

// Called by every thread of the workgroup after its last output store (all of them agent-scope stores).
// `consumers` = workgroups of this launch.
__device__ __forceinline__ void chain_signal(const ChainLink& c, unsigned consumers) {
    if (c.wait == nullptr && c.signal == nullptr) return;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
    __builtin_amdgcn_s_barrier();
    if (threadIdx.x == 0) {
        if (c.wait != nullptr) {
            // acknowledge on the producer's counter; whoever completes it resets it for the next replay
            const unsigned seen = __hip_atomic_fetch_add(c.wait, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (seen + 1u == c.wait_for + consumers) {
                store_agent(c.wait, 0u);
                __builtin_amdgcn_s_waitcnt(0);  // the reset lands before this launch reports itself complete
            }
        }
        if (c.signal != nullptr) __hip_atomic_fetch_add(c.signal, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
#endif

}  // namespace a81w41
