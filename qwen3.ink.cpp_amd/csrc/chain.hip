// Host side of a chain of overlapping launches (chain.h): two streams that take the launches in turn, the ring of
// completion counters, and the status word a wait that gave up sets.
#include "a81w41_kernels.h"

namespace a81w41 {
namespace {

__global__ void chain_clear_kernel(unsigned* __restrict__ counter) {
    if (threadIdx.x == 0 && blockIdx.x == 0) store_agent(counter, 0u);
}

}  // namespace

hipError_t chain_create(ChainState* st) {
    *st = ChainState{};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&st->cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess && st->cus < 1) e = hipErrorInvalidDevice;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&st->counters), (kChainRing + 1) * sizeof(unsigned));
    if (e == hipSuccess) e = hipMemset(st->counters, 0, (kChainRing + 1) * sizeof(unsigned));
    // default priority: streams of different priorities must not wait for each other's kernels
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&st->side, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&st->fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&st->join, hipEventDisableTiming);
    if (e != hipSuccess) chain_destroy(st);
    return e;
}

void chain_destroy(ChainState* st) {
    if (st->side) {
        (void)hipStreamSynchronize(st->side);
        (void)hipStreamDestroy(st->side);
    }
    if (st->fork) (void)hipEventDestroy(st->fork);
    if (st->join) (void)hipEventDestroy(st->join);
    (void)hipFree(st->counters);
    *st = ChainState{};
}

hipError_t chain_begin(ChainState* st, hipStream_t main) {
    if (st->open) return hipErrorInvalidValue;
    hipError_t e = hipEventRecord(st->fork, main);
    if (e == hipSuccess) e = hipStreamWaitEvent(st->side, st->fork, 0);
    if (e != hipSuccess) return e;
    st->main = main;
    st->open = true;
    st->n = 0;
    st->prev_grid = 0;
    return hipSuccess;
}

ChainLink chain_next(const ChainState* st, hipStream_t* stream) {
    ChainLink link;
    if (st->n > 0) {
        link.wait = st->counters + (st->n - 1) % kChainRing;
        link.wait_for = st->prev_grid;
    }
    link.signal = st->counters + st->n % kChainRing;
    link.status = st->counters + kChainRing;
    link.spin_limit = st->spin_limit;
    *stream = (st->n & 1) ? st->side : st->main;
    return link;
}

void chain_launched(ChainState* st, unsigned grid) {
    st->prev_grid = grid;
    st->n++;
}

hipError_t chain_end(ChainState* st) {
    if (!st->open) return hipErrorInvalidValue;
    st->open = false;
    hipError_t e = hipEventRecord(st->join, st->side);
    if (e == hipSuccess) e = hipStreamWaitEvent(st->main, st->join, 0);
    if (e != hipSuccess) return e;
    if (st->n > 0) {  // nobody waited for the last launch: its counter is still up
        hipLaunchKernelGGL(chain_clear_kernel, dim3(1), dim3(64), 0, st->main, st->counters + (st->n - 1) % kChainRing);
        e = hipGetLastError();
    }
    return e;
}

hipError_t chain_status(ChainState* st, bool* gave_up) {
    if (st->open) return hipErrorInvalidValue;
    hipError_t e = hipStreamSynchronize(st->side);
    if (e == hipSuccess && st->main) e = hipStreamSynchronize(st->main);
    unsigned word = 0;
    if (e == hipSuccess) e = hipMemcpy(&word, st->counters + kChainRing, sizeof(word), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return e;
    *gave_up = word != 0;
    // a chain whose wait gave up leaves counters behind: start from zero again
    if (word != 0) e = hipMemset(st->counters, 0, (kChainRing + 1) * sizeof(unsigned));
    return e;
}

}  // namespace a81w41
