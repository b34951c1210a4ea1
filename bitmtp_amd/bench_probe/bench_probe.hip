// libbonsai_probe.so: measurement aids for the benchmarks, kept apart from the drop-in
// libraries.  Nothing here computes anything of the GEMV; each probe isolates one cost of the
// machine so that a measured kernel time can be put beside it:
//   * bonsai_read_probe            the bytes of a launch read once with no arithmetic
//   * bonsai_probe_empty_launches  launches of a kernel that does nothing (cost of a launch)
//   * bonsai_probe_chain_launches  launches that each consume what the previous one wrote
//                                  (cost of a dependent launch)
//   * bonsai_probe_grid_barrier    a device-wide barrier among resident workgroups through one
//                                  counter (what a hand-over inside a persistent kernel costs);
//                                  the wait is bounded, so every wave exits whatever happens
// Declared in include/bonsai_probe.h.  No reference counterpart.
#include <hip/hip_runtime.h>

#include "read_probe.hip.h"

#include "../../include/bonsai_probe.h"

namespace {

__global__ void __launch_bounds__(1024) probe_empty_kernel(unsigned *sink, int never) {
    if (never != 0 && threadIdx.x == 0 && blockIdx.x == 0) *sink = 1;
}

// One link of a dependent chain: a single lane reads the word the previous launch wrote and
// writes its successor.
__global__ void __launch_bounds__(64) probe_chain_kernel(unsigned *word) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *word = *word + 1u;
}

constexpr unsigned kBarrierSpinLimit = 200000;  // polls per barrier before a workgroup gives up

// state[0] = arrival counter (zero at launch), state[1] = error flags (1: a wait ran into the
// spin limit, so the barrier did not complete and the kernel left early).
__global__ void __launch_bounds__(256) probe_barrier_kernel(unsigned *state, int barriers) {
    const unsigned n = gridDim.x;
    __shared__ unsigned s_bad;
    if (threadIdx.x == 0) s_bad = 0;
    for (int i = 0; i < barriers; ++i) {
        __syncthreads();
        if (threadIdx.x == 0) {
            __hip_atomic_fetch_add(&state[0], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned target = (unsigned)(i + 1) * n;
            unsigned spins = 0;
            while (__hip_atomic_load(&state[0], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) {
                if (++spins > kBarrierSpinLimit) {
                    s_bad = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        if (s_bad) break;  // every thread of the workgroup leaves together
    }
    if (s_bad && threadIdx.x == 0) atomicOr(&state[1], 1u);
}

// "Last arriver finishes": every workgroup writes a record of `words` 32-bit words (at most 64), makes it visible to the
// device and bumps an arrival counter; the workgroup that arrives last reads all records (what a
// fused consumer stage would do), writes one result word and resets the counter.  Nobody waits.
// mode 0: producers only (records written, no counter); mode 1: with the arrival counter and
// the finishing stage; mode 2: the finishing stage alone, as the separate launch it would replace.
__global__ void __launch_bounds__(256) probe_last_arriver_kernel(unsigned *records, unsigned *state,
                                                               int n_records, int words, int mode) {
    const unsigned wg = blockIdx.x;
    __shared__ unsigned s_last;
    if (mode != 2) {
        if ((int)threadIdx.x < words) records[wg * words + threadIdx.x] = wg + threadIdx.x;
        if (mode == 0) return;
        __syncthreads();
        if (threadIdx.x == 0) {
            __threadfence();  // the records of this workgroup before its arrival
            const unsigned old = __hip_atomic_fetch_add(&state[0], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            s_last = old == gridDim.x - 1 ? 1u : 0u;
        }
        __syncthreads();
        if (!s_last) return;
        __threadfence();
    }
    unsigned acc = 0;
    for (int i = threadIdx.x; i < n_records * words; i += 256)
        acc += records[i];  // ordinary loads: the fence above (mode 1) or the kernel boundary orders them
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    if ((threadIdx.x & 63) == 0) atomicAdd(&state[1], acc);  // one result word per wave
    if (threadIdx.x == 0 && mode == 1) __hip_atomic_store(&state[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

extern "C" {

int bonsai_probe_last_arriver(int launches, int workgroups, int words, int mode, void *records,
                              void *state, void *stream) {
    if (launches < 1 || workgroups < 1 || workgroups > 65536 || words < 1 || words > 64 || mode < 0 ||
        mode > 2 || records == nullptr || state == nullptr)
        return 1;
    for (int i = 0; i < launches; ++i)
        hipLaunchKernelGGL(probe_last_arriver_kernel, dim3(mode == 2 ? 1 : workgroups), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<unsigned *>(records),
                           static_cast<unsigned *>(state), workgroups, words, mode);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

int bonsai_read_probe(const void *src, size_t bytes, int workgroups, int persistent, void *sink,
                      void *stream) {
    return bonsai::launch_read_probe(src, bytes, workgroups, persistent, sink,
                                     static_cast<hipStream_t>(stream));
}

int bonsai_probe_empty_launches(int launches, int workgroups, int threads, int lds_bytes, void *sink,
                                void *stream) {
    if (launches < 1 || workgroups < 1 || threads < 64 || threads > 1024 || threads % 64 != 0 ||
        lds_bytes < 0 || lds_bytes > 65536 || sink == nullptr)
        return 1;
    for (int i = 0; i < launches; ++i)
        hipLaunchKernelGGL(probe_empty_kernel, dim3(workgroups), dim3(threads), lds_bytes,
                           static_cast<hipStream_t>(stream), static_cast<unsigned *>(sink), 0);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

int bonsai_probe_chain_launches(int launches, void *word, void *stream) {
    if (launches < 1 || word == nullptr || (reinterpret_cast<uintptr_t>(word) & 3) != 0) return 1;
    for (int i = 0; i < launches; ++i)
        hipLaunchKernelGGL(probe_chain_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                           static_cast<unsigned *>(word));
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

int bonsai_probe_grid_barrier(int workgroups, int barriers, void *state, void *stream) {
    if (workgroups < 1 || barriers < 1 || barriers > 1000 || state == nullptr ||
        (reinterpret_cast<uintptr_t>(state) & 3) != 0)
        return 1;
    // every workgroup must be resident at once, or the early ones wait for workgroups that
    // cannot start: at most four 256-thread workgroups per CU are asked for
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return 2;
    if (workgroups > 4 * cus) return 1;
    hipLaunchKernelGGL(probe_barrier_kernel, dim3(workgroups), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<unsigned *>(state), barriers);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // extern "C"
