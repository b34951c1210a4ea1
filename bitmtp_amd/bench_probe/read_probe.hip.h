// Measurement aid, not part of the GEMV: kernels that read a buffer once from HBM with the
// launch shape of a GEMV and no arithmetic, so that a measured GEMV time can be put beside
// what the same bytes cost on the same machine when nothing but the loads happens.
//   * read_once_kernel<NL>: the shape of a layer-sized launch -- every thread requests its NL
//     16-byte units up front and the wave ends when they have arrived;
//   * read_stream_kernel: the shape of the kernels for very long matrices -- persistent
//     workgroups, two batches of four 16-byte loads per lane in flight.
// The loaded words are combined and compared with a constant so that the loads cannot be
// dropped; the store behind the comparison practically never executes.
#ifndef BONSAI_READ_PROBE_HIP_H
#define BONSAI_READ_PROBE_HIP_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace bonsai {

typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeThreads = 256;
constexpr unsigned kProbeMagic = 0x9e3779b9u;

// A wave reads NL consecutive kilobytes (lane l takes 16-byte unit l of each), as a GEMV wave
// reads consecutive weight rows.
template <int NL>
__global__ void __launch_bounds__(kProbeThreads)
read_once_kernel(const probe_u32x4 *__restrict__ src, long units, unsigned *sink) {
    const long wave = (long)blockIdx.x * (kProbeThreads / 64) + (threadIdx.x >> 6);
    const long i0 = wave * (NL * 64) + (threadIdx.x & 63);
    probe_u32x4 v[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        long i = i0 + j * 64;
        i = i < units ? i : units - 1;  // unconditional load, the tail re-reads the last unit
        v[j] = src[i];
    }
    probe_u32x4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < NL; ++j) acc ^= v[j];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == kProbeMagic) *sink = 1;
}

// Persistent: a wave walks 4 KB blocks with the stride of the launch, the next block requested
// before the current one is consumed.
__global__ void __launch_bounds__(kProbeThreads)
read_stream_kernel(const probe_u32x4 *__restrict__ src, long units, unsigned *sink) {
    const long waves = (long)gridDim.x * (kProbeThreads / 64);
    const long wave = (long)blockIdx.x * (kProbeThreads / 64) + (threadIdx.x >> 6);
    const long last = units - 1;
    const long step = waves * 256;
    long i = wave * 256 + (threadIdx.x & 63);
    probe_u32x4 cur[4], nxt[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const long k = i + j * 64;
        cur[j] = src[k < last ? k : last];
    }
    probe_u32x4 acc = {0, 0, 0, 0};
    for (i += step; i < units; i += step) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long k = i + j * 64;
            nxt[j] = src[k < last ? k : last];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc ^= cur[j];
            cur[j] = nxt[j];
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) acc ^= cur[j];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == kProbeMagic) *sink = 1;
}

// Returns 0, 1 for bad arguments (null or misaligned pointers, a one-shot launch that would
// need more than eight loads per thread), 2 on a launch error.
inline int launch_read_probe(const void *src, size_t bytes, int workgroups, int persistent,
                             void *sink, hipStream_t stream) {
    if (src == nullptr || sink == nullptr || bytes < 16 || workgroups < 1) return 1;
    if ((reinterpret_cast<uintptr_t>(src) & 15) != 0 || (reinterpret_cast<uintptr_t>(sink) & 3) != 0)
        return 1;
    const long units = (long)(bytes / 16);
    const probe_u32x4 *p = static_cast<const probe_u32x4 *>(src);
    unsigned *s = static_cast<unsigned *>(sink);
    const dim3 grid(workgroups, 1, 1), block(kProbeThreads, 1, 1);
    if (persistent != 0) {
        hipLaunchKernelGGL(read_stream_kernel, grid, block, 0, stream, p, units, s);
    } else {
        const long T = (long)workgroups * kProbeThreads;
        const long nl = (units + T - 1) / T;
        switch (nl) {
            case 1: hipLaunchKernelGGL(read_once_kernel<1>, grid, block, 0, stream, p, units, s); break;
            case 2: hipLaunchKernelGGL(read_once_kernel<2>, grid, block, 0, stream, p, units, s); break;
            case 3: hipLaunchKernelGGL(read_once_kernel<3>, grid, block, 0, stream, p, units, s); break;
            case 4: hipLaunchKernelGGL(read_once_kernel<4>, grid, block, 0, stream, p, units, s); break;
            case 5: hipLaunchKernelGGL(read_once_kernel<5>, grid, block, 0, stream, p, units, s); break;
            case 6: hipLaunchKernelGGL(read_once_kernel<6>, grid, block, 0, stream, p, units, s); break;
            case 7: hipLaunchKernelGGL(read_once_kernel<7>, grid, block, 0, stream, p, units, s); break;
            case 8: hipLaunchKernelGGL(read_once_kernel<8>, grid, block, 0, stream, p, units, s); break;
            default: return 1;
        }
    }
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

}  // namespace bonsai
#endif  // BONSAI_READ_PROBE_HIP_H
