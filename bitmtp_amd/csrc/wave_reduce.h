// Whole-wave (64 lanes) reductions on the DPP network: six data-parallel moves instead of
// six LDS-crossbar permutes, result broadcast through a scalar register.
//
// Steps: quad_perm xor 1, quad_perm xor 2, row_half_mirror, row_mirror (after these every
// lane of a 16-lane row holds the row's result), row_bcast15 into rows 1 and 3, row_bcast31
// into rows 2 and 3; lane 63 then holds the wave's result.  Each step combines the same two
// partial results as the corresponding step of an xor butterfly with offsets 1, 2, 4, 8,
// 16, 32, so the value is bit-identical to that butterfly's (also for floating-point sums).
#ifndef BONSAI_WAVE_REDUCE_H
#define BONSAI_WAVE_REDUCE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bonsai_wave {

constexpr int kXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;  // lane i <-> 7-i inside each 8 lanes
constexpr int kMirror = 0x140;      // lane i <-> 15-i inside each 16 lanes
constexpr int kBcast15 = 0x142;     // lane 15 of each row -> the next row
constexpr int kBcast31 = 0x143;     // lane 31 -> rows 2 and 3

// value of the partner lane; lanes of rows outside ROW_MASK read their own value back
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float partner(float v) {
    const int x = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xF, false));
}

template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ double partner(double v) {
    const uint64_t b = (uint64_t)__double_as_longlong(v);
    const int lo = (int)(uint32_t)b, hi = (int)(uint32_t)(b >> 32);
    const uint32_t plo = (uint32_t)__builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xF, false);
    const uint32_t phi = (uint32_t)__builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xF, false);
    return __longlong_as_double((long long)(((uint64_t)phi << 32) | plo));
}

__device__ __forceinline__ float lane63(float v) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ double lane63(double v) {
    const uint64_t b = (uint64_t)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, 63);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), 63);
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}

// Rows outside the mask combine their value with itself: harmless for max, but a sum must
// not add it, so the masked steps of the sum select by lane instead.
__device__ __forceinline__ float max64(float v) {
    v = fmaxf(v, partner<kXor1>(v));
    v = fmaxf(v, partner<kXor2>(v));
    v = fmaxf(v, partner<kHalfMirror>(v));
    v = fmaxf(v, partner<kMirror>(v));
    v = fmaxf(v, partner<kBcast15, 0xA>(v));
    v = fmaxf(v, partner<kBcast31, 0xC>(v));
    return lane63(v);
}

// The same first four steps alone: every lane of a 16-lane row ends with its row's result.
__device__ __forceinline__ float max16(float v) {
    v = fmaxf(v, partner<kXor1>(v));
    v = fmaxf(v, partner<kXor2>(v));
    v = fmaxf(v, partner<kHalfMirror>(v));
    return fmaxf(v, partner<kMirror>(v));
}
__device__ __forceinline__ float sum16(float v) {
    v += partner<kXor1>(v);
    v += partner<kXor2>(v);
    v += partner<kHalfMirror>(v);
    return v + partner<kMirror>(v);
}

template <typename T>
__device__ __forceinline__ T sum64(T v) {
    const int lane = (int)(threadIdx.x & 63);
    v += partner<kXor1>(v);
    v += partner<kXor2>(v);
    v += partner<kHalfMirror>(v);
    v += partner<kMirror>(v);
    const T p15 = partner<kBcast15, 0xA>(v);
    if (lane & 16) v += p15;  // rows 1 and 3
    const T p31 = partner<kBcast31, 0xC>(v);
    if (lane & 32) v += p31;  // rows 2 and 3
    return lane63(v);
}

}  // namespace bonsai_wave
#endif  // BONSAI_WAVE_REDUCE_H
