// Per-lane arithmetic of the packed low-bit GEMV kernels.
//
// Everything here is plain integer code that compiles both as gfx950 device
// code (included by packed_gemv.hip.h) and as host C++ (included by the lane
// simulator under tests/host_sim/, which replays the exact staging layout and
// unpack/dot sequence on the CPU so that index mistakes are found without a GPU).
//
// Work decomposition.  A weight row is cut into 16-byte CHUNKS (one
// global_load_dwordx4 per lane): 64 weights for T2 (half a scale group), 128
// for Q1 (one scale group).  A packed dword p is turned into byte vectors with
// the cheapest possible sequence,
//     T2:  u_j = (p >> 2j) & 0x03030303   j = 0..3   byte b of u_j = code of weight 4b + j
//     Q1:  u_j = (p >>  j) & 0x01010101   j = 0..7   byte b of u_j = bit  of weight 8b + j
// i.e. the codes/bits are used as they are (0..3 / 0..1) and in an interleaved
// K order.  Both departures from the natural layout are paid for once per
// token, when the activations are staged:
//   * the activations are stored pre-permuted, so that dword j of an activation
//     unit lines up with u_j (a 4x4 byte transpose of the natural order), and
//   * the code offset is removed with the per-chunk activation sum:
//         T2:  sum a*(code-2)  = sum a*code - 2*asum
//         Q1:  sum a*(2*bit-1) = 2*sum a*bit - asum
// An integer dot product does not depend on the order of its terms, so the
// int32 group sums stay exact.
//
// Reference arithmetic being reproduced:
//   src/bonsai_sft/gpu/t2g128_kernels/t2g128_kernels.cu:21-27,62-81
//   src/bonsai_sft/gpu/q1g128_kernels/q1g128_kernels.h:47-68,388-410
#ifndef BONSAI_GEMV_CORE_H
#define BONSAI_GEMV_CORE_H

#include <stdint.h>

#if defined(__HIP_DEVICE_COMPILE__) || defined(__HIPCC__)
#define BONSAI_HD __host__ __device__ __forceinline__
#else
#define BONSAI_HD inline
#endif

namespace bonsai {

struct alignas(16) u32x4 {
    uint32_t x, y, z, w;
};

// Signed 4 x int8 dot product with int32 accumulate (v_dot4_i32_i8 on gfx950).
BONSAI_HD int dot4_i8(uint32_t a, uint32_t b, int acc) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_sdot4((int)a, (int)b, acc, false);
#else
    for (int i = 0; i < 4; ++i)
        acc += (int)(int8_t)(a >> (8 * i)) * (int)(int8_t)(b >> (8 * i));
    return acc;
#endif
}

template <int BITS>
struct Fmt;

template <>
struct Fmt<2> {
    static constexpr int kChunkWeights = 64;  // weights in one 16-byte chunk
    static constexpr int kUnits = 4;          // 16-byte activation units per chunk
    static constexpr int kUnitsPerDword = 1;  // activation units consumed per packed dword
    static constexpr int kVecPerDword = 4;    // byte vectors unpacked from one packed dword
    static constexpr int kGroupShift = 1;     // scale group = chunk >> kGroupShift
};

template <>
struct Fmt<1> {
    static constexpr int kChunkWeights = 128;
    static constexpr int kUnits = 8;
    static constexpr int kUnitsPerDword = 2;
    static constexpr int kVecPerDword = 8;
    static constexpr int kGroupShift = 0;
};

// out[d].byte[b] = in[b].byte[d]  (eight v_perm_b32 on the GPU)
BONSAI_HD u32x4 transpose4x4_bytes(uint32_t i0, uint32_t i1, uint32_t i2, uint32_t i3) {
    u32x4 o;
#if defined(__HIP_DEVICE_COMPILE__)
    // perm(hi, lo, sel): selector byte 0..3 picks a byte of lo, 4..7 a byte of hi
    const uint32_t l01 = __builtin_amdgcn_perm(i1, i0, 0x05010400u);  // i0.b0 i1.b0 i0.b1 i1.b1
    const uint32_t h01 = __builtin_amdgcn_perm(i1, i0, 0x07030602u);  // i0.b2 i1.b2 i0.b3 i1.b3
    const uint32_t l23 = __builtin_amdgcn_perm(i3, i2, 0x05010400u);
    const uint32_t h23 = __builtin_amdgcn_perm(i3, i2, 0x07030602u);
    o.x = __builtin_amdgcn_perm(l23, l01, 0x05040100u);
    o.y = __builtin_amdgcn_perm(l23, l01, 0x07060302u);
    o.z = __builtin_amdgcn_perm(h23, h01, 0x05040100u);
    o.w = __builtin_amdgcn_perm(h23, h01, 0x07060302u);
#else
    o.x = (i0 & 0xffu) | ((i1 & 0xffu) << 8) | ((i2 & 0xffu) << 16) | ((i3 & 0xffu) << 24);
    o.y = ((i0 >> 8) & 0xffu) | (((i1 >> 8) & 0xffu) << 8) | (((i2 >> 8) & 0xffu) << 16) |
          (((i3 >> 8) & 0xffu) << 24);
    o.z = ((i0 >> 16) & 0xffu) | (((i1 >> 16) & 0xffu) << 8) | (((i2 >> 16) & 0xffu) << 16) |
          (((i3 >> 16) & 0xffu) << 24);
    o.w = (i0 >> 24) | ((i1 >> 24) << 8) | ((i2 >> 24) << 16) | ((i3 >> 24) << 24);
#endif
    return o;
}

BONSAI_HD int sum4_i8(uint32_t a) { return dot4_i8(a, 0x01010101u, 0); }

// Staged-activation layout (LDS on the GPU).  Everything one weight chunk needs
// lives in one BLOCK of `block_words<BITS, MT>()` 16-byte words:
//     words [m*kUnits + unit]      permuted activation unit `unit` of tile token m
//     words [MT*kUnits ...]        MT int32 chunk activation sums (asum), then padding
// so that a lane addresses all of it with one base register and immediate
// offsets.  The block size is odd: lanes holding consecutive chunks then hit
// distinct 16-byte bank groups, whatever MT is.
template <int BITS, int MT>
BONSAI_HD constexpr int block_words() {
    return ((MT * Fmt<BITS>::kUnits + (MT * 4 + 15) / 16) | 1);
}

template <int BITS, int MT>
BONSAI_HD int act_index(int m, int unit, int chunk) {
    return chunk * block_words<BITS, MT>() + m * Fmt<BITS>::kUnits + unit;
}

// Index (in int32 units) of the activation sum of token m for `chunk`.
template <int BITS, int MT>
BONSAI_HD int asum_index(int m, int chunk) {
    return (chunk * block_words<BITS, MT>() + MT * Fmt<BITS>::kUnits) * 4 + m;
}

// Stage one quarter (`sub` = 0..3) of one chunk of one token.  `src` points at the
// quarter's natural-order int8 activations (16 for T2, 32 for Q1; 16-byte
// aligned).  Writes the permuted unit(s) into act[] and returns the sum of the
// quarter's activations; the four quarter sums of a chunk add up to its asum.
template <int BITS, int MT>
BONSAI_HD int stage_quarter(const u32x4 *src, u32x4 *act, int m, int chunk, int sub) {
    if (BITS == 2) {
        const u32x4 in = src[0];  // activations 16*sub .. 16*sub+15 of the chunk
        // unit sub, dword j, byte b  <-  activation 16*sub + 4b + j
        act[act_index<BITS, MT>(m, sub, chunk)] =
            transpose4x4_bytes(in.x, in.y, in.z, in.w);
        return sum4_i8(in.x) + sum4_i8(in.y) + sum4_i8(in.z) + sum4_i8(in.w);
    } else {
        const u32x4 lo = src[0], hi = src[1];  // activations 32*sub .. 32*sub+31
        // unit 2*sub+h, dword d, byte b  <-  activation 32*sub + 8b + 4h + d
        act[act_index<BITS, MT>(m, 2 * sub, chunk)] =
            transpose4x4_bytes(lo.x, lo.z, hi.x, hi.z);
        act[act_index<BITS, MT>(m, 2 * sub + 1, chunk)] =
            transpose4x4_bytes(lo.y, lo.w, hi.y, hi.w);
        return sum4_i8(lo.x) + sum4_i8(lo.y) + sum4_i8(lo.z) + sum4_i8(lo.w) +
               sum4_i8(hi.x) + sum4_i8(hi.y) + sum4_i8(hi.z) + sum4_i8(hi.w);
    }
}

// Stage a whole chunk (the four quarters in turn); returns the chunk's asum.
template <int BITS, int MT>
BONSAI_HD int stage_chunk(const u32x4 *src, u32x4 *act, int m, int chunk) {
    int sum = 0;
    for (int sub = 0; sub < 4; ++sub)
        sum += stage_quarter<BITS, MT>(src + sub * (Fmt<BITS>::kUnits / 4), act, m, chunk, sub);
    return sum;
}

// Raw dot products of one 16-byte weight chunk against MT staged tokens:
// raw[m] += sum_k a[m][k] * code[k] (codes 0..3 for T2, bits 0..1 for Q1).
template <int BITS, int MT>
BONSAI_HD void chunk_dot_raw(const u32x4 w, const u32x4 *act, int chunk, int raw[MT]) {
    const uint32_t p[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (BITS == 2) {
            const uint32_t u0 = p[t] & 0x03030303u;
            const uint32_t u1 = (p[t] >> 2) & 0x03030303u;
            const uint32_t u2 = (p[t] >> 4) & 0x03030303u;
            const uint32_t u3 = (p[t] >> 6) & 0x03030303u;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const u32x4 a = act[act_index<BITS, MT>(m, t, chunk)];
                int r = raw[m];
                r = dot4_i8(a.x, u0, r);
                r = dot4_i8(a.y, u1, r);
                r = dot4_i8(a.z, u2, r);
                r = dot4_i8(a.w, u3, r);
                raw[m] = r;
            }
        } else {
            uint32_t u[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) u[j] = (p[t] >> j) & 0x01010101u;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const u32x4 a0 = act[act_index<BITS, MT>(m, 2 * t, chunk)];
                const u32x4 a1 = act[act_index<BITS, MT>(m, 2 * t + 1, chunk)];
                int r = raw[m];
                r = dot4_i8(a0.x, u[0], r);
                r = dot4_i8(a0.y, u[1], r);
                r = dot4_i8(a0.z, u[2], r);
                r = dot4_i8(a0.w, u[3], r);
                r = dot4_i8(a1.x, u[4], r);
                r = dot4_i8(a1.y, u[5], r);
                r = dot4_i8(a1.z, u[6], r);
                r = dot4_i8(a1.w, u[7], r);
                raw[m] = r;
            }
        }
    }
}

// Exact signed dot product of the chunk from the raw code dot and the chunk's
// activation sum.
template <int BITS>
BONSAI_HD int chunk_dot_signed(int raw, int asum) {
    return BITS == 2 ? raw - 2 * asum : 2 * raw - asum;
}

// ---------------------------------------------------------------------------
// Matrix-core (MFMA) path: operand slots
// ---------------------------------------------------------------------------
// v_mfma_i32_16x16x64_i8 contracts 64 K-slots per instruction.  Lane l supplies,
// for matrix row/column l % 16, the 16 slots of K-block kb = l / 16 as four
// registers of four bytes, and slot (kb, reg, byte) of one operand meets the
// same slot of the other.  A 128-weight scale group is two MFMAs (t = 0, 1)
// into one accumulator.  Lane kb owns weights 32*kb .. 32*kb+31 of the group:
//   T2: packed dwords 2kb and 2kb+1 of the group's eight; MFMA t takes dword
//       2kb+t unpacked as u_j = (p >> 2j) & 0x03030303:
//           slot (reg j, byte b) = weight 32kb + 16t + 4b + j
//   Q1: packed dword kb of the group's four; u_j = 2 * ((p >> j) & 0x01010101),
//       i.e. bytes 0 / 2 for weights -1 / +1, and MFMA t takes u_{4t} .. u_{4t+3}:
//           slot (reg j, byte b) = weight 32kb + 8b + 4t + j
// In both formats the activation operand for (kb, t) is staged unit 2kb+t of
// the group, holding the activations of those weights in (reg, byte) order --
// the same 4x4 byte transposes the dot4 path stages.  The code offset is
// removed through the accumulator input of the first MFMA:
//     T2: sum a*(code-2)   = sum a*code    + (-2 * asum)
//     Q1: sum a*(2*bit-1)  = sum a*(2*bit) + (-asum)
// so the MFMA result IS the exact group sum.
template <int BITS>
BONSAI_HD void mfma_unpack(uint32_t p0, uint32_t p1, uint32_t b0[4], uint32_t b1[4]) {
    if (BITS == 2) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            b0[j] = (p0 >> (2 * j)) & 0x03030303u;
            b1[j] = (p1 >> (2 * j)) & 0x03030303u;
        }
    } else {
        b0[0] = (p0 << 1) & 0x02020202u;
#pragma unroll
        for (int j = 1; j < 4; ++j) b0[j] = (p0 >> (j - 1)) & 0x02020202u;
#pragma unroll
        for (int j = 0; j < 4; ++j) b1[j] = (p0 >> (3 + j)) & 0x02020202u;
    }
}

// Staged activations of the MFMA path: token-major, one 16-byte unit per (group,
// kb, t) in natural K order, each token padded by one unit so that the sixteen
// tokens a ds_read_b128 touches fall into distinct bank groups.
BONSAI_HD int mfma_token_words(int K) { return K / 16 + 1; }

// Natural-order activations per staging quarter: 16 (T2) or 32 (Q1).
template <int BITS>
BONSAI_HD constexpr int mfma_quarter_bytes() { return BITS == 2 ? 16 : 32; }

// Stage quarter q of one token (src = the quarter's natural-order activations);
// returns the sum of its activations.
template <int BITS>
BONSAI_HD int mfma_stage_quarter(const u32x4 *src, u32x4 *act_token, int q) {
    if (BITS == 2) {
        const u32x4 in = src[0];
        act_token[q] = transpose4x4_bytes(in.x, in.y, in.z, in.w);
        return sum4_i8(in.x) + sum4_i8(in.y) + sum4_i8(in.z) + sum4_i8(in.w);
    } else {
        const u32x4 lo = src[0], hi = src[1];
        act_token[2 * q] = transpose4x4_bytes(lo.x, lo.z, hi.x, hi.z);
        act_token[2 * q + 1] = transpose4x4_bytes(lo.y, lo.w, hi.y, hi.w);
        return sum4_i8(lo.x) + sum4_i8(lo.y) + sum4_i8(lo.z) + sum4_i8(lo.w) +
               sum4_i8(hi.x) + sum4_i8(hi.y) + sum4_i8(hi.z) + sum4_i8(hi.w);
    }
}

// Offset-removal term per (group, token), fed to the first MFMA as accumulator input.
template <int BITS>
BONSAI_HD int mfma_corr(int group_asum) { return BITS == 2 ? -2 * group_asum : -group_asum; }

}  // namespace bonsai
#endif  // BONSAI_GEMV_CORE_H
