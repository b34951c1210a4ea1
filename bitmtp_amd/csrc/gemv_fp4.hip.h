// FP4 x FP8 matrix-core kernel of the packed low-bit GEMV (gfx950 only).
//
// gfx950's v_mfma_f32_16x16x128_f8f6f4 takes FP4 (E2M1) operands whose codes
// 0..3 are 0, 0.5, 1.0, 1.5: a 2-bit T2 code or a Q1 bit placed in a nibble IS
// half its value, so the weights need no arithmetic unpack, only nibble masks --
// 6 (T2) / 7 (Q1) VALU operations per 16 rows x 128 weights instead of 14 / 15
// byte-vector operations for the int8 MFMA.  The int8 activations are staged as
// two exact FP8 (E4M3) planes, 16*(a >> 4) and a & 15; two MFMAs per group
// accumulate 0.5 * sum a*code exactly in fp32, the accumulator input removes the
// code offset, and the result D' = G/2 (T2) or G/4 (Q1) of the exact group sum G
// goes straight into the fp32 scale-accumulate (4 FMAs, no int->float convert):
//     acc[token][row] += D' * ws[row][group];   y = (F * acc) / s,  F = 2 or 4.
// F is a power of two, so F*acc is exactly what accumulating fp32(G)*ws gives.
//
// Data movement is that of the int8 MFMA kernel (gemv_mfma.hip.h): coalesced
// 16-byte weight loads parked in a wave-private LDS tile and read back in operand
// order, R 16-row tiles per wave, optional K split among the waves of a
// workgroup, optional row-block passes.  The staged activations take 2*K bytes
// per token, which bounds the token tile for long K.
#ifndef BONSAI_GEMV_FP4_HIP_H
#define BONSAI_GEMV_FP4_HIP_H

#include "gemv_mfma.hip.h"

namespace bonsai {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Bytes of one staged token: two 128-byte planes per group plus one 16-byte pad
// (odd pitch in 16-byte words: the tokens a ds_read_b128 touches hit distinct banks).
__host__ __device__ inline int fp4_token_bytes(int K) { return 2 * K + 16; }

template <int BITS, int R>
__host__ __device__ inline size_t fp4_lds_bytes(int mt, int K) {
    const size_t act = (size_t)mt * fp4_token_bytes(K);
    const size_t corr = (size_t)(K / kGroup) * kMfmaTokens * 4;
    const size_t tiles = (size_t)4 * mfma_wave_tile_bytes<BITS, R>();
    const size_t red = (size_t)4 * R * 4 * 64 * 4;
    return act + corr + tiles + red;
}

// Four int8 activations -> four FP8 (E4M3) bytes of each plane.  Both planes are
// exact: a & 15 is 0..15 and 16*(a >> 4) is a multiple of 16 in [-128, 112].
__device__ __forceinline__ void int8x4_to_fp8_planes(uint32_t x, uint32_t &hi, uint32_t &lo) {
    const uint32_t xl = x & 0x0f0f0f0fu;
    int l = __builtin_amdgcn_cvt_pk_fp8_f32((float)(xl & 0xffu), (float)((xl >> 8) & 0xffu), 0, false);
    l = __builtin_amdgcn_cvt_pk_fp8_f32((float)((xl >> 16) & 0xffu), (float)(xl >> 24), l, true);
    lo = (uint32_t)l;
    const uint32_t xh = x & 0xf0f0f0f0u;
    const float h0 = (float)(int)(int8_t)(xh & 0xffu);
    const float h1 = (float)(int)(int8_t)((xh >> 8) & 0xffu);
    const float h2 = (float)(int)(int8_t)((xh >> 16) & 0xffu);
    const float h3 = (float)((int)xh >> 24);
    int h = __builtin_amdgcn_cvt_pk_fp8_f32(h0, h1, 0, false);
    h = __builtin_amdgcn_cvt_pk_fp8_f32(h2, h3, h, true);
    hi = (uint32_t)h;
}

template <int BITS, int R, bool G32, bool SF16>
__global__ void __launch_bounds__(kMfmaThreads) gemv_fp4_kernel
(const int8_t *pA, const uint8_t *pB, void *pout, const float *ps, const uint16_t *pws, int pM,
 int pN, int pK, int pmt, int pks_log2, int pout_f32, int ppasses, uint32_t pdiv_magic) {
    // scalar parameters (instead of one struct) so that they can be preloaded into SGPRs
    const MfmaArgs a{pA, pB, pout, ps, pws, pM, pN, pK, pmt, pks_log2, pout_f32, ppasses, pdiv_magic};
    using MF = MfmaFmt<BITS>;
    extern __shared__ __align__(16) unsigned char smem[];

    const int K = a.K, N = a.N, M = a.M;
    const int G = K / kGroup;
    const int row_bytes = K * BITS / 8;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ks = 1 << a.ks_log2;
    const int kslice = wave & (ks - 1);
    const int rw = wave >> a.ks_log2;
    const int rws = 4 >> a.ks_log2;
    const int m0 = blockIdx.y * a.mt;
    const int mt = (M - m0) < a.mt ? (M - m0) : a.mt;
    const int pass_rows = rws * 16 * R;
    const int n_first = (int)blockIdx.x * a.passes * pass_rows + rw * (16 * R);

    // ---- LDS carve-up
    const int tb = fp4_token_bytes(K);
    unsigned char *act = smem;                                             // [a.mt][tb]
    float *corr = reinterpret_cast<float *>(smem + (size_t)a.mt * tb);     // [G][16]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(corr + (size_t)G * kMfmaTokens);
    unsigned char *wt = tiles + (size_t)wave * mfma_wave_tile_bytes<BITS, R>();
    float *red = reinterpret_cast<float *>(tiles + (size_t)4 * mfma_wave_tile_bytes<BITS, R>());

    const int ntiles = G / kMfmaGroupsPerTile;
    const int t_begin = (int)(((long)ntiles * kslice) >> a.ks_log2);
    const int t_end = (int)(((long)ntiles * (kslice + 1)) >> a.ks_log2);

    const int ld_row = lane / MF::kLanesPerRow;
    const int ld_col = lane % MF::kLanesPerRow;
    const int op_row = lane & 15;
    const int kb = lane >> 4;

    struct TileRegs {
        u32x4 w[R][MF::kLoads];
        uint2 sc[R];
    };
    auto load_tile = [&](TileRegs &tr, int n0, int kt) {
#pragma unroll
        for (int rt = 0; rt < R; ++rt) {
#pragma unroll
            for (int h = 0; h < MF::kLoads; ++h) {
                int row = n0 + rt * 16 + h * MF::kRowsPerLoad + ld_row;
                row = row < N ? row : N - 1;
                const unsigned char *p =
                    a.B + (size_t)row * row_bytes + (size_t)kt * MF::kTileBytes + ld_col * 16;
                tr.w[rt][h] = *reinterpret_cast<const u32x4 *>(p);
            }
            if (!G32) {
                int row = n0 + rt * 16 + op_row;
                row = row < N ? row : N - 1;
                tr.sc[rt] = *reinterpret_cast<const uint2 *>(a.ws + (size_t)row * G +
                                                             (size_t)kt * kMfmaGroupsPerTile);
            }
        }
    };
    auto park_tile = [&](const TileRegs &tr) {
#pragma unroll
        for (int rt = 0; rt < R; ++rt)
#pragma unroll
            for (int h = 0; h < MF::kLoads; ++h) {
                unsigned char *dst = wt + (rt * 16 + h * MF::kRowsPerLoad + ld_row) * MF::kPitch +
                                     ld_col * 16;
                uint2 *d2 = reinterpret_cast<uint2 *>(dst);
                d2[0] = make_uint2(tr.w[rt][h].x, tr.w[rt][h].y);
                d2[1] = make_uint2(tr.w[rt][h].z, tr.w[rt][h].w);
            }
    };

    TileRegs cur;
    if (t_begin < t_end) load_tile(cur, n_first, t_begin);

    float sdiv[4];
    if (!G32) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + 4 * kb + r;
            sdiv[r] = a.s[m < M ? m : M - 1];
        }
    }

    // ---- stage the token tile: per 32-activation block, reorder to operand K order,
    // split into the two FP8 planes, and sum for the group's offset-removal term.
    {
        constexpr int kSt = 2;      // blocks per thread and round (their loads go out together)
        const int qn = K / 32;      // blocks per token
        const int ntask = mt * qn;
        for (int base = tid; base < ntask; base += kSt * kMfmaThreads) {
            u32x4 in[kSt][2];
            int tok[kSt], q[kSt];
#pragma unroll
            for (int i = 0; i < kSt; ++i) {
                int task = base + i * kMfmaThreads;
                task = task < ntask ? task : ntask - 1;
                tok[i] = (int)__umulhi((uint32_t)task, a.div_magic);  // task / qn
                q[i] = task - tok[i] * qn;
                const u32x4 *src = reinterpret_cast<const u32x4 *>(
                    a.A + (size_t)(m0 + tok[i]) * K + (size_t)q[i] * 32);
                in[i][0] = src[0];
                in[i][1] = src[1];
            }
#pragma unroll
            for (int i = 0; i < kSt; ++i) {
                if (base + i * kMfmaThreads >= ntask) break;  // whole 4-lane groups drop out together
                const uint32_t x[8] = {in[i][0].x, in[i][0].y, in[i][0].z, in[i][0].w,
                                       in[i][1].x, in[i][1].y, in[i][1].z, in[i][1].w};
                int sum = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) sum += sum4_i8(x[j]);
                uint32_t o[8], hi[8], lo[8];
                fp4_order_block<BITS>(x, o);
#pragma unroll
                for (int j = 0; j < 8; ++j) int8x4_to_fp8_planes(o[j], hi[j], lo[j]);
                // group block: [hi plane 128 B][lo plane 128 B]; this block is bytes 32*(q%4)..+31
                unsigned char *dst = act + (size_t)tok[i] * tb + (q[i] >> 2) * 256 + (q[i] & 3) * 32;
                u32x4 *dh = reinterpret_cast<u32x4 *>(dst);
                u32x4 *dl = reinterpret_cast<u32x4 *>(dst + 128);
                dh[0] = u32x4{hi[0], hi[1], hi[2], hi[3]};
                dh[1] = u32x4{hi[4], hi[5], hi[6], hi[7]};
                dl[0] = u32x4{lo[0], lo[1], lo[2], lo[3]};
                dl[1] = u32x4{lo[4], lo[5], lo[6], lo[7]};
                sum += dpp_i32<kDppXor1>(sum);
                sum += dpp_i32<kDppXor2>(sum);
                if ((q[i] & 3) == 0) corr[(q[i] >> 2) * kMfmaTokens + tok[i]] = fp4_corr<BITS>(sum);
            }
        }
    }
    __syncthreads();

    float acc[R][4];
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[rt][r] = 0.0f;

    const int a_tok = op_row < mt ? op_row : mt - 1;
    const unsigned char *act_lane = act + (size_t)a_tok * tb + 16 * kb;
    constexpr float kF = (float)fp4_result_scale<BITS>();

    for (int pass = 0; pass < a.passes; ++pass) {
        const int n0 = n_first + pass * pass_rows;
        for (int kt = t_begin; kt < t_end; ++kt) {
            park_tile(cur);
            TileRegs nxt;
            const bool last_kt = kt + 1 == t_end;
            const bool more = !last_kt || pass + 1 < a.passes;
            if (more) load_tile(nxt, last_kt ? n0 + pass_rows : n0, last_kt ? t_begin : kt + 1);

#pragma unroll
            for (int gi = 0; gi < kMfmaGroupsPerTile; ++gi) {
                const int g = kt * kMfmaGroupsPerTile + gi;
                const unsigned char *ab = act_lane + (size_t)g * 256;
                const u32x4 h0 = *reinterpret_cast<const u32x4 *>(ab);        // K 16kb..
                const u32x4 h1 = *reinterpret_cast<const u32x4 *>(ab + 64);   // K 64+16kb..
                const u32x4 l0 = *reinterpret_cast<const u32x4 *>(ab + 128);
                const u32x4 l1 = *reinterpret_cast<const u32x4 *>(ab + 192);
                const v8i vah = {(int)h0.x, (int)h0.y, (int)h0.z, (int)h0.w,
                                 (int)h1.x, (int)h1.y, (int)h1.z, (int)h1.w};
                const v8i val = {(int)l0.x, (int)l0.y, (int)l0.z, (int)l0.w,
                                 (int)l1.x, (int)l1.y, (int)l1.z, (int)l1.w};
                const float4 cr = *reinterpret_cast<const float4 *>(corr + g * kMfmaTokens + 4 * kb);
                const v4f vcr = {cr.x, cr.y, cr.z, cr.w};
#pragma unroll
                for (int rt = 0; rt < R; ++rt) {
                    const unsigned char *src = wt + (rt * 16 + op_row) * MF::kPitch;
                    uint32_t p0, p1;
                    if (BITS == 2) {
                        const uint2 pp = *reinterpret_cast<const uint2 *>(src + gi * 32 + kb * 8);
                        p0 = pp.x;
                        p1 = pp.y;
                    } else {
                        p0 = *reinterpret_cast<const uint32_t *>(src + gi * 16 + kb * 4);
                        p1 = 0;
                    }
                    uint32_t nb[4];
                    fp4_unpack<BITS>(p0, p1, nb);
                    const v8i vb = {(int)nb[0], (int)nb[1], (int)nb[2], (int)nb[3], 0, 0, 0, 0};
                    // A operand: FP8 (format 0), B operand: FP4 (format 4), no block scales
                    v4f d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vah, vb, vcr, 0, 4, 0, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(val, vb, d, 0, 4, 0, 0, 0, 0);
                    // d[r] = G / F for token 4*kb + r and weight row op_row of tile rt
                    if (G32) {
                        const int row = n0 + rt * 16 + op_row;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int tok = 4 * kb + r;
                            if (row < N && tok < mt)
                                reinterpret_cast<int32_t *>(
                                    a.out)[((size_t)(m0 + tok) * N + row) * G + g] = (int32_t)(kF * d[r]);
                        }
                    } else {
                        const uint32_t raw = (gi & 2) ? cur.sc[rt].y : cur.sc[rt].x;
                        const float wsf = scale_to_f32<SF16>(
                            (uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rt][r] += d[r] * wsf;
                    }
                }
            }
            if (more) cur = nxt;
        }

        if (G32) continue;

        if (ks > 1) {
            float *mine = red + (size_t)wave * (R * 4 * 64);
#pragma unroll
            for (int rt = 0; rt < R; ++rt)
#pragma unroll
                for (int r = 0; r < 4; ++r) mine[(rt * 4 + r) * 64 + lane] = acc[rt][r];
            __syncthreads();
            if (kslice != 0) return;
            for (int k2 = 1; k2 < ks; ++k2) {
                const float *other = red + (size_t)(wave + k2) * (R * 4 * 64);
#pragma unroll
                for (int rt = 0; rt < R; ++rt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[rt][r] += other[(rt * 4 + r) * 64 + lane];
            }
        }
#pragma unroll
        for (int rt = 0; rt < R; ++rt) {
            const int row = n0 + rt * 16 + op_row;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int tok = 4 * kb + r;
                if (row < N && tok < mt) {
                    const float y = (kF * acc[rt][r]) / sdiv[r];
                    const size_t o = (size_t)(m0 + tok) * N + row;
                    if (a.out_f32)
                        reinterpret_cast<float *>(a.out)[o] = y;
                    else
                        reinterpret_cast<uint16_t *>(a.out)[o] = f32_to_bf16_rne(y);
                }
                acc[rt][r] = 0.0f;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
template <int BITS>
const MfmaTable<BITS> &fp4_table() {
    static const MfmaTable<BITS> t = [] {
        MfmaTable<BITS> x{};
        x.fn[0][0] = gemv_fp4_kernel<BITS, 1, false, false>;
        x.fn[0][1] = gemv_fp4_kernel<BITS, 1, false, true>;
        x.fn[0][2] = gemv_fp4_kernel<BITS, 1, true, false>;
        x.fn[1][0] = gemv_fp4_kernel<BITS, 2, false, false>;
        x.fn[1][1] = gemv_fp4_kernel<BITS, 2, false, true>;
        x.fn[1][2] = gemv_fp4_kernel<BITS, 2, true, false>;
        x.fn[2][0] = gemv_fp4_kernel<BITS, 4, false, false>;
        x.fn[2][1] = gemv_fp4_kernel<BITS, 4, false, true>;
        x.fn[2][2] = gemv_fp4_kernel<BITS, 4, true, false>;
        return x;
    }();
    return t;
}

template <int BITS>
int fp4_init_device(int max_lds) {
    const MfmaTable<BITS> &t = fp4_table<BITS>();
    for (int r = 0; r < 3; ++r)
        for (int v = 0; v < 3; ++v)
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(t.fn[r][v]),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    max_lds) != hipSuccess)
                return 2;
    return 0;
}

template <int BITS>
size_t fp4_lds_for(int ri, int mt, int K) {
    return ri == 0 ? fp4_lds_bytes<BITS, 1>(mt, K)
                   : (ri == 1 ? fp4_lds_bytes<BITS, 2>(mt, K) : fp4_lds_bytes<BITS, 4>(mt, K));
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_FP4_HIP_H
