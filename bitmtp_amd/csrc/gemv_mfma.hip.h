// Matrix-core kernel of the packed low-bit GEMV for block widths above one token.
//
// The dot4 kernel spends M dot instructions per packed weight byte, so from about
// four tokens on it is bound by VALU issue, not by HBM.  Here the weights of 16
// rows x one 128-wide group are unpacked once into the B operand of two
// v_mfma_i32_16x16x64_i8 and multiplied with up to 16 tokens at the cost the
// dot4 path pays for one: per group and 16 rows, 14 (T2) / 15 (Q1) unpack
// operations plus 9 for the exact-int32 -> fp32 scale-accumulate.
//
//   G[token][row] (int32, exact) = MFMA over the group's 128 slots, offset term as C input
//   acc[token][row] += fp32(G) * ws[row][group]                      (fp32)
//
// Data movement per wave: R tiles of 16 rows.  Weights are read from HBM with
// coalesced 16-byte loads (8 or 4 lanes per row), parked in a wave-private LDS
// tile and read back in operand order (row = lane % 16, K-block = lane / 16); the
// tile row pitch (tile bytes + 8) keeps both directions free of bank conflicts.
// The token tile's activations are staged once per workgroup in operand order
// together with the per-group offset-removal terms.  KS waves of a workgroup may
// split K among them; their fp32 partial sums are combined in a fixed order.
#ifndef BONSAI_GEMV_MFMA_HIP_H
#define BONSAI_GEMV_MFMA_HIP_H

#include "packed_gemv.hip.h"

namespace bonsai {

constexpr int kMfmaTokens = 16;   // token columns of one MFMA tile
constexpr int kMfmaThreads = 256; // four waves per workgroup
constexpr int kMfmaGroupsPerTile = 4;

typedef int v4i __attribute__((ext_vector_type(4)));

struct MfmaArgs {
    const int8_t *A;
    const uint8_t *B;
    void *out;
    const float *s;
    const uint16_t *ws;
    int M, N, K;
    int mt;        // tokens per token tile (<= 16); grid.y tiles cover M
    int ks_log2;   // log2 of the waves that split K inside a workgroup (0, 1, 2)
    int out_f32;
    int passes;          // row blocks a workgroup walks through (1 unless ks_log2 == 0)
    uint32_t div_magic;  // floor(2^32 / quarters-per-token) + 1: staging task -> token
};

template <int BITS>
struct MfmaFmt {
    // bytes of one weight row in a K tile of four groups, and its padded LDS pitch
    static constexpr int kTileBytes = BITS == 2 ? 128 : 64;
    static constexpr int kPitch = kTileBytes + 8;
    static constexpr int kLoads = kTileBytes / 64;        // 16-byte loads per lane and row tile
    static constexpr int kLanesPerRow = kTileBytes / 16;  // lanes sharing a row in one load
    static constexpr int kRowsPerLoad = 64 / kLanesPerRow;
};

template <int BITS, int R>
__host__ __device__ constexpr int mfma_wave_tile_bytes() {
    return R * 16 * MfmaFmt<BITS>::kPitch;
}

// LDS bytes of one workgroup: activations, correction terms, weight tiles, reduction.
template <int BITS, int R>
__host__ __device__ inline size_t mfma_lds_bytes(int mt, int K) {
    const size_t act = (size_t)mt * mfma_token_words(K) * 16;
    const size_t corr = (size_t)(K / kGroup) * kMfmaTokens * 4;
    const size_t tiles = (size_t)4 * mfma_wave_tile_bytes<BITS, R>();
    const size_t red = (size_t)4 * R * 4 * 64 * 4;
    return act + corr + tiles + red;
}

template <int BITS, int R, bool G32, bool SF16>
__global__ void __launch_bounds__(kMfmaThreads) gemv_mfma_kernel
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
    const int ks = 1 << a.ks_log2;         // waves along K
    const int kslice = wave & (ks - 1);
    const int rw = wave >> a.ks_log2;      // row-wave index inside the workgroup
    const int rws = 4 >> a.ks_log2;        // row-waves per workgroup
    const int m0 = blockIdx.y * a.mt;
    const int mt = (M - m0) < a.mt ? (M - m0) : a.mt;  // valid tokens of this tile
    const int pass_rows = rws * 16 * R;  // rows one pass of the workgroup covers
    const int n_first = (int)blockIdx.x * a.passes * pass_rows + rw * (16 * R);

    // ---- LDS carve-up
    const int tw = mfma_token_words(K);
    u32x4 *act = reinterpret_cast<u32x4 *>(smem);                       // [a.mt][tw]
    int *corr = reinterpret_cast<int *>(smem + (size_t)a.mt * tw * 16); // [G][16]
    unsigned char *tiles = reinterpret_cast<unsigned char *>(corr + (size_t)G * kMfmaTokens);
    unsigned char *wt = tiles + (size_t)wave * mfma_wave_tile_bytes<BITS, R>();
    float *red = reinterpret_cast<float *>(tiles + (size_t)4 * mfma_wave_tile_bytes<BITS, R>());

    // ---- K tiles of this wave
    const int ntiles = G / kMfmaGroupsPerTile;  // K % 512 == 0 is checked on the host
    const int t_begin = (int)(((long)ntiles * kslice) >> a.ks_log2);
    const int t_end = (int)(((long)ntiles * (kslice + 1)) >> a.ks_log2);

    // ---- lane roles
    const int ld_row = lane / MF::kLanesPerRow;  // row inside one load (of kRowsPerLoad)
    const int ld_col = lane % MF::kLanesPerRow;  // 16-byte chunk inside the tile row
    const int op_row = lane & 15;                // operand row (weight row / token)
    const int kb = lane >> 4;                    // operand K-block, also the token quad

    // Global loads of one K tile into registers: R*kLoads 16-byte loads + R scale loads.
    struct TileRegs {
        u32x4 w[R][MF::kLoads];
        uint2 sc[R];  // four bf16/fp16 scales of this lane's row
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
                uint2 *d2 = reinterpret_cast<uint2 *>(dst);  // pitch is 8- not 16-byte aligned
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

    // ---- stage the token tile (operand order) and the per-group correction terms.
    // Four quarter tasks per thread and round: their loads go out together.
    {
        constexpr int QB = mfma_quarter_bytes<BITS>();
        constexpr int QW = QB / 16;       // 16-byte words per quarter
        constexpr int QPG = kGroup / QB;  // quarters per group: 8 (T2) or 4 (Q1)
        constexpr int kSt = 4;
        const int qn = K / QB;            // quarters per token
        const int ntask = mt * qn;
        for (int base = tid; base < ntask; base += kSt * kMfmaThreads) {
            u32x4 in[kSt][QW];
            int tok[kSt], q[kSt];
#pragma unroll
            for (int i = 0; i < kSt; ++i) {
                int task = base + i * kMfmaThreads;
                task = task < ntask ? task : ntask - 1;  // clamped duplicates are not written
                tok[i] = (int)__umulhi((uint32_t)task, a.div_magic);  // task / qn
                q[i] = task - tok[i] * qn;
                const u32x4 *src = reinterpret_cast<const u32x4 *>(
                    a.A + (size_t)(m0 + tok[i]) * K + (size_t)q[i] * QB);
#pragma unroll
                for (int w = 0; w < QW; ++w) in[i][w] = src[w];
            }
#pragma unroll
            for (int i = 0; i < kSt; ++i) {
                if (base + i * kMfmaThreads >= ntask) break;  // whole lane groups drop out together
                int sum = mfma_stage_quarter<BITS>(in[i], act + (size_t)tok[i] * tw, q[i]);
                sum += dpp_i32<kDppXor1>(sum);
                sum += dpp_i32<kDppXor2>(sum);
                if (QPG == 8) sum += dpp_i32<kDppHalfMirror>(sum);
                if ((q[i] & (QPG - 1)) == 0)
                    corr[(q[i] / QPG) * kMfmaTokens + tok[i]] = mfma_corr<BITS>(sum);
            }
        }
    }
    __syncthreads();

    float acc[R][4];
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[rt][r] = 0.0f;

    // Tokens past the tile alias the last valid one: their columns are never stored.
    const int a_tok = op_row < mt ? op_row : mt - 1;
    const u32x4 *act_lane = act + (size_t)a_tok * tw + 2 * kb;

    for (int pass = 0; pass < a.passes; ++pass) {
        const int n0 = n_first + pass * pass_rows;
        for (int kt = t_begin; kt < t_end; ++kt) {
            park_tile(cur);
            TileRegs nxt;
            // next tile of this row block, or the first tile of the next row block
            const bool last_kt = kt + 1 == t_end;
            const bool more = !last_kt || pass + 1 < a.passes;
            if (more) load_tile(nxt, last_kt ? n0 + pass_rows : n0, last_kt ? t_begin : kt + 1);

#pragma unroll
            for (int gi = 0; gi < kMfmaGroupsPerTile; ++gi) {
                const int g = kt * kMfmaGroupsPerTile + gi;
                const u32x4 a0 = act_lane[g * 8];      // unit 8g + 2kb
                const u32x4 a1 = act_lane[g * 8 + 1];  // unit 8g + 2kb + 1
                const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
                const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                // offset-removal terms of tokens 4kb..4kb+3: the accumulator input
                const int4 cr = *reinterpret_cast<const int4 *>(corr + g * kMfmaTokens + 4 * kb);
                const v4i vcr = {cr.x, cr.y, cr.z, cr.w};
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
                    uint32_t b0[4], b1[4];
                    mfma_unpack<BITS>(p0, p1, b0, b1);
                    const v4i vb0 = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3]};
                    const v4i vb1 = {(int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
                    v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, vb0, vcr, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, vb1, d, 0, 0, 0);
                    // d[r]: exact group sum of token 4*kb + r and weight row op_row of tile rt
                    if (G32) {
                        const int row = n0 + rt * 16 + op_row;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int tok = 4 * kb + r;
                            if (row < N && tok < mt)
                                reinterpret_cast<int32_t *>(
                                    a.out)[((size_t)(m0 + tok) * N + row) * G + g] = d[r];
                        }
                    } else {
                        const uint32_t raw = (gi & 2) ? cur.sc[rt].y : cur.sc[rt].x;
                        const float wsf = scale_to_f32<SF16>(
                            (uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rt][r] += (float)d[r] * wsf;
                    }
                }
            }
            if (more) cur = nxt;
        }

        if (G32) continue;

        // ---- combine the K slices (fixed order; passes == 1 whenever ks > 1) and store
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
                    const float y = acc[rt][r] / sdiv[r];
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
// Same contraction without the activation staging pass: every wave loads the A operand of
// its K tiles straight from the row-major activations (lane = token, K-block: 32 contiguous
// bytes per group, an L2 hit) together with the weight tile, permutes them in registers to
// the order the unpack produces, and obtains the offset-removal terms from two more MFMAs
// against an all-ones operand (sum of a token's activations over the group, delivered in
// the accumulator layout).  No workgroup barrier before the K loop and no LDS for
// activations: the kernel is one memory round trip plus the K loop long.
// ---------------------------------------------------------------------------
// NW = waves per workgroup: four, or eight for long rows (K >= 4096), where a wave would
// otherwise walk through several K tiles one after the other.  NW = 0 is the form for tile
// counts that are no power of two (K = 2560, 6144, 9728 ...): one row block per workgroup
// and any number of waves up to twelve, each with its own K slice; the argument that
// otherwise carries log2 of the split then carries the split itself.
constexpr int kMfmaFlexMaxWaves = 12;

template <int BITS, int R>
__host__ __device__ inline size_t mfma_direct_lds_bytes_for(int nwaves) {
    return (size_t)nwaves * mfma_wave_tile_bytes<BITS, R>() + (size_t)nwaves * R * 4 * 64 * 4;
}

template <int BITS, int R, int NW = 4>
__host__ __device__ inline size_t mfma_direct_lds_bytes() {
    return mfma_direct_lds_bytes_for<BITS, R>(NW);
}

template <int BITS, int R, bool G32, bool SF16, int NW = 4>
__global__ void __launch_bounds__(NW == 0 ? kMfmaFlexMaxWaves * 64 : NW * 64)
gemv_mfma_direct_kernel
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
    constexpr bool kFlex = NW == 0;
    const int ks = kFlex ? a.ks_log2 : 1 << a.ks_log2;
    const int nwaves = kFlex ? ks : NW;
    const int kslice = kFlex ? wave : wave & (ks - 1);
    const int rw = kFlex ? 0 : wave >> a.ks_log2;
    const int rws = kFlex ? 1 : NW >> a.ks_log2;
    const int m0 = blockIdx.y * a.mt;
    const int mt = (M - m0) < a.mt ? (M - m0) : a.mt;
    const int pass_rows = rws * 16 * R;
    const int n_first = (int)blockIdx.x * a.passes * pass_rows + rw * (16 * R);

    unsigned char *tiles = smem;
    unsigned char *wt = tiles + (size_t)wave * mfma_wave_tile_bytes<BITS, R>();
    float *red =
        reinterpret_cast<float *>(tiles + (size_t)nwaves * mfma_wave_tile_bytes<BITS, R>());

    const int ntiles = G / kMfmaGroupsPerTile;
    const int t_begin = kFlex ? ntiles * kslice / ks : (int)(((long)ntiles * kslice) >> a.ks_log2);
    const int t_end = kFlex ? ntiles * (kslice + 1) / ks
                            : (int)(((long)ntiles * (kslice + 1)) >> a.ks_log2);

    const int ld_row = lane / MF::kLanesPerRow;
    const int ld_col = lane % MF::kLanesPerRow;
    const int op_row = lane & 15;
    const int kb = lane >> 4;
    const int a_tok = m0 + (op_row < mt ? op_row : mt - 1);  // tokens past the tile alias the last
    const int8_t *a_lane = a.A + (size_t)a_tok * K + 32 * kb;

    struct TileRegs {
        u32x4 w[R][MF::kLoads];
        uint2 sc[R];
    };
    struct ActRegs {
        u32x4 lo[kMfmaGroupsPerTile], hi[kMfmaGroupsPerTile];  // 32 natural-order bytes per group
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
    auto load_act = [&](ActRegs &ar, int kt) {
#pragma unroll
        for (int gi = 0; gi < kMfmaGroupsPerTile; ++gi) {
            const u32x4 *p = reinterpret_cast<const u32x4 *>(
                a_lane + (size_t)(kt * kMfmaGroupsPerTile + gi) * kGroup);
            ar.lo[gi] = p[0];
            ar.hi[gi] = p[1];
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
    ActRegs acur;
    if (t_begin < t_end) {
        load_act(acur, t_begin);
        load_tile(cur, n_first, t_begin);
    }
    float sdiv[4];
    if (!G32) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + 4 * kb + r;
            sdiv[r] = a.s[m < M ? m : M - 1];
        }
    }

    float acc[R][4];
#pragma unroll
    for (int rt = 0; rt < R; ++rt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[rt][r] = 0.0f;
    // the offset-removal term straight from the matrix cores: -2 (T2) / -1 (Q1) in every slot
    // of the B operand gives -2 * sum(a) / -sum(a) per token in the accumulator layout
    constexpr int kNegs = BITS == 2 ? (int)0xFEFEFEFEu : (int)0xFFFFFFFFu;
    const v4i negs = {kNegs, kNegs, kNegs, kNegs};
    const v4i zero = {0, 0, 0, 0};

    for (int pass = 0; pass < a.passes; ++pass) {
        const int n0 = n_first + pass * pass_rows;
        for (int kt = t_begin; kt < t_end; ++kt) {
            park_tile(cur);
            TileRegs nxt;
            ActRegs anxt;
            const bool last_kt = kt + 1 == t_end;
            const bool more = !last_kt || pass + 1 < a.passes;
            if (more) {
                load_act(anxt, last_kt ? t_begin : kt + 1);
                load_tile(nxt, last_kt ? n0 + pass_rows : n0, last_kt ? t_begin : kt + 1);
            }
#pragma unroll
            for (int gi = 0; gi < kMfmaGroupsPerTile; ++gi) {
                const int g = kt * kMfmaGroupsPerTile + gi;
                u32x4 a0, a1;
                if (BITS == 2) {
                    a0 = transpose4x4_bytes(acur.lo[gi].x, acur.lo[gi].y, acur.lo[gi].z, acur.lo[gi].w);
                    a1 = transpose4x4_bytes(acur.hi[gi].x, acur.hi[gi].y, acur.hi[gi].z, acur.hi[gi].w);
                } else {
                    a0 = transpose4x4_bytes(acur.lo[gi].x, acur.lo[gi].z, acur.hi[gi].x, acur.hi[gi].z);
                    a1 = transpose4x4_bytes(acur.lo[gi].y, acur.lo[gi].w, acur.hi[gi].y, acur.hi[gi].w);
                }
                const v4i va0 = {(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w};
                const v4i va1 = {(int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                v4i vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, negs, zero, 0, 0, 0);
                vcr = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, negs, vcr, 0, 0, 0);
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
                    uint32_t b0[4], b1[4];
                    mfma_unpack<BITS>(p0, p1, b0, b1);
                    const v4i vb0 = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3]};
                    const v4i vb1 = {(int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
                    v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(va0, vb0, vcr, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_i32_16x16x64_i8(va1, vb1, d, 0, 0, 0);
                    if (G32) {
                        const int row = n0 + rt * 16 + op_row;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int tok = 4 * kb + r;
                            if (row < N && tok < mt)
                                reinterpret_cast<int32_t *>(
                                    a.out)[((size_t)(m0 + tok) * N + row) * G + g] = d[r];
                        }
                    } else {
                        const uint32_t raw = (gi & 2) ? cur.sc[rt].y : cur.sc[rt].x;
                        const float wsf = scale_to_f32<SF16>(
                            (uint16_t)((gi & 1) ? (raw >> 16) : (raw & 0xffffu)));
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[rt][r] += (float)d[r] * wsf;
                    }
                }
            }
            if (more) {
                cur = nxt;
                acur = anxt;
            }
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
                    const float y = acc[rt][r] / sdiv[r];
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
struct MfmaTuning {
    int min_width = 0;   // smallest M sent to this kernel; 0 = built-in default
    int row_tiles = 0;   // R: 1, 2 or 4; 0 = heuristic
    int k_split = 0;     // waves along K: 1, 2, 4 (or 8: direct kernel, eight waves); 0 = heuristic
    int passes = 0;      // row blocks per workgroup; 0 = heuristic
    int engine = 0;      // 0 = choose, 1 = int8 MFMA (staged), 3 = int8 MFMA (direct), 4 = grouped kernel, 5 / 6 = streaming kernels
};

using MfmaKernelFn = void (*)(const int8_t *, const uint8_t *, void *, const float *,
                              const uint16_t *, int, int, int, int, int, int, int, uint32_t);

template <int BITS>
struct MfmaTable {
    MfmaKernelFn fn[3][3];  // [R index: 1,2,4][variant: bf16, fp16, G32]
    size_t tile_bytes[3];
};

template <int BITS>
const MfmaTable<BITS> &mfma_table() {
    static const MfmaTable<BITS> t = [] {
        MfmaTable<BITS> x{};
        x.fn[0][0] = gemv_mfma_kernel<BITS, 1, false, false>;
        x.fn[0][1] = gemv_mfma_kernel<BITS, 1, false, true>;
        x.fn[0][2] = gemv_mfma_kernel<BITS, 1, true, false>;
        x.fn[1][0] = gemv_mfma_kernel<BITS, 2, false, false>;
        x.fn[1][1] = gemv_mfma_kernel<BITS, 2, false, true>;
        x.fn[1][2] = gemv_mfma_kernel<BITS, 2, true, false>;
        x.fn[2][0] = gemv_mfma_kernel<BITS, 4, false, false>;
        x.fn[2][1] = gemv_mfma_kernel<BITS, 4, false, true>;
        x.fn[2][2] = gemv_mfma_kernel<BITS, 4, true, false>;
        return x;
    }();
    return t;
}

template <int BITS>
const MfmaTable<BITS> &mfma_direct_table() {
    static const MfmaTable<BITS> t = [] {
        MfmaTable<BITS> x{};
        x.fn[0][0] = gemv_mfma_direct_kernel<BITS, 1, false, false>;
        x.fn[0][1] = gemv_mfma_direct_kernel<BITS, 1, false, true>;
        x.fn[0][2] = gemv_mfma_direct_kernel<BITS, 1, true, false>;
        x.fn[1][0] = gemv_mfma_direct_kernel<BITS, 2, false, false>;
        x.fn[1][1] = gemv_mfma_direct_kernel<BITS, 2, false, true>;
        x.fn[1][2] = gemv_mfma_direct_kernel<BITS, 2, true, false>;
        x.fn[2][0] = gemv_mfma_direct_kernel<BITS, 4, false, false>;
        x.fn[2][1] = gemv_mfma_direct_kernel<BITS, 4, false, true>;
        x.fn[2][2] = gemv_mfma_direct_kernel<BITS, 4, true, false>;
        return x;
    }();
    return t;
}

// the form with one K slice per wave for any number of waves (one row tile per wave only)
template <int BITS>
const MfmaTable<BITS> &mfma_direct_flex_table() {
    static const MfmaTable<BITS> t = [] {
        MfmaTable<BITS> x{};
        x.fn[0][0] = gemv_mfma_direct_kernel<BITS, 1, false, false, 0>;
        x.fn[0][1] = gemv_mfma_direct_kernel<BITS, 1, false, true, 0>;
        x.fn[0][2] = gemv_mfma_direct_kernel<BITS, 1, true, false, 0>;
        return x;
    }();
    return t;
}

// the eight-wave form of the direct kernel
template <int BITS>
const MfmaTable<BITS> &mfma_direct8_table() {
    static const MfmaTable<BITS> t = [] {
        MfmaTable<BITS> x{};
        x.fn[0][0] = gemv_mfma_direct_kernel<BITS, 1, false, false, 8>;
        x.fn[0][1] = gemv_mfma_direct_kernel<BITS, 1, false, true, 8>;
        x.fn[0][2] = gemv_mfma_direct_kernel<BITS, 1, true, false, 8>;
        x.fn[1][0] = gemv_mfma_direct_kernel<BITS, 2, false, false, 8>;
        x.fn[1][1] = gemv_mfma_direct_kernel<BITS, 2, false, true, 8>;
        x.fn[1][2] = gemv_mfma_direct_kernel<BITS, 2, true, false, 8>;
        x.fn[2][0] = gemv_mfma_direct_kernel<BITS, 4, false, false, 8>;
        x.fn[2][1] = gemv_mfma_direct_kernel<BITS, 4, false, true, 8>;
        x.fn[2][2] = gemv_mfma_direct_kernel<BITS, 4, true, false, 8>;
        return x;
    }();
    return t;
}

template <int BITS>
size_t mfma_direct_lds_for(int ri, int nw = 4) {
    return ri == 0 ? mfma_direct_lds_bytes_for<BITS, 1>(nw)
                   : (ri == 1 ? mfma_direct_lds_bytes_for<BITS, 2>(nw)
                              : mfma_direct_lds_bytes_for<BITS, 4>(nw));
}

template <int BITS>
MfmaTuning &mfma_tuning() {
    static MfmaTuning t;
    return t;
}

template <int BITS>
int mfma_init_device(int max_lds) {
    const MfmaTable<BITS> *tables[4] = {&mfma_table<BITS>(), &mfma_direct_table<BITS>(),
                                        &mfma_direct8_table<BITS>(),
                                        &mfma_direct_flex_table<BITS>()};
    for (const MfmaTable<BITS> *t : tables)
        for (int r = 0; r < 3; ++r)
            for (int v = 0; v < 3; ++v)
                if (t->fn[r][v] != nullptr &&
                    hipFuncSetAttribute(reinterpret_cast<const void *>(t->fn[r][v]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                        max_lds) != hipSuccess)
                    return 2;
    return 0;
}

template <int BITS>
size_t mfma_lds_for(int ri, int mt, int K) {
    return ri == 0 ? mfma_lds_bytes<BITS, 1>(mt, K)
                   : (ri == 1 ? mfma_lds_bytes<BITS, 2>(mt, K) : mfma_lds_bytes<BITS, 4>(mt, K));
}

// True when the matrix-core kernels can take the shape: whole K tiles of four
// groups, 16-byte aligned weight rows and 8-byte aligned scale rows.
inline bool mfma_shape_ok(const void *B, const void *ws, int K) {
    return K % 512 == 0 && (reinterpret_cast<uintptr_t>(B) & 15) == 0 &&
           (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 7) == 0);
}

}  // namespace bonsai
#endif  // BONSAI_GEMV_MFMA_HIP_H
