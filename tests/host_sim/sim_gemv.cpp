// CPU lane simulator for the per-lane arithmetic in bitmtp_amd/csrc/gemv_core.h.
// Replays, lane by lane, what one weight row's lanes do in the gfx950 kernel:
// stage the activations in the permuted layout, unpack each 16-byte chunk with
// the kernel's own shift/mask sequence, form the raw code dot products and fix
// them up with the chunk activation sums.  The result is the int32 group sums,
// which tests compare bit for bit with the oracle.  Built with g++ (no GPU).
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../bitmtp_amd/csrc/gemv_core.h"

using namespace bonsai;

template <int BITS, int MT>
static void run_tile(const int8_t *A, const uint8_t *B, int32_t *G, int m0, int M, int N, int K) {
    using F = Fmt<BITS>;
    const int C = K / F::kChunkWeights;
    const int ng = K / 128;
    std::vector<u32x4> act((size_t)C * block_words<BITS, MT>());
    int *asum = reinterpret_cast<int *>(act.data());
    for (int task = 0; task < MT * C; ++task) {
        const int m = task / C, chunk = task - m * C;
        const int msrc = (m0 + m) < M ? (m0 + m) : M - 1;
        std::vector<u32x4> src(F::kUnits);
        std::memcpy(src.data(), A + (size_t)msrc * K + (size_t)chunk * F::kChunkWeights,
                    F::kChunkWeights);
        asum[asum_index<BITS, MT>(m, chunk)] = stage_chunk<BITS, MT>(src.data(), act.data(), m, chunk);
    }
    for (int n = 0; n < N; ++n)
        for (int chunk = 0; chunk < C; ++chunk) {
            u32x4 w;
            std::memcpy(&w, B + (size_t)n * C * 16 + (size_t)chunk * 16, 16);
            int raw[MT];
            for (int m = 0; m < MT; ++m) raw[m] = 0;
            chunk_dot_raw<BITS, MT>(w, act.data(), chunk, raw);
            for (int m = 0; m < MT; ++m) {
                if (m0 + m >= M) continue;
                const int g = chunk_dot_signed<BITS>(raw[m], asum[asum_index<BITS, MT>(m, chunk)]);
                int32_t *dst = &G[((size_t)(m0 + m) * N + n) * ng + (chunk >> F::kGroupShift)];
                if (BITS == 2 && (chunk & 1)) *dst += g; else *dst = g;
            }
        }
}

extern "C" int sim_group_sums(const int8_t *A, const uint8_t *B, int32_t *G, int M, int N, int K,
                              int bits, int mt) {
    if (K % 128 != 0 || mt < 1 || mt > 3) return 1;
    for (int m0 = 0; m0 < M; m0 += mt) {
        if (bits == 2) {
            if (mt == 1) run_tile<2, 1>(A, B, G, m0, M, N, K);
            if (mt == 2) run_tile<2, 2>(A, B, G, m0, M, N, K);
            if (mt == 3) run_tile<2, 3>(A, B, G, m0, M, N, K);
        } else {
            if (mt == 1) run_tile<1, 1>(A, B, G, m0, M, N, K);
            if (mt == 2) run_tile<1, 2>(A, B, G, m0, M, N, K);
            if (mt == 3) run_tile<1, 3>(A, B, G, m0, M, N, K);
        }
    }
    return 0;
}

// ---------------------------------------------------------------------------
// Matrix-core path.  The MFMA is modelled by its contract: slot (kb, reg, byte) of
// the token operand meets the same slot of the weight operand, D[token][row] is
// the sum over the 64 slots.  Everything else -- activation staging order, the
// correction terms, which packed dword a lane unpacks for which of the two MFMAs
// of a group -- is the kernel's own code from gemv_core.h.
// ---------------------------------------------------------------------------
template <int BITS>
static void run_mfma(const int8_t *A, const uint8_t *B, int32_t *G, int M, int N, int K) {
    const int ng = K / 128;
    const int tw = mfma_token_words(K);
    constexpr int QB = mfma_quarter_bytes<BITS>();
    constexpr int QPG = 128 / QB;
    std::vector<u32x4> act((size_t)M * tw);
    std::vector<int> corr((size_t)ng * M);
    for (int tok = 0; tok < M; ++tok)
        for (int g = 0; g < ng; ++g) {
            int sum = 0;
            for (int qi = 0; qi < QPG; ++qi) {
                const int q = g * QPG + qi;
                u32x4 src[2];
                std::memcpy(src, A + (size_t)tok * K + (size_t)q * QB, QB);
                sum += mfma_stage_quarter<BITS>(src, act.data() + (size_t)tok * tw, q);
            }
            corr[(size_t)g * M + tok] = mfma_corr<BITS>(sum);
        }
    const int row_bytes = K * BITS / 8;
    for (int n = 0; n < N; ++n)
        for (int g = 0; g < ng; ++g)
            for (int tok = 0; tok < M; ++tok) {
                int d = corr[(size_t)g * M + tok];  // accumulator input of the first MFMA
                for (int kb = 0; kb < 4; ++kb) {
                    uint32_t p0, p1 = 0;
                    const uint8_t *grp = B + (size_t)n * row_bytes + (size_t)g * (128 * BITS / 8);
                    if (BITS == 2) {
                        std::memcpy(&p0, grp + kb * 8, 4);
                        std::memcpy(&p1, grp + kb * 8 + 4, 4);
                    } else {
                        std::memcpy(&p0, grp + kb * 4, 4);
                    }
                    uint32_t b0[4], b1[4];
                    mfma_unpack<BITS>(p0, p1, b0, b1);
                    const u32x4 a0 = act[(size_t)tok * tw + g * 8 + 2 * kb];
                    const u32x4 a1 = act[(size_t)tok * tw + g * 8 + 2 * kb + 1];
                    const uint32_t av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
                    for (int j = 0; j < 4; ++j) {
                        d = dot4_i8(av0[j], b0[j], d);
                        d = dot4_i8(av1[j], b1[j], d);
                    }
                }
                G[((size_t)tok * N + n) * ng + g] = d;
            }
}

extern "C" int sim_group_sums_mfma(const int8_t *A, const uint8_t *B, int32_t *G, int M, int N, int K,
                                   int bits) {
    if (K % 128 != 0) return 1;
    if (bits == 2) run_mfma<2>(A, B, G, M, N, K); else run_mfma<1>(A, B, G, M, N, K);
    return 0;
}
