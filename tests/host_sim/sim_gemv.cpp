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
