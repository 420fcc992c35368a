// Internal interface of the MFMA GEMM kernel (shared by the Linear and attention
// entry points).
#pragma once
#include "common.hip.h"

namespace et {

struct GemmArgs {
    const _Float16 *A, *B;
    _Float16 *C;
    int M, N, K;
    int lda, ldb, ldc;
    // Problem z of a batch is (outer, inner) = (z / batch_inner, z % batch_inner);
    // operand offsets are outer*s?o + inner*s?i elements.
    int batch_inner;
    long long sAo, sAi, sBo, sBi, sCo, sCi;
    const _Float16 *bias;     // indexed by output column (after c_scatter)
    long long sBias_o, sBias_i;
    const int32_t *a_gather;  // [K] or nullptr
    const int32_t *c_scatter; // [N] or nullptr
    const int32_t *bias_idx;  // [N] or nullptr: bias index of result column n (default: the output column)
    int act;
    // direct-to-LDS kernel only, set by its launcher: tile rows of a group of tiles (x 8 tile columns) that one XCD
    // works on at a time: 4, 2 or 1
    int group_rows;
};

// Launches the MFMA GEMM kernel over batch_outer*batch_inner problems.
int launch_gemm(const GemmArgs &g, int batch_total, bool trans_b, hipStream_t stream);

// The direct-to-LDS kernel (gemm_dma.hip) for problems without an A-column gather whose M, N and K are
// multiples of 16 and whose operands are 16-byte aligned; launch_gemm tries it first.
bool gemm_dma_applies(const GemmArgs &g, int batch_total, bool trans_b);
int launch_gemm_dma(const GemmArgs &g, int batch_total, bool trans_b, hipStream_t stream);

inline GemmArgs gemm_args(const _Float16 *A, const _Float16 *B, _Float16 *C, int M, int N, int K, int lda,
                          int ldb, int ldc) {
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.batch_inner = 1;
    g.act = ET_ACT_NONE;
    return g;
}

}  // namespace et
