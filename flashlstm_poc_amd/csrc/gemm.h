// fp16 x fp16 -> fp32-accumulate MFMA GEMM for gfx950, "NT" form: both operands K-contiguous.
#pragma once
#include "common.h"

namespace flstm_hip {

struct GemmNT {
    // C[M][N] (+)= sum_k A[m][k] * B[n][k]
    const half_t* A; size_t lda;   // M x K, row-major, lda multiple of 8
    const half_t* B; size_t ldb;   // N x K, row-major, ldb multiple of 8
    int M, N, K;                   // K multiple of 32
    // output: exactly one of C16 / C32 is non-null
    half_t* C16; float* C32; size_t ldc;
    float alpha;                   // C = alpha * (A * B^T)
    // split-K: when splits > 1 partial z is written to C32 + z * split_stride (fp32 only)
    int splits; size_t split_stride;
    // optional per-column term: C = alpha * (A * B^T) + bias[n]  (NT form only)
    const float* bias;
    // TN form only: a second B operand.  With B2 set, columns [0, N1) of C come from B (N1 columns) and columns
    // [N1, N) from B2 (N - N1 columns, row pitch ldb2): one launch forms A^T * [B | B2] and reads A once.  N1 must
    // be a multiple of 8; output tiles never straddle the seam (each side is tiled on its own).
    const half_t* B2; size_t ldb2; int N1;
};

// Enqueue on `stream`. Returns hipSuccess or the launch error.
hipError_t launch_gemm_nt(const GemmNT& g, hipStream_t stream);

// Same contraction with k-major operands: A is [K][M] (lda = row pitch, M % 8 == 0), B is [K][N]
// (N % 8 == 0); K is arbitrary.  C[M][N] as above.
hipError_t launch_gemm_tn(const GemmNT& g, hipStream_t stream);

// Number of K slices the launchers really produce when `wanted` are asked for (every slice gets a
// whole number of 64-wide K slabs). Size split-K partial buffers with this.
int gemm_effective_splits(int K, int wanted);
// The split count launch_gemm_tn runs fastest with for fp32 partials of an M x (N1 + N2) product over K (two B operands
// side by side when N2 > 0), at most max_splits.
int gemm_tn_auto_splits(int M, int N1, int N2, int K, int max_splits);

}  // namespace flstm_hip
