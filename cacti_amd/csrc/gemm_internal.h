// Shared between the generic GEMM kernel (any alignment) and the 16-byte-aligned fast path.
#pragma once
#include "common.h"

namespace cacti {

struct GemmArgs {
    int64_t M, N, K;
    float alpha, beta;
    const half_t *A;
    int64_t lda, sa;
    const half_t *B;
    int64_t ldb, sb;
    half_t *C;
    int64_t ldc, sc;
    int tiles_m, tiles_n;
    // triangular structure of square attention operands (0 = none):
    //  1: only the lower triangle (n <= m) of C is wanted: tiles wholly above it are skipped
    //     and left unwritten;
    //  2: op(A) = A is lower triangular (zero for k > m): the k loop stops at the tile's
    //     last row;
    //  3: op(A) = A^T with A lower triangular (zero for k < m): the k loop starts at the
    //     tile's first row.
    // For 2 and 3 the entries of A above the diagonal must be zero up to the next multiple
    // of 256 columns; beyond that they are never read.
    int tri;
    int gm, xcd;          // tile walk: rows per group; 1 = XCD-banded numbering
    int pair;             // 1: a workgroup computes tile rows r and tiles_m - 1 - r (tri 2 / 3)
    // 1: B ([K][N] row-major) and C are addressed per block from the 16-byte boundary at or
    // below their first column (column window); set by the entry point when A is 16-byte
    // aligned and B, C are only 8-byte aligned because of their batch stride
    int win;
    // 1: the blocks of the batch are separate arrays: block z starts at A + za[z], B + zb[z],
    // C + zc[z] (element offsets) instead of z times the batch strides; at most kMaxPtrBatch blocks
    int ztab;
    int64_t za[4], zb[4], zc[4];
};
constexpr int kMaxPtrBatch = 4;
constexpr int kTriPad = 256;

// tile < 0: chosen by shape
// align = 8 (16-byte aligned operands) or 4 (8-byte aligned, e.g. head_dim 100)
int gemm_mfma_launch(int ta, int tb, const GemmArgs &p, int64_t nblk, int align, int tile,
                     hipStream_t st);

// C = f16(alpha A B^T) with K <= 128 (attention scores): A [M,K], B [N,K] row-major, rows
// 8-byte aligned, K % 4 == 0, beta = 0, tri 0 or 1
int gemm_nt_smallk_launch(const GemmArgs &p, int64_t nblk, hipStream_t st);

// C[M,N] = f16(alpha A B^T) for 1 <= M <= 4: a stream over B ([N,K] row-major, rows 16-byte
// aligned, K % 8 == 0), beta = 0; A rows 16-byte aligned
int gemm_skinny_nt_launch(int64_t M, int64_t N, int64_t K, float alpha, const half_t *A, int64_t lda,
                          const half_t *B, int64_t ldb, half_t *C, int64_t ldc, hipStream_t st);

}  // namespace cacti
