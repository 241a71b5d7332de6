// C[M,N] = f16(alpha * A[M,K] B[N,K]^T) for M <= 4 rows (decoding: one or a few tokens against a
// weight matrix).  The product is a stream over B: every byte of the weights is read once and
// used M times, so the kernel is built for HBM, not for the matrix cores.
//
// A workgroup of 256 lanes owns R = 4 rows of B (4 output columns) and splits K over its lanes
// in 16-byte pieces; each lane issues its 4 row loads together, accumulates M x 4 fp32 sums, and
// the sums are reduced over the wave (cross-lane adds) and over the 4 waves (LDS).  N / 4
// workgroups: 800 for N = 3200, 8 resident per CU, i.e. some 200 KiB of weight loads in flight
// per CU.  A (a few KiB) is re-read from L2 by every workgroup.
#include "gemm_internal.h"

namespace cacti {

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 4;

template <int M>
__global__ void __launch_bounds__(kThreads)
gemm_skinny_nt_kernel(int64_t N, int64_t K, float alpha, const half_t *__restrict__ A, int64_t lda,
                      const half_t *__restrict__ B, int64_t ldb, half_t *__restrict__ C, int64_t ldc)
{
    __shared__ float part[kThreads / 64][M * kRows];
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t n0 = (int64_t)blockIdx.x * kRows;
    float acc[M][kRows];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int r = 0; r < kRows; r++) acc[m][r] = 0.f;
    // rows past N re-read the last row (their sums are dropped)
    const half_t *brow[kRows];
#pragma unroll
    for (int r = 0; r < kRows; r++) brow[r] = B + (n0 + r < N ? n0 + r : N - 1) * ldb;
    const int64_t chunks = K / 8;
    for (int64_t c = tid; c < chunks; c += kThreads) {
        half8_t b[kRows];
        h8 a[M];
#pragma unroll
        for (int r = 0; r < kRows; r++)
            b[r] = __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(brow[r]) + c);
#pragma unroll
        for (int m = 0; m < M; m++) a[m] = ld8(A + m * lda + c * 8);
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++)
#pragma unroll
                for (int k = 0; k < 8; k++) acc[m][r] += h2f(a[m].v[k]) * h2f(b[r][k]);
    }
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int r = 0; r < kRows; r++) {
            float v = acc[m][r];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            if (lane == 0) part[wid][m * kRows + r] = v;
        }
    __syncthreads();
    if (tid < M * kRows) {
        const int m = tid / kRows, r = tid % kRows;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kThreads / 64; w++) v += part[w][tid];
        if (n0 + r < N) C[m * ldc + n0 + r] = f2h(alpha * v);
    }
}

}  // namespace

// A, B rows 16-byte aligned (lda, ldb multiples of 8), K % 8 == 0, 1 <= M <= 4
int gemm_skinny_nt_launch(int64_t M, int64_t N, int64_t K, float alpha, const half_t *A, int64_t lda,
                          const half_t *B, int64_t ldb, half_t *C, int64_t ldc, hipStream_t st)
{
    const dim3 grid((unsigned)((N + kRows - 1) / kRows)), block(kThreads);
    switch (M) {
        case 1: hipLaunchKernelGGL((gemm_skinny_nt_kernel<1>), grid, block, 0, st, N, K, alpha, A, lda, B, ldb, C, ldc); break;
        case 2: hipLaunchKernelGGL((gemm_skinny_nt_kernel<2>), grid, block, 0, st, N, K, alpha, A, lda, B, ldb, C, ldc); break;
        case 3: hipLaunchKernelGGL((gemm_skinny_nt_kernel<3>), grid, block, 0, st, N, K, alpha, A, lda, B, ldb, C, ldc); break;
        default: hipLaunchKernelGGL((gemm_skinny_nt_kernel<4>), grid, block, 0, st, N, K, alpha, A, lda, B, ldb, C, ldc); break;
    }
    return launch_status("gemm_skinny_nt");
}

}  // namespace cacti
