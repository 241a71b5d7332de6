// f16 x f16 -> fp32-accumulate -> f16 GEMM on gfx950 MFMA (v_mfma_f32_32x32x16_f16),
// C = alpha op(A) op(B) + beta C, row-major, all four transpose cases, optional
// strided batch (the per-head blocks of attention tensors).
//
// Block tile BM x BN x BK, 256 lanes = 4 wavefronts in a 2 x 2 grid, each wavefront
// owning a (BM/2) x (BN/2) tile of 32 x 32 MFMA accumulators.  Both operands are staged
// in LDS as [row][k] with k contiguous (row = m for A, n for B) and a padded row stride
// so that the 16-byte operand reads of a wavefront hit distinct banks.  An operand whose
// k index is not contiguous in memory (A^T, or B not transposed) is transposed in
// registers on its way from global memory to LDS, so the MFMA read path is the same for
// all four cases.  Global loads for tile t+1 are issued before the MFMAs of tile t and
// land in the other LDS buffer afterwards: one barrier per k tile.
//
// The MFMA is issued with the B fragment as first operand, so a lane ends up with 4
// consecutive columns of one row of C per accumulator group and stores 8 bytes at a time.
#include <stdlib.h>

#include "common.h"
#include "gemm_internal.h"

using namespace cacti;

namespace {

template <int VEC> struct VecT;
template <> struct VecT<8> { typedef uint4 type; };
template <> struct VecT<4> { typedef uint2 type; };
template <> struct VecT<1> { typedef uint16_t type; };

template <int VEC>
__device__ __forceinline__ typename VecT<VEC>::type vzero();
template <> __device__ __forceinline__ uint4 vzero<8>() { return make_uint4(0, 0, 0, 0); }
template <> __device__ __forceinline__ uint2 vzero<4>() { return make_uint2(0, 0); }
template <> __device__ __forceinline__ uint16_t vzero<1>() { return 0; }

template <int VEC>
__device__ __forceinline__ uint16_t vget(const typename VecT<VEC>::type &v, int j)
{
    return reinterpret_cast<const uint16_t *>(&v)[j];
}

constexpr int BM = 128, BN = 128, BK = 32, PAD = 8, LDS_LD = BK + PAD, NT = 256;

// ---- global -> registers ----------------------------------------------------
// K-contiguous operand: tile [ROWS][BK], vectors of VEC halves along k.
template <int ROWS, int VEC>
struct LoadKC {
    static constexpr int CPR = BK / VEC;                  // chunks per row
    static constexpr int ITEMS = ROWS * CPR;
    static constexpr int NL = (ITEMS + NT - 1) / NT;
    typename VecT<VEC>::type st[NL];

    __device__ __forceinline__ void load(const half_t *base, int64_t ld, int64_t row0, int64_t R,
                                         int64_t k0, int64_t K)
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int row = c / CPR, kc = c % CPR;
            const int64_t gr = row0 + row, gk = k0 + kc * VEC;
            if (c < ITEMS && gr < R && gk < K)
                st[it] = *reinterpret_cast<const typename VecT<VEC>::type *>(base + gr * ld + gk);
            else
                st[it] = vzero<VEC>();
        }
    }
    __device__ __forceinline__ void store(half_t *lds)
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int row = c / CPR, kc = c % CPR;
            if (c < ITEMS)
                *reinterpret_cast<typename VecT<VEC>::type *>(lds + row * LDS_LD + kc * VEC) =
                    st[it];
        }
    }
};

// K-strided operand: memory is [k][row]; blocks of 4 k x VEC rows, transposed in registers.
template <int ROWS, int VEC>
struct LoadKS {
    static constexpr int RC = ROWS / VEC;                 // row chunks
    static constexpr int ITEMS = (BK / 4) * RC;
    static constexpr int NL = (ITEMS + NT - 1) / NT;
    typename VecT<VEC>::type st[NL][4];

    __device__ __forceinline__ void load(const half_t *base, int64_t ld, int64_t row0, int64_t R,
                                         int64_t k0, int64_t K)
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int rc = c % RC, kq = c / RC;
            const int64_t gr = row0 + rc * VEC;
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                const int64_t gk = k0 + kq * 4 + kk;
                if (c < ITEMS && gr < R && gk < K)
                    st[it][kk] =
                        *reinterpret_cast<const typename VecT<VEC>::type *>(base + gk * ld + gr);
                else
                    st[it][kk] = vzero<VEC>();
            }
        }
    }
    __device__ __forceinline__ void store(half_t *lds)
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int rc = c % RC, kq = c / RC;
            if (c < ITEMS) {
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    uint2 w;
                    w.x = (uint32_t)vget<VEC>(st[it][0], j) | ((uint32_t)vget<VEC>(st[it][1], j) << 16);
                    w.y = (uint32_t)vget<VEC>(st[it][2], j) | ((uint32_t)vget<VEC>(st[it][3], j) << 16);
                    *reinterpret_cast<uint2 *>(lds + (rc * VEC + j) * LDS_LD + kq * 4) = w;
                }
            }
        }
    }
};

template <bool KSTRIDED, int ROWS, int VEC> struct Loader;
template <int ROWS, int VEC> struct Loader<false, ROWS, VEC> : LoadKC<ROWS, VEC> {};
template <int ROWS, int VEC> struct Loader<true, ROWS, VEC> : LoadKS<ROWS, VEC> {};

template <bool TA, bool TB, int VEC>
__global__ void __launch_bounds__(NT) gemm_f16_kernel(GemmArgs p)
{
    __shared__ __attribute__((aligned(16))) half_t As[2][BM * LDS_LD];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][BN * LDS_LD];

    const int tile = blockIdx.x;
    const int tm = tile % p.tiles_m, tn = tile / p.tiles_m;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t bz = blockIdx.z;
    const half_t *A = p.A + bz * p.sa;
    const half_t *B = p.B + bz * p.sb;
    half_t *C = p.C + bz * p.sc;

    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int wm = wid & 1, wn = wid >> 1;
    const int l32 = lane & 31, lh = lane >> 5;

    // A is k-strided in memory when transposed; B when not transposed
    Loader<TA, BM, VEC> la;
    Loader<!TB, BN, VEC> lb;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    int nk = (int)((p.K + BK - 1) / BK), kt0 = 0;
    if (p.tri == 1 && n0 > m0 + BM - 1) return;               // uniform for the block
    if (p.tri == 2) nk = min(nk, (int)((m0 + BM + BK - 1) / BK));
    if (p.tri == 3) kt0 = (int)(m0 / BK);
    la.load(A, p.lda, m0, p.M, (int64_t)kt0 * BK, p.K);
    lb.load(B, p.ldb, n0, p.N, (int64_t)kt0 * BK, p.K);
    la.store(As[kt0 & 1]);
    lb.store(Bs[kt0 & 1]);
    __syncthreads();

    for (int kt = kt0; kt < nk; kt++) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {
            la.load(A, p.lda, m0, p.M, (int64_t)(kt + 1) * BK, p.K);
            lb.load(B, p.ldb, n0, p.N, (int64_t)(kt + 1) * BK, p.K);
        }
        const half_t *as = As[cur] + (wm * 64 + l32) * LDS_LD + lh * 8;
        const half_t *bs = Bs[cur] + (wn * 64 + l32) * LDS_LD + lh * 8;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            half8_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[i] = *reinterpret_cast<const half8_t *>(as + i * 32 * LDS_LD + ks * 16);
                bf[i] = *reinterpret_cast<const half8_t *>(bs + i * 32 * LDS_LD + ks * 16);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] =
                        __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            la.store(As[cur ^ 1]);
            lb.store(Bs[cur ^ 1]);
        }
        __syncthreads();
    }

    // epilogue: lane holds row m = .. + l32 and, per accumulator group q, the 4
    // consecutive columns n = .. + 8 q + 4 lh + {0..3}
    const bool has_beta = p.beta != 0.f;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int64_t m = m0 + wm * 64 + i * 32 + l32;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int64_t n = n0 + wn * 64 + j * 32 + q * 8 + lh * 4;
                half_t *cp = C + m * p.ldc + n;
                if (VEC >= 4) {
                    if (n < p.N) {
                        half4_t o;
                        if (has_beta) {
                            half4_t old = *reinterpret_cast<const half4_t *>(cp);
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                o[r] = f2h(p.alpha * acc[i][j][q * 4 + r] + p.beta * h2f(old[r]));
                        } else {
#pragma unroll
                            for (int r = 0; r < 4; r++) o[r] = f2h(p.alpha * acc[i][j][q * 4 + r]);
                        }
                        *reinterpret_cast<half4_t *>(cp) = o;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        if (n + r < p.N) {
                            float v = p.alpha * acc[i][j][q * 4 + r];
                            if (has_beta) v += p.beta * h2f(cp[r]);
                            cp[r] = f2h(v);
                        }
                    }
                }
            }
        }
    }
}

template <bool TA, bool TB>
int launch_vec(int vec, const GemmArgs &p, int64_t nblk, hipStream_t st)
{
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)nblk), block(NT);
    if (vec == 8)
        hipLaunchKernelGGL((gemm_f16_kernel<TA, TB, 8>), grid, block, 0, st, p);
    else if (vec == 4)
        hipLaunchKernelGGL((gemm_f16_kernel<TA, TB, 4>), grid, block, 0, st, p);
    else
        hipLaunchKernelGGL((gemm_f16_kernel<TA, TB, 1>), grid, block, 0, st, p);
    return launch_status("gemm_f16");
}

inline bool mult(int64_t v, int64_t a) { return v % a == 0; }

}  // namespace

CACTI_API int cacti_hip_gemm_f16_strided_batched_tri(int ta, int tb, int64_t nblk, int64_t M,
                                                     int64_t N, int64_t K, float alpha, const void *A,
                                                     int64_t lda, int64_t stride_a, const void *B,
                                                     int64_t ldb, int64_t stride_b, float beta,
                                                     void *C, int64_t ldc, int64_t stride_c, int tri,
                                                     void *stream)
{
    CACTI_REQUIRE(tri >= 0 && tri <= 3, CACTI_E_INVALID, "gemm: tri must be 0..3");
    CACTI_REQUIRE(tri == 0 || (tri == 1 && M == N) || (tri == 2 && !ta && M == K) ||
                      (tri == 3 && ta && M == K),
                  CACTI_E_INVALID, "gemm: tri=%d needs a square (sequence x sequence) operand", tri);
    CACTI_REQUIRE(A && B && C, CACTI_E_INVALID, "gemm: null operand");
    CACTI_REQUIRE(M > 0 && N > 0 && K > 0 && nblk > 0 && nblk <= 65535, CACTI_E_INVALID,
                  "gemm: bad shape M=%lld N=%lld K=%lld nblk=%lld", (long long)M, (long long)N,
                  (long long)K, (long long)nblk);
    CACTI_REQUIRE(beta == 0.f || beta == 1.f, CACTI_E_INVALID, "gemm: beta must be 0 or 1");
    CACTI_REQUIRE(lda >= (ta ? M : K) && ldb >= (tb ? K : N) && ldc >= N, CACTI_E_INVALID,
                  "gemm: leading dimension smaller than the row length");
    CACTI_REQUIRE(aligned(A, 2) && aligned(B, 2) && aligned(C, 2), CACTI_E_INVALID,
                  "gemm: operands must be 2-byte aligned");
    GemmArgs p;
    p.M = M; p.N = N; p.K = K; p.alpha = alpha; p.beta = beta;
    p.A = (const half_t *)A; p.lda = lda; p.sa = stride_a;
    p.B = (const half_t *)B; p.ldb = ldb; p.sb = stride_b;
    p.C = (half_t *)C; p.ldc = ldc; p.sc = stride_c;
    p.tiles_m = (int)((M + BM - 1) / BM);
    p.tiles_n = (int)((N + BN - 1) / BN);
    p.tri = tri;
    CACTI_REQUIRE((int64_t)p.tiles_m * p.tiles_n < (1LL << 31), CACTI_E_NOTIMPL, "gemm: too many tiles");

    // widest vector every operand supports: contiguous extent, leading dimension,
    // batch stride and base address must all be multiples of it
    const int64_t ca = ta ? M : K, cb = tb ? K : N;
    int vec = 1;
    for (int v : {8, 4}) {
        const bool multi = nblk > 1;
        if (mult(ca, v) && mult(cb, v) && mult(N, v) && mult(lda, v) && mult(ldb, v) &&
            mult(ldc, v) && (!multi || (mult(stride_a, v) && mult(stride_b, v) && mult(stride_c, v))) &&
            aligned(A, 2 * v) && aligned(B, 2 * v) && aligned(C, 2 * v)) {
            vec = v;
            break;
        }
    }
    hipStream_t st = (hipStream_t)stream;
    p.win = 0;
    p.ztab = 0;
    if (vec >= 4 && !ta && tb && K <= 128 && beta == 0.f && tri <= 1)
        return gemm_nt_smallk_launch(p, nblk, st);
    // one to four rows against a weight matrix (decoding): a stream over B
    if (vec == 8 && !ta && tb && M <= 4 && nblk == 1 && beta == 0.f && tri == 0)
        return gemm_skinny_nt_launch(M, N, K, alpha, p.A, lda, p.B, ldb, p.C, ldc, st);
    // The attention products with a [sequence, heads, head_dim] operand: A (probabilities or
    // their adjoint) is 16-byte aligned, B and C are per-head slabs whose offset (head_dim 100)
    // is only a multiple of 8 bytes.  Addressed from the 16-byte boundary below each slab they
    // take the direct-load path; the extra columns read stay inside the columns the blocks
    // cover in one row of B (checked here).
    if (vec == 4 && !tb && nblk > 1 && mult(K, 64) && mult(ta ? M : K, 8) && mult(lda, 8) &&
        mult(stride_a, 8) && aligned(A, 16) && mult(ldb, 8) && mult(ldc, 8) && aligned(B, 16) &&
        aligned(C, 16) && (stride_b & 7) == (stride_c & 7)) {
        const int64_t row_end = (nblk - 1) * stride_b + N;
        bool inside = stride_b >= 0 && row_end <= ldb;
        for (int64_t bz = 0; bz < nblk && inside; bz++) {
            const int64_t shift = (bz * stride_b) & 7;
            const int64_t first = bz * stride_b - shift;          // >= 0: bz * stride_b >= shift
            inside = first + (shift + N + 7) / 8 * 8 <= row_end;
        }
        if (inside) {
            p.win = 1;
            return gemm_mfma_launch(ta, tb, p, nblk, 8, -1, st);
        }
    }
    if (vec >= 4) return gemm_mfma_launch(ta, tb, p, nblk, vec, -1, st);
    if (!ta && !tb) return launch_vec<false, false>(vec, p, nblk, st);
    if (!ta && tb) return launch_vec<false, true>(vec, p, nblk, st);
    if (ta && !tb) return launch_vec<true, false>(vec, p, nblk, st);
    return launch_vec<true, true>(vec, p, nblk, st);
}

// Pointer-array batch (cublasGemmBatchedEx shape): the products must have one shape; up to
// kMaxPtrBatch of them share a launch when every operand is 16-byte aligned, otherwise they run
// one after another.
CACTI_API int cacti_hip_gemm_f16_batched(int ta, int tb, int64_t nblk, int64_t M, int64_t N, int64_t K,
                                         float alpha, const void *const *A, int64_t lda, const void *const *B,
                                         int64_t ldb, float beta, void *const *C, int64_t ldc, void *stream)
{
    CACTI_REQUIRE(nblk > 0 && A && B && C, CACTI_E_INVALID, "gemm_batched: null pointer array or empty batch");
    for (int64_t z = 0; z < nblk; z++)
        CACTI_REQUIRE(A[z] && B[z] && C[z], CACTI_E_INVALID, "gemm_batched: null operand in block %lld", (long long)z);
    const int64_t ca = ta ? M : K, cb = tb ? K : N;
    bool fast = M > 0 && N > 0 && K > 0 && (beta == 0.f || beta == 1.f) && mult(ca, 8) && mult(cb, 8) && mult(N, 8) &&
                mult(lda, 8) && mult(ldb, 8) && mult(ldc, 8) && lda >= ca && ldb >= cb && ldc >= N && K > 128;
    for (int64_t z = 0; z < nblk && fast; z++) fast = aligned(A[z], 16) && aligned(B[z], 16) && aligned(C[z], 16);
    for (int64_t z0 = 0; z0 < nblk; z0 += kMaxPtrBatch) {
        const int64_t cnt = nblk - z0 < kMaxPtrBatch ? nblk - z0 : kMaxPtrBatch;
        if (!fast || cnt == 1) {
            for (int64_t z = z0; z < z0 + cnt; z++) {
                const int rc = cacti_hip_gemm_f16(ta, tb, M, N, K, alpha, A[z], lda, B[z], ldb, beta, C[z], ldc, stream);
                if (rc) return rc;
            }
            continue;
        }
        GemmArgs p;
        p.M = M; p.N = N; p.K = K; p.alpha = alpha; p.beta = beta;
        p.A = (const half_t *)A[z0]; p.lda = lda; p.sa = 0;
        p.B = (const half_t *)B[z0]; p.ldb = ldb; p.sb = 0;
        p.C = (half_t *)C[z0]; p.ldc = ldc; p.sc = 0;
        p.tiles_m = (int)((M + BM - 1) / BM);
        p.tiles_n = (int)((N + BN - 1) / BN);
        p.tri = 0;
        p.win = 0;
        p.ztab = 1;
        for (int64_t z = 0; z < kMaxPtrBatch; z++) {
            const int64_t zz = z0 + (z < cnt ? z : 0);
            p.za[z] = (const half_t *)A[zz] - p.A;
            p.zb[z] = (const half_t *)B[zz] - p.B;
            p.zc[z] = (half_t *)C[zz] - p.C;
        }
        const int rc = gemm_mfma_launch(ta, tb, p, cnt, 8, -1, (hipStream_t)stream);
        if (rc) return rc;
    }
    return 0;
}

CACTI_API int cacti_hip_gemm_f16_strided_batched(int ta, int tb, int64_t nblk, int64_t M, int64_t N,
                                                 int64_t K, float alpha, const void *A, int64_t lda,
                                                 int64_t stride_a, const void *B, int64_t ldb,
                                                 int64_t stride_b, float beta, void *C, int64_t ldc,
                                                 int64_t stride_c, void *stream)
{
    return cacti_hip_gemm_f16_strided_batched_tri(ta, tb, nblk, M, N, K, alpha, A, lda, stride_a, B,
                                                  ldb, stride_b, beta, C, ldc, stride_c, 0, stream);
}

CACTI_API int cacti_hip_gemm_f16(int ta, int tb, int64_t M, int64_t N, int64_t K, float alpha,
                                 const void *A, int64_t lda, const void *B, int64_t ldb, float beta,
                                 void *C, int64_t ldc, void *stream)
{
    return cacti_hip_gemm_f16_strided_batched(ta, tb, 1, M, N, K, alpha, A, lda, 0, B, ldb, 0, beta,
                                              C, ldc, 0, stream);
}

// Column-major C[m x n] = alpha op(a) op(b) + beta C is the row-major product
// C^T[n x m] = op(b)^T op(a)^T, i.e. the row-major kernel with the operands swapped:
// a column-major "N" operand is a row-major transposed one's transpose.
CACTI_API int cacti_hip_gemm_colmajor_f16(int tr_a, int tr_b, int m, int n, int k,
                                          const float *alpha, const void *a, int lda, const void *b,
                                          int ldb, const float *beta, void *c, int ldc, void *stream)
{
    CACTI_REQUIRE(alpha && beta, CACTI_E_INVALID, "gemm_colmajor: null alpha/beta");
    // row-major view: C'[n,m]; first operand op'(b): col-major b (k x n if N) is row-major [n,k]
    // = "transposed" storage of the K x N... expressed through (ta', tb') below.
    // col-major b, tr_b = N: memory holds b[k][n] at n*ldb + k  -> row-major [n][k]: op'(A') = A' (M'=n, K=k): ta' = 0
    // col-major b, tr_b = T: memory holds b[n][k] at k*ldb + n  -> row-major [k][n]: ta' = 1
    // col-major a, tr_a = N: memory a[m][k] at k*lda + m        -> row-major [k][m] = K x N' : tb' = 0
    // col-major a, tr_a = T: memory a[k][m] at m*lda + k        -> row-major [m][k] = N' x K : tb' = 1
    return cacti_hip_gemm_f16(tr_b ? 1 : 0, tr_a ? 1 : 0, n, m, k, *alpha, b, ldb, a, lda, *beta, c,
                              ldc, stream);
}
