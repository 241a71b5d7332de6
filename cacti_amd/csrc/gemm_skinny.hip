// C[M,N] = f16(alpha * A[M,K] B[N,K]^T) for M <= 4 rows (decoding: one or a few positions against
// a weight matrix).  The product is a stream over B: every byte of the weights is read once and
// used M times, so the kernel is built for HBM, not for the matrix cores.
//
// A workgroup of 256 lanes owns R = 4 rows of B (4 output columns) and splits K over its lanes
// in 16-byte pieces; a lane issues the loads of 2 or 4 pieces x 4 rows before it uses the first,
// accumulates M x 4 fp32 sums with v_dot2_f32_f16 (the scalar form, 3 instructions per product
// with the conversions, made the kernel compute-bound), and the sums are reduced over the wave (cross-lane adds) and
// over the 4 waves (LDS).  N / 4 workgroups: 800 for N = 3200, 8 resident per CU.  A (a few KiB)
// is re-read from L2 by every workgroup.
//
// Two fusions keep a decoding step from paying a launch for every small thunk:
//  * NORM: A is not read but formed per workgroup as the RMSNorm of a row x (optionally of the
//    residual sum f16(x + x2), which workgroup 0 also writes out): the lanes' own pieces of the
//    row give the sum of squares (every piece of the row belongs to exactly one lane), one
//    workgroup reduction, then a = f16(w * (x * rinv)) exactly as the RMSNorm kernel rounds it.
//  * GATE: two weight matrices share the rows (gate and up projection); the epilogue stores
//    f16(f16(silu(g)) * u) of the two rounded products, as the SiLU-gate kernel computes it.
//  * QKV: one launch covers the query, key and value projections; a workgroup owns two rotation
//    pairs of a head, rotates queries and keys in the epilogue and adds keys and values to the
//    cache rows of the new positions.
#include "gemm_internal.h"

namespace cacti {

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 4;
constexpr int kMaxPre = 4;                 // pieces of K per lane whose loads are in flight together (2 or 4)

struct SkinnyArgs {
    int64_t N, K;
    float alpha;
    const half_t *A;         // [M, lda] (plain) or the row source x (NORM)
    int64_t lda;
    const half_t *x2;        // NORM: optional second summand of the row
    const half_t *w;         // NORM: norm weights [K]
    float eps;
    half_t *sum_out;         // NORM with x2: the residual sum [M, lda], written by workgroup 0
    const half_t *B;         // [N, ldb]
    const half_t *B2;        // GATE: the second weight matrix [N, ldb]; QKV: the key projection
    int64_t ldb;
    half_t *C;               // QKV: the rotated queries [M, ldc]
    int64_t ldc;
    // QKV: value projection, position tables (row 0 = the first new position), caches (row 0 = the
    // first new position, pitch ldc), heads
    const half_t *B3;
    const half_t *cos16, *sin16;
    half_t *kc, *vc;
    int H, Dh;
};
enum : int { E_PLAIN = 0, E_GATE = 1, E_QKV = 2 };

__device__ __forceinline__ float block_sum(float v, float *scratch)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; w++) r += scratch[w];
    return r;
}

// sum of 8 products, fp32 accumulate: four v_dot2_f32_f16 (no conversions, two products each)
__device__ __forceinline__ float dot8(const half8_t &a, const half8_t &b, float acc)
{
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const half2_t a2 = {a[2 * i], a[2 * i + 1]}, b2 = {b[2 * i], b[2 * i + 1]};
        acc = __builtin_amdgcn_fdot2(a2, b2, acc, false);
    }
    return acc;
}

template <int M, bool NORM, int EPI, int kPre>
__global__ void __launch_bounds__(kThreads)
gemm_skinny_nt_kernel(SkinnyArgs p)
{
    constexpr bool GATE = EPI == E_GATE;
    constexpr int NB = GATE ? 2 : 1;
    __shared__ float part[kThreads / 64][NB * M * kRows];
    __shared__ float scratch[kThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int64_t n0 = (int64_t)blockIdx.x * kRows;
    float acc[NB][M][kRows];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) acc[b][m][r] = 0.f;
    // rows past N re-read the last row (their sums are dropped)
    const half_t *brow[NB][kRows];
    int64_t col[kRows];
    if (EPI == E_QKV) {
        // the workgroup owns two rotation pairs of one head: columns d, d + 1, d + Dh/2, d + 1 + Dh/2;
        // blockIdx.y picks the query, key or value projection
        const int hf = p.Dh / 2, per_head = hf / 2;
        const int head = blockIdx.x / per_head, d0 = 2 * (blockIdx.x - head * per_head);
        const half_t *Bsel = blockIdx.y == 0 ? p.B : blockIdx.y == 1 ? p.B2 : p.B3;
#pragma unroll
        for (int r = 0; r < kRows; r++) {
            col[r] = (int64_t)head * p.Dh + d0 + (r & 1) + (r >> 1) * hf;
            brow[0][r] = Bsel + col[r] * p.ldb;
        }
    } else {
#pragma unroll
        for (int r = 0; r < kRows; r++) {
            col[r] = n0 + r;
            const int64_t n = n0 + r < p.N ? n0 + r : p.N - 1;
            brow[0][r] = p.B + n * p.ldb;
            if (GATE) brow[NB - 1][r] = p.B2 + n * p.ldb;
        }
    }
    const int64_t chunks = p.K / 8;
    for (int64_t base = 0; base < chunks; base += (int64_t)kPre * kThreads) {
        half8_t b[kPre][NB][kRows];
        h8 a[kPre][M];
        // Every load of the batch is issued before the first use, unconditionally (pieces past the
        // row re-read its last piece): a load inside a branch is waited for at the end of the branch.
#pragma unroll
        for (int j = 0; j < kPre; j++) {
            const int64_t cr = base + j * kThreads + tid, c = cr < chunks ? cr : chunks - 1;
#pragma unroll
            for (int q = 0; q < NB; q++)
#pragma unroll
                for (int r = 0; r < kRows; r++)
                    b[j][q][r] = __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(brow[q][r]) + c);
#pragma unroll
            for (int m = 0; m < M; m++) a[j][m] = ld8(p.A + m * p.lda + c * 8);
        }
        if (NORM) {
            // the whole row is in this one batch (K <= 8 * kPre * kThreads, seen to by the launcher)
            h8 wv[kPre], x2v[kPre][M];
#pragma unroll
            for (int j = 0; j < kPre; j++) {
                const int64_t cr = base + j * kThreads + tid, c = cr < chunks ? cr : chunks - 1;
                wv[j] = ld8(p.w + c * 8);
                if (p.x2) {                                       // uniform over the launch
#pragma unroll
                    for (int m = 0; m < M; m++) x2v[j][m] = ld8(p.x2 + m * p.lda + c * 8);
                }
            }
#pragma unroll
            for (int m = 0; m < M; m++) {
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < kPre; j++) {
                    const int64_t c = base + j * kThreads + tid;
                    if (c < chunks) {
                        if (p.x2) {
#pragma unroll
                            for (int i = 0; i < 8; i++) a[j][m].v[i] = f2h(h2f(a[j][m].v[i]) + h2f(x2v[j][m].v[i]));
                            if (blockIdx.x == 0 && blockIdx.y == 0 && p.sum_out) st8(p.sum_out + m * p.lda + c * 8, a[j][m]);
                        }
#pragma unroll
                        for (int i = 0; i < 8; i++) {
                            const float f = h2f(a[j][m].v[i]);
                            ss += f * f;
                        }
                    }
                }
                ss = block_sum(ss, scratch);
                const float rinv = 1.0f / sqrtf(ss / (float)p.K + p.eps);
#pragma unroll
                for (int j = 0; j < kPre; j++) {
                    const int64_t c = base + j * kThreads + tid;
                    if (c < chunks) {
#pragma unroll
                        for (int i = 0; i < 8; i++) a[j][m].v[i] = f2h(h2f(wv[j].v[i]) * (h2f(a[j][m].v[i]) * rinv));
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kPre; j++) {
            const int64_t c = base + j * kThreads + tid;
            if (c < chunks) {
#pragma unroll
                for (int m = 0; m < M; m++) {
                    half8_t av;
#pragma unroll
                    for (int k = 0; k < 8; k++) av[k] = a[j][m].v[k];
#pragma unroll
                    for (int q = 0; q < NB; q++)
#pragma unroll
                        for (int r = 0; r < kRows; r++) acc[q][m][r] = dot8(av, b[j][q][r], acc[q][m][r]);
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NB; q++)
#pragma unroll
        for (int m = 0; m < M; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) {
                float v = acc[q][m][r];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
                if (lane == 0) part[wid][(q * M + m) * kRows + r] = v;
            }
    __syncthreads();
    if (EPI == E_QKV) {
        // rotate (queries, keys) and add to the caches (keys, values) with the rounding points of
        // the separate thunks: y = f16(f16(x cos) + f16(rot(x) sin)), cache = f16(cache + y)
        __shared__ float xr[M][kRows];
        const int m = tid / kRows, r = tid % kRows;
        if (tid < M * kRows) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kThreads / 64; w++) v += part[w][m * kRows + r];
            xr[m][r] = rnd16(p.alpha * v);
        }
        __syncthreads();
        if (tid < M * kRows) {
            float y = xr[m][r];
            if (blockIdx.y < 2) {
                const bool left = r < 2;
                const float xp = xr[m][r ^ 2];
                const int64_t d = col[r] % p.Dh;
                const float cs = h2f(p.cos16[m * p.Dh + d]), sn = h2f(p.sin16[m * p.Dh + d]);
                y = rnd16(rnd16(y * cs) + rnd16((left ? -xp : xp) * sn));
            }
            if (blockIdx.y == 0) {
                p.C[m * p.ldc + col[r]] = f2h(y);
            } else {
                half_t *dst = (blockIdx.y == 1 ? p.kc : p.vc) + m * p.ldc + col[r];
                *dst = f2h(h2f(*dst) + y);
            }
        }
        return;
    }
    if (tid < M * kRows) {
        const int m = tid / kRows, r = tid % kRows;
        float v[NB];
#pragma unroll
        for (int q = 0; q < NB; q++) {
            v[q] = 0.f;
#pragma unroll
            for (int w = 0; w < kThreads / 64; w++) v[q] += part[w][(q * M + m) * kRows + r];
        }
        if (n0 + r < p.N) {
            if (GATE) {
                // g = f16(alpha dot_g), u = f16(alpha dot_u); h = f16(f16(silu g) * u)
                const float g = rnd16(p.alpha * v[0]), u = rnd16(p.alpha * v[NB - 1]);
                const float y = rnd16(g / (1.0f + expf(-g)));
                p.C[m * p.ldc + n0 + r] = f2h(y * u);
            } else {
                p.C[m * p.ldc + n0 + r] = f2h(p.alpha * v[0]);
            }
        }
    }
}

template <bool NORM, int EPI, int kPre>
int launch_pre(int64_t M, const SkinnyArgs &p, hipStream_t st)
{
    const dim3 grid((unsigned)((p.N + kRows - 1) / kRows), EPI == E_QKV ? 3 : 1), block(kThreads);
    switch (M) {
        case 1: hipLaunchKernelGGL((gemm_skinny_nt_kernel<1, NORM, EPI, kPre>), grid, block, 0, st, p); break;
        case 2: hipLaunchKernelGGL((gemm_skinny_nt_kernel<2, NORM, EPI, kPre>), grid, block, 0, st, p); break;
        case 3: hipLaunchKernelGGL((gemm_skinny_nt_kernel<3, NORM, EPI, kPre>), grid, block, 0, st, p); break;
        default: hipLaunchKernelGGL((gemm_skinny_nt_kernel<4, NORM, EPI, kPre>), grid, block, 0, st, p); break;
    }
    return launch_status("gemm_skinny_nt");
}

// rows of at most 4096 elements fit two pieces per lane: fewer registers, more workgroups per CU
template <bool NORM, int EPI>
int launch(int64_t M, const SkinnyArgs &p, hipStream_t st)
{
    return p.K <= 8 * 2 * kThreads ? launch_pre<NORM, EPI, 2>(M, p, st) : launch_pre<NORM, EPI, kMaxPre>(M, p, st);
}

}  // namespace

// A, B rows 16-byte aligned (lda, ldb multiples of 8), K % 8 == 0, 1 <= M <= 4
int gemm_skinny_nt_launch(int64_t M, int64_t N, int64_t K, float alpha, const half_t *A, int64_t lda,
                          const half_t *B, int64_t ldb, half_t *C, int64_t ldc, hipStream_t st)
{
    SkinnyArgs p = {N, K, alpha, A, lda, nullptr, nullptr, 0.f, nullptr, B, nullptr, ldb, C, ldc,
                    nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
    return launch<false, E_PLAIN>(M, p, st);
}

}  // namespace cacti

using namespace cacti;

CACTI_API int cacti_hip_rows_norm_matmul_f16(int64_t M, int64_t N, int64_t K, const void *x, const void *x2,
                                             const void *w_norm, float eps, void *sum_out, const void *B,
                                             const void *B_mul, void *C, void *stream)
{
    CACTI_REQUIRE(M >= 1 && M <= 4, CACTI_E_NOTIMPL, "rows_norm_matmul: 1 to 4 rows are handled here (M=%lld)", (long long)M);
    CACTI_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && K <= 8 * kMaxPre * kThreads, CACTI_E_NOTIMPL,
                  "rows_norm_matmul: need K %% 8 == 0 and K <= %d (K=%lld)", 8 * kMaxPre * kThreads, (long long)K);
    CACTI_REQUIRE(x && B && C && (w_norm || (!x2 && !sum_out)), CACTI_E_INVALID, "rows_norm_matmul: null pointer");
    CACTI_REQUIRE(aligned(x, 16) && aligned(x2, 16) && aligned(w_norm, 16) && aligned(sum_out, 16) && aligned(B, 16) &&
                      aligned(B_mul, 16) && aligned(C, 2),
                  CACTI_E_INVALID, "rows_norm_matmul: operands must be 16-byte aligned");
    SkinnyArgs p = {N, K, 1.0f, (const half_t *)x, K, (const half_t *)x2, (const half_t *)w_norm, eps,
                    (half_t *)sum_out, (const half_t *)B, (const half_t *)B_mul, K, (half_t *)C, N,
                    nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
    hipStream_t st = (hipStream_t)stream;
    if (w_norm) return B_mul ? launch<true, E_GATE>(M, p, st) : launch<true, E_PLAIN>(M, p, st);
    return B_mul ? launch<false, E_GATE>(M, p, st) : launch<false, E_PLAIN>(M, p, st);
}

CACTI_API int cacti_hip_rows_qkv_rope_cache_f16(int64_t M, int64_t H, int64_t Dh, const void *x, const void *x2,
                                                const void *w_norm, float eps, void *sum_out, const void *Wq,
                                                const void *Wk, const void *Wv, const void *cos16, const void *sin16,
                                                void *q_rot, void *k_cache_rows, void *v_cache_rows, void *stream)
{
    const int64_t D = H * Dh;
    CACTI_REQUIRE(M >= 1 && M <= 4, CACTI_E_NOTIMPL, "rows_qkv: 1 to 4 rows are handled here (M=%lld)", (long long)M);
    CACTI_REQUIRE(H > 0 && Dh > 0 && Dh % 4 == 0 && D % 8 == 0 && D <= 8 * kMaxPre * kThreads, CACTI_E_NOTIMPL,
                  "rows_qkv: need Dh %% 4 == 0, H*Dh %% 8 == 0 and H*Dh <= %d", 8 * kMaxPre * kThreads);
    CACTI_REQUIRE(x && w_norm && Wq && Wk && Wv && cos16 && sin16 && q_rot && k_cache_rows && v_cache_rows, CACTI_E_INVALID,
                  "rows_qkv: null pointer");
    CACTI_REQUIRE(aligned(x, 16) && aligned(x2, 16) && aligned(w_norm, 16) && aligned(sum_out, 16) && aligned(Wq, 16) &&
                      aligned(Wk, 16) && aligned(Wv, 16) && aligned(cos16, 2) && aligned(sin16, 2) && aligned(q_rot, 2) &&
                      aligned(k_cache_rows, 2) && aligned(v_cache_rows, 2),
                  CACTI_E_INVALID, "rows_qkv: rows and weights must be 16-byte aligned");
    SkinnyArgs p = {D, D, 1.0f, (const half_t *)x, D, (const half_t *)x2, (const half_t *)w_norm, eps,
                    (half_t *)sum_out, (const half_t *)Wq, (const half_t *)Wk, D, (half_t *)q_rot, D,
                    (const half_t *)Wv, (const half_t *)cos16, (const half_t *)sin16, (half_t *)k_cache_rows,
                    (half_t *)v_cache_rows, (int)H, (int)Dh};
    return launch<true, E_QKV>(M, p, (hipStream_t)stream);
}
