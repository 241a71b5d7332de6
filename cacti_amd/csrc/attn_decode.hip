// Attention of one to four new positions over the key / value cache (decoding): the chain
//   block_matmul_scale(q, k_cache^T, 1/sqrt(Dh)) -> f32 -> row-causal mask -> softmax -> f16
//   -> block_matmul(., v_cache)                      src/librarium/llama.rs:895-915
// with the reference's rounding points (scores and probabilities are f16 values, both products
// accumulate in fp32 and round once).
//
// With a single query row per head the tiled GEMM kernels cannot fill the chip (one tile per
// head), so the cache is cut into slices of 128 positions and every (head, slice) pair is a
// workgroup, in three launches:
//   scores : s16[t,h,j] = f16(alpha q[t,h,:] . K[j,h,:]) for the slice's j
//   values : the row maximum and sum over the live columns are recomputed from s16 by every
//            workgroup (a row is a few KiB in L2), p = f16(e / sum) for the slice, partial
//            out[t,h,:] = sum_j p[j] V[j,h,:] per slice, in fp32
//   reduce : the slices' partial sums added in slice order and rounded once.  (Letting the last
//            workgroup of a head do this inside the second launch needs a device-wide fence,
//            which writes back and invalidates a whole L2 on this chip: it cost 40 us.)
// K and V rows of a head are Dh contiguous halves, read as 8-byte pieces: consecutive lanes take
// consecutive pieces, rows follow one another, so every wave access is a few contiguous runs.
#include "common.h"
#include "softmax_math.h"

using namespace cacti;

namespace {

constexpr int kThreads = 256;
constexpr int kSlice = 128;                // cached positions per workgroup
constexpr int kMaxPieces = 32;             // Dh <= 128

struct __attribute__((aligned(8))) h4 {
    half_t v[4];
};

template <int T>
__global__ void __launch_bounds__(kThreads)
decode_scores_kernel(int C, int H, int Dh, float alpha, const half_t *__restrict__ q, int64_t ldq,
                     const half_t *__restrict__ kc, int64_t ldk, int64_t hsk, half_t *__restrict__ s16, int64_t ld)
{
    __shared__ float part[T][kSlice * 25 + kSlice];        // [t][row * pieces + piece], pieces <= 26 here
    const int tid = threadIdx.x, h = blockIdx.y, j0 = blockIdx.x * kSlice;
    const int pieces = Dh / 4;
    const int nrow = min(kSlice, C - j0);
    const int total = nrow * pieces;
    // All of the lane's loads are issued before the first use: at most 13 pieces of K of 8 bytes,
    // each with the matching piece of every query row (those hit in L2).  The loads are
    // unconditional (pieces past the slice re-read its last piece): a load inside a branch is
    // waited for at the end of the branch, which would turn the 13 loads into 13 round trips.
    constexpr int kMaxIter = (kSlice * 25 + kThreads - 1) / kThreads;
    h4 kv[kMaxIter], qv[kMaxIter][T];
#pragma unroll
    for (int it = 0; it < kMaxIter; it++) {
        const int p = min(tid + it * kThreads, total - 1);
        const int r = p / pieces, c = p - r * pieces;
        kv[it] = *reinterpret_cast<const h4 *>(kc + (int64_t)(j0 + r) * ldk + h * hsk + 4 * c);
#pragma unroll
        for (int t = 0; t < T; t++) qv[it][t] = *reinterpret_cast<const h4 *>(q + t * ldq + h * Dh + 4 * c);
    }
#pragma unroll
    for (int it = 0; it < kMaxIter; it++) {
        const int p = tid + it * kThreads;
        if (p < total) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                float a = 0.f;
#pragma unroll
                for (int i = 0; i < 4; i++) a += h2f(qv[it][t].v[i]) * h2f(kv[it].v[i]);
                part[t][p] = a;
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < T * nrow; idx += kThreads) {
        const int t = idx / nrow, r = idx - t * nrow;
        float a = 0.f;
        for (int c = 0; c < pieces; c++) a += part[t][r * pieces + c];
        s16[((int64_t)t * H + h) * ld + j0 + r] = f2h(alpha * a);
    }
}

__device__ __forceinline__ float block_reduce(float v, bool is_max, float *scratch)
{
    v = is_max ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; w++) r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

constexpr int kRowIter = 4;                // 8-column pieces of a score row per lane: rows up to 8192 columns

template <int T>
__global__ void __launch_bounds__(kThreads)
decode_values_kernel(int C, int H, int Dh, int64_t row0, const half_t *__restrict__ s16, int64_t ld,
                     const half_t *__restrict__ vc, int64_t ldv, int64_t hsv, float *__restrict__ partial)
{
    __shared__ float ps[T][kSlice];
    __shared__ float red[8][T][kMaxPieces * 4];
    __shared__ float scratch[kThreads / 64];
    const int tid = threadIdx.x, h = blockIdx.y, split = blockIdx.x, nsplit = gridDim.x;
    const int j0 = split * kSlice;
    const int pieces = Dh / 4;
    const int nrow = min(kSlice, C - j0);
    // Every load of the workgroup is issued here, before the first wait: the slice of V (lane
    // groups of `pieces` lanes, group g takes rows g, g + 8, ...), the score rows (8 columns per
    // lane and step) and the lane's own column of the slice.
    constexpr int G = 8;                       // pieces <= 25 lanes per group: 8 groups fit in 256 lanes
    constexpr int kRowsPerGroup = kSlice / G;
    const int g = tid / pieces, c = tid - g * pieces;
    h4 vv[kRowsPerGroup];
    {
        // unconditional loads (clamped to the slice's last row and to a piece of the head): see above
        const int cc = g < G ? c : 0;
#pragma unroll
        for (int it = 0; it < kRowsPerGroup; it++) {
            const int r = min((g < G ? g : 0) + it * G, nrow - 1);
            vv[it] = *reinterpret_cast<const h4 *>(vc + (int64_t)(j0 + r) * ldv + h * hsv + 4 * cc);
        }
    }
    h8 rowv[T][kRowIter];
    half_t own[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const half_t *sr = s16 + ((int64_t)t * H + h) * ld;
        const int live = (int)min((int64_t)C, (int64_t)t + row0 + 1);
        const int last8 = ((live - 1) / 8) * 8;                        // live >= 1
#pragma unroll
        for (int it = 0; it < kRowIter; it++) {
            const int j8 = min((tid + it * kThreads) * 8, last8);      // rows are 16-byte aligned, ld % 8 == 0
            rowv[t][it] = ld8(sr + j8);
        }
        own[t] = sr[min(j0 + tid, live - 1)];
    }
    // probabilities of the slice: every row's maximum and sum run over all its live columns
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int live = (int)min((int64_t)C, (int64_t)t + row0 + 1);
        float mx = -INFINITY;
#pragma unroll
        for (int it = 0; it < kRowIter; it++) {
            const int j8 = (tid + it * kThreads) * 8;
            if (j8 < live) {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (j8 + i < live) mx = fmaxf(mx, h2f(rowv[t][it].v[i]));
            }
        }
        mx = block_reduce(mx, true, scratch);
        float sum = 0.f;
#pragma unroll
        for (int it = 0; it < kRowIter; it++) {
            const int j8 = (tid + it * kThreads) * 8;
            if (j8 < live) {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (j8 + i < live) sum += exp_nonpos(fmaxf(h2f(rowv[t][it].v[i]) - mx, -100.0f));
            }
        }
        sum = block_reduce(sum, false, scratch);
        const RowDivide div(sum);
        if (tid < kSlice) {
            float p = 0.f;
            if (tid < nrow && j0 + tid < live) p = h2f(f2h(div(exp_nonpos(fmaxf(h2f(own[t]) - mx, -100.0f)))));
            ps[t][tid] = p;
        }
    }
    __syncthreads();
    float acc[T][4];
#pragma unroll
    for (int t = 0; t < T; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[t][i] = 0.f;
    if (g < G) {
#pragma unroll
        for (int it = 0; it < kRowsPerGroup; it++) {
            const int r = g + it * G;
            if (r < nrow) {
#pragma unroll
                for (int t = 0; t < T; t++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[t][i] += ps[t][r] * h2f(vv[it].v[i]);
            }
        }
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[g][t][4 * c + i] = acc[t][i];
    }
    __syncthreads();
    float *mine = partial + ((int64_t)h * nsplit + split) * T * Dh;
    for (int idx = tid; idx < T * Dh; idx += kThreads) {
        const int t = idx / Dh, d = idx - t * Dh;
        float a = 0.f;
        for (int gg = 0; gg < G; gg++) a += red[gg][t][d];
        mine[idx] = a;
    }
}

// out[t,h,:] = f16(sum over the slices, in slice order, of the partial products)
template <int T>
__global__ void __launch_bounds__(128)
decode_reduce_kernel(int nsplit, int Dh, const float *__restrict__ partial, half_t *__restrict__ out, int64_t ldo)
{
    const int h = blockIdx.x;
    const float *all = partial + (int64_t)h * nsplit * T * Dh;
    for (int idx = threadIdx.x; idx < T * Dh; idx += 128) {
        const int t = idx / Dh, d = idx - t * Dh;
        float a = 0.f;
        for (int s = 0; s < nsplit; s++) a += all[(int64_t)s * T * Dh + idx];
        out[(int64_t)t * ldo + h * Dh + d] = f2h(a);
    }
}

}  // namespace

CACTI_API size_t cacti_hip_attn_decode_workspace(int64_t T, int64_t H, int64_t Dh, int64_t C)
{
    if (T <= 0 || H <= 0 || Dh <= 0 || C <= 0) return 0;
    const int64_t ld = (C + 7) / 8 * 8, nsplit = (C + kSlice - 1) / kSlice;
    // scores [T,H,ld] f16, then the per-slice partial outputs [H,nsplit,T,Dh] f32
    return (size_t)((T * H * ld * 2 + 255) / 256 * 256 + H * nsplit * T * Dh * 4);
}

CACTI_API int cacti_hip_attn_decode_f16(int64_t T, int64_t H, int64_t Dh, int64_t C, int64_t initial_row, float alpha,
                                        const void *q, int64_t ldq, const void *k_cache, const void *v_cache,
                                        int64_t ldkv, int64_t head_stride, void *out, int64_t ldo, void *workspace,
                                        size_t workspace_bytes, void *stream)
{
    CACTI_REQUIRE(T >= 1 && T <= 4 && H > 0 && C > 0 && initial_row >= 0, CACTI_E_NOTIMPL,
                  "attn_decode: 1 to 4 rows are handled here (T=%lld)", (long long)T);
    CACTI_REQUIRE(Dh % 4 == 0 && Dh >= 4 && Dh <= 100, CACTI_E_NOTIMPL, "attn_decode: need Dh %% 4 == 0 and Dh <= 100");
    CACTI_REQUIRE(q && k_cache && v_cache && out && workspace, CACTI_E_INVALID, "attn_decode: null pointer");
    CACTI_REQUIRE(C <= (int64_t)kRowIter * kThreads * 8, CACTI_E_NOTIMPL, "attn_decode: at most %d cached positions",
                  kRowIter * kThreads * 8);
    CACTI_REQUIRE(ldq % 4 == 0 && ldkv % 4 == 0 && head_stride % 4 == 0 && aligned(q, 8) && aligned(k_cache, 8) && aligned(v_cache, 8) &&
                      aligned(workspace, 16),
                  CACTI_E_INVALID, "attn_decode: operands must be 8-byte aligned with row pitches that are multiples of 4");
    CACTI_REQUIRE(workspace_bytes >= cacti_hip_attn_decode_workspace(T, H, Dh, C), CACTI_E_INVALID,
                  "attn_decode: workspace too small");
    // columns beyond the last row's position are masked for every row: they are not formed
    const int64_t live = C < T + initial_row ? C : T + initial_row;
    const int64_t ld = (C + 7) / 8 * 8;
    half_t *s16 = static_cast<half_t *>(workspace);
    float *partial = reinterpret_cast<float *>(static_cast<char *>(workspace) + (T * H * ld * 2 + 255) / 256 * 256);
    const dim3 grid((unsigned)((live + kSlice - 1) / kSlice), (unsigned)H), block(kThreads);
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(TT)                                                                                                     \
    do {                                                                                                               \
        hipLaunchKernelGGL((decode_scores_kernel<TT>), grid, block, 0, st, (int)live, (int)H, (int)Dh, alpha,          \
                           (const half_t *)q, ldq, (const half_t *)k_cache, ldkv, head_stride, s16, ld);               \
        hipLaunchKernelGGL((decode_values_kernel<TT>), grid, block, 0, st, (int)live, (int)H, (int)Dh, initial_row, s16, \
                           ld, (const half_t *)v_cache, ldkv, head_stride, partial);                                   \
        hipLaunchKernelGGL((decode_reduce_kernel<TT>), dim3((unsigned)H), dim3(128), 0, st, (int)grid.x, (int)Dh,      \
                           (const float *)partial, (half_t *)out, ldo);                                                \
    } while (0)
    switch (T) {
        case 1: LAUNCH(1); break;
        case 2: LAUNCH(2); break;
        case 3: LAUNCH(3); break;
        default: LAUNCH(4); break;
    }
#undef LAUNCH
    return launch_status("attn_decode");
}
