// Row softmax kernels: causal softmax over attention scores (forward, adjoint) with one
// wavefront per row, and the LM-head softmax / cross-entropy (forward, adjoint) with one
// block per vocabulary row.  Rows are read from HBM once and held in registers.
#include "common.h"
#include "softmax_math.h"

using namespace cacti;

namespace {

// ---------------------------------------------------------------------------
// Causal softmax on [S,H,S]: row (i,h), columns j <= i are live, the rest are -inf.
//   forward: P16 = f16( exp(u - max) / sum ),  u = f32(S16)
//   adjoint: P' as above (fp32), T = P' f32(dP16), dS16 = f16( T - (sum T) P' ), 0 above
//            the diagonal
// (Cast, BlockTriElemAffine src/thunk/op.rs:4189-4278, InnerSoftmax :3257-3383,
//  InnerSoftmaxPostAdj :3386-3457.)
constexpr int kRowsPerBlock = 4;

// A wave owns one row and holds it in registers; chunk c covers columns [512 c, 512 c + 512)
// (8 per lane).  Per chunk the wave is in one of three uniform states: wholly above the
// diagonal (skipped), wholly below it (no masking code at all) or on it (per-element masks).
template <int CH, bool BWD>
__global__ void __launch_bounds__(kRowsPerBlock * 64)
causal_softmax_kernel(int64_t S, int H, const half_t *__restrict__ s16,
                      const half_t *__restrict__ dp16, half_t *__restrict__ out)
{
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + wid;
    if (row >= S * H) return;
    const int i = (int)(row / H);                 // query position
    const int nchunk = (int)(S / 8);
    const half_t *sr = s16 + row * S;
    const half_t *gr = BWD ? dp16 + row * S : nullptr;
    float e[CH][8];
    h8 g[CH], sv[CH];
    float mx = -INFINITY;
    // Forward: all loads of the row first and unconditional (pieces past the diagonal re-read the
    // piece that holds it): a load followed by its use inside each chunk's branch makes the chunks
    // of a lane as many round trips (61.5 -> 56.8 us at 2048 x 32 x 2048).  The adjoint, with two
    // operands and twice the registers, measured no better that way (85 -> 88 us) and loads per chunk.
    if (!BWD) {
#pragma unroll
        for (int c = 0; c < CH; c++) sv[c] = ld8(sr + min((c * 64 + lane) * 8, i & ~7));
    }
#pragma unroll
    for (int c = 0; c < CH; c++) {
        if (c * 512 > i) continue;
        const int j0 = (c * 64 + lane) * 8;
        if (c * 512 + 511 <= i) {                 // whole chunk live (and inside the row: i < S)
            const h8 v = BWD ? ld8(sr + j0) : sv[c];
            if (BWD) g[c] = ld8(gr + j0);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                e[c][k] = h2f(v.v[k]);
                mx = fmaxf(mx, e[c][k]);
            }
        } else if (j0 <= i) {
            const h8 v = BWD ? ld8(sr + j0) : sv[c];
            if (BWD) g[c] = ld8(gr + j0);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                e[c][k] = (j0 + k <= i) ? h2f(v.v[k]) : -INFINITY;
                mx = fmaxf(mx, e[c][k]);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                e[c][k] = -INFINITY;
                if (BWD) g[c].v[k] = (half_t)0.f;
            }
        }
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        if (c * 512 > i) continue;
        const int j0 = (c * 64 + lane) * 8;
        const bool full = c * 512 + 511 <= i;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            // below -100 the term is under half an ulp of the sum (>= 1) and rounds to a zero
            // probability, exactly as exp(-inf) = 0 does
            float t = exp_nonpos(fmaxf(e[c][k] - mx, -100.0f));
            if (!full) t = (j0 + k <= i) ? t : 0.f;
            e[c][k] = t;
            sum += t;
        }
    }
    sum = wave_sum(sum);
    const RowDivide div(sum);
    half_t *orow = out + row * S;
    // columns written: j <= i, then zeros to the next multiple of 256 (the triangular GEMMs
    // read no further); the rest of the row is left untouched
    const int wchunk = min(nchunk, ((i + 256) & ~255) >> 3);
    if (!BWD) {
#pragma unroll
        for (int c = 0; c < CH; c++) {
            if (c * 512 > i) continue;
            const int ch = c * 64 + lane;
            if (ch < wchunk) {
                h8 o;
#pragma unroll
                for (int k = 0; k < 8; k++) o.v[k] = f2h(div(e[c][k]));
                st8(orow + ch * 8, o);
            }
        }
    } else {
        float tsum = 0.f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            if (c * 512 > i) continue;
            const int j0 = (c * 64 + lane) * 8;
            const bool full = c * 512 + 511 <= i;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float p = div(e[c][k]);           // 0 above the diagonal
                e[c][k] = p;
                if (full || j0 + k <= i) tsum += p * h2f(g[c].v[k]);
            }
        }
        tsum = wave_sum(tsum);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            if (c * 512 > i) continue;
            const int ch = c * 64 + lane;
            const int j0 = ch * 8;
            const bool full = c * 512 + 511 <= i;
            if (ch < wchunk) {
                h8 o;
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float p = e[c][k];
                    const float t = p * h2f(g[c].v[k]);
                    o.v[k] = (full || j0 + k <= i) ? f2h(t - tsum * p) : (half_t)0.f;
                }
                st8(orow + ch * 8, o);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// LM-head softmax / cross-entropy on [N,V], one block of 1024 lanes per row.
constexpr int kCeThreads = 1024;

// The row lives in registers as fp32 (CH x 8 values per lane); chunks past the row hold -inf, and
// differences from the maximum below -100 contribute nothing to an fp32 sum that is at least 1.
// The kernels are bound by their arithmetic as much as by HBM (per element: convert, maximum,
// exponential, sum, quotient, one-hot, scale, round), hence exp_nonpos and RowDivide.
template <int CH>
struct CeRow {
    float e[CH][8];
    __device__ float load_max(const half_t *row, int nchunk)
    {
        // every load first and unconditional (a chunk past the row re-reads the last one): a load
        // inside `if (ch < nchunk)` is waited for at the end of that branch, one round trip per chunk
        h8 raw[CH];
#pragma unroll
        for (int c = 0; c < CH; c++) raw[c] = ld8(row + min(c * kCeThreads + (int)threadIdx.x, nchunk - 1) * 8);
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const bool valid = c * kCeThreads + (int)threadIdx.x < nchunk;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                e[c][k] = valid ? h2f(raw[c].v[k]) : -INFINITY;
                mx = fmaxf(mx, e[c][k]);
            }
        }
        return mx;
    }
    // e := exp(e - mx); returns the lane's partial sum
    __device__ float exp_sum(float mx)
    {
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < CH; c++)
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float x = e[c][k] - mx;
                e[c][k] = x >= -100.f ? exp_nonpos(x) : 0.f;
                s += e[c][k];
            }
        return s;
    }
};

template <int CH>
__global__ void __launch_bounds__(kCeThreads)
softmax_ce_fwd_kernel(int64_t N, int V, const half_t *__restrict__ logit,
                      const uint16_t *__restrict__ tok, float *__restrict__ prob,
                      float *__restrict__ loss, uint16_t *__restrict__ amax, int *status)
{
    __shared__ float red[16];
    __shared__ float xt_s;
    const int64_t n = blockIdx.x;
    const int nchunk = V / 8;
    const int t = tok ? (int)tok[n] : 0;
    if (tok && t >= V) {
        if (threadIdx.x == 0 && status) atomicMax(status, (int)n + 1);
        return;                                    // uniform for the block
    }
    CeRow<CH> row;
    const float mx = block_reduce(row.load_max(logit + n * V, nchunk), OpMax(), -INFINITY, red);
    if (amax) {
        // first index holding the maximum
        float best = 3.0e38f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * kCeThreads + threadIdx.x;
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (row.e[c][k] == mx) best = fminf(best, (float)(ch * 8 + k));
        }
        best = -block_reduce(-best, OpMax(), -3.0e38f, red);
        if (threadIdx.x == 0) amax[n] = (uint16_t)best;
    }
    if (loss) {
        // the label's logit: selected in a register, stored by the one lane that holds it
        float xt = 0.f;
        bool mine = false;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * kCeThreads + threadIdx.x;
            mine = mine || ch == (t >> 3);
#pragma unroll
            for (int k = 0; k < 8; k++) xt = (ch * 8 + k == t) ? row.e[c][k] : xt;
        }
        if (mine) xt_s = xt;
    }
    const float sum = block_reduce(row.exp_sum(mx), OpSum(), 0.f, red);     // barriers inside publish xt_s
    if (loss && threadIdx.x == 0) loss[n] = -logf(expf(xt_s - mx) / sum);
    if (prob) {
        float *pr = prob + n * V;
        const RowDivide div(sum);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * kCeThreads + threadIdx.x;
            if (ch < nchunk) {
                const float *e = row.e[c];
                float4 a = make_float4(div(e[0]), div(e[1]), div(e[2]), div(e[3]));
                float4 b = make_float4(div(e[4]), div(e[5]), div(e[6]), div(e[7]));
                *reinterpret_cast<float4 *>(pr + ch * 8) = a;
                *reinterpret_cast<float4 *>(pr + ch * 8 + 4) = b;
            }
        }
    }
}

// dlogit16 (+)= f16( scale[n] * (softmax - one_hot(tok)) )
template <int CH>
__global__ void __launch_bounds__(kCeThreads)
softmax_ce_bwd_kernel(int64_t N, int V, const half_t *__restrict__ logit,
                      const uint16_t *__restrict__ tok, const float *__restrict__ scale,
                      half_t *dlogit, int acc)
{
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const int nchunk = V / 8;
    const int t = (int)tok[n];
    const float sc = scale[n];
    half_t *dr = dlogit + n * V;
    CeRow<CH> row;
    const float mx = block_reduce(row.load_max(logit + n * V, nchunk), OpMax(), -INFINITY, red);
    const float sum = block_reduce(row.exp_sum(mx), OpSum(), 0.f, red);
    const RowDivide div(sum);
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int ch = c * kCeThreads + threadIdx.x;
        if (ch < nchunk) {
            h8 o, old;
            // loaded here, not with the row: the accumulating form runs once per cycle at most (the
            // first write of dlogit overwrites)
            if (acc) old = ld8(dr + ch * 8);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                float p = div(row.e[c][k]);
                float z = p - ((ch * 8 + k == t) ? 1.0f : 0.0f);
                float d = sc * z;
                o.v[k] = acc ? f2h(h2f(old.v[k]) + rnd16(d)) : f2h(d);
            }
            st8(dr + ch * 8, o);
        }
    }
}

__global__ void check_tok_kernel(int64_t N, int V, const uint16_t *tok, int *status)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N && (int)tok[i] >= V) atomicMax(status, (int)i + 1);
}

}  // namespace

#define CACTI_DISPATCH_SM(ch, CALL)                                  \
    switch (ch) {                                                    \
        case 1: { constexpr int CH = 1; CALL; } break;               \
        case 2: { constexpr int CH = 2; CALL; } break;               \
        case 3: case 4: { constexpr int CH = 4; CALL; } break;       \
        case 5: case 6: case 7: case 8: { constexpr int CH = 8; CALL; } break; \
        default: { constexpr int CH = 16; CALL; } break;             \
    }

namespace {

// Row-causal softmax for the cached forward pass: T new rows at positions row0 .. row0 + T - 1
// against C cached columns; column j of row t is live when j <= t + row0.  One wave per row
// (t, h); the row is read three times (it is short and stays in cache): maximum, sum, quotient.
// The per-lane partial sums run over the same 8-column pieces in the same order as in
// causal_softmax_kernel, so a whole sequence processed as one block gives the same bits.
__global__ void __launch_bounds__(kRowsPerBlock * 64)
row_causal_softmax_kernel(int64_t T, int H, int64_t C, int64_t ld, int64_t row0, const half_t *__restrict__ s16,
                          half_t *__restrict__ p16)
{
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + wid;
    if (row >= T * H) return;
    const int64_t i = row / H + row0;             // last live column
    const half_t *sr = s16 + row * ld;
    half_t *pr = p16 + row * ld;
    const int64_t live = (i + 1 < C ? i + 1 : C); // number of live columns
    float mx = -INFINITY;
    for (int64_t j0 = (int64_t)lane * 8; j0 < live; j0 += 512) {
        const h8 v = ld8(sr + j0);
#pragma unroll
        for (int k = 0; k < 8; k++)
            if (j0 + k < live) mx = fmaxf(mx, h2f(v.v[k]));
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int64_t j0 = (int64_t)lane * 8; j0 < live; j0 += 512) {
        const h8 v = ld8(sr + j0);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float t = exp_nonpos(fmaxf(h2f(v.v[k]) - mx, -100.0f));
            sum += (j0 + k < live) ? t : 0.f;
        }
    }
    sum = wave_sum(sum);
    const RowDivide div(sum);
    for (int64_t j0 = (int64_t)lane * 8; j0 < C; j0 += 512) {
        h8 o;
        if (j0 < live) {
            const h8 v = ld8(sr + j0);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float t = exp_nonpos(fmaxf(h2f(v.v[k]) - mx, -100.0f));
                o.v[k] = (j0 + k < live) ? f2h(div(t)) : (half_t)0.f;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) o.v[k] = (half_t)0.f;
        }
        st8(pr + j0, o);
    }
}

// in_tok[pos] += out_tok[last]: the generated token appended to the input (u16 add as the
// reference's `+=` on a zero-filled slot, src/librarium/llama.rs:958-959)
__global__ void append_token_kernel(uint16_t *in_tok, int64_t pos, const uint16_t *out_tok, int64_t last)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) in_tok[pos] = (uint16_t)(in_tok[pos] + out_tok[last]);
}

}  // namespace

CACTI_API int cacti_hip_row_causal_softmax_fwd(int64_t T, int64_t H, int64_t C, int64_t ld, int64_t initial_row,
                                               const void *s16, void *p16, void *stream)
{
    CACTI_REQUIRE(T > 0 && H > 0 && C > 0 && s16 && p16 && initial_row >= 0, CACTI_E_INVALID,
                  "row_causal_softmax_fwd: null pointer or empty shape");
    CACTI_REQUIRE(C % 8 == 0 && ld % 8 == 0 && ld >= C, CACTI_E_NOTIMPL,
                  "row_causal_softmax_fwd: need C %% 8 == 0 and a row pitch that is a multiple of 8 and >= C");
    CACTI_REQUIRE(aligned(s16, 16) && aligned(p16, 16), CACTI_E_INVALID,
                  "row_causal_softmax_fwd: tensors must be 16-byte aligned");
    const unsigned grid = (unsigned)((T * H + kRowsPerBlock - 1) / kRowsPerBlock);
    hipLaunchKernelGGL(row_causal_softmax_kernel, dim3(grid), dim3(kRowsPerBlock * 64), 0, (hipStream_t)stream, T,
                       (int)H, C, ld, initial_row, (const half_t *)s16, (half_t *)p16);
    return launch_status("row_causal_softmax_fwd");
}

CACTI_API int cacti_hip_append_token_u16(void *in_tok, int64_t pos, const void *out_tok, int64_t last, void *stream)
{
    CACTI_REQUIRE(in_tok && out_tok && pos >= 0 && last >= 0, CACTI_E_INVALID, "append_token: bad argument");
    hipLaunchKernelGGL(append_token_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (uint16_t *)in_tok, pos,
                       (const uint16_t *)out_tok, last);
    return launch_status("append_token");
}

static int causal_check(int64_t S, int64_t H, const void *a, const void *b, const char *who)
{
    CACTI_REQUIRE(S > 0 && H > 0 && a && b, CACTI_E_INVALID, "%s: null pointer or empty shape", who);
    CACTI_REQUIRE(S % 8 == 0 && S <= 8192, CACTI_E_NOTIMPL,
                  "%s: need S %% 8 == 0 and S <= 8192 (S=%lld)", who, (long long)S);
    CACTI_REQUIRE(aligned(a, 16) && aligned(b, 16), CACTI_E_INVALID,
                  "%s: tensors must be 16-byte aligned", who);
    return 0;
}

CACTI_API int cacti_hip_causal_softmax_fwd(int64_t S, int64_t H, const void *s16, void *p16,
                                           void *stream)
{
    int rc = causal_check(S, H, s16, p16, "causal_softmax_fwd");
    if (rc) return rc;
    const unsigned grid = (unsigned)((S * H + kRowsPerBlock - 1) / kRowsPerBlock);
    const int ch = (int)((S / 8 + 63) / 64);
    CACTI_DISPATCH_SM(ch, hipLaunchKernelGGL((causal_softmax_kernel<CH, false>), dim3(grid),
                                             dim3(kRowsPerBlock * 64), 0, (hipStream_t)stream, S,
                                             (int)H, (const half_t *)s16, (const half_t *)nullptr,
                                             (half_t *)p16));
    return launch_status("causal_softmax_fwd");
}

CACTI_API int cacti_hip_causal_softmax_bwd(int64_t S, int64_t H, const void *s16, const void *dp16,
                                           void *ds16, void *stream)
{
    int rc = causal_check(S, H, s16, ds16, "causal_softmax_bwd");
    if (rc) return rc;
    CACTI_REQUIRE(dp16 && aligned(dp16, 16), CACTI_E_INVALID,
                  "causal_softmax_bwd: dp16 null or not 16-byte aligned");
    const unsigned grid = (unsigned)((S * H + kRowsPerBlock - 1) / kRowsPerBlock);
    const int ch = (int)((S / 8 + 63) / 64);
    CACTI_DISPATCH_SM(ch, hipLaunchKernelGGL((causal_softmax_kernel<CH, true>), dim3(grid),
                                             dim3(kRowsPerBlock * 64), 0, (hipStream_t)stream, S,
                                             (int)H, (const half_t *)s16, (const half_t *)dp16,
                                             (half_t *)ds16));
    return launch_status("causal_softmax_bwd");
}

static int ce_check(int64_t N, int64_t V, const void *logit, const char *who)
{
    CACTI_REQUIRE(N > 0 && V > 0 && logit, CACTI_E_INVALID, "%s: null pointer or empty shape", who);
    CACTI_REQUIRE(V % 8 == 0 && V <= 65536, CACTI_E_NOTIMPL,
                  "%s: need V %% 8 == 0 and V <= 65536 (V=%lld)", who, (long long)V);
    CACTI_REQUIRE(aligned(logit, 16), CACTI_E_INVALID, "%s: logits must be 16-byte aligned", who);
    return 0;
}

CACTI_API int cacti_hip_softmax_ce_fwd(int64_t N, int64_t V, const void *logit16, const void *tok,
                                       void *prob, void *loss, void *amax, void *status,
                                       void *stream)
{
    int rc = ce_check(N, V, logit16, "softmax_ce_fwd");
    if (rc) return rc;
    CACTI_REQUIRE(!loss || tok, CACTI_E_INVALID, "softmax_ce_fwd: loss requested without tokens");
    CACTI_REQUIRE(!prob || aligned(prob, 16), CACTI_E_INVALID,
                  "softmax_ce_fwd: prob must be 16-byte aligned");
    const int ch = (int)((V / 8 + kCeThreads - 1) / kCeThreads);
    CACTI_REQUIRE(ch <= 8, CACTI_E_NOTIMPL, "softmax_ce_fwd: V too large");
    CACTI_DISPATCH_SM(ch, hipLaunchKernelGGL(softmax_ce_fwd_kernel<CH>, dim3((unsigned)N),
                                             dim3(kCeThreads), 0, (hipStream_t)stream, N, (int)V,
                                             (const half_t *)logit16, (const uint16_t *)tok,
                                             (float *)prob, (float *)loss, (uint16_t *)amax,
                                             (int *)status));
    return launch_status("softmax_ce_fwd");
}

CACTI_API int cacti_hip_softmax_ce_bwd(int64_t N, int64_t V, const void *logit16, const void *tok,
                                       const void *scale, void *dlogit16, int acc, void *stream)
{
    int rc = ce_check(N, V, logit16, "softmax_ce_bwd");
    if (rc) return rc;
    CACTI_REQUIRE(tok && scale && dlogit16 && aligned(dlogit16, 16), CACTI_E_INVALID,
                  "softmax_ce_bwd: null pointer or misaligned output");
    const int ch = (int)((V / 8 + kCeThreads - 1) / kCeThreads);
    CACTI_REQUIRE(ch <= 8, CACTI_E_NOTIMPL, "softmax_ce_bwd: V too large");
    CACTI_DISPATCH_SM(ch, hipLaunchKernelGGL(softmax_ce_bwd_kernel<CH>, dim3((unsigned)N),
                                             dim3(kCeThreads), 0, (hipStream_t)stream, N, (int)V,
                                             (const half_t *)logit16, (const uint16_t *)tok,
                                             (const float *)scale, (half_t *)dlogit16, acc));
    return launch_status("softmax_ce_bwd");
}

// Wave-reduction self-test (the DPP / swizzle path against a plain LDS loop).
namespace {
__global__ void selftest_wave_reduce_kernel(float *out)
{
    __shared__ float buf[64];
    const int lane = threadIdx.x;
    float v = (float)((lane * 37 + 11) % 101) - 50.0f;
    buf[lane] = v;
    __syncthreads();
    float s = wave_sum(v), m = wave_max(v);
    float rs = 0.f, rm = -INFINITY;
    for (int i = 0; i < 64; i++) {
        rs += buf[i];
        rm = fmaxf(rm, buf[i]);
    }
    // every lane must agree with the loop; count the lanes that do
    int ok = (s == rs) && (m == rm);
    int cnt = __syncthreads_count(ok);
    if (lane == 0) {
        out[0] = s;
        out[1] = rs;
        out[2] = m;
        out[3] = (float)cnt + (rm == m ? 0.f : 1000.f);
    }
}
}  // namespace

CACTI_API int cacti_hip_selftest_wave_reduce(void *out4, void *stream)
{
    CACTI_REQUIRE(out4, CACTI_E_INVALID, "selftest_wave_reduce: null pointer");
    hipLaunchKernelGGL(selftest_wave_reduce_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream,
                       (float *)out4);
    return launch_status("selftest_wave_reduce");
}
