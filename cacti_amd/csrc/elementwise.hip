// HBM-bound elementwise / gather kernels: RoPE (tables, forward, adjoint), SiLU gate
// (forward, adjoint), residual add, accumulate_1d, embedding gather and scatter-add.
//
// Every kernel moves 16 bytes per lane per access and reproduces, in registers, the
// f16 rounding points of the reference's thunk chain (rnd16 = one thunk boundary).
#include "common.h"

using namespace cacti;

namespace {

constexpr int kThreads = 256;

inline int grid_for(int64_t work_items, int per_block, int max_blocks = 1 << 20)
{
    int64_t g = (work_items + per_block - 1) / per_block;
    if (g < 1) g = 1;
    if (g > max_blocks) g = max_blocks;
    return (int)g;
}

// ---------------------------------------------------------------------------
// RoPE tables: inv_freq_i = 10000^(i * (-2/Dh)) in f32; freq = f32(s) * inv_freq;
// cos16/sin16 = f16(cos/sin(freq)), duplicated to width Dh (src/librarium/llama.rs:389-411).
__global__ void rope_tables_kernel(int64_t S, int Dh, half_t *__restrict__ cos16,
                                   half_t *__restrict__ sin16)
{
    const int hf = Dh / 2;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= S * hf) return;
    int64_t s = idx / hf;
    int i = (int)(idx % hf);
    float ex = -2.0f / (float)Dh;
    float inv = powf(10000.0f, (float)i * ex);
    float fr = (float)s * inv;
    half_t c = f2h(cosf(fr)), sn = f2h(sinf(fr));
    cos16[s * Dh + i] = c;
    cos16[s * Dh + hf + i] = c;
    sin16[s * Dh + i] = sn;
    sin16[s * Dh + hf + i] = sn;
}

// ---------------------------------------------------------------------------
// RoPE forward / adjoint on [S,H,Dh].  A block stages TOK whole token rows (H*Dh
// halves each, contiguous) plus their table rows in LDS with 16-byte loads, so the
// partner element d +- Dh/2 is an LDS read whatever Dh's alignment is (Dh = 100 puts
// the half-row boundary at 100 bytes).  Reads complete before any write, so the
// kernel may run in place.
//
// forward : a = f16(x cos); b = f16(rot(x) sin), rot(x) = [-x_r, x_l]; y = f16(a + b)
// adjoint : drx = f16(dy sin); dx (+)= [drx_r, -drx_l]; dx += f16(dy cos)
template <bool BWD>
__global__ void __launch_bounds__(kThreads)
rope_kernel(int64_t S, int H, int Dh, int tok_per_block, const half_t *__restrict__ in,
            const half_t *__restrict__ cos16, const half_t *__restrict__ sin16, half_t *out,
            int acc)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int row = H * Dh;             // halves per token
    const int cpt = row / 8;            // 16-byte chunks per token
    const int hf = Dh / 2;
    half_t *tile = reinterpret_cast<half_t *>(smem_raw);
    half_t *tc = tile + (size_t)tok_per_block * row;
    half_t *ts = tc + (size_t)tok_per_block * Dh;

    const int64_t t0 = (int64_t)blockIdx.x * tok_per_block;
    const int ntok = (int)((S - t0) < tok_per_block ? (S - t0) : tok_per_block);
    const half_t *src = in + t0 * row;

    for (int c = threadIdx.x; c < ntok * cpt; c += blockDim.x) st8(tile + c * 8, ld8(src + c * 8));
    for (int i = threadIdx.x; i < ntok * Dh; i += blockDim.x) {
        tc[i] = cos16[t0 * Dh + i];
        ts[i] = sin16[t0 * Dh + i];
    }
    __syncthreads();

    half_t *dst = out + t0 * row;
    for (int c = threadIdx.x; c < ntok * cpt; c += blockDim.x) {
        const int tok = c / cpt;
        const int e0 = (c - tok * cpt) * 8;
        const half_t *trow = tile + (size_t)tok * row;
        const half_t *cr = tc + tok * Dh, *sr = ts + tok * Dh;
        int d = e0 % Dh;
        h8 old;
        if (BWD && acc) old = ld8(dst + c * 8);
        h8 res;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int e = e0 + i;
            const bool left = d < hf;
            const int pe = left ? e + hf : e - hf;      // partner element
            const int pd = left ? d + hf : d - hf;
            const float x = h2f(trow[e]), xp = h2f(trow[pe]);
            if (!BWD) {
                float a = rnd16(x * h2f(cr[d]));
                float rx = left ? -xp : xp;
                float b = rnd16(rx * h2f(sr[d]));
                res.v[i] = f2h(a + b);
            } else {
                float drx_p = rnd16(xp * h2f(sr[pd]));  // f16(dy sin) at the partner
                float dx1 = left ? drx_p : -drx_p;      // [drx_r, -drx_l]
                float c2 = rnd16(x * h2f(cr[d]));       // f16(dy cos)
                float base = acc ? rnd16(h2f(old.v[i]) + dx1) : dx1;
                res.v[i] = f2h(base + c2);
            }
            if (++d == Dh) d = 0;
        }
        st8(dst + c * 8, res);
    }
}

// ---------------------------------------------------------------------------
// RoPE without LDS, for head dimensions that are multiples of 4 (Dh/2 even, so an aligned
// pair of halves never straddles the middle of a head).  A lane owns the pair (d, d+1) of the
// left half AND its partner pair (d + Dh/2, ..) of the right half: it reads both, then writes
// both, so no lane reads what another lane writes and the kernel may run in place.  All
// accesses are 4 bytes per lane and consecutive across lanes.
// blockIdx.y = 1 works on a second tensor (in1 -> out1, acc1) with the same tables: the query and the
// key of a layer in one launch.
template <bool BWD>
__global__ void __launch_bounds__(kThreads)
rope_pair_kernel(int64_t S, int H, int Dh, const half_t *__restrict__ in0,
                 const half_t *__restrict__ cos16, const half_t *__restrict__ sin16, half_t *out0,
                 int acc0, const half_t *__restrict__ in1, half_t *out1, int acc1)
{
    const half_t *__restrict__ in = blockIdx.y ? in1 : in0;
    half_t *out = blockIdx.y ? out1 : out0;
    const int acc = blockIdx.y ? acc1 : acc0;
    const int hf = Dh / 2, pph = hf / 2;            // pairs per half head
    const int64_t per_tok = (int64_t)H * pph, total = S * per_tok;
    for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < total;
         it += (int64_t)gridDim.x * blockDim.x) {
        const int64_t s = it / per_tok;
        const int r = (int)(it - s * per_tok);
        const int h = r / pph, d = (r - h * pph) * 2;
        const int64_t eL = (s * H + h) * Dh + d, eR = eL + hf;
        const int64_t tL = s * Dh + d, tR = tL + hf;
        const half2_t xL = *reinterpret_cast<const half2_t *>(in + eL);
        const half2_t xR = *reinterpret_cast<const half2_t *>(in + eR);
        const half2_t cL = *reinterpret_cast<const half2_t *>(cos16 + tL);
        const half2_t cR = *reinterpret_cast<const half2_t *>(cos16 + tR);
        const half2_t sL = *reinterpret_cast<const half2_t *>(sin16 + tL);
        const half2_t sR = *reinterpret_cast<const half2_t *>(sin16 + tR);
        half2_t oL, oR, qL, qR;
        if (BWD && acc) {
            qL = *reinterpret_cast<const half2_t *>(out + eL);
            qR = *reinterpret_cast<const half2_t *>(out + eR);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float xl = h2f(xL[i]), xr = h2f(xR[i]);
            if (!BWD) {
                // a + f16(-x_r sin) == a - f16(x_r sin): rounding is symmetric in sign
                oL[i] = f2h(rnd16(xl * h2f(cL[i])) - rnd16(xr * h2f(sL[i])));
                oR[i] = f2h(rnd16(xr * h2f(cR[i])) + rnd16(xl * h2f(sR[i])));
            } else {
                const float dl = rnd16(xr * h2f(sR[i]));        // drx_r = f16(dy sin) at d + Dh/2
                const float tl = rnd16(xl * h2f(sL[i]));        // drx_l; enters dx_r negated
                const float c2l = rnd16(xl * h2f(cL[i])), c2r = rnd16(xr * h2f(cR[i]));
                if (acc) {
                    oL[i] = f2h(rnd16(h2f(qL[i]) + dl) + c2l);
                    oR[i] = f2h(rnd16(h2f(qR[i]) - tl) + c2r);
                } else {
                    oL[i] = f2h(dl + c2l);
                    oR[i] = f2h(c2r - tl);
                }
            }
        }
        *reinterpret_cast<half2_t *>(out + eL) = oL;
        *reinterpret_cast<half2_t *>(out + eR) = oR;
    }
}

// ---------------------------------------------------------------------------
// SiLU gate.  forward: y = f16(g / (1 + exp(-g))); h = f16(y u).
__global__ void __launch_bounds__(kThreads)
silu_gate_fwd_kernel(int64_t nchunk, const half_t *__restrict__ g, const half_t *__restrict__ u,
                     half_t *__restrict__ h)
{
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunk;
         c += (int64_t)gridDim.x * blockDim.x) {
        h8 gv = ld8(g + c * 8), uv = ld8(u + c * 8), r;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float x = h2f(gv.v[i]);
            float y = rnd16(x / (1.0f + expf(-x)));
            r.v[i] = f2h(y * h2f(uv.v[i]));
        }
        st8(h + c * 8, r);
    }
}

// adjoint (Mul::pop_adj then StandardSilu::pop_adj, src/thunk/op.rs:2050-2054, 2901-2908):
//   du (+)= f16(y dh);  dy = f16(dh u);
//   y' = f16(silu g); t = f16(logistic g); a = f16(1 - t); b = f16(y' a); c = f16(b + t);
//   dg (+)= f16(dy c)
__global__ void __launch_bounds__(kThreads)
silu_gate_bwd_kernel(int64_t nchunk, const half_t *__restrict__ g, const half_t *__restrict__ u,
                     const half_t *__restrict__ dh, half_t *dg, int dg_acc, half_t *du, int du_acc)
{
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunk;
         c += (int64_t)gridDim.x * blockDim.x) {
        h8 gv = ld8(g + c * 8), uv = ld8(u + c * 8), dv = ld8(dh + c * 8), og, ou, rg, ru;
        if (dg_acc) og = ld8(dg + c * 8);
        if (du_acc) ou = ld8(du + c * 8);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float x = h2f(gv.v[i]), uu = h2f(uv.v[i]), d = h2f(dv.v[i]);
            float e = expf(-x);
            float y = rnd16(x / (1.0f + e));
            float t = rnd16(1.0f / (1.0f + e));
            float vdu = rnd16(y * d);
            float dy = rnd16(d * uu);
            float a = rnd16(1.0f - t);
            float b = rnd16(y * a);
            float cc = rnd16(b + t);
            float vdg = rnd16(dy * cc);
            rg.v[i] = dg_acc ? f2h(h2f(og.v[i]) + vdg) : f2h(vdg);
            ru.v[i] = du_acc ? f2h(h2f(ou.v[i]) + vdu) : f2h(vdu);
        }
        st8(dg + c * 8, rg);
        st8(du + c * 8, ru);
    }
}

// ---------------------------------------------------------------------------
// y = f16(a + b), 16 bytes per lane, scalar tail
__global__ void __launch_bounds__(kThreads)
add_f16_kernel(int64_t n, const half_t *a, const half_t *b, half_t *y)
{
    const int64_t nchunk = n / 8;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nth = (int64_t)gridDim.x * blockDim.x;
    for (int64_t c = tid; c < nchunk; c += nth) {
        h8 av = ld8(a + c * 8), bv = ld8(b + c * 8), r;
#pragma unroll
        for (int i = 0; i < 8; i++) r.v[i] = f2h(h2f(av.v[i]) + h2f(bv.v[i]));
        st8(y + c * 8, r);
    }
    for (int64_t i = nchunk * 8 + tid; i < n; i += nth) y[i] = f2h(h2f(a[i]) + h2f(b[i]));
}

template <class T>
__global__ void __launch_bounds__(kThreads) accumulate_1d_kernel(T *dst, const T *src, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = (T)(dst[i] + src[i]);
}

// ---------------------------------------------------------------------------
// Embedding gather: one block per position, 16-byte copies; ids >= V flag `status`.
__global__ void __launch_bounds__(kThreads)
embed_fwd_kernel(int64_t V, int64_t D, const half_t *__restrict__ W,
                 const uint16_t *__restrict__ tok, half_t *__restrict__ y, int *status)
{
    const int64_t s = blockIdx.x;
    const int64_t id = tok[s];
    if (id >= V) {
        if (threadIdx.x == 0 && status) atomicMax(status, (int)s + 1);
        return;
    }
    const half_t *src = W + id * D;
    half_t *dst = y + s * D;
    for (int c = threadIdx.x; c < D / 8; c += blockDim.x) st8(dst + c * 8, ld8(src + c * 8));
}

__global__ void __launch_bounds__(kThreads) fill_zero16_kernel(uint4 *p, int64_t n16)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
         i += (int64_t)gridDim.x * blockDim.x)
        p[i] = make_uint4(0, 0, 0, 0);
}

// Scatter-add, deterministic: the block of position s owns row tok[s] iff s is the
// first position holding that id; it then sums the dy rows of every position with
// the same id in position order in fp32 and rounds once.  The later positions of the id are
// collected, in order, by the first wave with ballots (64 positions per step), so a block
// with duplicates costs a few microseconds instead of a serial scan by every lane.
__global__ void __launch_bounds__(kThreads)
embed_bwd_kernel(int64_t V, int64_t D, int64_t S, const uint16_t *__restrict__ tok,
                 const half_t *__restrict__ dy, half_t *dW, int acc)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t *ids = reinterpret_cast<uint16_t *>(smem_raw);           // [S]
    uint16_t *dup = ids + S;                                          // [S] later positions of the id
    __shared__ int ndup;
    const int64_t s = blockIdx.x;
    for (int64_t j = threadIdx.x; j < S; j += blockDim.x) ids[j] = tok[j];
    __syncthreads();
    const uint16_t id = ids[s];
    if ((int64_t)id >= V) return;
    int earlier = 0;
    for (int64_t j = threadIdx.x; j < s; j += blockDim.x) earlier += ids[j] == id;
    earlier = __syncthreads_count(earlier);
    if (earlier) return;
    if (threadIdx.x < 64) {
        int n = 0;
        for (int64_t j0 = s + 1; j0 < S; j0 += 64) {
            const int64_t j = j0 + threadIdx.x;
            unsigned long long m = __ballot(j < S && ids[j] == id);
            while (m) {
                const int b = __builtin_ctzll(m);
                if (threadIdx.x == 0) dup[n] = (uint16_t)(j0 + b);
                n++;
                m &= m - 1;
            }
        }
        if (threadIdx.x == 0) ndup = n;
    }
    __syncthreads();
    const int n = ndup;
    half_t *dst = dW + (int64_t)id * D;
    for (int c = threadIdx.x; c < D / 8; c += blockDim.x) {
        h8 v = ld8(dy + s * D + c * 8);
        float a[8];
#pragma unroll
        for (int i = 0; i < 8; i++) a[i] = h2f(v.v[i]);
        int t = 0;
        for (; t + 4 <= n; t += 4) {                  // four independent loads in flight
            h8 w[4];
#pragma unroll
            for (int u = 0; u < 4; u++) w[u] = ld8(dy + (int64_t)dup[t + u] * D + c * 8);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int i = 0; i < 8; i++) a[i] += h2f(w[u].v[i]);
        }
        for (; t < n; t++) {
            const h8 w = ld8(dy + (int64_t)dup[t] * D + c * 8);
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] += h2f(w.v[i]);
        }
        h8 r;
        if (acc) {
            h8 o = ld8(dst + c * 8);
#pragma unroll
            for (int i = 0; i < 8; i++) r.v[i] = f2h(h2f(o.v[i]) + rnd16(a[i]));
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) r.v[i] = f2h(a[i]);
        }
        st8(dst + c * 8, r);
    }
}

}  // namespace

// ===========================================================================
// C ABI

CACTI_API int cacti_hip_rope_tables(int64_t S, int64_t Dh, void *cos16, void *sin16, void *stream)
{
    CACTI_REQUIRE(S > 0 && Dh > 0 && Dh % 2 == 0 && cos16 && sin16, CACTI_E_INVALID,
                  "rope_tables: bad arguments (S=%lld Dh=%lld)", (long long)S, (long long)Dh);
    int64_t n = S * (Dh / 2);
    hipLaunchKernelGGL(rope_tables_kernel, dim3(grid_for(n, kThreads)), dim3(kThreads), 0,
                       (hipStream_t)stream, S, (int)Dh, (half_t *)cos16, (half_t *)sin16);
    return launch_status("rope_tables");
}

// in1 / out1 / acc1: an optional second tensor for the same launch (nullptr: none)
static int rope_launch(bool bwd, int64_t S, int64_t H, int64_t Dh, const void *in, const void *c,
                       const void *s, void *out, int acc, void *stream, const void *in1 = nullptr,
                       void *out1 = nullptr, int acc1 = 0)
{
    CACTI_REQUIRE(S > 0 && H > 0 && Dh > 0 && in && c && s && out, CACTI_E_INVALID,
                  "rope: null pointer or empty shape");
    if (in1) {
        CACTI_REQUIRE(out1 && Dh % 4 == 0 && aligned(c, 4) && aligned(s, 4) && aligned(in1, 16) && aligned(out1, 16),
                      CACTI_E_NOTIMPL, "rope: two tensors in one launch need Dh %% 4 == 0 and aligned tensors");
    }
    CACTI_REQUIRE(Dh % 2 == 0 && (H * Dh) % 8 == 0, CACTI_E_NOTIMPL,
                  "rope: need Dh even and H*Dh %% 8 == 0 (H=%lld Dh=%lld)", (long long)H,
                  (long long)Dh);
    CACTI_REQUIRE(aligned(in, 16) && aligned(out, 16), CACTI_E_INVALID,
                  "rope: tensors must be 16-byte aligned");
    const int64_t row = H * Dh;
    if (Dh % 4 == 0 && aligned(c, 4) && aligned(s, 4)) {
        const int64_t items = S * H * (Dh / 4);
        const int grid = grid_for(items, kThreads, 4096);
        const dim3 g(grid, in1 ? 2 : 1);
        if (bwd)
            hipLaunchKernelGGL(rope_pair_kernel<true>, g, dim3(kThreads), 0,
                               (hipStream_t)stream, S, (int)H, (int)Dh, (const half_t *)in,
                               (const half_t *)c, (const half_t *)s, (half_t *)out, acc,
                               (const half_t *)in1, (half_t *)out1, acc1);
        else
            hipLaunchKernelGGL(rope_pair_kernel<false>, g, dim3(kThreads), 0,
                               (hipStream_t)stream, S, (int)H, (int)Dh, (const half_t *)in,
                               (const half_t *)c, (const half_t *)s, (half_t *)out, 0,
                               (const half_t *)in1, (half_t *)out1, 0);
        return launch_status("rope");
    }
    int tok = 2;
    size_t smem = (size_t)tok * (row + 2 * Dh) * 2;
    if (smem > 64 * 1024) {
        tok = 1;
        smem = (size_t)(row + 2 * Dh) * 2;
    }
    CACTI_REQUIRE(smem <= 64 * 1024, CACTI_E_NOTIMPL, "rope: token row of %lld halves too large",
                  (long long)row);
    int grid = (int)((S + tok - 1) / tok);
    if (bwd)
        hipLaunchKernelGGL(rope_kernel<true>, dim3(grid), dim3(kThreads), smem, (hipStream_t)stream,
                           S, (int)H, (int)Dh, tok, (const half_t *)in, (const half_t *)c,
                           (const half_t *)s, (half_t *)out, acc);
    else
        hipLaunchKernelGGL(rope_kernel<false>, dim3(grid), dim3(kThreads), smem,
                           (hipStream_t)stream, S, (int)H, (int)Dh, tok, (const half_t *)in,
                           (const half_t *)c, (const half_t *)s, (half_t *)out, 0);
    return launch_status("rope");
}

CACTI_API int cacti_hip_rope_fwd(int64_t S, int64_t H, int64_t Dh, const void *x,
                                 const void *cos16, const void *sin16, void *y, void *stream)
{
    return rope_launch(false, S, H, Dh, x, cos16, sin16, y, 0, stream);
}

CACTI_API int cacti_hip_rope_bwd(int64_t S, int64_t H, int64_t Dh, const void *dy,
                                 const void *cos16, const void *sin16, void *dx, int dx_acc,
                                 void *stream)
{
    CACTI_REQUIRE(!(dx_acc && dx == dy), CACTI_E_INVALID, "rope_bwd: accumulate cannot run in place");
    return rope_launch(true, S, H, Dh, dy, cos16, sin16, dx, dx_acc, stream);
}

CACTI_API int cacti_hip_rope_fwd_pair(int64_t S, int64_t H, int64_t Dh, const void *x0, const void *x1,
                                      const void *cos16, const void *sin16, void *y0, void *y1, void *stream)
{
    CACTI_REQUIRE(x1 && y1, CACTI_E_INVALID, "rope_fwd_pair: null pointer");
    if (Dh % 4 != 0) {                            // the staged kernel takes one tensor per launch
        const int rc = rope_launch(false, S, H, Dh, x0, cos16, sin16, y0, 0, stream);
        return rc ? rc : rope_launch(false, S, H, Dh, x1, cos16, sin16, y1, 0, stream);
    }
    return rope_launch(false, S, H, Dh, x0, cos16, sin16, y0, 0, stream, x1, y1, 0);
}

CACTI_API int cacti_hip_rope_bwd_pair(int64_t S, int64_t H, int64_t Dh, const void *dy0, const void *dy1,
                                      const void *cos16, const void *sin16, void *dx0, int dx0_acc, void *dx1,
                                      int dx1_acc, void *stream)
{
    CACTI_REQUIRE(dy1 && dx1, CACTI_E_INVALID, "rope_bwd_pair: null pointer");
    CACTI_REQUIRE(!(dx0_acc && dx0 == dy0) && !(dx1_acc && dx1 == dy1), CACTI_E_INVALID,
                  "rope_bwd_pair: accumulate cannot run in place");
    if (Dh % 4 != 0) {
        const int rc = rope_launch(true, S, H, Dh, dy0, cos16, sin16, dx0, dx0_acc, stream);
        return rc ? rc : rope_launch(true, S, H, Dh, dy1, cos16, sin16, dx1, dx1_acc, stream);
    }
    return rope_launch(true, S, H, Dh, dy0, cos16, sin16, dx0, dx0_acc, stream, dy1, dx1, dx1_acc);
}

CACTI_API int cacti_hip_silu_gate_fwd(int64_t n, const void *g, const void *u, void *h,
                                      void *stream)
{
    CACTI_REQUIRE(n > 0 && g && u && h, CACTI_E_INVALID, "silu_gate_fwd: null pointer or n <= 0");
    CACTI_REQUIRE(n % 8 == 0, CACTI_E_NOTIMPL, "silu_gate_fwd: n %% 8 != 0 (n=%lld)", (long long)n);
    CACTI_REQUIRE(aligned(g, 16) && aligned(u, 16) && aligned(h, 16), CACTI_E_INVALID,
                  "silu_gate_fwd: tensors must be 16-byte aligned");
    hipLaunchKernelGGL(silu_gate_fwd_kernel, dim3(grid_for(n / 8, kThreads, 8192)), dim3(kThreads),
                       0, (hipStream_t)stream, n / 8, (const half_t *)g, (const half_t *)u,
                       (half_t *)h);
    return launch_status("silu_gate_fwd");
}

CACTI_API int cacti_hip_silu_gate_bwd(int64_t n, const void *g, const void *u, const void *dh,
                                      void *dg, int dg_acc, void *du, int du_acc, void *stream)
{
    CACTI_REQUIRE(n > 0 && g && u && dh && dg && du, CACTI_E_INVALID,
                  "silu_gate_bwd: null pointer or n <= 0");
    CACTI_REQUIRE(n % 8 == 0, CACTI_E_NOTIMPL, "silu_gate_bwd: n %% 8 != 0 (n=%lld)", (long long)n);
    CACTI_REQUIRE(aligned(g, 16) && aligned(u, 16) && aligned(dh, 16) && aligned(dg, 16) &&
                      aligned(du, 16),
                  CACTI_E_INVALID, "silu_gate_bwd: tensors must be 16-byte aligned");
    hipLaunchKernelGGL(silu_gate_bwd_kernel, dim3(grid_for(n / 8, kThreads, 8192)), dim3(kThreads),
                       0, (hipStream_t)stream, n / 8, (const half_t *)g, (const half_t *)u,
                       (const half_t *)dh, (half_t *)dg, dg_acc, (half_t *)du, du_acc);
    return launch_status("silu_gate_bwd");
}

CACTI_API int cacti_hip_add_f16(int64_t n, const void *a, const void *b, void *y, void *stream)
{
    CACTI_REQUIRE(n > 0 && a && b && y, CACTI_E_INVALID, "add_f16: null pointer or n <= 0");
    CACTI_REQUIRE(aligned(a, 16) && aligned(b, 16) && aligned(y, 16), CACTI_E_INVALID,
                  "add_f16: tensors must be 16-byte aligned");
    hipLaunchKernelGGL(add_f16_kernel, dim3(grid_for((n + 7) / 8, kThreads, 8192)), dim3(kThreads),
                       0, (hipStream_t)stream, n, (const half_t *)a, (const half_t *)b,
                       (half_t *)y);
    return launch_status("add_f16");
}

template <class T>
static int accumulate_launch(void *dst, const void *src, int64_t n, void *stream)
{
    CACTI_REQUIRE(dst && src && n >= 0 && n <= INT32_MAX, CACTI_E_INVALID,
                  "accumulate_1d: null pointer or n outside [0, 2^31)");
    if (n == 0) return 0;
    hipLaunchKernelGGL(accumulate_1d_kernel<T>, dim3(grid_for(n, kThreads, 16384)), dim3(kThreads),
                       0, (hipStream_t)stream, (T *)dst, (const T *)src, n);
    return launch_status("accumulate_1d");
}
CACTI_API int cacti_hip_accumulate_1d_f32(void *dst, const void *src, int64_t n, void *stream)
{
    return accumulate_launch<float>(dst, src, n, stream);
}
CACTI_API int cacti_hip_accumulate_1d_f16(void *dst, const void *src, int64_t n, void *stream)
{
    return accumulate_launch<half_t>(dst, src, n, stream);
}
CACTI_API int cacti_hip_accumulate_1d_u16(void *dst, const void *src, int64_t n, void *stream)
{
    return accumulate_launch<uint16_t>(dst, src, n, stream);
}

CACTI_API int cacti_hip_embed_fwd(int64_t V, int64_t D, const void *W, int64_t S, const void *tok,
                                  void *y, void *status, void *stream)
{
    CACTI_REQUIRE(V > 0 && D > 0 && S > 0 && W && tok && y, CACTI_E_INVALID,
                  "embed_fwd: null pointer or empty shape");
    CACTI_REQUIRE(D % 8 == 0, CACTI_E_NOTIMPL, "embed_fwd: D %% 8 != 0 (D=%lld)", (long long)D);
    CACTI_REQUIRE(aligned(W, 16) && aligned(y, 16), CACTI_E_INVALID,
                  "embed_fwd: tensors must be 16-byte aligned");
    hipLaunchKernelGGL(embed_fwd_kernel, dim3((unsigned)S), dim3(kThreads), 0, (hipStream_t)stream,
                       V, D, (const half_t *)W, (const uint16_t *)tok, (half_t *)y, (int *)status);
    return launch_status("embed_fwd");
}

CACTI_API int cacti_hip_embed_bwd(int64_t V, int64_t D, int64_t S, const void *tok, const void *dy,
                                  void *dW, int acc, void *stream)
{
    CACTI_REQUIRE(V > 0 && D > 0 && S > 0 && tok && dy && dW, CACTI_E_INVALID,
                  "embed_bwd: null pointer or empty shape");
    CACTI_REQUIRE(D % 8 == 0 && S <= 16384, CACTI_E_NOTIMPL,      // 4 S bytes of LDS per block
                  "embed_bwd: need D %% 8 == 0 and S <= 16384 (D=%lld S=%lld)", (long long)D,
                  (long long)S);
    CACTI_REQUIRE(aligned(dy, 16) && aligned(dW, 16), CACTI_E_INVALID,
                  "embed_bwd: tensors must be 16-byte aligned");
    if (!acc) {
        int64_t n16 = V * D / 8;
        hipLaunchKernelGGL(fill_zero16_kernel, dim3(grid_for(n16, kThreads, 8192)), dim3(kThreads),
                           0, (hipStream_t)stream, (uint4 *)dW, n16);
    }
    hipLaunchKernelGGL(embed_bwd_kernel, dim3((unsigned)S), dim3(kThreads), (size_t)S * 4,
                       (hipStream_t)stream, V, D, S, (const uint16_t *)tok, (const half_t *)dy,
                       (half_t *)dW, acc);
    return launch_status("embed_bwd");
}
