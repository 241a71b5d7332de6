// Causal attention of one layer as fused kernels: the reference's chain
//   S16 = f16(a Q K^T) -> f32 -> causal mask -> softmax -> P16 = f16(P) -> O = f16(P16 V)
// (src/librarium/llama.rs:501-507; BlockMatrixMul src/thunk/op.rs:4719-5471, BlockTriElemAffine
// :4189-4278, InnerSoftmax :3257-3383) and its adjoint
//   dV = f16(P16^T dO), dP16 = f16(dO V^T), dS16 = f16(tril(T - (sum_j T) P')), T = P' f32(dP16),
//   dQ = f16(a dS16 K), dK = f16(a dS16^T Q)
// (pop_adj :4882-4912, InnerSoftmaxPostAdj :3386-3457) without the sequence x sequence tensors
// ever reaching memory.  Every rounding point of the chain is kept, in registers: scores and
// probabilities are rounded to f16 before they are used, each product accumulates in fp32 and is
// rounded once.
//
// Layout: q, k, v, o and their adjoints are [S, H, Dh] (row stride ld), 8-byte aligned.
//
// Forward (a workgroup = 128 query rows of one head, 4 waves x 32 rows; keys in tiles of 64):
// the scores are computed twice.  Pass 1 keeps a running row maximum m and sum l of exp(S16 - m);
// pass 2 recomputes S16 (same instructions, same bits), forms P16 = f16(exp(S16 - m) / l) -- the
// reference's probabilities, not an unnormalised stand-in -- and accumulates O += P16 V.  Only
// (m, l) per row are kept for the adjoint.
//
// Adjoint: two kernels, each deterministic (no atomics).  The dQ kernel has the forward's shape
// (queries fixed, loop over keys); the dK/dV kernel fixes 128 keys and loops over the queries at
// or after them.  Both recompute S16, P' and dP16 per tile.  The row sums sigma_i = sum_j P'_ij
// f32(dP16_ij) are formed as the reference forms them, from the rounded dP16, by a first pass of the
// dQ kernel over its key tiles (the shortcut sum_d dO_id O_id is the same number only in exact
// arithmetic: it misses the cancellation between dP16 and sigma in rows whose probability sits on
// one key, where the reference's dS is exactly zero).
//
// MFMA data flow (v_mfma_f32_32x32x16_f16, D = X Y^T: lane <-> row of Y, registers <-> rows of X).
// With the fixed operand as Y, a lane owns one query (key) and 16 of a 32-key (query) tile's
// entries, 4 q + r <-> index 8 q + 4 lh + r.  Rounded to f16 and packed, registers 8 kk .. 8 kk + 7
// are directly the Y operand of k step kk of the next product (contraction over that index); the
// X operand is read from the [row][d] LDS tile by ds_read_b64_tr_b16 with the matching row
// permutation (rows 16 kk + 4 lh + 0..3 and 16 kk + 8 + 4 lh + 0..3).  No probability ever goes
// through LDS.
//
// LDS tiles are [rows][128 halves] (256 bytes per row, head dim zero-padded); 16-byte chunk c of
// row r sits at chunk c ^ g(r), g(r) = 2 (r & 3) | ((r >> 2) & 1): conflict-free both for the
// 16-byte operand reads of 8 consecutive rows and for the transposing reads of 4 consecutive rows.
#include "common.h"
#include "softmax_math.h"

#include <type_traits>

using namespace cacti;

namespace {

constexpr int kDP = 128;                 // padded head dim of an LDS tile
constexpr int kRowB = kDP * 2;           // bytes per tile row
constexpr int kTileRows = 64;
constexpr int kTileB = kTileRows * kRowB;   // 16 KB
constexpr int kNT = 256;                 // threads per workgroup
constexpr int kBM = 128;                 // rows of the fixed operand per workgroup

struct AttnArgs {
    int S, H, Dh;
    int64_t ld;
    float alpha;
    const half_t *q, *k, *v, *dO;
    half_t *out, *dq, *dk, *dv;
    float *m, *l;                        // [H][S] row maximum and sum (forward output)
    float *y, *sig;                      // [H][S] reciprocal of l, sigma (adjoint scratch)
    int acc_dq, acc_dk, acc_dv;
};

typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

__device__ __forceinline__ int gsw(int r) { return ((r & 3) << 1) | ((r >> 2) & 1); }
__device__ __forceinline__ int toff(int r, int c) { return r * kRowB + ((c ^ gsw(r)) << 4); }

__device__ __forceinline__ uint2 lds_read_tr(const unsigned char *q)
{
    typedef __attribute__((address_space(3))) fp16x4_t *lds_ptr;
    const fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_ptr)q);
    uint2 r;
    __builtin_memcpy(&r, &v, 8);
    return r;
}

__device__ __forceinline__ half8_t as_h8(uint2 lo, uint2 hi)
{
    const uint4 v = make_uint4(lo.x, lo.y, hi.x, hi.y);
    half8_t f;
    __builtin_memcpy(&f, &v, 16);
    return f;
}

// 64 rows x Dh of a [S, H, Dh] tensor -> registers -> LDS tile (zero beyond Dh and beyond the last row)
struct TileLoader {
    static constexpr int NP = kTileRows * 32 / kNT;      // 8-byte pieces per lane
    uint2 v[NP];
    // src = &X[row0][head column 0]; rows_left = S - row0 >= 1
    __device__ __forceinline__ void load(const half_t *src, int64_t ld, int rows_left, int Dh)
    {
#pragma unroll
        for (int it = 0; it < NP; it++) {
            const int p = threadIdx.x + it * kNT;
            const int row = p >> 5, pc = p & 31;
            const bool ok = row < rows_left && pc * 4 < Dh;
            // always a valid address (the tile's first element), zeroed by a select: a load inside a
            // branch would be waited for at the end of that branch
            const uint2 t = *reinterpret_cast<const uint2 *>(src + (ok ? (int64_t)row * ld + pc * 4 : 0));
            v[it] = ok ? t : make_uint2(0u, 0u);
        }
    }
    __device__ __forceinline__ void store(unsigned char *tile) const
    {
#pragma unroll
        for (int it = 0; it < NP; it++) {
            const int p = threadIdx.x + it * kNT;
            const int row = p >> 5, pc = p & 31;
            *reinterpret_cast<uint2 *>(tile + toff(row, pc >> 1) + ((pc & 1) << 3)) = v[it];
        }
    }
};

// The fixed operand of a lane: row `row` of a [S, H, Dh] tensor as KS fragments (k step ks: the 8
// halves at d = 16 ks + 8 lh ..), zero beyond Dh and for rows beyond S
template <int KS>
__device__ __forceinline__ void load_frags(half8_t (&f)[KS], const half_t *X, int64_t ld, int row, int S, int Dh,
                                           int lh)
{
    const bool rok = row < S;
    const half_t *xr = X + (int64_t)(rok ? row : 0) * ld;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int d0 = 16 * ks + 8 * lh;
        const bool ok0 = rok && d0 < Dh, ok1 = rok && d0 + 4 < Dh;
        const uint2 a = *reinterpret_cast<const uint2 *>(xr + (d0 < Dh ? d0 : 0));
        const uint2 b = *reinterpret_cast<const uint2 *>(xr + (d0 + 4 < Dh ? d0 + 4 : 0));
        f[ks] = as_h8(ok0 ? a : make_uint2(0u, 0u), ok1 ? b : make_uint2(0u, 0u));
    }
}

// acc = sum over d of X[row_base + .][d] Y[.][d]: X from the LDS tile (16-byte reads), Y = fixed fragments
template <int KS>
__device__ __forceinline__ float16_t prod_direct(const unsigned char *tile, int row_base, const half8_t (&yf)[KS],
                                                 int l32, int lh)
{
    float16_t acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    const int row = row_base + l32;
    const unsigned char *rp = tile + row * kRowB;
    const int g = gsw(row);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const half8_t x = *reinterpret_cast<const half8_t *>(rp + (((2 * ks + lh) ^ g) << 4));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, yf[ks], acc, 0, 0, 0);
    }
    return acc;
}

// acc[dt] += sum over the 32 tile rows k_base .. k_base + 31 of X[row][32 dt + .] Y[.][row]: X by
// transposing reads of the LDS tile, Y = the packed registers y0 (rows 0..15) and y1 (rows 16..31) in
// the row permutation described at the top
template <int DT>
__device__ __forceinline__ void prod_tr(float16_t (&acc)[DT], const unsigned char *tile, int k_base, half8_t y0,
                                        half8_t y1, int lane)
{
    const int a4 = (lane >> 2) & 3, b4 = lane & 3, n16 = (lane >> 4) & 1, lh = lane >> 5;
    const int colb = 16 * n16 + 4 * b4;                 // first of the lane's 4 columns inside a 32-wide tile
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
        const int r1 = k_base + 16 * kk + 4 * lh + a4, r2 = r1 + 8;
        const unsigned char *p1 = tile + r1 * kRowB + ((colb & 4) << 1);
        const unsigned char *p2 = tile + r2 * kRowB + ((colb & 4) << 1);
        const int g1 = gsw(r1), g2 = gsw(r2);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            const int c = (32 * dt + colb) >> 3;
            const half8_t x = as_h8(lds_read_tr(p1 + ((c ^ g1) << 4)), lds_read_tr(p2 + ((c ^ g2) << 4)));
            acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, kk ? y1 : y0, acc[dt], 0, 0, 0);
        }
    }
}

__device__ __forceinline__ half8_t pack8(const float *p)
{
    half8_t h;
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f2h(p[i]);
    return h;
}

// exp(s - m) as every kernel here forms it (s <= m; differences below -100 count as -100, whose
// exponential is far below half an ulp of a sum that is at least 1)
__device__ __forceinline__ float exp_diff(float s, float m) { return exp_nonpos(fmaxf(s - m, -100.0f)); }

// e / l with the reciprocal y of l given (the arithmetic of RowDivide, softmax_math.h)
__device__ __forceinline__ float div_by(float e, float l, float y)
{
    const float q0 = e * y;
    return __builtin_fmaf(__builtin_fmaf(-q0, l, e), y, q0);
}
__device__ __forceinline__ float recip_refined(float l)
{
    const float y0 = __builtin_amdgcn_rcpf(l);
    return __builtin_fmaf(__builtin_fmaf(-l, y0, 1.0f), y0, y0);
}

// which 128-row tile a workgroup takes: the first half of the grid the long ones (descending), the
// second half the short ones (ascending), so that the two workgroups a CU holds add up evenly
__device__ __forceinline__ int balanced_tile(int t, int ntiles, bool long_is_high)
{
    const int half = (ntiles + 1) / 2;
    const int rank = t < half ? t : ntiles - 1 - (t - half);     // 0 = longest
    return long_is_high ? ntiles - 1 - rank : rank;
}

// 4 consecutive d of one output row: f16(scale acc[4 q + r] [+ old])
__device__ __forceinline__ void store_row4(half_t *dst, const float16_t &acc, int q, float scale, int acc_old)
{
    const float a[4] = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    half4_t o;
    if (acc_old) {
        const half4_t old = *reinterpret_cast<const half4_t *>(dst);
#pragma unroll
        for (int r = 0; r < 4; r++) o[r] = f2h(scale * a[r] + h2f(old[r]));
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++) o[r] = f2h(scale * a[r]);
    }
    *reinterpret_cast<half4_t *>(dst) = o;
}

// ---------------------------------------------------------------------------------------------
template <int KS, int DT>
__global__ void __launch_bounds__(kNT, 2) attn_fwd_kernel(AttnArgs p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem, *Vs = smem + 2 * kTileB;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, l32 = lane & 31, lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int nqt = (S + kBM - 1) / kBM;
    const int h = blockIdx.x % p.H;
    const int qt = balanced_tile(blockIdx.x / p.H, nqt, true);
    const int i0 = qt * kBM, r0 = i0 + wid * 32, myrow = r0 + l32;
    const half_t *Q = p.q + (int64_t)h * Dh, *K = p.k + (int64_t)h * Dh, *V = p.v + (int64_t)h * Dh;

    half8_t qf[KS];
    load_frags<KS>(qf, Q, ld, myrow, S, Dh, lh);

    const int kend = min(i0 + kBM, S);                 // keys [0, kend) are visible to the tile
    const int njt = (kend + kTileRows - 1) / kTileRows;
    TileLoader tk, tv;

    // ---- pass 1: row maximum and sum, each lane over its half of the keys, merged at the end
    float m_run = -INFINITY, l_run = 0.f;
    tk.load(K, ld, S, Dh);
    tk.store(Ks);
    __syncthreads();
    for (int jt = 0; jt < njt; jt++) {
        const int cur = jt & 1;
        if (jt + 1 < njt) tk.load(K + (int64_t)(jt + 1) * kTileRows * ld, ld, S - (jt + 1) * kTileRows, Dh);
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            const int kb = jt * kTileRows + 32 * kt;
            if (kb > r0 + 31) continue;                  // every key of the tile is beyond every row of the wave
            const float16_t acc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
            const bool full = kb + 31 <= r0;
            float sv[16], mt = -INFINITY;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                const float s = rnd16(p.alpha * acc[e]);
                sv[e] = (full || key <= myrow) ? s : -INFINITY;
                mt = fmaxf(mt, sv[e]);
            }
            const float m_new = fmaxf(m_run, mt);
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 16; e++) sum += (sv[e] == -INFINITY) ? 0.f : exp_diff(sv[e], m_new);
            l_run = ((m_run == -INFINITY) ? 0.f : l_run * exp_diff(m_run, m_new)) + sum;
            m_run = m_new;
        }
        if (jt + 1 < njt) tk.store(Ks + (cur ^ 1) * kTileB);
        __syncthreads();
    }
    float m, l;
    {
        const float m_o = __shfl_xor(m_run, 32, 64), l_o = __shfl_xor(l_run, 32, 64);
        const float ma = lh ? m_o : m_run, la = lh ? l_o : l_run;      // the lower half of the keys' lanes first
        const float mb = lh ? m_run : m_o, lb = lh ? l_run : l_o;
        m = fmaxf(ma, mb);
        l = ((ma == -INFINITY) ? 0.f : la * exp_diff(ma, m)) + ((mb == -INFINITY) ? 0.f : lb * exp_diff(mb, m));
        if (myrow >= S) { m = 0.f; l = 1.f; }
        if (lh == 0 && myrow < S) {
            p.m[(int64_t)h * S + myrow] = m;
            p.l[(int64_t)h * S + myrow] = l;
        }
    }
    const float y = recip_refined(l);

    // ---- pass 2: probabilities and O
    float16_t oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
    tk.load(K, ld, S, Dh);
    tv.load(V, ld, S, Dh);
    tk.store(Ks);
    tv.store(Vs);
    __syncthreads();
    for (int jt = 0; jt < njt; jt++) {
        const int cur = jt & 1;
        if (jt + 1 < njt) {
            tk.load(K + (int64_t)(jt + 1) * kTileRows * ld, ld, S - (jt + 1) * kTileRows, Dh);
            tv.load(V + (int64_t)(jt + 1) * kTileRows * ld, ld, S - (jt + 1) * kTileRows, Dh);
        }
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
            const int kb = jt * kTileRows + 32 * kt;
            if (kb > r0 + 31) continue;
            const float16_t acc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
            const bool full = kb + 31 <= r0;
            float pe[16];
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                const float s = rnd16(p.alpha * acc[e]);
                const float pr = div_by(exp_diff(s, m), l, y);
                pe[e] = (full || key <= myrow) ? pr : 0.f;
            }
            prod_tr<DT>(oacc, Vs + cur * kTileB, 32 * kt, pack8(pe), pack8(pe + 8), lane);
        }
        if (jt + 1 < njt) {
            tk.store(Ks + (cur ^ 1) * kTileB);
            tv.store(Vs + (cur ^ 1) * kTileB);
        }
        __syncthreads();
    }
    if (myrow < S) {
        half_t *orow = p.out + (int64_t)myrow * ld + (int64_t)h * Dh;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int d0 = 32 * dt + 8 * q + 4 * lh;
                if (d0 < Dh) store_row4(orow + d0, oacc[dt], q, 1.0f, 0);
            }
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: queries fixed (128 per workgroup), loop over the key tiles at or before them.  Also leaves
// y = 1 / l and sigma per row for the dK / dV kernel.
template <int KS, int DT>
__global__ void __launch_bounds__(kNT, 2) attn_bwd_dq_kernel(AttnArgs p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem, *Vs = smem + 2 * kTileB;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, l32 = lane & 31, lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int nqt = (S + kBM - 1) / kBM;
    const int h = blockIdx.x % p.H;
    const int qt = balanced_tile(blockIdx.x / p.H, nqt, true);
    const int i0 = qt * kBM, r0 = i0 + wid * 32, myrow = r0 + l32;
    const int64_t hoff = (int64_t)h * Dh;
    const half_t *K = p.k + hoff, *V = p.v + hoff;

    half8_t qf[KS], gf[KS];
    load_frags<KS>(qf, p.q + hoff, ld, myrow, S, Dh, lh);
    load_frags<KS>(gf, p.dO + hoff, ld, myrow, S, Dh, lh);
    float m = 0.f, l = 1.f, sig = 0.f;
    if (myrow < S) {
        m = p.m[(int64_t)h * S + myrow];
        l = p.l[(int64_t)h * S + myrow];
    }
    const float y = recip_refined(l);

    const int kend = min(i0 + kBM, S);
    const int njt = (kend + kTileRows - 1) / kTileRows;
    TileLoader tk, tv;
    float16_t dacc[DT];
    // pass 0: sigma = sum_j P' f32(dP16); pass 1: dS16 and dQ
    auto run_pass = [&](auto pass_c) __attribute__((always_inline)) {
        constexpr int PASS = decltype(pass_c)::value;
        float part = 0.f;
        tk.load(K, ld, S, Dh);
        tv.load(V, ld, S, Dh);
        tk.store(Ks);
        tv.store(Vs);
        __syncthreads();
        for (int jt = 0; jt < njt; jt++) {
            const int cur = jt & 1;
            if (jt + 1 < njt) {
                tk.load(K + (int64_t)(jt + 1) * kTileRows * ld, ld, S - (jt + 1) * kTileRows, Dh);
                tv.load(V + (int64_t)(jt + 1) * kTileRows * ld, ld, S - (jt + 1) * kTileRows, Dh);
            }
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
                const int kb = jt * kTileRows + 32 * kt;
                if (kb > r0 + 31) continue;
                const float16_t sacc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
                const float16_t pacc = prod_direct<KS>(Vs + cur * kTileB, 32 * kt, gf, l32, lh);
                const bool full = kb + 31 <= r0;
                float de[16];
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                    const float s = rnd16(p.alpha * sacc[e]);
                    const float pr = div_by(exp_diff(s, m), l, y);
                    const float dp = rnd16(pacc[e]);
                    const float tt = pr * dp;
                    const bool live = full || key <= myrow;
                    if (PASS == 0) {
                        part += live ? tt : 0.f;
                    } else {
                        const float ds = tt - sig * pr;
                        de[e] = live ? ds : 0.f;
                    }
                }
                if (PASS == 1) prod_tr<DT>(dacc, Ks + cur * kTileB, 32 * kt, pack8(de), pack8(de + 8), lane);
            }
            if (jt + 1 < njt) {
                tk.store(Ks + (cur ^ 1) * kTileB);
                tv.store(Vs + (cur ^ 1) * kTileB);
            }
            __syncthreads();
        }
        return part;
    };
    {
        const float part = run_pass(std::integral_constant<int, 0>{});
        sig = part + __shfl_xor(part, 32, 64);
        if (lh == 0 && myrow < S) {
            p.y[(int64_t)h * S + myrow] = y;
            p.sig[(int64_t)h * S + myrow] = sig;
        }
    }
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) dacc[dt][r] = 0.f;
    run_pass(std::integral_constant<int, 1>{});
    if (myrow < S) {
        half_t *drow = p.dq + (int64_t)myrow * ld + hoff;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int d0 = 32 * dt + 8 * q + 4 * lh;
                if (d0 < Dh) store_row4(drow + d0, dacc[dt], q, p.alpha, p.acc_dq);
            }
    }
}

// ---------------------------------------------------------------------------------------------
// dK, dV: keys fixed (128 per workgroup, a lane owns one), loop over the query tiles at or after them.
template <int KS, int DT>
__global__ void __launch_bounds__(kNT, 1) attn_bwd_dkv_kernel(AttnArgs p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Qs = smem, *Gs = smem + 2 * kTileB;
    float *St = reinterpret_cast<float *>(smem + 4 * kTileB);          // [2][4][64]: m, l, y, sigma of the tile's rows
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, l32 = lane & 31, lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int nkt = (S + kBM - 1) / kBM;
    const int h = blockIdx.x % p.H;
    const int kt_ = balanced_tile(blockIdx.x / p.H, nkt, false);       // low key tiles see the most queries
    const int c00 = kt_ * kBM, c0 = c00 + wid * 32, mykey = c0 + l32;
    const int64_t hoff = (int64_t)h * Dh;
    const half_t *Q = p.q + hoff, *G = p.dO + hoff;

    half8_t kf[KS], vf[KS];
    load_frags<KS>(kf, p.k + hoff, ld, mykey, S, Dh, lh);
    load_frags<KS>(vf, p.v + hoff, ld, mykey, S, Dh, lh);

    float16_t kacc[DT], vacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            kacc[dt][r] = 0.f;
            vacc[dt][r] = 0.f;
        }
    const int iq0 = c00 / kTileRows, niq = (S + kTileRows - 1) / kTileRows;
    // the four per-row statistics of a 64-query tile: lane t of wave w fetches array w, row t
    const float *stat_src = (wid == 0 ? p.m : wid == 1 ? p.l : wid == 2 ? p.y : p.sig) + (int64_t)h * S;
    const float stat_pad = (wid == 1 || wid == 2) ? 1.f : 0.f;
    TileLoader tq, tg;
    float st;
    auto load_stat = [&](int iq) __attribute__((always_inline)) {
        const int row = iq * kTileRows + lane;
        const float t = stat_src[row < S ? row : S - 1];
        st = row < S ? t : stat_pad;
    };
    tq.load(Q + (int64_t)iq0 * kTileRows * ld, ld, S - iq0 * kTileRows, Dh);
    tg.load(G + (int64_t)iq0 * kTileRows * ld, ld, S - iq0 * kTileRows, Dh);
    load_stat(iq0);
    tq.store(Qs);
    tg.store(Gs);
    St[wid * 64 + lane] = st;
    __syncthreads();
    for (int iq = iq0; iq < niq; iq++) {
        const int cur = (iq - iq0) & 1;
        if (iq + 1 < niq) {
            tq.load(Q + (int64_t)(iq + 1) * kTileRows * ld, ld, S - (iq + 1) * kTileRows, Dh);
            tg.load(G + (int64_t)(iq + 1) * kTileRows * ld, ld, S - (iq + 1) * kTileRows, Dh);
            load_stat(iq + 1);
        }
        const float *stc = St + cur * 256;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const int qb0 = iq * kTileRows + 32 * qb;
            if (qb0 + 31 < c0 || qb0 >= S) continue;     // every query of the block is before every key of the wave
            const float16_t sacc = prod_direct<KS>(Qs + cur * kTileB, 32 * qb, kf, l32, lh);
            const float16_t pacc = prod_direct<KS>(Gs + cur * kTileB, 32 * qb, vf, l32, lh);
            const bool full = qb0 >= c0 + 31 && qb0 + 32 <= S;
            float pe[16], de[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int qi = 32 * qb + 8 * q + 4 * lh;
                const float4_t mm = *reinterpret_cast<const float4_t *>(stc + 0 * 64 + qi);
                const float4_t ll = *reinterpret_cast<const float4_t *>(stc + 1 * 64 + qi);
                const float4_t yy = *reinterpret_cast<const float4_t *>(stc + 2 * 64 + qi);
                const float4_t sg = *reinterpret_cast<const float4_t *>(stc + 3 * 64 + qi);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int e = 4 * q + r, query = iq * kTileRows + qi + r;
                    const float s = rnd16(p.alpha * sacc[e]);
                    const float pr = div_by(exp_diff(s, mm[r]), ll[r], yy[r]);
                    const float dp = rnd16(pacc[e]);
                    const float tt = pr * dp;
                    const float ds = tt - sg[r] * pr;
                    const bool live = full || (query >= mykey && query < S);
                    pe[e] = live ? pr : 0.f;
                    de[e] = live ? ds : 0.f;
                }
            }
            prod_tr<DT>(vacc, Gs + cur * kTileB, 32 * qb, pack8(pe), pack8(pe + 8), lane);
            prod_tr<DT>(kacc, Qs + cur * kTileB, 32 * qb, pack8(de), pack8(de + 8), lane);
        }
        if (iq + 1 < niq) {
            tq.store(Qs + (cur ^ 1) * kTileB);
            tg.store(Gs + (cur ^ 1) * kTileB);
            St[(cur ^ 1) * 256 + wid * 64 + lane] = st;
        }
        __syncthreads();
    }
    if (mykey < S) {
        half_t *krow = p.dk + (int64_t)mykey * ld + hoff, *vrow = p.dv + (int64_t)mykey * ld + hoff;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int d0 = 32 * dt + 8 * q + 4 * lh;
                if (d0 < Dh) {
                    store_row4(vrow + d0, vacc[dt], q, 1.0f, p.acc_dv);
                    store_row4(krow + d0, kacc[dt], q, p.alpha, p.acc_dk);
                }
            }
    }
}

constexpr size_t kFwdSmem = 4 * kTileB;
constexpr size_t kDkvSmem = 4 * kTileB + 2 * 4 * 64 * sizeof(float);

template <class K>
int set_smem(K kern, size_t bytes)
{
    CACTI_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return 0;
}

template <int KS, int DT>
int launch_fwd(const AttnArgs &p, hipStream_t st)
{
    static bool ready = false;
    if (!ready) {
        int rc = set_smem(attn_fwd_kernel<KS, DT>, kFwdSmem);
        if (rc) return rc;
        ready = true;
    }
    const int nqt = (p.S + kBM - 1) / kBM;
    hipLaunchKernelGGL((attn_fwd_kernel<KS, DT>), dim3((unsigned)(nqt * p.H)), dim3(kNT), kFwdSmem, st, p);
    return launch_status("attention_fwd");
}

template <int KS, int DT>
int launch_bwd(const AttnArgs &p, hipStream_t st)
{
    static bool ready = false;
    if (!ready) {
        int rc = set_smem(attn_bwd_dq_kernel<KS, DT>, kFwdSmem);
        if (rc) return rc;
        if ((rc = set_smem(attn_bwd_dkv_kernel<KS, DT>, kDkvSmem))) return rc;
        ready = true;
    }
    const int nqt = (p.S + kBM - 1) / kBM;
    hipLaunchKernelGGL((attn_bwd_dq_kernel<KS, DT>), dim3((unsigned)(nqt * p.H)), dim3(kNT), kFwdSmem, st, p);
    int rc = launch_status("attention_bwd_dq");
    if (rc) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<KS, DT>), dim3((unsigned)(nqt * p.H)), dim3(kNT), kDkvSmem, st, p);
    return launch_status("attention_bwd_dkv");
}

int check_shape(const char *who, int64_t S, int64_t H, int64_t Dh, int64_t ld)
{
    CACTI_REQUIRE(S > 0 && H > 0 && Dh > 0, CACTI_E_INVALID, "%s: empty shape", who);
    CACTI_REQUIRE(Dh % 4 == 0 && Dh <= kDP, CACTI_E_NOTIMPL, "%s: need Dh %% 4 == 0 and Dh <= %d (Dh=%lld)", who, kDP,
                  (long long)Dh);
    CACTI_REQUIRE(ld >= H * Dh && ld % 4 == 0, CACTI_E_INVALID, "%s: row stride %lld must be a multiple of 4 and >= H*Dh",
                  who, (long long)ld);
    CACTI_REQUIRE(S <= (1 << 24) && S * H < ((int64_t)1 << 31) / 2, CACTI_E_NOTIMPL, "%s: S = %lld is too large", who,
                  (long long)S);
    return 0;
}

}  // namespace

CACTI_API size_t cacti_hip_attention_stats_bytes(int64_t S, int64_t H)
{
    return (S > 0 && H > 0) ? (size_t)(2 * S * H) * sizeof(float) : 0;
}

CACTI_API size_t cacti_hip_attention_bwd_workspace(int64_t S, int64_t H)
{
    return (S > 0 && H > 0) ? (size_t)(2 * S * H) * sizeof(float) : 0;
}

CACTI_API int cacti_hip_attention_fwd(int64_t S, int64_t H, int64_t Dh, float alpha, const void *q, const void *k,
                                      const void *v, int64_t ld, void *o, void *stats, void *stream)
{
    int rc = check_shape("attention_fwd", S, H, Dh, ld);
    if (rc) return rc;
    CACTI_REQUIRE(q && k && v && o && stats, CACTI_E_INVALID, "attention_fwd: null pointer");
    CACTI_REQUIRE(aligned(q, 8) && aligned(k, 8) && aligned(v, 8) && aligned(o, 8) && aligned(stats, 4),
                  CACTI_E_INVALID, "attention_fwd: tensors must be 8-byte aligned");
    AttnArgs p = {};
    p.S = (int)S; p.H = (int)H; p.Dh = (int)Dh; p.ld = ld; p.alpha = alpha;
    p.q = (const half_t *)q; p.k = (const half_t *)k; p.v = (const half_t *)v;
    p.out = (half_t *)o;
    p.m = (float *)stats;
    p.l = p.m + S * H;
    hipStream_t st = (hipStream_t)stream;
    if (Dh <= 64) return launch_fwd<4, 2>(p, st);
    if (Dh <= 112) return launch_fwd<7, 4>(p, st);
    return launch_fwd<8, 4>(p, st);
}

CACTI_API int cacti_hip_attention_bwd(int64_t S, int64_t H, int64_t Dh, float alpha, const void *q, const void *k,
                                      const void *v, const void *dO, int64_t ld, const void *stats,
                                      void *dq, int dq_acc, void *dk, int dk_acc, void *dv, int dv_acc,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = check_shape("attention_bwd", S, H, Dh, ld);
    if (rc) return rc;
    CACTI_REQUIRE(q && k && v && dO && stats && dq && dk && dv && workspace, CACTI_E_INVALID,
                  "attention_bwd: null pointer");
    CACTI_REQUIRE(aligned(q, 8) && aligned(k, 8) && aligned(v, 8) && aligned(dO, 8) &&
                      aligned(dq, 8) && aligned(dk, 8) && aligned(dv, 8) && aligned(stats, 4) && aligned(workspace, 4),
                  CACTI_E_INVALID, "attention_bwd: tensors must be 8-byte aligned");
    CACTI_REQUIRE(workspace_bytes >= cacti_hip_attention_bwd_workspace(S, H), CACTI_E_INVALID,
                  "attention_bwd: workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                  cacti_hip_attention_bwd_workspace(S, H));
    AttnArgs p = {};
    p.S = (int)S; p.H = (int)H; p.Dh = (int)Dh; p.ld = ld; p.alpha = alpha;
    p.q = (const half_t *)q; p.k = (const half_t *)k; p.v = (const half_t *)v;
    p.dO = (const half_t *)dO;
    p.dq = (half_t *)dq; p.dk = (half_t *)dk; p.dv = (half_t *)dv;
    p.acc_dq = dq_acc; p.acc_dk = dk_acc; p.acc_dv = dv_acc;
    p.m = (float *)const_cast<void *>(stats);
    p.l = p.m + S * H;
    p.y = (float *)workspace;
    p.sig = p.y + S * H;
    hipStream_t st = (hipStream_t)stream;
    if (Dh <= 64) return launch_bwd<4, 2>(p, st);
    if (Dh <= 112) return launch_bwd<7, 4>(p, st);
    return launch_bwd<8, 4>(p, st);
}
