// C[M,N] = f16(alpha A B^T) for a short inner dimension (K <= 128): the attention scores
// Q K^T and dP = dO V^T, where K is the head dimension and the output is sequence x sequence
// per head.  Such a product is bound by writing C, not by its MFMAs, so the general tile kernel's
// load -> barrier -> compute -> barrier chain per 128 x 128 tile (two k tiles, nothing to
// overlap them with) leaves the chip idle most of the time.  Here a workgroup keeps its 128
// rows of A as MFMA fragments in registers for its whole life and walks up to kTilesPerBlock
// column tiles: while the MFMAs and the store of tile t run, the rows of B for tile t + 1 are
// already on their way into registers.
//
//   per column tile:  B rows (regs) -> LDS | 28..32 MFMAs per wave | accumulators -> f16 -> LDS
//                     (row-contiguous staging) -> 16-byte global stores of whole row segments
//
// LDS: B tile 128 x (K padded to 16) halves with an 8-half pad per row (the 16-byte fragment
// reads of 8 consecutive rows then fall into distinct bank groups), C staging 128 x 128.
// Two workgroups fit a CU.  Operands need 8-byte alignment only (head_dim 100).
#include "common.h"
#include <stdlib.h>
#include "gemm_internal.h"

using namespace cacti;

namespace {

constexpr int kThreads = 256;
constexpr int kTile = 128;
constexpr int kTilesPerBlock = 4;

struct SmallKArgs {
    GemmArgs g;
    int chunks;         // column chunks (of kTilesPerBlock tiles) per row tile
    int store16;        // C rows allow 16-byte stores
    int tpb;            // column tiles per block
};

// 8 halves starting at k of a row of K halves (K % 4 == 0, k % 8 == 0, row 8-byte aligned):
// two 8-byte loads clamped into the row, zero beyond K
__device__ __forceinline__ uint4 load_chunk(const half_t *row, int k, int K)
{
    const int left = K - k;                                   // valid halves from k on
    const int k0 = left >= 4 ? k : K - 4, k1 = left >= 8 ? k + 4 : K - 4;
    const uint2 lo = *reinterpret_cast<const uint2 *>(row + k0);
    const uint2 hi = *reinterpret_cast<const uint2 *>(row + k1);
    uint4 v = make_uint4(lo.x, lo.y, hi.x, hi.y);
    if (left < 4) { v.x = 0; v.y = 0; }
    if (left < 8) { v.z = 0; v.w = 0; }
    return v;
}

template <int KS>
__global__ void __launch_bounds__(kThreads, 2)
gemm_nt_smallk_kernel(SmallKArgs a)
{
    constexpr int PITCH = KS * 16 + 8;                        // halves per LDS row of B
    constexpr int CHUNKS = 2 * KS;                            // 16-byte chunks per row
    constexpr int NLD = (kTile * CHUNKS) / kThreads;          // chunks per lane per tile (= KS)
    static_assert((kTile * CHUNKS) % kThreads == 0, "whole chunks per lane");
    __shared__ __attribute__((aligned(16))) half_t Ks[kTile * PITCH];
    // C staging; also parks the A tile (pitch PITCH) before the first column tile
    __shared__ __attribute__((aligned(16))) half_t Cs[kTile * (PITCH > kTile ? PITCH : kTile)];
    const GemmArgs &p = a.g;

    // XCD-aware numbering (dispatch order i lands on XCD i % 8): a contiguous band of the
    // (batch block, row tile, column chunk) sequence per XCD, i.e. whole heads when the
    // batch is a multiple of 8, which balances the triangular case
    const int nb = gridDim.x;
    int bid = blockIdx.x;
    {
        const int per = nb >> 3, rem = nb & 7;
        const int xcd = bid & 7, idx = bid >> 3;
        bid = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    const int per_head = p.tiles_m * a.chunks;
    const int64_t bz = bid / per_head;
    const int r = bid - (int)bz * per_head;
    const int tm = p.tiles_m - 1 - r / a.chunks;              // long rows first
    const int tn0 = (r % a.chunks) * a.tpb;
    int tn1 = min(p.tiles_n, tn0 + a.tpb);
    if (p.tri == 1) tn1 = min(tn1, tm + 1);                   // tiles wholly above the diagonal
    if (tn0 >= tn1) return;                                   // uniform for the block

    const half_t *A = p.A + bz * p.sa;
    const half_t *B = p.B + bz * p.sb;
    half_t *C = p.C + bz * p.sc;
    const int64_t m0 = (int64_t)tm * kTile;
    const int K = (int)p.K;

    const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
    const int wm = wid & 1, wn = wid >> 1;
    const int l32 = lane & 31, lh = lane >> 5;

    half8_t aq[2][KS];          // A fragments, filled below

    // B tile loads: chunk c = tid + it * 256 of the tile is (row c / CHUNKS, k chunk c % CHUNKS).
    // Byte offsets from the tile's first row and the zero masks of the k tail depend on the lane
    // only and are computed once; a tile that reaches past N clamps its rows instead.
    uint4 kreg[NLD];
    uint32_t boff[NLD];         // byte offset (a multiple of 8) | 1: low half valid | 2: high half valid
#pragma unroll
    for (int it = 0; it < NLD; it++) {
        const int c = tid + it * kThreads;
        const int row = c / CHUNKS, k = (c - row * CHUNKS) * 8;
        const int left = K - k;
        const int k0 = left >= 4 ? k : K - 4;                 // an invalid half re-reads a valid one
        boff[it] = (uint32_t)((row * p.ldb + k0) * 2) | (left >= 4 ? 1u : 0u) | (left >= 8 ? 2u : 0u);
    }
    auto load_b = [&](int tn) __attribute__((always_inline)) {
        const int64_t n0 = (int64_t)tn * kTile;
        const char *base = reinterpret_cast<const char *>(B + n0 * p.ldb);
        if (n0 + kTile <= p.N) {                              // uniform
#pragma unroll
            for (int it = 0; it < NLD; it++) {
                const uint32_t m0_ = (uint32_t)__builtin_amdgcn_sbfe((int)boff[it], 0, 1);   // 0 or ~0
                const uint32_t m1_ = (uint32_t)__builtin_amdgcn_sbfe((int)boff[it], 1, 1);
                const uint32_t off = boff[it] & ~7u;
                const uint2 lo = *reinterpret_cast<const uint2 *>(base + off);
                const uint2 hi = *reinterpret_cast<const uint2 *>(base + off + (m1_ & 8u));
                kreg[it] = make_uint4(lo.x & m0_, lo.y & m0_, hi.x & m1_, hi.y & m1_);
            }
        } else {
#pragma unroll
            for (int it = 0; it < NLD; it++) {
                const int c = tid + it * kThreads;
                const int row = c / CHUNKS, kc = c - row * CHUNKS;
                int64_t n = n0 + row;
                if (n > p.N - 1) n = p.N - 1;
                kreg[it] = load_chunk(B + n * p.ldb, kc * 8, K);
            }
        }
    };
    auto store_b = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < NLD; it++) {
            const int c = tid + it * kThreads;
            const int row = c / CHUNKS, kc = c - row * CHUNKS;
            *reinterpret_cast<uint4 *>(Ks + row * PITCH + kc * 8) = kreg[it];
        }
    };

    // staging addresses of the epilogue: row & 15 == l32 & 15 for every 32-row tile of a wave
    int cs_wr[2][4];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int chunk = wn * 8 + j * 4 + q;
            cs_wr[j][q] = (wm * 64 + l32) * kTile + (((chunk ^ (l32 & 15)) << 3) | (lh * 4));
        }
    // store side: lane = (row tid / 16 + 16 it, 16-byte chunk tid % 16)
    const int srow = tid >> 4, scc = tid & 15;
    const half_t *cs_rd = Cs + srow * kTile + ((scc ^ (srow & 15)) << 3);
    half_t *c_lane = C + (m0 + srow) * p.ldc + scc * 8;
    const bool rows_full = m0 + kTile <= p.M;

    // A tile: loaded like a B tile (consecutive lanes take consecutive 16-byte chunks of a row:
    // fragment-shaped global loads would touch 32 rows per instruction), parked in the C staging
    // buffer, and read back as MFMA fragments (lane = row l32 of a 32-row tile, k chunk lh of
    // each 16-wide k step) that stay in registers for the block's life
    {
        uint4 areg[NLD];
#pragma unroll
        for (int it = 0; it < NLD; it++) {
            const int c = tid + it * kThreads;
            const int row = c / CHUNKS, kc = c - row * CHUNKS;
            int64_t m = m0 + row;
            if (m > p.M - 1) m = p.M - 1;
            areg[it] = load_chunk(A + m * p.lda, kc * 8, K);
        }
        load_b(tn0);
#pragma unroll
        for (int it = 0; it < NLD; it++) {
            const int c = tid + it * kThreads;
            const int row = c / CHUNKS, kc = c - row * CHUNKS;
            *reinterpret_cast<uint4 *>(Cs + row * PITCH + kc * 8) = areg[it];
        }
        store_b();
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                aq[i][ks] = *reinterpret_cast<const half8_t *>(Cs + (wm * 64 + i * 32 + l32) * PITCH +
                                                               (ks * 2 + lh) * 8);
        if (tn0 + 1 < tn1) load_b(tn0 + 1);
        __syncthreads();                      // the staging buffer is free for the first C tile
    }

    for (int tn = tn0; tn < tn1; tn++) {
        float16_t acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            half8_t bf[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
                bf[j] = *reinterpret_cast<const half8_t *>(Ks + (wn * 64 + j * 32 + l32) * PITCH +
                                                           (ks * 2 + lh) * 8);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], aq[i][ks], acc[i][j], 0, 0, 0);
        }

        // a lane holds row l32 and, per accumulator group q, the 4 consecutive columns
        // 8 q + 4 lh + {0..3} of each 32 x 32 tile: staged as Cs[row][128] with the 16-byte
        // chunks of a row swizzled by the row, the tile leaves as contiguous row segments
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    half4_t o;
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = f2h(p.alpha * acc[i][j][q * 4 + e]);
                    *reinterpret_cast<half4_t *>(Cs + i * 32 * kTile + cs_wr[j][q]) = o;
                }
        __syncthreads();                      // B tile consumed, C tile staged
        // the loads of the tile after next are issued BEFORE this tile's stores: the wait for
        // them (one iteration later) then leaves the younger stores outstanding instead of
        // draining the whole write queue every tile
        if (tn + 1 < tn1) store_b();
        if (tn + 2 < tn1) load_b(tn + 2);

        const int64_t n0 = (int64_t)tn * kTile;
        if (rows_full && n0 + kTile <= p.N && a.store16) {    // uniform: whole tile, 16-byte rows
#pragma unroll
            for (int it = 0; it < kTile / 16; it++)
                *reinterpret_cast<uint4 *>(c_lane + n0 + (int64_t)it * 16 * p.ldc) =
                    *reinterpret_cast<const uint4 *>(cs_rd + it * 16 * kTile);
        } else {
#pragma unroll
            for (int it = 0; it < kTile / 16; it++) {
                const int64_t m = m0 + srow + it * 16, n = n0 + scc * 8;
                if (m >= p.M || n >= p.N) continue;
                const uint4 v = *reinterpret_cast<const uint4 *>(cs_rd + it * 16 * kTile);
                half_t *cp = c_lane + n0 + (int64_t)it * 16 * p.ldc;
                if (a.store16 && n + 8 <= p.N) {
                    *reinterpret_cast<uint4 *>(cp) = v;
                } else {
                    *reinterpret_cast<uint2 *>(cp) = make_uint2(v.x, v.y);
                    if (n + 8 <= p.N) *reinterpret_cast<uint2 *>(cp + 4) = make_uint2(v.z, v.w);
                }
            }
        }
        __syncthreads();                      // next B tile in LDS, staging buffer free
    }
}

template <int KS>
int launch(const SmallKArgs &a, int64_t nblk, hipStream_t st)
{
    const int64_t nwg = (int64_t)a.g.tiles_m * a.chunks * nblk;
    CACTI_REQUIRE(nwg < (int64_t)1 << 31, CACTI_E_NOTIMPL, "gemm: %lld workgroups exceed the grid limit",
                  (long long)nwg);
    hipLaunchKernelGGL(gemm_nt_smallk_kernel<KS>, dim3((unsigned)nwg), dim3(kThreads), 0, st, a);
    return launch_status("gemm_nt_smallk");
}

}  // namespace

namespace cacti {

// A [M,K] and B [N,K] row-major with K <= 128, K % 4 == 0 and 8-byte aligned rows; beta = 0;
// tri 0 or 1.
int gemm_nt_smallk_launch(const GemmArgs &p, int64_t nblk, hipStream_t st)
{
    SmallKArgs a;
    a.g = p;
    a.g.tiles_m = (int)((p.M + kTile - 1) / kTile);
    a.g.tiles_n = (int)((p.N + kTile - 1) / kTile);
    // Column tiles per workgroup: a third of the tile row once it is long enough.  Measured at
    // 32 heads x 2048 x 2048, lower triangle (us per launch inside the training step): 1: 69.0,
    // 2: 64.3, 3: 58.3, 4: 68.7, 5: 74.9, 6: 56.9, 7: 59.4, 8: 69.5, 16: 75.3 -- the counts of
    // workgroups per head that are powers of two (16 x 4, 16 x 2, ..) are the slow ones: the
    // workgroups resident together then write tiles whose addresses differ by multiples of the
    // same large power of two.
    a.tpb = a.g.tiles_n >= 6 ? (a.g.tiles_n + 2) / 3 : kTilesPerBlock;
    a.chunks = (a.g.tiles_n + a.tpb - 1) / a.tpb;
    CACTI_REQUIRE(p.ldb < ((int64_t)1 << 22), CACTI_E_NOTIMPL, "gemm: ldb %lld too large for the short-K kernel",
                  (long long)p.ldb);
    a.store16 = (p.ldc % 8 == 0) && (nblk == 1 || p.sc % 8 == 0) && aligned(p.C, 16);
    if (p.K <= 64) return launch<4>(a, nblk, st);
    if (p.K <= 112) return launch<7>(a, nblk, st);
    return launch<8>(a, nblk, st);
}

}  // namespace cacti
