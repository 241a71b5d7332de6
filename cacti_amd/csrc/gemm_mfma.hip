// Fast path of the f16 GEMM for operands whose rows are at least 8-byte aligned (every
// projection, LM-head and attention GEMM of the step; head_dim 100 gives 8-byte alignment).
//
//   C[M,N] = alpha op(A) op(B) + beta C,   f16 in, fp32 MFMA accumulate, f16 out.
//
// Block tile BM x BN x 64, WM x WN wavefronts, each owning BM / WM x BN / WN outputs as 32 x 32
// blocks that are interleaved with those of the other waves (32 WM rows / 32 WN columns apart).
// The register path forms a block with v_mfma_f32_32x32x16_f16; the direct path, which carries the
// large products of the step, as four 16 x 16 results of v_mfma_f32_16x16x32_f16: under a sustained
// load the device is limited by power, and that instruction needs less of it per flop.  Shapes
// instantiated: 128 x 128 on 4 waves (two workgroups per CU), 256 x 128 and 256 x 256 on 8
// waves (one per CU), 64 x 64 on 4 waves (remainder columns).
//
// Two ways from global memory to LDS.  Through registers (any alignment >= 8 bytes, k tails):
// described below.  Direct (16-byte aligned operands, K a multiple of 64; the large dense
// products): global_load_lds_dwordx4 writes each wave's 1 KB straight into LDS, NBUF - 1 k
// tiles ahead, with no staging registers, no LDS store instructions and no transposes in
// registers; a k-contiguous operand lands in the swizzled [row][k] layout below (the swizzle
// is applied to the global address), a k-strided one in its own [k][row] layout and is
// transposed on the way out of LDS by ds_read_b64_tr_b16.
//
// LDS layout (both operands): [row][64 k] = 128 bytes per row, no padding; the 16-byte
// k-chunk q of row r sits at chunk position q ^ f(r), f(r) = (r ^ (r >> 3)) & 7.
// With this swizzle (a) the 16-byte MFMA operand reads of 8 consecutive rows, (b) the
// 16-byte writes of a k-contiguous global row and (c) the writes of the register
// transpose (lanes 8 rows apart) each cover all eight 16-byte bank groups of a 128-byte
// LDS line, and 16 consecutive rows also spread over both halves of a 256-byte line.
//
// An operand whose k index is not contiguous in memory (A^T, or B not transposed) is
// loaded as blocks of k-rows x 8 tile-rows per lane with fully coalesced 16-byte loads,
// transposed in registers with v_perm_b32, and written as 8 row pieces: the MFMA read path is
// identical for NN / NT / TN / TT.  The block of a lane is 8, 4 or 2 k-rows deep, whichever
// spreads the operand tile over every lane of the workgroup.
//
// The main loop has no branch: every lane's global offsets (32-bit, relative to the tile
// origin, clamped into the operand) are computed once, a k step only moves a uniform base
// pointer.  Rows beyond the edge read a duplicate of the last rows (they only feed outputs
// that are never stored); a k tail is zeroed with selects (KTAIL instantiations only).
// With STAGES = 2 the global loads of k tile t+2 are issued before the MFMAs of tile t and
// stored to LDS after the MFMAs of tile t+1 (two register stages + double-buffered LDS);
// STAGES = 1 looks one tile ahead.  One barrier per k tile; in the direct kernels it sits before
// the tile's last k step, so that the loads of a later tile and the first fragments of the next
// one are issued between the MFMAs of that step and no wave waits on LDS behind a barrier.  Workgroups are numbered so
// that the 8 XCDs (round-robin dispatch) each walk a contiguous band of tiles and reuse
// the operand panels in their own L2.
#include "common.h"
#include "gemm_internal.h"

#include <type_traits>

using namespace cacti;

namespace {

constexpr int BK = 64;

__device__ __forceinline__ int swz(int r) { return ((r >> 3) ^ r) & 7; }
// The same for the direct path, whose fragments (v_mfma_f32_16x16x32_f16) are 16 rows x four 16-byte k
// chunks per wave instruction instead of 32 rows x two: with swz() those reads take two passes through
// LDS (measured: 286 against 493 GB/s per CU), with this one a single pass (484).  Period 32 rows.
__device__ __forceinline__ int swz16(int r) { return ((r >> 2) ^ r) & 7; }

// 16-byte chunk q (0..7) of tile row r
__device__ __forceinline__ int lds_off(int r, int q) { return r * BK + ((q ^ swz(r)) << 3); }

__device__ __forceinline__ const half_t *at(const half_t *base, uint32_t byte_off)
{
    return reinterpret_cast<const half_t *>(reinterpret_cast<const char *>(base) + byte_off);
}

// 8 halves as one 16-byte load (AL = 8) or two 8-byte loads (AL = 4: operands that are only
// 8-byte aligned, whose extents are multiples of 4); off1 = offset of the second half
template <int AL>
__device__ __forceinline__ uint4 ld8(const half_t *base, uint32_t off0, uint32_t off1)
{
    if (AL == 8) return *reinterpret_cast<const uint4 *>(at(base, off0));
    const uint2 lo = *reinterpret_cast<const uint2 *>(at(base, off0));
    const uint2 hi = *reinterpret_cast<const uint2 *>(at(base, off1));
    return make_uint4(lo.x, lo.y, hi.x, hi.y);
}

// ---- k-contiguous operand (memory [row][k]): chunk c -> row c / 8, k-chunk c % 8 ----------
template <int ROWS, int NT, int AL, bool KTAIL>
struct LoadKC {
    static constexpr int ITEMS = ROWS * 8;
    static constexpr int NL = (ITEMS + NT - 1) / NT;
    uint32_t off[NL];              // byte offset of the chunk from (row0, k = 0)
    int64_t ld, K;

    // rows_left = R - row0 > 0
    __device__ __forceinline__ void init(int64_t ld_, int64_t rows_left, int64_t K_)
    {
        ld = ld_;
        K = K_;
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            int row = (c >> 3) % ROWS;
            const int kc = c & 7;
            if (row >= rows_left) row = (int)rows_left - 1;
            off[it] = (uint32_t)((row * ld + kc * 8) * 2);
        }
    }
    // origin = &op[row0][0]
    __device__ __forceinline__ void load(uint4 *st, const half_t *origin, int64_t k0) const
    {
        const half_t *base = origin + k0;
        const bool whole = !KTAIL || k0 + BK <= K;     // uniform: only the last k tile has a tail
#pragma unroll
        for (int it = 0; it < NL; it++) {
            if (whole) {
                st[it] = ld8<AL>(base, off[it], off[it] + 8);
            } else {
                const int kc = (threadIdx.x + it * NT) & 7;
                const int left = (int)(K - k0) - kc * 8;        // valid halves from this chunk on
                // clamp both halves back into the row; zero what lies beyond K
                const uint32_t back0 = left >= AL ? 0 : (uint32_t)(AL - left) * 2;
                const uint32_t back1 = left >= 8 ? 0 : (uint32_t)(8 - (left > 4 ? left : 4)) * 2;
                uint4 v = ld8<AL>(base, off[it] - back0, off[it] + 8 - back0 - back1);
                if (AL == 8) {
                    if (left <= 0) v = make_uint4(0, 0, 0, 0);
                } else {
                    if (left <= 0) { v.x = 0; v.y = 0; }
                    if (left <= 4) { v.z = 0; v.w = 0; }
                }
                st[it] = v;
            }
        }
    }
    __device__ __forceinline__ void store(const uint4 *st, half_t *lds) const
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int row = c >> 3, kc = c & 7;
            if (ITEMS % NT == 0 || c < ITEMS)
                *reinterpret_cast<uint4 *>(lds + lds_off(row, kc)) = st[it];
        }
    }
    static constexpr int NREG = NL;
    static constexpr int NDMA = 0;
    __device__ __forceinline__ void dma(uint32_t, const half_t *, int64_t) const {}
};

// ---- k-contiguous operand fetched straight into LDS (global_load_lds_dwordx4: the 16 bytes
// of lane l land at LDS address M0 + 16 l, no register staging and no LDS store instruction).
// A wave fills 1 KB = 8 consecutive tile rows per instruction; the chunk swizzle of the LDS
// layout is applied on the global side: the lane at chunk position p of row r fetches k chunk
// p ^ f(r), which stays inside the row's 128-byte segment.  The loads are issued from inline
// assembly, so the compiler neither counts them nor knows that they write LDS: the kernel
// waits for them itself (vmcnt) before the barrier that publishes the tile.
template <int ROWS, int NT>
struct LoadKCD {
    static_assert(ROWS * 8 % NT == 0, "whole instructions per wave");
    static constexpr int NL = ROWS * 8 / NT;
    uint32_t off[NL];              // byte offset of the lane's chunk from (row0, k = 0)

    __device__ __forceinline__ void init(int64_t ld, int64_t rows_left, int64_t)
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int r = c >> 3, q = (c & 7) ^ swz16(r);
            const int64_t row = r < rows_left ? r : rows_left - 1;
            off[it] = (uint32_t)((row * ld + q * 8) * 2);
        }
    }
    // lds = byte address in LDS of the tile buffer to fill; origin = &op[row0][0]
    __device__ __forceinline__ void dma(uint32_t lds, const half_t *origin, int64_t k0) const
    {
        const half_t *base = origin + k0;
        const uint32_t wave = lds + (threadIdx.x & ~63u) * 16;
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const uint32_t m0 = __builtin_amdgcn_readfirstlane(wave + it * NT * 16);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :
                         : "s"(m0), "v"(off[it]), "s"(base)
                         : "memory");
        }
    }
    // instruction `it` of the NL alone (base = origin + k0): lets the caller place each load between MFMAs
    __device__ __forceinline__ void dma1(int it, uint32_t lds, const half_t *base) const
    {
        const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds + (threadIdx.x & ~63u) * 16 + it * NT * 16);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(m0), "v"(off[it]), "s"(base)
                     : "memory");
    }
    __device__ __forceinline__ const half_t *kbase(const half_t *origin, int64_t k0) const { return origin + k0; }
    __device__ __forceinline__ void load(uint4 *, const half_t *, int64_t) const {}
    __device__ __forceinline__ void store(const uint4 *, half_t *) const {}
    static constexpr int NREG = 1;
    static constexpr int NDMA = NL;
};

// ---- k-strided operand (memory [k][row]) fetched straight into LDS in its own layout,
// [64 k][ROWS] with the 16-byte chunks of k row k swizzled by 2 (k & 3); the MFMA fragments
// come out of it through ds_read_b64_tr_b16, which hands each lane of a 16-lane group 4
// consecutive k of one row from a 4 k x 16 rows block (the swizzle spreads the 4 k rows of such
// a block over all banks).  A wave fills 1 KB = 1024 / (2 ROWS) whole k rows per instruction.
template <int ROWS, int NT>
struct LoadKSD {
    static constexpr int CPR = ROWS / 8;           // 16-byte chunks per k row
    static_assert(BK * CPR % NT == 0 && CPR >= 8, "whole instructions per wave");
    static constexpr int NL = BK * CPR / NT;
    uint32_t off[NL];              // byte offset of the lane's chunk from (k = 0, row0)
    int64_t ld;

    __device__ __forceinline__ void init(int64_t ld_, int64_t rows_left, int64_t)
    {
        ld = ld_;
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = threadIdx.x + it * NT;
            const int k = c / CPR, q = (c % CPR) ^ (2 * (k & 3));
            int64_t col = q * 8;
            if (col > rows_left - 8) col = rows_left - 8;          // rows_left is a multiple of 8
            off[it] = (uint32_t)((k * ld_ + col) * 2);
        }
    }
    // lds = byte address in LDS of the tile buffer to fill; origin = &op[0][row0]
    __device__ __forceinline__ void dma(uint32_t lds, const half_t *origin, int64_t k0) const
    {
        const half_t *base = origin + k0 * ld;
        const uint32_t wave = lds + (threadIdx.x & ~63u) * 16;
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const uint32_t m0 = __builtin_amdgcn_readfirstlane(wave + it * NT * 16);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :
                         : "s"(m0), "v"(off[it]), "s"(base)
                         : "memory");
        }
    }
    __device__ __forceinline__ void dma1(int it, uint32_t lds, const half_t *base) const
    {
        const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds + (threadIdx.x & ~63u) * 16 + it * NT * 16);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(m0), "v"(off[it]), "s"(base)
                     : "memory");
    }
    __device__ __forceinline__ const half_t *kbase(const half_t *origin, int64_t k0) const { return origin + k0 * ld; }
    __device__ __forceinline__ void load(uint4 *, const half_t *, int64_t) const {}
    __device__ __forceinline__ void store(const uint4 *, half_t *) const {}
    static constexpr int NREG = 1;
    static constexpr int NDMA = NL;
};

// ---- k-strided operand (memory [k][row]): item c -> row chunk c % (ROWS/8), k group
// c / (ROWS/8); an item is 8 k x 8 rows.  T0 = first thread that takes part (lets two
// strided operands use disjoint halves of the block).
template <int ROWS, int NT, int T0, int AL, bool KTAIL>
struct LoadKS {
    static constexpr int RC = ROWS / 8;
    static constexpr int ITEMS = RC * 8;
    static constexpr int NTH = NT - T0 >= ITEMS ? ITEMS : NT;      // threads taking part
    static constexpr int TB = NT - T0 >= ITEMS ? T0 : 0;
    static constexpr int NL = (ITEMS + NTH - 1) / NTH;
    uint32_t off[NL], off1[NL];    // byte offset of the item's first k row from (k = 0, row0)
    uint32_t ldb2;                 // ld in bytes
    int64_t ld, K;

    __device__ __forceinline__ int item(int it) const
    {
        const int t = ((int)threadIdx.x - TB + NT) % NT;           // non-members wrap harmlessly
        return (t + it * NTH) % ITEMS;
    }
    __device__ __forceinline__ bool mine(int it) const
    {
        const int t = (int)threadIdx.x - TB;
        return t >= 0 && t < NTH && t + it * NTH < ITEMS;
    }
    __device__ __forceinline__ void init(int64_t ld_, int64_t rows_left, int64_t K_)
    {
        ld = ld_;
        K = K_;
        ldb2 = (uint32_t)(ld_ * 2);
#pragma unroll
        for (int it = 0; it < NL; it++) {
            const int c = item(it);
            const int rc = c % RC, kq = c / RC;
            // clamp the row chunk(s) into the operand (rows_left is a multiple of AL)
            int r0 = rc * 8, r1 = rc * 8 + 4;
            if (AL == 8) {
                if (r0 > rows_left - 8) r0 = (int)rows_left - 8;
            } else {
                if (r0 > rows_left - 4) r0 = (int)rows_left - 4;
                if (r1 > rows_left - 4) r1 = (int)rows_left - 4;
            }
            off[it] = (uint32_t)(((int64_t)kq * 8 * ld + r0) * 2);
            off1[it] = (uint32_t)(((int64_t)kq * 8 * ld + r1) * 2);
        }
    }
    // origin = &op[0][row0]
    __device__ __forceinline__ void load(uint4 *st, const half_t *origin, int64_t k0) const
    {
        const half_t *base = origin + k0 * ld;
#pragma unroll
        for (int it = 0; it < NL; it++) {
            if (!mine(it)) continue;          // whole wavefronts: a uniform skip, not a lane mask
            const int kq = item(it) / RC;
#pragma unroll
            for (int kk = 0; kk < 8; kk++) {
                if (!KTAIL || k0 + BK <= K) {
                    st[it * 8 + kk] = ld8<AL>(base, off[it] + kk * ldb2, off1[it] + kk * ldb2);
                } else {
                    const int left = (int)(K - k0) - (kq * 8 + kk);   // > 0 iff this k row exists
                    const uint32_t back = left > 0 ? 0 : (uint32_t)(1 - left) * ldb2;
                    uint4 v = ld8<AL>(base, off[it] + kk * ldb2 - back, off1[it] + kk * ldb2 - back);
                    if (left <= 0) v = make_uint4(0, 0, 0, 0);
                    st[it * 8 + kk] = v;
                }
            }
        }
    }
    __device__ __forceinline__ void store(const uint4 *st, half_t *lds) const
    {
#pragma unroll
        for (int it = 0; it < NL; it++) {
            if (!mine(it)) continue;
            const int c = item(it);
            const int rc = c % RC, kq = c / RC;
            const uint32_t *w = reinterpret_cast<const uint32_t *>(st + it * 8);   // [kk][4 words]
#pragma unroll
            for (int j = 0; j < 8; j++) {
                // row j of the 8 x 8 block: halves (k = 0..7) = word j/2, half j%2 of each k row
                const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                uint4 o;
                o.x = __builtin_amdgcn_perm(w[1 * 4 + (j >> 1)], w[0 * 4 + (j >> 1)], sel);
                o.y = __builtin_amdgcn_perm(w[3 * 4 + (j >> 1)], w[2 * 4 + (j >> 1)], sel);
                o.z = __builtin_amdgcn_perm(w[5 * 4 + (j >> 1)], w[4 * 4 + (j >> 1)], sel);
                o.w = __builtin_amdgcn_perm(w[7 * 4 + (j >> 1)], w[6 * 4 + (j >> 1)], sel);
                *reinterpret_cast<uint4 *>(lds + lds_off(rc * 8 + j, kq)) = o;
            }
        }
    }
    static constexpr int NREG = NL * 8;
    static constexpr int NDMA = 0;
    __device__ __forceinline__ void dma(uint32_t, const half_t *, int64_t) const {}
};

// ---- both operands k-strided (A^T and B), square block tile with exactly one 8 k x 8 rows
// item per lane: the first half of the block takes A items, the second half B items.  Which
// operand a wave works on only changes its base pointer, leading dimension and LDS target, so
// the load / transpose / store sequence is one straight line for the whole block (no branch
// splits the k loop into several scheduling regions).
template <int BT, int NT, int AL, bool KTAIL>
struct LoadKS2 {
    static_assert(2 * BT == NT, "one item per lane");
    static constexpr int RC = BT / 8;
    uint32_t off, off1, ldb2;
    const half_t *origin;
    int64_t ld, K;
    int lds_extra;                 // halves from the A stage buffer to this lane's operand buffer
    int rc, kq;

    __device__ __forceinline__ void init(const half_t *Ao, int64_t lda, int64_t rows_a,
                                         const half_t *Bo, int64_t ldb, int64_t rows_b, int64_t K_)
    {
        const bool is_b = threadIdx.x >= BT;
        const int c = threadIdx.x - (is_b ? BT : 0);
        const int64_t rows_left = is_b ? rows_b : rows_a;
        origin = is_b ? Bo : Ao;
        ld = is_b ? ldb : lda;
        lds_extra = is_b ? 2 * BT * BK : 0;
        K = K_;
        ldb2 = (uint32_t)(ld * 2);
        rc = c % RC;
        kq = c / RC;
        int r0 = rc * 8, r1 = rc * 8 + 4;
        if (AL == 8) {
            if (r0 > rows_left - 8) r0 = (int)rows_left - 8;
        } else {
            if (r0 > rows_left - 4) r0 = (int)rows_left - 4;
            if (r1 > rows_left - 4) r1 = (int)rows_left - 4;
        }
        off = (uint32_t)(((int64_t)kq * 8 * ld + r0) * 2);
        off1 = (uint32_t)(((int64_t)kq * 8 * ld + r1) * 2);
    }
    __device__ __forceinline__ void load(uint4 *st, const half_t *, int64_t k0) const
    {
        const half_t *base = origin + k0 * ld;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            if (!KTAIL || k0 + BK <= K) {
                st[kk] = ld8<AL>(base, off + kk * ldb2, off1 + kk * ldb2);
            } else {
                const int left = (int)(K - k0) - (kq * 8 + kk);
                const uint32_t back = left > 0 ? 0 : (uint32_t)(1 - left) * ldb2;
                uint4 v = ld8<AL>(base, off + kk * ldb2 - back, off1 + kk * ldb2 - back);
                if (left <= 0) v = make_uint4(0, 0, 0, 0);
                st[kk] = v;
            }
        }
    }
    // lds = the A buffer of the stage being filled
    __device__ __forceinline__ void store(const uint4 *st, half_t *lds) const
    {
        const uint32_t *w = reinterpret_cast<const uint32_t *>(st);
        half_t *dst = lds + lds_extra;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
            uint4 o;
            o.x = __builtin_amdgcn_perm(w[1 * 4 + (j >> 1)], w[0 * 4 + (j >> 1)], sel);
            o.y = __builtin_amdgcn_perm(w[3 * 4 + (j >> 1)], w[2 * 4 + (j >> 1)], sel);
            o.z = __builtin_amdgcn_perm(w[5 * 4 + (j >> 1)], w[4 * 4 + (j >> 1)], sel);
            o.w = __builtin_amdgcn_perm(w[7 * 4 + (j >> 1)], w[6 * 4 + (j >> 1)], sel);
            *reinterpret_cast<uint4 *>(dst + lds_off(rc * 8 + j, kq)) = o;
        }
    }
    static constexpr int NREG = 8;
    static constexpr int NDMA = 0;
    __device__ __forceinline__ void dma(uint32_t, const half_t *, int64_t) const {}
};

// ---- one k-strided operand, every lane of the block taking part: an item is KPI k x 8 rows
// (KPI = 4 or 2, a half or a quarter of LoadKS's), so that the ROWS / 8 x 64 / KPI items spread
// over exactly NT lanes with no idle wavefronts and no branch in the k loop.  Each of the 8
// tile rows of an item gets KPI k values (2 KPI bytes of its 16-byte k chunk).
template <int ROWS, int NT, int AL, bool KTAIL>
struct LoadKSH {
    static constexpr int RC = ROWS / 8;
    static constexpr int KPI = BK * RC / NT;
    static_assert(KPI == 4 || KPI == 2, "a half or a quarter item per lane");
    uint32_t off, off1, ldb2;
    int64_t ld, K;
    int rc, kq;                    // row chunk; group of KPI k rows

    __device__ __forceinline__ void init(int64_t ld_, int64_t rows_left, int64_t K_)
    {
        ld = ld_;
        K = K_;
        ldb2 = (uint32_t)(ld_ * 2);
        rc = threadIdx.x % RC;
        kq = threadIdx.x / RC;
        int r0 = rc * 8, r1 = rc * 8 + 4;
        if (AL == 8) {
            if (r0 > rows_left - 8) r0 = (int)rows_left - 8;
        } else {
            if (r0 > rows_left - 4) r0 = (int)rows_left - 4;
            if (r1 > rows_left - 4) r1 = (int)rows_left - 4;
        }
        off = (uint32_t)(((int64_t)kq * KPI * ld + r0) * 2);
        off1 = (uint32_t)(((int64_t)kq * KPI * ld + r1) * 2);
    }
    __device__ __forceinline__ void load(uint4 *st, const half_t *origin, int64_t k0) const
    {
        const half_t *base = origin + k0 * ld;
#pragma unroll
        for (int kk = 0; kk < KPI; kk++) {
            if (!KTAIL || k0 + BK <= K) {
                st[kk] = ld8<AL>(base, off + kk * ldb2, off1 + kk * ldb2);
            } else {
                const int left = (int)(K - k0) - (kq * KPI + kk);
                const uint32_t back = left > 0 ? 0 : (uint32_t)(1 - left) * ldb2;
                uint4 v = ld8<AL>(base, off + kk * ldb2 - back, off1 + kk * ldb2 - back);
                if (left <= 0) v = make_uint4(0, 0, 0, 0);
                st[kk] = v;
            }
        }
    }
    __device__ __forceinline__ void store(const uint4 *st, half_t *lds) const
    {
        const uint32_t *w = reinterpret_cast<const uint32_t *>(st);       // [kk][4 words]
        const int k = kq * KPI;                                           // first k of the item
        half_t *dst = lds + (k & 7);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
            const uint32_t lo = __builtin_amdgcn_perm(w[1 * 4 + (j >> 1)], w[0 * 4 + (j >> 1)], sel);
            if (KPI == 4) {
                uint2 o;
                o.x = lo;
                o.y = __builtin_amdgcn_perm(w[(KPI - 1) * 4 + (j >> 1)], w[(KPI - 2) * 4 + (j >> 1)], sel);
                *reinterpret_cast<uint2 *>(dst + lds_off(rc * 8 + j, k >> 3)) = o;
            } else {
                *reinterpret_cast<uint32_t *>(dst + lds_off(rc * 8 + j, k >> 3)) = lo;
            }
        }
    }
    static constexpr int NREG = KPI;
    static constexpr int NDMA = 0;
    __device__ __forceinline__ void dma(uint32_t, const half_t *, int64_t) const {}
};

// stands in for the B loader when LoadKS2 serves both operands
struct LoadNone {
    __device__ __forceinline__ void init(int64_t, int64_t, int64_t) {}
    __device__ __forceinline__ void load(uint4 *, const half_t *, int64_t) const {}
    __device__ __forceinline__ void store(const uint4 *, half_t *) const {}
    __device__ __forceinline__ void dma(uint32_t, const half_t *, int64_t) const {}
    static constexpr int NREG = 1;
    static constexpr int NDMA = 0;
};

template <bool STRIDED, int ROWS, int NT, int T0, int AL, bool KTAIL> struct Loader;
template <int ROWS, int NT, int T0, int AL, bool KTAIL>
struct Loader<false, ROWS, NT, T0, AL, KTAIL> : LoadKC<ROWS, NT, AL, KTAIL> {};
template <int ROWS, int NT, int T0, int AL, bool KTAIL>
struct Loader<true, ROWS, NT, T0, AL, KTAIL> : LoadKS<ROWS, NT, T0, AL, KTAIL> {};

// scheduling pattern of one k step: NM MFMAs with NR LDS reads spread evenly between them
template <int NM, int NR, int R>
struct SchedStep {
    static __device__ __forceinline__ void run()
    {
        __builtin_amdgcn_sched_group_barrier(0x008, (NM * (R + 1)) / NR - (NM * R) / NR, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        SchedStep<NM, NR, R + 1>::run();
    }
};
template <int NM, int NR>
struct SchedStep<NM, NR, NR> {
    static __device__ __forceinline__ void run() {}
};

// waves per SIMD the register allocation must leave room for: two 128 x 128 blocks (or one
// 8-wave block) per CU, one 4-wave 256 x 256 block
constexpr int min_waves(int bm, int bn, int waves, int nbuf)
{
    const int blocks = 160 * 1024 / (nbuf * (bm + bn) * BK * 2);  // workgroups per CU by LDS
    const int w = blocks * waves / 4;
    return w >= 2 ? 2 : 1;
}

// wait until at most n vector memory loads are outstanding (s_waitcnt vmcnt only)
template <int N>
__device__ __forceinline__ void wait_vmem()
{
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

// 4 consecutive k of this lane's row out of a [k][row] tile (ds_read_b64_tr_b16)
__device__ __forceinline__ uint2 lds_read_tr(const unsigned char *q)
{
    typedef __attribute__((address_space(3))) fp16x4_t *lds_ptr;
    const fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_ptr)q);
    uint2 r;
    __builtin_memcpy(&r, &v, 8);
    return r;
}

// DMA = true: both operands are fetched straight into LDS, NBUF - 1 tiles ahead, no register
// stages (STAGES is 1); DMA = false: through registers, two LDS buffers.
template <bool TA, bool TB, int BM, int BN, int WM, int WN, int AL, bool KTAIL, int STAGES, int NBUF, bool DMA>
__global__ void __launch_bounds__(WM * WN * 64, min_waves(BM, BN, WM * WN, NBUF))
gemm_mfma_kernel(GemmArgs p)
{
    // the whole argument block in scalar registers before anything else: read field by field where the control
    // flow first wants it, it costs five dependent round trips to memory before the first operand load
    asm volatile("" ::"s"(p.M), "s"(p.N), "s"(p.K), "s"(p.alpha), "s"(p.beta), "s"(p.A), "s"(p.lda), "s"(p.sa), "s"(p.B),
                 "s"(p.ldb), "s"(p.sb), "s"(p.C), "s"(p.ldc), "s"(p.sc), "s"(p.tiles_m), "s"(p.tiles_n), "s"(p.tri),
                 "s"(p.gm), "s"(p.xcd), "s"(p.pair), "s"(p.win), "s"(p.ztab));
    static_assert(DMA ? (STAGES == 1 && AL == 8 && !KTAIL) : NBUF == 2,
                  "direct loads: 16-byte aligned operands, whole k tiles");
    constexpr bool TR_A = DMA && TA, TR_B = DMA && !TB;           // fragments by transposing reads
    static_assert((WM % 2 == 0 || BM / WM == 32) && (WN % 2 == 0 || BN / WN == 32),
                  "tiles of a wave lie 32 WM rows apart: a multiple of 64 keeps their swizzle equal");
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;          // 32x32 tiles per wave
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    half_t *As = reinterpret_cast<half_t *>(smem_raw);            // [NBUF][BM*BK]
    half_t *Bs = As + NBUF * BM * BK;                             // [NBUF][BN*BK]

    // XCD-aware numbering over the flattened (block of the batch, tile) sequence: dispatch
    // order i lands on XCD i % 8; give each XCD a contiguous band.  With a batch that is a
    // multiple of 8 an XCD then owns whole blocks of the batch, which also balances the
    // triangular modes (their work per tile row grows or shrinks along M).
    const int nb = gridDim.x;
    int bid = blockIdx.x;
    if (p.xcd) {
        const int per = nb >> 3, rem = nb & 7;
        const int xcd = bid & 7, idx = bid >> 3;
        bid = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    // pair mode (triangular operands): a workgroup takes tile row r and then tile row
    // tiles_m - 1 - r, whose k ranges add up to the same length for every r
    const int rows_m = p.pair ? p.tiles_m / 2 : p.tiles_m;
    const int tiles = rows_m * p.tiles_n;
    int64_t bz;
    if (p.ztab) {
        // a pointer-table batch is a handful of whole products that share an operand (the projections of one
        // input, the weight gradients against one input): product fastest, so that the workgroups resident
        // together on an XCD work on the same tile of every product and fetch the shared panel once
        const int nz = nb / tiles;
        bz = bid % nz;
        bid /= nz;
    } else {
        bz = bid / tiles;
        bid -= (int)bz * tiles;
    }
    // within a block of the batch, tiles are walked in groups of 8 tile rows x all tile
    // columns, row fastest: the ~64 blocks resident on an XCD then form an 8 x 8 patch of C
    // and each operand panel fetched into its L2 is shared by 8 blocks
    const int GM = p.gm;
    const int per_group = GM * p.tiles_n;
    const int first_m = (bid / per_group) * GM;
    const int gsz = min(GM, rows_m - first_m);
    const int tm_base = first_m + (bid % per_group) % gsz;
    const int tn = (bid % per_group) / gsz;
    for (int rep = 0; rep <= p.pair; rep++) {
    int tm = rep ? p.tiles_m - 1 - tm_base : tm_base;
    if (p.tri == 2 && !p.pair) tm = p.tiles_m - 1 - tm;           // longest k ranges first
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    int nk = (int)((p.K + BK - 1) / BK), kt0 = 0;
    if (p.tri == 1 && n0 > m0 + BM - 1) return;                   // uniform for the block
    if (p.tri == 2) nk = min(nk, (int)((m0 + BM + BK - 1) / BK));
    if (p.tri == 3) kt0 = (int)(m0 / BK);

    const half_t *A = p.A + (p.ztab ? p.za[bz] : bz * p.sa);
    // column window (p.win): the [k][n] operand B and C of block bz start 8 bytes off a 16-byte
    // boundary when bz * sb is an odd multiple of 4 (head_dim 100).  Both are then addressed
    // from the boundary before: column `shift` of this view is the block's column 0, columns
    // below it and from nw on hold the neighbouring blocks' data, are multiplied like the rest
    // and never stored.
    const int shift = p.win ? (int)((bz * p.sb) & 7) : 0;
    const int64_t nw = p.N + shift;                               // end of the window
    const half_t *B = p.B + (p.ztab ? p.zb[bz] : bz * p.sb) - shift;
    half_t *C = p.C + (p.ztab ? p.zc[bz] : bz * p.sc) - shift;
    // tile origins: &op[row0][0] for a k-contiguous operand, &op[0][row0] for a strided one
    const half_t *Ao = TA ? A + m0 : A + m0 * p.lda;
    const half_t *Bo = TB ? B + n0 * p.ldb : B + n0;

    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int wm = wid % WM, wn = wid / WM;
    const int l32 = lane & 31, lh = lane >> 5;

    // when both operands are strided they use disjoint halves of the block
    constexpr bool UNI = !DMA && TA && !TB && BM == BN && BM + BN == NT;  // one combined strided loader
    // strided operands whose 8-row x 64-k items divide into 4- or 2-k pieces over all lanes
    // (128 rows on 256 lanes, 256 or 128 rows on 512 lanes): branch-free on every lane
    constexpr bool FITS_A = BM * 2 == NT || BM * 4 == NT, FITS_B = BN * 2 == NT || BN * 4 == NT;
    constexpr bool HALF_A = TA && !UNI && FITS_A && (TB || FITS_B);
    constexpr bool HALF_B = !TB && !UNI && FITS_B && (!TA || FITS_A);
    typedef typename std::conditional<
        UNI, LoadKS2<BM, NT, AL, KTAIL>,
        typename std::conditional<HALF_A, LoadKSH<BM, NT, AL, KTAIL>,
                                  Loader<TA, BM, NT, 0, AL, KTAIL>>::type>::type LA_REG;
    typedef typename std::conditional<
        UNI, LoadNone,
        typename std::conditional<HALF_B, LoadKSH<BN, NT, AL, KTAIL>,
                                  Loader<!TB, BN, NT, (TA && !TB) ? NT / 2 : 0, AL, KTAIL>>::type>::type LB_REG;
    typedef typename std::conditional<
        DMA, typename std::conditional<TA, LoadKSD<BM, NT>, LoadKCD<BM, NT>>::type, LA_REG>::type LA;
    typedef typename std::conditional<
        DMA, typename std::conditional<TB, LoadKCD<BN, NT>, LoadKSD<BN, NT>>::type, LB_REG>::type LB;
    LA la;
    LB lb;
    if constexpr (UNI) {
        la.init(Ao, p.lda, p.M - m0, Bo, p.ldb, nw - n0, p.K);
    } else {
        la.init(p.lda, p.M - m0, p.K);
        lb.init(p.ldb, (p.win ? (nw + 7) / 8 * 8 : nw) - n0, p.K);
    }
    uint4 ra[STAGES][LA::NREG], rb[STAGES][LB::NREG];
    // direct loads: the first NBUF tiles are requested here, before the accumulators are cleared and the
    // fragment addresses worked out (some thousand cycles of set-up that need not stand in front of them)
    if constexpr (DMA) {
#pragma unroll
        for (int u = 0; u < NBUF; u++)
            if (kt0 + u < nk) {
                la.dma((uint32_t)(uintptr_t)(As + u * BM * BK), Ao, (int64_t)(kt0 + u) * BK);
                lb.dma((uint32_t)(uintptr_t)(Bs + u * BN * BK), Bo, (int64_t)(kt0 + u) * BK);
            }
        __builtin_amdgcn_sched_barrier(0);
    }

    // direct path: 16 x 16 results of v_mfma_f32_16x16x32_f16, [A fragment][B fragment]; lane l holds row
    // l % 16 of the fragment pair's block and columns 4 (l / 16) .. + 3
    float4_t c16[DMA ? 2 * TM : 1][DMA ? 2 * TN : 1];
    const int l16 = lane & 15, kg = lane >> 4;
    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // per-lane row offsets and swizzles of the operand fragments.  The 32 x 32 tiles of a wave
    // lie 32 WM rows (32 WN columns) apart, a multiple of 64 rows, so every tile of a lane has
    // the same swizzle and differs from the first only by a constant LDS offset.
    const int ar0 = wm * 32 + l32, br0 = wn * 32 + l32;
    const int asw = swz(ar0), bsw = swz(br0);
    constexpr int ASTEP = (TM > 1 ? 32 * WM : 0) * BK, BSTEP = (TN > 1 ? 32 * WN : 0) * BK;
    // [k][row] tiles: byte offset of the lane's first transposing read (k step 0, first 32 x 32
    // tile).  In its 16-lane group the lane addresses k row a4 (of 4), rows 4 b4 .. 4 b4 + 3
    // (of 16); k steps, the second half of a fragment and further tiles add constants.
    const int a4 = (lane >> 2) & 3, b4 = lane & 3, n16 = (lane >> 4) & 1;
    auto tr_base = [&](int w32, int pitch) __attribute__((always_inline)) {
        const int chunk = (w32 + 16 * n16) / 8 + (b4 >> 1);
        return (8 * lh + a4) * pitch + ((chunk ^ (2 * a4)) << 4) + ((b4 & 1) << 3);
    };
    const int atr = tr_base(wm * 32, BM * 2), btr = tr_base(wn * 32, BN * 2);

    // MFMAs of k step ks run while the operand fragments of step ks + 1 are in flight from
    // LDS (two fragment sets): the wait before a step's MFMAs leaves the next step's reads
    // outstanding
    auto compute = [&](int cur) __attribute__((always_inline)) {
        const half_t *as = As + cur * BM * BK + ar0 * BK;
        const half_t *bs = Bs + cur * BN * BK + br0 * BK;
        // fragment double-buffering costs (TM + TN) * 4 registers: used where it fits without
        // spilling (16-byte aligned operands, small patches)
        constexpr bool PIPE = AL == 8 || TM * TN <= 2;
        half8_t af[PIPE ? 2 : 1][TM], bf[PIPE ? 2 : 1][TN];
        auto frag_tr = [&](const unsigned char *q, int pitch) __attribute__((always_inline)) {
            const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * pitch);
            const uint4 v = make_uint4(lo.x, lo.y, hi.x, hi.y);
            half8_t f;
            __builtin_memcpy(&f, &v, 16);
            return f;
        };
        auto frags = [&](int set, int ks) __attribute__((always_inline)) {
            const int q = ks * 2 + lh;
#pragma unroll
            for (int i = 0; i < TM; i++) {
                if (TR_A)
                    af[set][i] = frag_tr(reinterpret_cast<const unsigned char *>(As + cur * BM * BK) + atr +
                                             ks * 16 * (BM * 2) + i * (32 * WM * 2),
                                         BM * 2);
                else
                    af[set][i] = *reinterpret_cast<const half8_t *>(as + i * ASTEP + ((q ^ asw) << 3));
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (TR_B)
                    bf[set][j] = frag_tr(reinterpret_cast<const unsigned char *>(Bs + cur * BN * BK) + btr +
                                             ks * 16 * (BN * 2) + j * (32 * WN * 2),
                                         BN * 2);
                else
                    bf[set][j] = *reinterpret_cast<const half8_t *>(bs + j * BSTEP + ((q ^ bsw) << 3));
            }
        };
        if (PIPE) frags(0, 0);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            const int cur_set = PIPE ? (ks & 1) : 0;
            if (!PIPE) frags(0, ks);
            else if (ks + 1 < BK / 16) frags((ks + 1) & 1, ks + 1);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur_set][j], af[cur_set][i],
                                                                       acc[i][j], 0, 0, 0);
        }
        if (PIPE) {
            // pin that order for the instruction scheduler (it would otherwise sink each read
            // to just before its use): the first fragment set, then per k step its MFMAs
            // with the next step's LDS reads spread between them
            constexpr int NM = TM * TN, NR = (TR_A ? 2 : 1) * TM + (TR_B ? 2 : 1) * TN;
            // with one register stage the global loads of the next tile (same scheduling region
            // when no operand is strided) must go first, so that their latency overlaps the
            // whole k tile; with two stages they are a tile ahead anyway and are left to the
            // scheduler (measured: pinning them first costs 5 %)
            if (STAGES == 1 && !DMA) __builtin_amdgcn_sched_group_barrier(0x020, LA::NREG + LB::NREG, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
#pragma unroll
            for (int ks = 0; ks + 1 < BK / 16; ks++) SchedStep<NM, NR, 0>::run();
            __builtin_amdgcn_sched_group_barrier(0x008, NM, 0);
        }
    };

    // Software pipeline over k tiles.  Through registers (STAGES register sets, two LDS
    // buffers): at the start of tile t, LDS[t & 1] holds tile t, register set
    // (t + j - kt0) % STAGES holds tile t + j for j = 1 .. STAGES - 1 and set (t - kt0) % STAGES
    // is free; a step loads tile t + STAGES into the free set, runs the MFMAs of tile t, moves
    // tile t + 1 from its set to the other LDS buffer and ends in the one barrier of the k tile.
    // The main loop has no branch (all its loads are inside K); the last tiles are peeled
    // into steps that test what still exists.  (Direct loads: the rotated pipeline further down.)
    constexpr int LOOK = STAGES;                                  // tiles between load and use
    auto next_buf = [](int b) __attribute__((always_inline)) { return b + 1 == NBUF ? 0 : b + 1; };
    auto lds_addr = [](const half_t *q) __attribute__((always_inline)) {
        return (uint32_t)(uintptr_t)q;                            // LDS byte address of a shared pointer
    };
    auto step = [&](auto set_c, auto main_c, int t, int cbv) __attribute__((always_inline)) {
        constexpr int U = decltype(set_c)::value, UN = (U + 1) % STAGES;
        constexpr bool MAIN = decltype(main_c)::value;
        (void)cbv;
        const int cb = t & 1, nb1 = next_buf(cb);
        if (MAIN || t + LOOK < nk) {
            la.load(ra[U], Ao, (int64_t)(t + LOOK) * BK);
            lb.load(rb[U], Bo, (int64_t)(t + LOOK) * BK);
        }
        compute(cb);
        if (MAIN || t + 1 < nk) {
            la.store(ra[UN], As + nb1 * BM * BK);
            lb.store(rb[UN], Bs + nb1 * BN * BK);
        }
        __syncthreads();
    };
    if constexpr (DMA) {
        // Direct loads: v_mfma_f32_16x16x32_f16 and a rotated pipeline.
        //
        // The 16 x 16 x 32 product: under a sustained load with real operands the device is limited by
        // power, not by cycles, and per flop this instruction costs less of it than the 32 x 32 x 16 one (a
        // quarter of the accumulator registers read and written per flop): measured on random operands,
        // same fragment traffic, 1570 .. 1600 against 1435 TFLOP/s sustained.  A wave's 32-row blocks are
        // the same as in the register path, each cut into two 16-row fragments; a k tile of 64 is two k steps
        // of 32, each k step two halves (the first / second TM of the wave's 2 TM A fragments against all
        // 2 TN B fragments).  Lane l supplies, for row l % 16 of a fragment, the 8 k values of group l / 16,
        // and holds row l % 16, columns 4 (l / 16) .. + 3 of a 16 x 16 result.
        //
        // The pipeline: while the MFMAs of one half run, the A fragments of the next half (and, in a second
        // half, the B fragments of the next k step) are read.  The one barrier of a k tile sits before its
        // LAST half: by then a wave has every fragment of the tile in registers, so behind the barrier (a) the
        // tile's own buffer is free and takes the loads of the tile NBUF tiles further on, and (b) the next
        // tile, complete behind the same barrier, gives its first fragments while the MFMAs of this tile's
        // last half run.  The fragment ring never drains and nothing but MFMAs stands right behind the
        // barrier, where all waves of the workgroup are in step: loads and reads are placed between them.
        constexpr int ND = LA::NDMA + LB::NDMA;
        static_assert(BK == 64 && NBUF >= 2, "two k steps of 32 per tile");
        constexpr int NA = 2 * TM, NB = 2 * TN;                   // 16-row fragments of a wave per k step
        constexpr int NMH = TM * NB;                              // MFMAs of a half
        constexpr int RA = (TR_A ? 2 : 1) * TM, RB = (TR_B ? 2 : 1) * NB;   // LDS reads: A fragments of a half, all B
#pragma unroll
        for (int a = 0; a < NA; a++)
#pragma unroll
            for (int b = 0; b < NB; b++) c16[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
        half8_t fa[2][TM], fb[2][NB];                             // A fragments of a half, B fragments of a k step
        // [row][k] tiles: halves offset of the lane's row in a block's upper / lower 16 rows, and its swizzle
        const int ar[2] = {wm * 32 + l16, wm * 32 + 16 + l16}, br[2] = {wn * 32 + l16, wn * 32 + 16 + l16};
        const int asw2[2] = {swz16(ar[0]), swz16(ar[1])}, bsw2[2] = {swz16(br[0]), swz16(br[1])};
        // [k][row] tiles: byte offset of the lane's first transposing read; its 16-lane group (= k group)
        // fetches k rows 8 kg + a4 of rows 4 b4 .. 4 b4 + 3 of the 16
        auto tr16 = [&](int w16, int pitch) __attribute__((always_inline)) {
            const int chunk = w16 / 8 + (b4 >> 1);
            return (8 * kg + a4) * pitch + ((chunk ^ (2 * a4)) << 4) + ((b4 & 1) << 3);
        };
        const int atr2[2] = {tr16(wm * 32, BM * 2), tr16(wm * 32 + 16, BM * 2)};
        const int btr2[2] = {tr16(wn * 32, BN * 2), tr16(wn * 32 + 16, BN * 2)};
        auto frag_tr = [&](const unsigned char *q, int pitch) __attribute__((always_inline)) {
            const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * pitch);
            const uint4 v = make_uint4(lo.x, lo.y, hi.x, hi.y);
            half8_t f;
            __builtin_memcpy(&f, &v, 16);
            return f;
        };
        // A fragment a (0 .. NA - 1) / B fragment b of k step ks (0, 1) of the tile in buffer `buf`
        auto read_a = [&](int buf, int ks, int a) __attribute__((always_inline)) {
            const int blk = a >> 1, sub = a & 1;
            if (TR_A)
                return frag_tr(reinterpret_cast<const unsigned char *>(As + buf * BM * BK) + atr2[sub] +
                                   ks * 32 * (BM * 2) + blk * (32 * WM * 2),
                               BM * 2);
            return *reinterpret_cast<const half8_t *>(As + buf * BM * BK + ar[sub] * BK + blk * ASTEP +
                                                      (((ks * 4 + kg) ^ asw2[sub]) << 3));
        };
        auto read_b = [&](int buf, int ks, int b) __attribute__((always_inline)) {
            const int blk = b >> 1, sub = b & 1;
            if (TR_B)
                return frag_tr(reinterpret_cast<const unsigned char *>(Bs + buf * BN * BK) + btr2[sub] +
                                   ks * 32 * (BN * 2) + blk * (32 * WN * 2),
                               BN * 2);
            return *reinterpret_cast<const half8_t *>(Bs + buf * BN * BK + br[sub] * BK + blk * BSTEP +
                                                      (((ks * 4 + kg) ^ bsw2[sub]) << 3));
        };
        // the reads a half issues for what follows it, in the order the MFMAs there first need them (an A
        // fragment outer, the B fragments inner): A 0, every B, A 1 ..  `nxt` = (buffer, k step, half) of what
        // follows; unit u of NU
        auto next_read = [&](int u, int nbuf, int nks, int nh) __attribute__((always_inline)) {
            if (nh == 1) {                                        // second half of the same k step: its A fragments
                fa[1][u] = read_a(nbuf, nks, TM + u);
            } else if (u == 0) {
                fa[0][0] = read_a(nbuf, nks, 0);
            } else if (u <= NB) {
                fb[nks][u - 1] = read_b(nbuf, nks, u - 1);
            } else {
                fa[0][u - NB] = read_a(nbuf, nks, u - NB);
            }
        };
        auto mfma1 = [&](int h, int ks, int m) __attribute__((always_inline)) {
            const int a = m / NB, b = m % NB;
            c16[h * TM + a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[ks][b], fa[h][a], c16[h * TM + a][b], 0, 0, 0);
        };
        // a half with the reads for the next one spread between its MFMAs by the scheduler's groups
        auto half_pinned = [&](int h, int ks, int buf, int nbuf, int nks, int nh) __attribute__((always_inline)) {
            const int nu = nh == 1 ? TM : TM + NB;
#pragma unroll
            for (int u = 0; u < TM + NB; u++)
                if (u < nu) next_read(u, nbuf, nks, nh);
#pragma unroll
            for (int m = 0; m < NMH; m++) mfma1(h, ks, m);
        };
        auto issue_all = [&](int tile, int buf) __attribute__((always_inline)) {
            la.dma(lds_addr(As + buf * BM * BK), Ao, (int64_t)tile * BK);
            lb.dma(lds_addr(Bs + buf * BN * BK), Bo, (int64_t)tile * BK);
        };
        // the first three halves of the tile in buffer cb (fa[0], fb[0] hold the first half's fragments)
        auto first_halves = [&](int cb) __attribute__((always_inline)) {
            half_pinned(0, 0, cb, cb, 0, 1);
            SchedStep<NMH, RA, 0>::run();
            half_pinned(1, 0, cb, cb, 1, 0);
            SchedStep<NMH, RA + RB, 0>::run();
            half_pinned(0, 1, cb, cb, 1, 1);
            SchedStep<NMH, RA, 0>::run();
            __builtin_amdgcn_sched_barrier(0);
        };
        if (kt0 + NBUF <= nk) wait_vmem<(NBUF - 1) * ND>();       // the first tile; the others stay in flight
        else wait_vmem<0>();
        __syncthreads();
        int t = kt0, cb = 0;
        if constexpr (TM * TN == 1) {
        // One 32 x 32 block per wave: a half is two MFMAs (32 cycles), far less than an LDS read takes, so
        // reads issued one half ahead leave the wave waiting in every half.  Here the fragments of a whole
        // k tile (two register sets) are read while the eight MFMAs of the tile before run: behind the
        // barrier of tile t (tile t + 1 has landed; every wave holds tile t in registers, the barrier's own
        // wait for LDS sees to that) come the reads of tile t + 1, the loads of tile t + NBUF into the
        // buffer of tile t, and then the MFMAs of tile t.
        half8_t ga[2][2][NA], gb[2][2][NB];
        auto read_tile = [&](auto set_c, int buf) __attribute__((always_inline)) {
            constexpr int S = decltype(set_c)::value;
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
#pragma unroll
                for (int a = 0; a < NA; a++) ga[S][ks][a] = read_a(buf, ks, a);
#pragma unroll
                for (int b = 0; b < NB; b++) gb[S][ks][b] = read_b(buf, ks, b);
            }
        };
        auto body = [&](auto set_c, auto main_c) __attribute__((always_inline)) {
            constexpr int S = decltype(set_c)::value;
            constexpr bool MAIN = decltype(main_c)::value;
            const int nb = next_buf(cb);
            if (MAIN || t + 1 < nk) {
                if (MAIN) wait_vmem<(NBUF - 2) * ND>();
                else wait_vmem<0>();
                __syncthreads();
                read_tile(std::integral_constant<int, S ^ 1>{}, nb);
                __builtin_amdgcn_sched_barrier(0);
                if (MAIN || t + NBUF < nk) issue_all(t + NBUF, cb);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int a = 0; a < NA; a++)
#pragma unroll
                    for (int b = 0; b < NB; b++)
                        c16[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(gb[S][ks][b], ga[S][ks][a], c16[a][b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            cb = nb;
            t++;
        };
        read_tile(std::integral_constant<int, 0>{}, 0);
        while (t + NBUF + 1 < nk) {                               // both steps load inside K
            body(std::integral_constant<int, 0>{}, std::true_type{});
            body(std::integral_constant<int, 1>{}, std::true_type{});
        }
        while (t < nk) {
            body(std::integral_constant<int, 0>{}, std::false_type{});
            if (t < nk) body(std::integral_constant<int, 1>{}, std::false_type{});
        }
        __syncthreads();
        } else {
#pragma unroll
        for (int u = 0; u < TM + NB; u++) next_read(u, 0, 0, 0);
        for (; t + NBUF < nk; t++) {                              // every load of the body lies inside K
            first_halves(cb);
            const int nb = next_buf(cb);
            wait_vmem<(NBUF - 2) * ND>();                         // tile t + 1 has landed (this wave's part of it)
            __syncthreads();
            // last half: MFMA by MFMA, with the loads of tile t + NBUF (into the buffer of this tile) and
            // the first fragments of tile t + 1 between them
            const half_t *abase = la.kbase(Ao, (int64_t)(t + NBUF) * BK), *bbase = lb.kbase(Bo, (int64_t)(t + NBUF) * BK);
            const uint32_t alds = lds_addr(As + cb * BM * BK), blds = lds_addr(Bs + cb * BN * BK);
            constexpr int NU = TM + NB;
#pragma unroll
            for (int m = 0; m < NMH; m++) {
                mfma1(1, 1, m);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int d = m * ND / NMH; d < (m + 1) * ND / NMH; d++) {
                    if (d < LA::NDMA) la.dma1(d, alds, abase);
                    else lb.dma1(d - LA::NDMA, blds, bbase);
                }
#pragma unroll
                for (int u = m * NU / NMH; u < (m + 1) * NU / NMH; u++) next_read(u, nb, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            cb = nb;
        }
        for (; t < nk; t++) {                                     // the last NBUF tiles: nothing left to load
            first_halves(cb);
            const int nb = next_buf(cb);
            if (t + 1 < nk) {
                wait_vmem<0>();
                __syncthreads();
#pragma unroll
                for (int u = 0; u < TM + NB; u++) next_read(u, nb, 0, 0);
            }
#pragma unroll
            for (int m = 0; m < NMH; m++) mfma1(1, 1, m);
            __builtin_amdgcn_sched_barrier(0);
            cb = nb;
        }
        __syncthreads();                                          // every wave is done with the operand buffers
        }
    } else {
        la.load(ra[0], Ao, (int64_t)kt0 * BK);
        lb.load(rb[0], Bo, (int64_t)kt0 * BK);
#pragma unroll
        for (int u = 1; u < STAGES; u++)
            if (kt0 + u < nk) {
                la.load(ra[u], Ao, (int64_t)(kt0 + u) * BK);
                lb.load(rb[u], Bo, (int64_t)(kt0 + u) * BK);
            }
        la.store(ra[0], As + (kt0 & 1) * BM * BK);
        lb.store(rb[0], Bs + (kt0 & 1) * BN * BK);
        __syncthreads();
        int kt = kt0, cb = 0;
        for (; kt + STAGES - 1 + LOOK < nk; kt += STAGES) {
            step(std::integral_constant<int, 0>{}, std::true_type{}, kt, cb);
            cb = next_buf(cb);
            if (STAGES > 1) {
                step(std::integral_constant<int, 1 % STAGES>{}, std::true_type{}, kt + 1, cb);
                cb = next_buf(cb);
            }
            if (STAGES > 2) {
                step(std::integral_constant<int, 2 % STAGES>{}, std::true_type{}, kt + 2, cb);
                cb = next_buf(cb);
            }
        }
        constexpr int TAIL = STAGES - 1 + LOOK;                   // tiles left at most
        static_assert(STAGES >= 1 && STAGES <= 3 && TAIL <= 5, "peeled tail below covers up to 5 tiles");
        if (TAIL > 0 && kt + 0 < nk) { step(std::integral_constant<int, 0 % STAGES>{}, std::false_type{}, kt + 0, cb); cb = next_buf(cb); }
        if (TAIL > 1 && kt + 1 < nk) { step(std::integral_constant<int, 1 % STAGES>{}, std::false_type{}, kt + 1, cb); cb = next_buf(cb); }
        if (TAIL > 2 && kt + 2 < nk) { step(std::integral_constant<int, 2 % STAGES>{}, std::false_type{}, kt + 2, cb); cb = next_buf(cb); }
        if (TAIL > 3 && kt + 3 < nk) { step(std::integral_constant<int, 3 % STAGES>{}, std::false_type{}, kt + 3, cb); cb = next_buf(cb); }
        if (TAIL > 4 && kt + 4 < nk) { step(std::integral_constant<int, 4 % STAGES>{}, std::false_type{}, kt + 4, cb); cb = next_buf(cb); }
    }

    // Epilogue through LDS (the operand buffers are free after the last barrier): a lane
    // holds row m = .. + l32 and, per accumulator group q, the 4 consecutive columns
    // n = .. + 8 q + 4 lh + {0..3}, i.e. 8 bytes in each of 32 different rows of C; staged as
    // Cs[row][BN] (16-byte chunks swizzled by the row) the tile leaves as whole contiguous
    // rows, 16 bytes per lane.  With beta the old C tile is staged the same way first, so
    // alpha acc + beta C is still rounded to f16 exactly once.
    half_t *Cs = reinterpret_cast<half_t *>(smem_raw);
    constexpr int CPRC = BN / 8;                                  // 16-byte chunks per row
    constexpr int CSW = (CPRC & (CPRC - 1)) == 0 ? CPRC - 1 : 7;  // chunk swizzle mask
    static_assert(CPRC % (CSW + 1) == 0, "the chunk swizzle must stay inside the row");
    const bool has_beta = p.beta != 0.f;
    // (the lane's index as a value the compiler cannot trace back: the addresses of the batched paths below are
    // otherwise computed before the k loop, kept across it and spilled inside it)
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    // a tile wholly inside C, 16-byte aligned: all of a lane's pieces of the old tile requested before the first is
    // stored (the general loop below waits for every piece in turn: 9,000 cycles more per workgroup measured)
    // (tiles of up to 256 x 128: the larger ones have no registers for it and spill in their main loop with it)
    constexpr bool C_BATCH = BM * BN <= 256 * 128 && BM * CPRC % NT == 0;
    const bool c_inside = C_BATCH && AL == 8 && shift == 0 && m0 + BM <= p.M && n0 + BN <= nw;
    if (has_beta && c_inside) {
        constexpr int NC = C_BATCH ? BM * CPRC / NT : 1;
        uint4 old[NC];
#pragma unroll
        for (int i = 0; i < NC; i++) {
            const int c = tid + i * NT, row = c / CPRC, cc = c % CPRC;
            old[i] = *reinterpret_cast<const uint4 *>(C + (m0 + row) * p.ldc + n0 + cc * 8);
        }
#pragma unroll
        for (int i = 0; i < NC; i++) {
            const int c = tid + i * NT, row = c / CPRC, cc = c % CPRC;
            *reinterpret_cast<uint4 *>(Cs + row * BN + ((cc ^ (row & CSW)) << 3)) = old[i];
        }
        __syncthreads();
    } else if (has_beta) {
        for (int c = threadIdx.x; c < BM * CPRC; c += NT) {
            const int row = c / CPRC, cc = c % CPRC;
            const int64_t m = m0 + row, n = n0 + cc * 8;
            const bool lo = m < p.M && n >= shift && n < nw, hi = m < p.M && n + 4 >= shift && n + 4 < nw;
            const half_t *cp = C + m * p.ldc + n;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (AL == 8 && lo && hi) {
                v = *reinterpret_cast<const uint4 *>(cp);
            } else {
                if (lo) {
                    const uint2 t = *reinterpret_cast<const uint2 *>(cp);
                    v.x = t.x;
                    v.y = t.y;
                }
                if (hi) {
                    const uint2 t = *reinterpret_cast<const uint2 *>(cp + 4);
                    v.z = t.x;
                    v.w = t.y;
                }
            }
            *reinterpret_cast<uint4 *>(Cs + row * BN + ((cc ^ (row & CSW)) << 3)) = v;
        }
        __syncthreads();
    }
    if constexpr (DMA) {
#pragma unroll
        for (int a = 0; a < 2 * TM; a++) {
            const int row = (a >> 1) * (32 * WM) + wm * 32 + (a & 1) * 16 + l16;
#pragma unroll
            for (int b = 0; b < 2 * TN; b++) {
                const int col = (b >> 1) * (32 * WN) + wn * 32 + (b & 1) * 16 + kg * 4;
                half_t *sp = Cs + row * BN + ((((col >> 3) ^ (row & CSW)) << 3) | (col & 4));
                half4_t o;
                if (has_beta) {
                    const half4_t old = *reinterpret_cast<const half4_t *>(sp);
#pragma unroll
                    for (int r = 0; r < 4; r++) o[r] = f2h(p.alpha * c16[a][b][r] + p.beta * h2f(old[r]));
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++) o[r] = f2h(p.alpha * c16[a][b][r]);
                }
                *reinterpret_cast<half4_t *>(sp) = o;
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int row = i * (32 * WM) + wm * 32 + l32;
    #pragma unroll
            for (int j = 0; j < TN; j++) {
    #pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int col = j * (32 * WN) + wn * 32 + q * 8 + lh * 4;
                    half_t *sp = Cs + row * BN + ((((col >> 3) ^ (row & CSW)) << 3) | (col & 4));
                    half4_t o;
                    if (has_beta) {
                        const half4_t old = *reinterpret_cast<const half4_t *>(sp);
    #pragma unroll
                        for (int r = 0; r < 4; r++)
                            o[r] = f2h(p.alpha * acc[i][j][q * 4 + r] + p.beta * h2f(old[r]));
                    } else {
    #pragma unroll
                        for (int r = 0; r < 4; r++) o[r] = f2h(p.alpha * acc[i][j][q * 4 + r]);
                    }
                    *reinterpret_cast<half4_t *>(sp) = o;
                }
            }
        }
}
    __syncthreads();
    for (int c = threadIdx.x; c < BM * CPRC; c += NT) {
        const int row = c / CPRC, cc = c % CPRC;
        const int64_t m = m0 + row, n = n0 + cc * 8;
        if (m >= p.M) continue;
        const bool lo = n >= shift && n < nw, hi = n + 4 >= shift && n + 4 < nw;   // 4-column halves
        const uint4 v = *reinterpret_cast<const uint4 *>(Cs + row * BN + ((cc ^ (row & CSW)) << 3));
        half_t *cp = C + m * p.ldc + n;
        if (AL == 8 && lo && hi) {
            *reinterpret_cast<uint4 *>(cp) = v;
        } else {
            if (lo) *reinterpret_cast<uint2 *>(cp) = make_uint2(v.x, v.y);
            if (hi) *reinterpret_cast<uint2 *>(cp + 4) = make_uint2(v.z, v.w);
        }
    }
    __syncthreads();                          // the staging buffer is read out before the next tile's operands land
    }
}

template <bool TA, bool TB, int BM, int BN, int WM, int WN, int AL, bool KTAIL, int STAGES, int NBUF = 2, bool DMA = false>
int launch_cfg(GemmArgs p, int64_t nblk, hipStream_t st)
{
    p.tiles_m = (int)((p.M + BM - 1) / BM);
    p.tiles_n = (int)((p.N + (p.win ? 4 : 0) + BN - 1) / BN);
    const size_t smem = (size_t)NBUF * (BM + BN) * BK * sizeof(half_t);
    auto kern = gemm_mfma_kernel<TA, TB, BM, BN, WM, WN, AL, KTAIL, STAGES, NBUF, DMA>;
    static DeviceOnce attr_set;                   // one per instantiation
    if (!attr_set.fresh()) {
        CACTI_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)smem));
        attr_set.mark();
    }
    if (p.gm <= 0) {
        // tile rows per group of the walk.  An XCD works on a band of tiles / 8 consecutive tiles,
        // i.e. on gm tile rows x band / gm tile columns at a time, and fetches gm A panels and
        // band / gm B panels per k tile into its L2: the power of two with the fewest rows fetched.  (Run
        // time hardly reacts, the re-reads being served by the MALL; the L2-miss traffic does:
        // -25 % at 2048 x 3200 x 8640.)
        p.gm = 8;
        if (nblk == 1) {
            const double band = (double)p.tiles_m * p.tiles_n / 8.0;
            double best = 0;
            for (int g = 8; g >= 2; g /= 2) {             // ties: the larger group
                const double fetched = g * (double)BM + band / g * (double)BN;
                if (best == 0 || fetched < best) {
                    best = fetched;
                    p.gm = g;
                }
            }
        }
    }
    p.pair = (p.tri >= 2 && p.tiles_m % 2 == 0) ? 1 : 0;
    const int64_t nwg = (int64_t)(p.pair ? p.tiles_m / 2 : p.tiles_m) * p.tiles_n * nblk;
    CACTI_REQUIRE(nwg < (int64_t)1 << 31, CACTI_E_NOTIMPL, "gemm: %lld workgroups exceed the grid limit",
                  (long long)nwg);
    dim3 grid((unsigned)nwg), block(WM * WN * 64);
    hipLaunchKernelGGL(kern, grid, block, smem, st, p);
    return launch_status("gemm_mfma");
}

// tile: 0 = 128 x 128 on 4 waves, two register stages (every loader is branch-free on 256
// lanes); 1 = 256 x 128 on 8 waves, two register stages; 3 = 64 x 64 on 4 waves; 4 = 256 x 128,
// 5 = 256 x 256 (128 x 64 per wave), 6 = 256 x 192 (64 x 96 per wave) and 7 = 128 x 128 (64 x 32
// per wave) on 8 waves with both operands loaded straight into LDS; 8 = 64 x 64 on 4 waves the same way,
// five k tiles ahead
template <bool TA, bool TB>
int launch_tile(int tile, int align, const GemmArgs &p, int64_t nblk, hipStream_t st)
{
    const bool ktail = (p.K % BK) != 0;
    if (align < 8) {
        // 8-byte aligned operands (the attention blocks): 8 waves of 64 x 32 on the 128 x 128 tile;
        // with one workgroup per CU (32 heads x 8 tile-row pairs) two waves per SIMD hide each
        // other's LDS latency (-9..13 % against 4 waves of 64 x 64)
        return ktail ? launch_cfg<TA, TB, 128, 128, 2, 2, 4, true, 1>(p, nblk, st)
                     : launch_cfg<TA, TB, 128, 128, 2, 4, 4, false, 2>(p, nblk, st);
    }
    if (ktail) return launch_cfg<TA, TB, 128, 128, 2, 2, 8, true, 1>(p, nblk, st);
    switch (tile) {
        case 0: return launch_cfg<TA, TB, 128, 128, 2, 2, 8, false, 2>(p, nblk, st);
        case 3: return launch_cfg<TA, TB, 64, 64, 2, 2, 8, false, 2>(p, nblk, st);
        case 4: return launch_cfg<TA, TB, 256, 128, 4, 2, 8, false, 1, 3, true>(p, nblk, st);
        case 5: return launch_cfg<TA, TB, 256, 256, 2, 4, 8, false, 1, 2, true>(p, nblk, st);
        case 6: return launch_cfg<TA, TB, 256, 192, 4, 2, 8, false, 1, 2, true>(p, nblk, st);
        case 7: return launch_cfg<TA, TB, 128, 128, 2, 4, 8, false, 1, 3, true>(p, nblk, st);
        case 8: return launch_cfg<TA, TB, 64, 64, 2, 2, 8, false, 1, 6, true>(p, nblk, st);
        default: return launch_cfg<TA, TB, 256, 128, 4, 2, 8, false, 2>(p, nblk, st);
    }
}

int cu_count()
{
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

// How a large product with A not transposed (M = tokens) is cut into workgroups.  One workgroup
// per CU runs in rounds of `cus` tiles, and a last round that holds only a few tiles costs as
// much as a full one (N = 8640 at 2048 tokens: 544 tiles of 256 x 128 = 2 rounds + 32 tiles).
// The columns of the full rounds can instead go to one launch and the few remaining ones to a
// second launch of 64 x 64 tiles, which spreads them over every CU.  The plan compares
// 256 x 128 tiles with 256 x 256 tiles (measured 1.2 x the rate per tile area: 883 -> 1075
// TFLOP/s on 2048 x 8192 x 3200) by rounds x tile area / rate, the second launch costing 3/8 of
// a 256 x 128 round.  At 2048 tokens: N = 3200 -> 200 tiles of 256 x 128 (one round); N = 8640
// -> 256 tiles of 256 x 256 + 448 columns (135 -> 122 us); N = 32000 -> 1000 tiles of 256 x 256.
struct Plan {
    int tile;               // 4 or 5
    int64_t cols_main;      // columns of the first launch (N: a single launch)
};
Plan plan_tokens_product(int64_t M, int64_t N, bool may_split)
{
    const int64_t cus = cu_count();
    Plan best{4, N};
    int64_t best_cost = -1;
    const int tiles[2] = {4, 5};
    const int64_t widths[2] = {128, 256}, round_cost[2] = {32768, 54613};   // 256 bn / rate
    for (int c = 0; c < 2; c++) {
        const int64_t bn = widths[c], tiles_m = (M + 255) / 256, tiles_n = (N + bn - 1) / bn;
        const int64_t total = tiles_m * tiles_n, full = total / cus;
        const int64_t cols_main = full * cus / tiles_m, rest = tiles_m * (tiles_n - cols_main);
        int64_t cost, main_cols;
        if (may_split && full >= 1 && cols_main < tiles_n && rest * bn * 4 <= cus * 128) {
            cost = full * round_cost[c] + 12288;
            main_cols = cols_main * bn;
        } else {
            cost = (total + cus - 1) / cus * round_cost[c];
            main_cols = N;
        }
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = Plan{tiles[c], main_cols};
        }
    }
    return best;
}

template <bool TA, bool TB>
int launch_auto(int tile, int64_t cols_main, int align, const GemmArgs &p, int64_t nblk, hipStream_t st)
{
    if (cols_main > 0 && cols_main < p.N) {
        GemmArgs a = p, b = p;
        a.N = cols_main;
        b.N = p.N - a.N;
        b.B = p.B + (TB ? a.N * p.ldb : a.N);
        b.C = p.C + a.N;
        const int rc = launch_tile<TA, TB>(tile, align, a, nblk, st);
        // the remaining columns on 64 x 64 tiles loaded straight into LDS, six buffers: a tile this
        // small has 4 MFMAs per wave and k tile, so a k step costs the latency of its loads unless
        // they were issued several steps earlier (448 columns at K = 3200: register path with two
        // stages 23.7 us, three buffers 21.4, six 15.2 .. 16.5)
        return rc ? rc : launch_tile<TA, TB>(8, align, b, nblk, st);
    }
    return launch_tile<TA, TB>(tile, align, p, nblk, st);
}

}  // namespace

namespace cacti {

// tile: as launch_tile; -1 = pick by shape
int gemm_mfma_launch(int ta, int tb, const GemmArgs &p, int64_t nblk, int align, int tile,
                     hipStream_t st)
{
    GemmArgs q = p;
    q.gm = -1;                                    // rows of tiles per group: chosen per launch
    q.xcd = 1;                                    // consecutive tiles to the workgroups of one XCD
    int64_t cols_main = 0;                        // > 0: a second launch takes the columns from here on
    if (tile < 0) {
        {
            // measured on MI355X at the step's shapes (TFLOP/s on cold operands, register
            // path 128 x 128 or 256 x 128 -> direct loads).  A not transposed (forward and dgrad,
            // M = tokens): NT 661..821 -> 707..881, NN 702..787 -> 773..864 on 256 x 128, one
            // workgroup per CU; 256 x 256 where its rounds fit (plan_tokens_product).  Wgrad (both
            // operands strided, weight-sized outputs): 256 x 256, 558..715 -> 755..932.
            // Small and batched products stay on 128 x 128 through registers.
            tile = 0;
            // the attention products on per-head slabs: 128 x 128, 8 waves of 64 x 32, three
            // LDS buffers (-5 us per launch against the register path with 8 waves)
            if (p.win) tile = 7;
            // (a pointer-table batch is a handful of whole products: planned like a single one)
            if ((nblk == 1 || p.ztab) && p.M >= 1024 && p.N >= 1024) {
                if (!ta) {
                    const bool direct_ok = align >= 8 && p.K % BK == 0;     // else launch_tile ignores the tile
                    const Plan plan = plan_tokens_product(p.M, p.N, direct_ok && p.tri == 0);
                    tile = plan.tile;
                    cols_main = plan.cols_main;
                } else if (p.M >= 2048 && p.N >= 2048) {
                    // 256 x 192 where its tile count fills the CUs markedly better (3200 x 3200:
                    // 221 tiles in one round against 169; +5 %)
                    const int64_t cus = cu_count();
                    const int64_t tiles256 = ((p.M + 255) / 256) * ((p.N + 255) / 256);
                    const int64_t tiles192 = ((p.M + 255) / 256) * ((p.N + 191) / 192);
                    auto fill = [&](int64_t tiles) { return (double)tiles / (double)((tiles + cus - 1) / cus * cus); };
                    tile = fill(tiles192) > 1.2 * fill(tiles256) ? 6 : 5;
                }
            }
        }
    }
    if (!ta && !tb) return launch_auto<false, false>(tile, cols_main, align, q, nblk, st);
    if (!ta && tb) return launch_auto<false, true>(tile, cols_main, align, q, nblk, st);
    if (ta && !tb) return launch_auto<true, false>(tile, cols_main, align, q, nblk, st);
    return launch_auto<true, true>(tile, cols_main, align, q, nblk, st);
}

}  // namespace cacti
