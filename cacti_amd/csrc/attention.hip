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
// LDS tiles are [rows][128 halves] (256 bytes per row = one pass over all 64 banks, head dim
// zero-padded); 16-byte chunk c of row r sits at chunk c ^ g(r), g(r) = 2 (r & 3) | ((r >> 2) & 1) |
// 8 (((r >> 3) ^ r) & 1): a permutation of r mod 16, so the 16-byte operand reads of 16 consecutive rows
// cover all 16 bank groups, and the 8 rows of a transposing read (64 bytes each out of one aligned
// 64-byte quarter of the row) fall two to a quarter, which is all 64 banks twice -- the least 512 bytes
// can take.  (With bit 3 of g taken from bit 3 of r alone those 8 rows shared two quarters: a quarter of
// all LDS cycles were bank conflicts then, 4 % now.)
//
// How a K / V (Q / dO) tile gets there: straight from memory by global_load_lds_dwordx4 where the tensors
// allow it (16-byte aligned, see DmaTileMap: every head addressed from the 16-byte boundary at or below
// its start), else through registers (FastTileLoader, TileLoader8).  Measured at 32 heads x 2048 x 100:
// forward 108.7 -> 92.9 us, adjoint 235.5 -> 209.8 us, 48 vector registers fewer per kernel.  On that path the
// fixed operand of a workgroup (its 128 rows) arrives as tiles in LDS as well and every wave picks its fragments
// out of them (frags_from_tile), and the outputs leave through LDS as whole row segments (stage_rows,
// write_rows): a load or store in which every lane addresses its own row costs about a clock per lane.
// Forward 85.9 -> 79.0 us, dQ 95.8 -> 84.8, dK / dV 101.9 -> 97.0.
#include "common.h"
#include "softmax_math.h"

#include <algorithm>
#include <atomic>
#include <initializer_list>
#include <type_traits>

using namespace cacti;

namespace {

constexpr int kDP = 128;                 // padded head dim of an LDS tile
constexpr int kRowB = kDP * 2;           // bytes per tile row
constexpr int kTileRows = 64;
constexpr int kTileB = kTileRows * kRowB;   // 16 KB
constexpr int kNT = 256;                 // threads of a wave group (4 waves): the unit that loads a tile
constexpr int kBM = 128;                 // rows of the fixed operand per wave group (32 per wave)
constexpr float kSpread = 8.f;           // least row sum of exponentials for the short form of sigma (dQ kernel)

struct AttnArgs {
    int S, H, Dh;
    int64_t ld;
    float alpha;
    const half_t *q, *k, *v, *dO;
    const half_t *o;                     // the forward output (adjoint only; may be null)
    half_t *out, *dq, *dk, *dv;
    float *m, *l;                        // [H][S] row maximum and sum (forward output)
    float *y, *sig;                      // [H][S] adjoint scratch: sigma, and 1 / l (exact arithmetic) or the
                                         // exponent offset m log2(e) + log2(l) (fast arithmetic) of each row
    int acc_dq, acc_dk, acc_dv;
};

typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
// pointers into device memory, said so: inside a function that is not inlined into the kernel the
// compiler would otherwise use flat loads, which also count as LDS operations when it waits for one
typedef const __attribute__((address_space(1))) half_t *gptr_t;
typedef const __attribute__((address_space(1))) float *gfptr_t;
__device__ __forceinline__ gptr_t gp(const half_t *q) { return (gptr_t)q; }
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
// 8 bytes from device memory
__device__ __forceinline__ uint2 gload8(gptr_t q)
{
    const u32x2_t t = *(const __attribute__((address_space(1))) u32x2_t *)q;
    return make_uint2(t.x, t.y);
}

__device__ __forceinline__ int gsw(int r) { return ((r & 3) << 1) | ((r >> 2) & 1) | ((r & 8) ^ ((r & 1) << 3)); }
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

// The K / V (Q / dO) tiles through registers into LDS: the path for tensors whose tiles cannot be loaded
// straight into LDS (DmaTileMap further down).

// 16 bytes from device memory at an address that is only 8-byte aligned (the heads of a [S, H, 100]
// tensor start every 200 bytes): one global_load_dwordx4, which needs dword alignment only
typedef uint32_t u32x4_a8_t __attribute__((ext_vector_type(4), aligned(8)));
__device__ __forceinline__ uint4 gload16(gptr_t q)
{
    const u32x4_a8_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a8_t *>(q);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Per-lane constants of the mapping between a 64 x Dh tile of a [S, H, Dh] tensor and its LDS tile, for
// the 256 lanes of one wave group: piece `it` of a lane (16 bytes, 4 per lane) is row r0 + 16 it,
// columns 8 pc .. 8 pc + 7, r0 = lane / 16, pc = lane % 16.  Its element offset from the tile's first
// row is goff0 + 16 it ld (a wave-uniform step), its byte offset in the LDS tile loff + 4096 it (16
// more rows leave the chunk swizzle g(r) as it is).  A memory instruction costs the address unit the
// same for 8 as for 16 bytes per lane, and the address unit, not the arithmetic, is what these kernels
// wait for: 4 loads per tile and lane instead of 8.  Lanes whose columns lie beyond the head load a
// duplicate and store nothing: the pad columns of every tile buffer are zeroed once when the kernel
// starts.  The piece that straddles the end of the head (Dh % 8 = 4: columns Dh - 4 .. Dh + 3) is
// loaded 4 columns early, so that it stays inside the head, and shifted into place.
struct FastTileMap {
    unsigned goff0, loff;
    int r0, gcol;
    int64_t ld;
    bool colok, tail, narrow;                            // narrow: a head of 4 columns, one 8-byte piece per row
    __device__ __forceinline__ FastTileMap(int64_t ld_, int Dh, int)
    {
        const int t = threadIdx.x & (kNT - 1), pc = t & 15;
        r0 = t >> 4;
        ld = ld_;
        narrow = Dh < 8;
        colok = pc * 8 < Dh;
        tail = !narrow && colok && pc * 8 + 8 > Dh;
        gcol = narrow ? 0 : tail ? Dh - 8 : min(pc * 8, Dh - 8);
        goff0 = (unsigned)(r0 * ld_ + gcol);
        loff = (unsigned)toff(r0, pc);
    }
};

__device__ __forceinline__ void zero_lds(unsigned char *smem, int bytes)
{
    for (int o = threadIdx.x * 16; o < bytes; o += blockDim.x * 16) *reinterpret_cast<uint4 *>(smem + o) = make_uint4(0, 0, 0, 0);
    __syncthreads();
}
// The same for tiles that are loaded straight into LDS: only the chunks no load writes (window chunks nch .. 15 of
// every row), without a barrier of its own -- the loads of the first tiles are already in flight when this runs
// and touch none of these chunks; the barrier that publishes those tiles publishes the zeros.
__device__ __forceinline__ void zero_pads(unsigned char *smem, int rows, int nch)
{
    const int npad = 16 - nch;
    for (int i = threadIdx.x; i < rows * npad; i += blockDim.x) {
        const int r = i / npad, c = nch + i % npad;
        *reinterpret_cast<uint4 *>(smem + toff(r, c)) = make_uint4(0, 0, 0, 0);
    }
}

// 64 rows x Dh of a [S, H, Dh] tensor -> registers -> LDS tile, by the 256 lanes of one wave group, with
// the constants above (the forward and the dK / dV kernel; the dQ kernel has no registers to spare for
// it -- it spills 56 registers with it -- and uses the 8-byte form further down).
// Whole tiles take the straight path: 4 loads at a lane-constant offset from 4 uniform row pointers, 4
// stores at a lane-constant LDS address with immediate offsets.  The last tile of a ragged sequence
// clamps its rows and zeroes the ones beyond the end.
struct FastTileLoader {
    static constexpr int NP = kTileRows * 16 / kNT;      // 16-byte pieces per lane
    uint4 v[NP];
    int rows;                                            // rows of the tile inside the tensor (uniform)
    // src = &X[row0][head column 0]; rows_left = S - row0 >= 1
    __device__ __forceinline__ void load(const FastTileMap &m, gptr_t src, int rows_left, unsigned char *)
    {
        rows = __builtin_amdgcn_readfirstlane(min(rows_left, kTileRows));
        if (m.narrow) {
#pragma unroll
            for (int it = 0; it < NP; it++) {
                const uint2 a = gload8(src + (int64_t)min(m.r0 + 16 * it, rows - 1) * m.ld);
                v[it] = make_uint4(a.x, a.y, 0u, 0u);
            }
        } else if (rows == kTileRows) {
#pragma unroll
            for (int it = 0; it < NP; it++) v[it] = gload16(src + (int64_t)(16 * it) * m.ld + m.goff0);
        } else {
#pragma unroll
            for (int it = 0; it < NP; it++) v[it] = gload16(src + (int64_t)min(m.r0 + 16 * it, rows - 1) * m.ld + m.gcol);
        }
    }
    // the straddling piece moves into place by four selects per piece and the test for a ragged tile is
    // made once (a shuffle under a lane mask per piece took five times the instructions: forward and
    // dK / dV kernel -4 us each)
    __device__ __forceinline__ void store(const FastTileMap &m, unsigned char *tile) const
    {
        if (!m.colok) return;
        if (rows == kTileRows) {
#pragma unroll
            for (int it = 0; it < NP; it++) {
                uint4 x;
                x.x = m.tail ? v[it].z : v[it].x;
                x.y = m.tail ? v[it].w : v[it].y;
                x.z = m.tail ? 0u : v[it].z;
                x.w = m.tail ? 0u : v[it].w;
                *reinterpret_cast<uint4 *>(tile + m.loff + 4096 * it) = x;
            }
        } else {
#pragma unroll
            for (int it = 0; it < NP; it++) {
                const bool in = m.r0 + 16 * it < rows;
                uint4 x;
                x.x = !in ? 0u : m.tail ? v[it].z : v[it].x;
                x.y = !in ? 0u : m.tail ? v[it].w : v[it].y;
                x.z = (!in || m.tail) ? 0u : v[it].z;
                x.w = (!in || m.tail) ? 0u : v[it].w;
                *reinterpret_cast<uint4 *>(tile + m.loff + 4096 * it) = x;
            }
        }
    }
};

// The same with 8-byte pieces (8 per lane: row r0 + 8 it, columns 4 pc .. 4 pc + 3, r0 = lane / 32,
// pc = lane % 32), for the kernel whose registers do not hold the 16-byte loader: no piece straddles the
// end of a head (Dh % 4 = 0), the chunk swizzle of rows r0 + 8 it alternates between two values.  With
// per-piece index arithmetic instead of these lane constants a tile cost 5 times the instructions
// (dQ kernel 129 -> 125 us).
struct TileMap8 {
    unsigned goff0, loff0, loff1;
    int r0, gcol;
    int64_t ld;
    bool colok;
    __device__ __forceinline__ TileMap8(int64_t ld_, int Dh, int)
    {
        const int t = threadIdx.x & (kNT - 1), pc = t & 31;
        r0 = t >> 5;
        ld = ld_;
        colok = pc * 4 < Dh;
        gcol = min(pc * 4, Dh - 4);
        goff0 = (unsigned)(r0 * ld_ + gcol);
        loff0 = (unsigned)(toff(r0, pc >> 1) + ((pc & 1) << 3));
        loff1 = (unsigned)(toff(r0 + 8, pc >> 1) + ((pc & 1) << 3)) - 8 * kRowB;
    }
};
struct TileLoader8 {
    static constexpr int NP = kTileRows * 32 / kNT;      // 8-byte pieces per lane
    uint2 v[NP];
    int rows;
    __device__ __forceinline__ void load(const TileMap8 &m, gptr_t src, int rows_left, unsigned char *)
    {
        rows = __builtin_amdgcn_readfirstlane(min(rows_left, kTileRows));
        if (rows == kTileRows) {
#pragma unroll
            for (int it = 0; it < NP; it++) v[it] = gload8(src + (int64_t)(8 * it) * m.ld + m.goff0);
        } else {
#pragma unroll
            for (int it = 0; it < NP; it++) v[it] = gload8(src + (int64_t)min(m.r0 + 8 * it, rows - 1) * m.ld + m.gcol);
        }
    }
    __device__ __forceinline__ void store(const TileMap8 &m, unsigned char *tile) const
    {
        if (!m.colok) return;
        if (rows == kTileRows) {
#pragma unroll
            for (int it = 0; it < NP; it++)
                *reinterpret_cast<uint2 *>(tile + ((it & 1) ? m.loff1 : m.loff0) + 8 * kRowB * it) = v[it];
        } else {
#pragma unroll
            for (int it = 0; it < NP; it++) {
                const bool in = m.r0 + 8 * it < rows;
                *reinterpret_cast<uint2 *>(tile + ((it & 1) ? m.loff1 : m.loff0) + 8 * kRowB * it) =
                    make_uint2(in ? v[it].x : 0u, in ? v[it].y : 0u);
            }
        }
    }
};

// Tiles straight into LDS (global_load_lds_dwordx4: the 16 bytes of lane l land at LDS address M0 + 16 l; no
// staging registers, no LDS store instructions, no selects).  The load wants 16-byte aligned addresses and the
// heads of a [S, H, Dh] tensor with Dh % 8 = 4 start on 8-byte boundaries every other head, so a head is
// addressed from the 16-byte boundary at or below its start: a *window* of ceil((Dh + shift) / 8) chunks that
// begins shift = (h Dh) % 8 elements (0 or 4) before the head.  Everything a kernel holds per head -- LDS tiles,
// the fragments of the fixed operand, accumulator columns -- is in window positions, column d of the head at
// position d + shift; the positions outside the head hold the neighbouring heads' elements in the tiles and
// zeros in the fixed operand's fragments, so they add nothing to a product over the head dimension, and output
// columns there are not stored.  (What that costs: a non-finite value in the 4 elements next to a head makes
// that head's result non-finite too, where the reference keeps it to the neighbour until the output projection
// mixes the heads.)  One instruction of a wave fills 4 tile rows; the chunk swizzle g(r) is applied on the
// global side (the lane at chunk position p of row r fetches window chunk p ^ g(r)), lanes whose chunk lies
// beyond the window stay out of the instruction, and those positions keep the zeros the kernel wrote at its
// start.  The compiler neither counts these loads nor knows that they write LDS: the kernels wait for them
// (vmcnt) before the barrier that publishes a tile.
struct DmaTileMap {
    uint32_t voff, slot;
    int r0;
    int64_t ld;
    bool act;
    __device__ __forceinline__ DmaTileMap(int64_t ld_, int Dh, int shift)
    {
        const int t = threadIdx.x & (kNT - 1), pc = t & 15;
        r0 = t >> 4;
        ld = ld_;
        const int c = pc ^ gsw(r0);                      // g(r0 + 16 it) = g(r0)
        act = c * 8 < Dh + shift;
        voff = (uint32_t)((r0 * ld_ + c * 8) * 2);
        slot = (uint32_t)(r0 * kRowB + pc * 16);
    }
};
__device__ __forceinline__ void dma16(uint32_t lds, uint32_t voff, gptr_t base)
{
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(m0), "v"(voff), "s"(base) : "memory");
}
struct DmaTileLoader {
    // src = the window's first element in the tile's first row; rows beyond the tensor are zeroed by the lanes
    // that would have fetched them
    __device__ __forceinline__ void load(const DmaTileMap &m, gptr_t src, int rows_left, unsigned char *tile) const
    {
        const int rows = __builtin_amdgcn_readfirstlane(min(rows_left, kTileRows));
        const uint32_t wave = (uint32_t)(uintptr_t)tile + ((threadIdx.x & (kNT - 1)) >> 6) * 4 * kRowB;
        if (rows == kTileRows) {
            if (m.act) {
#pragma unroll
                for (int it = 0; it < 4; it++) dma16(wave + it * 16 * kRowB, m.voff, src + (int64_t)(16 * it) * m.ld);
            }
        } else {
#pragma unroll
            for (int it = 0; it < 4; it++) {
                if (m.r0 + 16 * it < rows) {
                    if (m.act) dma16(wave + it * 16 * kRowB, m.voff, src + (int64_t)(16 * it) * m.ld);
                } else {
                    *reinterpret_cast<uint4 *>(tile + m.slot + it * 16 * kRowB) = make_uint4(0, 0, 0, 0);
                }
            }
        }
    }
    __device__ __forceinline__ void store(const DmaTileMap &, unsigned char *) const {}
};

// the barrier that publishes the tiles just loaded (and retires the ones just read)
template <bool DMA>
__device__ __forceinline__ void tile_sync()
{
    if (DMA) __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));          // vmcnt(0) alone
    __syncthreads();
}

// The fixed operand of a lane: row `row` of a [S, H, Dh] tensor as KS fragments (k step ks: the 8
// halves at positions 16 ks + 8 lh .., position = column + shift), zero outside the head and for rows beyond S
template <int KS>
__device__ __forceinline__ void load_frags(half8_t (&f)[KS], gptr_t X, int64_t ld, int row, int S, int Dh, int lh,
                                           int shift = 0)
{
    const bool rok = row < S;
    gptr_t xr = X + (int64_t)min(row, S - 1) * ld;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int d0 = 16 * ks + 8 * lh - shift;          // the head's column at the fragment's first position
        const bool ok0 = rok && d0 >= 0 && d0 < Dh, ok1 = rok && d0 + 4 < Dh;
        const uint2 a = gload8(xr + max(min(d0, Dh - 4), 0));
        const uint2 b = gload8(xr + min(d0 + 4, Dh - 4));
        f[ks] = as_h8(make_uint2(ok0 ? a.x : 0u, ok0 ? a.y : 0u), make_uint2(ok1 ? b.x : 0u, ok1 ? b.y : 0u));
    }
}

// The same fragments out of an LDS tile that holds the operand's rows in window positions (a tile loaded
// straight into LDS; row = the lane's row inside the tile): what lies outside the head there is the
// neighbouring heads' data, cleared here.  Rows beyond S are zero in such a tile already.
template <int KS>
__device__ __forceinline__ void frags_from_tile(half8_t (&f)[KS], const unsigned char *tile, int row, int Dh, int lh,
                                                int shift)
{
    const unsigned char *rp = tile + row * kRowB;
    const int g = gsw(row);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const uint4 v = *reinterpret_cast<const uint4 *>(rp + (((2 * ks + lh) ^ g) << 4));
        const int d0 = 16 * ks + 8 * lh - shift;
        const bool ok0 = d0 >= 0 && d0 < Dh, ok1 = d0 + 4 < Dh;
        f[ks] = as_h8(make_uint2(ok0 ? v.x : 0u, ok0 ? v.y : 0u), make_uint2(ok1 ? v.z : 0u, ok1 ? v.w : 0u));
    }
}

// acc = sum over d of X[row_base + .][d] Y[.][d]: X from the LDS tile (16-byte reads), Y = fixed fragments.
// PRIO: the wave runs its chain of dependent MFMAs at raised priority, so that the other wave of the SIMD
// fills the gaps of the chain with its arithmetic instead of delaying it (forward and dQ kernel -2 %; the
// dK / dV kernel has a SIMD to itself and only pays for the two extra instructions)
template <int KS, bool PRIO = true>
__device__ __forceinline__ float16_t prod_direct(const unsigned char *tile, int row_base, const half8_t (&yf)[KS],
                                                 int l32, int lh)
{
    float16_t acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    const int row = row_base + l32;
    const unsigned char *rp = tile + row * kRowB;
    const int g = gsw(row);
    half8_t x[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) x[ks] = *reinterpret_cast<const half8_t *>(rp + (((2 * ks + lh) ^ g) << 4));
    if (PRIO) __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[ks], yf[ks], acc, 0, 0, 0);
    if (PRIO) __builtin_amdgcn_s_setprio(0);
    // all fragment reads in flight before the first product (the scheduler would otherwise pair each
    // read with its use and expose the LDS latency once per k step)
    __builtin_amdgcn_sched_group_barrier(0x100, KS, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, KS, 0);
    return acc;
}

// The same product with independent vector arithmetic issued between its MFMAs (the softmax arithmetic of the
// score tile before this one): a chain of dependent MFMAs leaves the wave nothing to issue for 32 cycles per
// link, and the two waves of a SIMD do not fill each other's gaps reliably.  `work(integral_constant<i>)` is
// piece i of NP pieces of that arithmetic: piece 0 covers the latency of the fragment reads, the others follow
// the MFMAs in equal shares; scheduling barriers keep the order as written.
template <int KS, int NP, class F>
__device__ __forceinline__ float16_t prod_direct_with(const unsigned char *tile, int row_base, const half8_t (&yf)[KS],
                                                      int l32, int lh, F &&work)
{
    float16_t acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    const int row = row_base + l32;
    const unsigned char *rp = tile + row * kRowB;
    const int g = gsw(row);
    half8_t x[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) x[ks] = *reinterpret_cast<const half8_t *>(rp + (((2 * ks + lh) ^ g) << 4));
    __builtin_amdgcn_sched_barrier(0);
    work(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    auto link = [&](auto ks_c) __attribute__((always_inline)) {
        constexpr int ks = decltype(ks_c)::value;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[ks], yf[ks], acc, 0, 0, 0);
        constexpr int p0 = 1 + ks * (NP - 1) / KS, p1 = 1 + (ks + 1) * (NP - 1) / KS;
        if constexpr (p0 < p1) work(std::integral_constant<int, p0>{});
        if constexpr (p0 + 1 < p1) work(std::integral_constant<int, p0 + 1>{});
        static_assert(p1 - p0 <= 2, "at most two pieces per MFMA");
        __builtin_amdgcn_sched_barrier(0);
    };
    link(std::integral_constant<int, 0>{});
    link(std::integral_constant<int, 1>{});
    link(std::integral_constant<int, 2>{});
    link(std::integral_constant<int, 3>{});
    if constexpr (KS > 4) link(std::integral_constant<int, 4>{});
    if constexpr (KS > 5) link(std::integral_constant<int, 5>{});
    if constexpr (KS > 6) link(std::integral_constant<int, 6>{});
    if constexpr (KS > 7) link(std::integral_constant<int, 7>{});
    static_assert(KS >= 4 && KS <= 8, "4 to 8 k steps");
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

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// The same with independent vector arithmetic between its 2 DT MFMAs (NP pieces, `work(integral_constant<i>)`):
// every transposing read is issued first, scheduling barriers keep the order as written.
template <int DT, int NP, class F>
__device__ __forceinline__ void prod_tr_with(float16_t (&acc)[DT], const unsigned char *tile, int k_base, half8_t y0,
                                             half8_t y1, int lane, F &&work)
{
    const int a4 = (lane >> 2) & 3, b4 = lane & 3, n16 = (lane >> 4) & 1, lh = lane >> 5;
    const int colb = 16 * n16 + 4 * b4;
    half8_t x[2][DT];
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
        const int r1 = k_base + 16 * kk + 4 * lh + a4, r2 = r1 + 8;
        const unsigned char *p1 = tile + r1 * kRowB + ((colb & 4) << 1);
        const unsigned char *p2 = tile + r2 * kRowB + ((colb & 4) << 1);
        const int g1 = gsw(r1), g2 = gsw(r2);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            const int c = (32 * dt + colb) >> 3;
            x[kk][dt] = as_h8(lds_read_tr(p1 + ((c ^ g1) << 4)), lds_read_tr(p2 + ((c ^ g2) << 4)));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 2 * DT>([&](auto j_c) __attribute__((always_inline)) {
        constexpr int j = decltype(j_c)::value, kk = j / DT, dt = j % DT;
        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[kk][dt], kk ? y1 : y0, acc[dt], 0, 0, 0);
        constexpr int p0 = j * NP / (2 * DT), p1 = (j + 1) * NP / (2 * DT);
        if constexpr (p0 < p1) work(std::integral_constant<int, p0>{});
        if constexpr (p0 + 1 < p1) work(std::integral_constant<int, p0 + 1>{});
        static_assert(p1 - p0 <= 2, "at most two pieces per MFMA");
        __builtin_amdgcn_sched_barrier(0);
    });
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

// The f32 arithmetic between the rounding points.  EXACT: exponential with range reduction and a
// correctly rounded quotient, the arithmetic of the separate softmax kernels; FAST: v_exp_f32 of the
// scaled difference, with the division folded into the exponent (exp2_mix below; a few ulp of f32
// away, under half of the instructions).
constexpr float kLog2e = 0x1.715476p+0f;
template <bool FAST>
struct AttnMath {
    // exp(s - m) of two f32 values (merging row statistics; every score in the exact form)
    static __device__ __forceinline__ float ex(float s, float m)
    {
        if (FAST) return __builtin_amdgcn_exp2f((s - m) * kLog2e);
        return exp_diff(s, m);
    }
    // a probability in the exact form (the fast form goes through exp2_mix)
    static __device__ __forceinline__ float prob(float s, float m, float l, float y)
    {
        return div_by(exp_diff(s, m), l, y);
    }
};

// FAST arithmetic on scores that stay f16 between their rounding point and the exponent: one fused
// multiply-add that reads the f16 value (v_fma_mix_f32) forms s log2(e) - c, where c holds the row's
// maximum (and, for a probability, log2 of the row's sum as well), and v_exp_f32 does the rest.
typedef _Float16 half2v_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float exp2_mix(half_t s, float c)
{
    return __builtin_amdgcn_exp2f(__builtin_fmaf((float)s, kLog2e, -c));
}
// maximum of 16 f16 values (exact in f16), two per instruction
__device__ __forceinline__ float max16(const half_t (&h)[16])
{
    half2v_t mx = {h[0], h[1]};
#pragma unroll
    for (int e = 2; e < 16; e += 2) mx = __builtin_elementwise_max(mx, half2v_t{h[e], h[e + 1]});
    return (float)__builtin_fmaxf16(mx[0], mx[1]);
}
// 16 f32 -> f16 (round to nearest even), two per instruction
typedef float float2v_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void round16(half_t (&h)[16], const float16_t &a)
{
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        const half2v_t t = __builtin_convertvector(float2v_t{a[e], a[e + 1]}, half2v_t);
        h[e] = t[0];
        h[e + 1] = t[1];
    }
}
// two f32 -> packed f16 (round to nearest even) as one v_cvt_pk_f16_f32, said so: left to itself the compiler
// may fold the multiplication in front into two v_fma_mixlo / mixhi_f16, which cost 4.4 ns each per SIMD where
// a multiplication costs 2.1 and this instruction 2.8 for the pair
__device__ __forceinline__ half2v_t cvt_pk(float a, float b)
{
    uint32_t u;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(u) : "v"(a), "v"(b));
    half2v_t h;
    __builtin_memcpy(&h, &u, 4);
    return h;
}
// the exponent offset of a row's probabilities: m log2(e) + log2(l)
__device__ __forceinline__ float prob_shift(float m, float l)
{
    return __builtin_fmaf(m, kLog2e, __builtin_amdgcn_logf(l));
}

// a x as an f32 value of its own: the reference scales a product in f32 and rounds the result to f16, two
// roundings; written as f2h(a * x) the compiler is free to use one instruction that multiplies and rounds to f16
// once (v_fma_mixlo_f16), which differs from that in one element of some 20,000 by an f16 ulp -- and costs
// more than the multiplication and half a packed conversion
__device__ __forceinline__ float scaled(float a, float x)
{
    float t = a * x;
    asm volatile("" : "+v"(t));
    return t;
}

// 4 consecutive d of one output row: f16(scale a[0..3] [+ old])
__device__ __forceinline__ void store_row4(half_t *dst, float a0, float a1, float a2, float a3, float scale,
                                           int acc_old)
{
    const float a[4] = {a0, a1, a2, a3};
    half4_t o;
    if (acc_old) {
        const half4_t old = *reinterpret_cast<const half4_t *>(dst);
#pragma unroll
        for (int r = 0; r < 4; r++) o[r] = f2h(scaled(scale, a[r]) + h2f(old[r]));
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++) o[r] = f2h(scaled(scale, a[r]));
    }
    *reinterpret_cast<half4_t *>(dst) = o;
}

// An output tile of 128 rows leaves through LDS when the tiles are direct (16-byte aligned rows): stores in which
// every lane addresses its own row are served at about one lane per clock and CU like such loads (16 of them per
// lane and output: 4 k cycles per workgroup), whole row segments of 16 bytes per lane are not.  stage_rows: a
// wave's 32 rows as f16(scale acc), in window positions, in the layout of an operand tile; write_rows: the
// staged rows [0, rows) to memory by all threads, the head's columns only (dst = the window's first element in
// row 0).  The same values as store_row4 writes.
template <int DT>
__device__ __forceinline__ void stage_rows(unsigned char *stage, const float16_t (&acc)[DT], int row, int lh, float scale)
{
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            half4_t o;
#pragma unroll
            for (int r = 0; r < 4; r++) o[r] = f2h(scaled(scale, acc[dt][4 * q + r]));
            *reinterpret_cast<half4_t *>(stage + toff(row, 4 * dt + q) + 8 * lh) = o;
        }
}
__device__ __forceinline__ void write_rows(const unsigned char *stage, half_t *dst, int64_t ld, int rows, int Dh,
                                           int shift, int tid, int nthr)
{
    const int nch = (Dh + shift + 7) >> 3;
    for (int i = tid; i < kBM * 16; i += nthr) {
        const int row = i >> 4, c = i & 15;
        if (row >= rows || c >= nch) continue;
        const uint4 v = *reinterpret_cast<const uint4 *>(stage + toff(row, c));
        const int d0 = 8 * c - shift;                    // the head's column at the chunk's first position
        const bool lo = d0 >= 0 && d0 < Dh, hi = d0 + 4 < Dh;
        half_t *q = dst + (int64_t)row * ld + 8 * c;
        if (lo && hi) *reinterpret_cast<uint4 *>(q) = v;
        else if (lo) *reinterpret_cast<uint2 *>(q) = make_uint2(v.x, v.y);
        else if (hi) *reinterpret_cast<uint2 *>(q + 4) = make_uint2(v.z, v.w);
    }
}

// Work split of the query-major kernels (forward, dQ).  A workgroup is two wave groups of 4 waves on
// the same 128 query rows; group g takes the key tiles g, g + 2, ... with its own LDS buffers, and the
// two partial results (row statistics, output tile) meet in LDS at the end: the 2 waves a SIMD holds
// have the same amount of work from start to end.
constexpr int kNT2 = 2 * kNT;
constexpr int kGroupLds = 4 * kTileB;                   // K and V tiles, two buffers each
constexpr int kXsOff = 2 * kGroupLds;                   // float [2 groups][2][128]: statistics exchange
constexpr size_t kQmSmem = 2 * kGroupLds + 2 * 2 * kBM * sizeof(float);

// partial output tiles (DT x 16 floats per lane) of wave group 1 -> LDS -> added onto group 0's
template <int DT>
__device__ __forceinline__ void merge_partials(float16_t (&acc)[DT], unsigned char *region, int g, int tig)
{
    float *x = reinterpret_cast<float *>(region);
    if (g == 1) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) x[(dt * 16 + r) * kNT + tig] = acc[dt][r];
    }
    __syncthreads();
    if (g == 0) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[dt][r] += x[(dt * 16 + r) * kNT + tig];
    }
}

// ---------------------------------------------------------------------------------------------
// Workgroups take the tiles in descending order of their key count; a CU holds one workgroup at a
// time (LDS), so the dispatcher hands the next tile to whichever CU is done first.
template <int KS, int DT, bool FAST, bool DMA>
__global__ void __launch_bounds__(kNT2, 2) attn_fwd_kernel(AttnArgs p)
{
    // the whole argument block in scalar registers at once (read field by field where the control flow first
    // wants it, it costs several dependent round trips to memory before the first tile is requested)
    asm volatile("" ::"s"(p.S), "s"(p.H), "s"(p.Dh), "s"(p.ld), "s"(p.alpha), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.dO),
                 "s"(p.o), "s"(p.out), "s"(p.dq), "s"(p.dk), "s"(p.dv), "s"(p.m), "s"(p.l), "s"(p.y), "s"(p.sig),
                 "s"(p.acc_dq), "s"(p.acc_dk), "s"(p.acc_dv));
    typedef AttnMath<FAST> M;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    if constexpr (!DMA) zero_lds(smem, 2 * kGroupLds);   // the pad columns of the tile buffers: zero from here on
    // wave-uniform values kept in scalar registers, so that the branches on them are scalar branches
    const int g = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8), tig = threadIdx.x & (kNT - 1);
    unsigned char *Ks = smem + g * kGroupLds, *Vs = Ks + 2 * kTileB;
    float *xs = reinterpret_cast<float *>(smem + kXsOff);
    const int lane = tig & 63, wid = __builtin_amdgcn_readfirstlane(tig >> 6), l32 = lane & 31, lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int nqt = (S + kBM - 1) / kBM;
    const int h = blockIdx.x % p.H, qt = nqt - 1 - blockIdx.x / p.H;
    const int shift = DMA ? (int)(((int64_t)h * Dh) & 7) : 0;          // the head's first column in its window
    gptr_t Q = gp(p.q) + (int64_t)h * Dh, K = gp(p.k) + (int64_t)h * Dh - shift, V = gp(p.v) + (int64_t)h * Dh - shift;
    {
        const int i0 = qt * kBM, r0 = i0 + wid * 32, myrow = r0 + l32;

        // the queries: with direct tiles they come as two tiles straight into LDS below, beside the first key
        // and value tiles (a load in which every lane addresses its own row is served at one lane per clock)
        half8_t qf[KS];
        if constexpr (!DMA) load_frags<KS>(qf, Q, ld, myrow, S, Dh, lh, shift);

        const int kend = min(i0 + kBM, S);                 // keys [0, kend) are visible to the tile
        const int njt = (kend + kTileRows - 1) / kTileRows, niter = (njt + 1) / 2;
        typedef typename std::conditional<DMA, DmaTileMap, FastTileMap>::type Map;
        typedef typename std::conditional<DMA, DmaTileLoader, FastTileLoader>::type Loader;
        const Map tm(ld, Dh, shift);
        Loader tk, tv;

        // ---- pass 1: row maximum and sum; each lane over its half of the keys of its group's tiles
        float m_run = -INFINITY, l_run = 0.f;
        if (g < njt) {
            tk.load(tm, K + (int64_t)g * kTileRows * ld, S - g * kTileRows, Ks);
            tk.store(tm, Ks);
            // the V buffers idle through pass 1: the first V tile of pass 2 comes in now
            if constexpr (DMA) tv.load(tm, V + (int64_t)g * kTileRows * ld, S - g * kTileRows, Vs);
        }
        if constexpr (DMA) {
            // rows 64 g .. 64 g + 63 of the workgroup's queries into this group's second V buffer, which idles
            // until the second pass; every wave then takes its fragments from the tile that holds its rows
            tv.load(tm, Q - shift + (int64_t)(i0 + g * kTileRows) * ld, S - (i0 + g * kTileRows), Vs + kTileB);
            zero_pads(smem, 2 * kGroupLds / kRowB, (Dh + shift + 7) >> 3);
        }
        tile_sync<DMA>();
        if constexpr (DMA)
            frags_from_tile<KS>(qf, smem + (wid >> 1) * kGroupLds + 3 * kTileB, (wid & 1) * 32 + l32, Dh, lh, shift);
        int it0 = 0;
        if constexpr (FAST) {
            // The key tiles wholly below the diagonal for every wave (iterations 0 .. qt - 1 of both groups) as a
            // pipeline: the products of a score tile run while the statistics of the tile before it are updated.
            // The same operations on the same values in the same order as the general loop below.
            // in 8 pieces: round the scores; their maximum; 4 x (4 exponentials and their sum); the running pair
            half2v_t sp[8];
            float m_new, cexp, sum;
            auto stat_piece = [&](const float16_t &acc, auto i_c) __attribute__((always_inline)) {
                constexpr int i = decltype(i_c)::value;
                if constexpr (i == 0) {
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        sp[e] = __builtin_convertvector(float2v_t{scaled(p.alpha, acc[2 * e]), scaled(p.alpha, acc[2 * e + 1])}, half2v_t);
                } else if constexpr (i == 1) {
                    half2v_t mx = sp[0];
#pragma unroll
                    for (int e = 1; e < 8; e++) mx = __builtin_elementwise_max(mx, sp[e]);
                    m_new = fmaxf(m_run, (float)__builtin_fmaxf16(mx[0], mx[1]));
                    cexp = m_new * kLog2e;
                    sum = 0.f;
                } else if constexpr (i < 6) {
#pragma unroll
                    for (int e = 4 * (i - 2); e < 4 * (i - 1); e++) sum += exp2_mix(sp[e >> 1][e & 1], cexp);
                } else if constexpr (i == 6) {
                    l_run = ((m_run == -INFINITY) ? 0.f : l_run * M::ex(m_run, m_new)) + sum;
                    m_run = m_new;
                }
            };
            auto stat_full = [&](const float16_t &acc) __attribute__((always_inline)) {
                stat_piece(acc, std::integral_constant<int, 0>{});
                stat_piece(acc, std::integral_constant<int, 1>{});
                stat_piece(acc, std::integral_constant<int, 2>{});
                stat_piece(acc, std::integral_constant<int, 3>{});
                stat_piece(acc, std::integral_constant<int, 4>{});
                stat_piece(acc, std::integral_constant<int, 5>{});
                stat_piece(acc, std::integral_constant<int, 6>{});
            };
            const int nfull = min(qt, niter);
            if (nfull > 0) {
                float16_t accp = prod_direct<KS>(Ks, 0, qf, l32, lh);
                for (int it = 0; it < nfull; it++) {
                    const int jt = 2 * it + g, cur = it & 1;
                    const bool nxt = jt + 2 < njt;
                    if (nxt) tk.load(tm, K + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Ks + (cur ^ 1) * kTileB);
                    accp = prod_direct_with<KS, 7>(Ks + cur * kTileB, 32, qf, l32, lh, [&](auto i_c) { stat_piece(accp, i_c); });
                    if (nxt) tk.store(tm, Ks + (cur ^ 1) * kTileB);
                    tile_sync<DMA>();
                    if (it + 1 < nfull)
                        accp = prod_direct_with<KS, 7>(Ks + (cur ^ 1) * kTileB, 0, qf, l32, lh, [&](auto i_c) { stat_piece(accp, i_c); });
                    else
                        stat_full(accp);
                }
                it0 = nfull;
            }
        }
        for (int it = it0; it < niter; it++) {
            const int jt = 2 * it + g, cur = it & 1;
            const bool nxt = jt + 2 < njt;
            if (nxt) tk.load(tm, K + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Ks + (cur ^ 1) * kTileB);
            if (jt < njt) {
#pragma unroll
                for (int kt = 0; kt < 2; kt++) {
                    const int kb = jt * kTileRows + 32 * kt;
                    if (kb > r0 + 31) continue;          // every key of the tile is beyond every row of the wave
                    const float16_t acc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
                    const bool full = kb + 31 <= r0;
                    float sv[16], mt = -INFINITY, sum = 0.f;
                    if constexpr (FAST) {
                        half_t sh[16];
                        if (full) {
#pragma unroll
                            for (int e = 0; e < 16; e++) sh[e] = f2h(scaled(p.alpha, acc[e]));
                        } else {
#pragma unroll
                            for (int e = 0; e < 16; e++) {
                                const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                                sh[e] = key <= myrow ? f2h(scaled(p.alpha, acc[e])) : (half_t)-INFINITY;
                            }
                        }
                        const float m_new = fmaxf(m_run, max16(sh)), c = m_new * kLog2e;
                        if (full) {
#pragma unroll
                            for (int e = 0; e < 16; e++) sum += exp2_mix(sh[e], c);
                        } else {
#pragma unroll
                            for (int e = 0; e < 16; e++)
                                sum += (sh[e] == (half_t)-INFINITY) ? 0.f : exp2_mix(sh[e], c);
                        }
                        l_run = ((m_run == -INFINITY) ? 0.f : l_run * M::ex(m_run, m_new)) + sum;
                        m_run = m_new;
                    } else if (full) {                   // no masks on tiles wholly below the diagonal
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            sv[e] = rnd16(scaled(p.alpha, acc[e]));
                            mt = fmaxf(mt, sv[e]);
                        }
                        const float m_new = fmaxf(m_run, mt);
#pragma unroll
                        for (int e = 0; e < 16; e++) sum += M::ex(sv[e], m_new);
                        l_run = ((m_run == -INFINITY) ? 0.f : l_run * M::ex(m_run, m_new)) + sum;
                        m_run = m_new;
                    } else {
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                            const float s = rnd16(scaled(p.alpha, acc[e]));
                            sv[e] = key <= myrow ? s : -INFINITY;
                            mt = fmaxf(mt, sv[e]);
                        }
                        const float m_new = fmaxf(m_run, mt);
#pragma unroll
                        for (int e = 0; e < 16; e++) sum += (sv[e] == -INFINITY) ? 0.f : M::ex(sv[e], m_new);
                        l_run = ((m_run == -INFINITY) ? 0.f : l_run * M::ex(m_run, m_new)) + sum;
                        m_run = m_new;
                    }
                }
            }
            if (nxt) tk.store(tm, Ks + (cur ^ 1) * kTileB);
            tile_sync<DMA>();
        }
        // pass 2 starts from the group's first K tile again: on its way while the statistics are merged
        if constexpr (DMA) {
            if (g < njt) tk.load(tm, K + (int64_t)g * kTileRows * ld, S - g * kTileRows, Ks);
        }
        float m, l;
        {
            // the four partial (maximum, sum) pairs of a row -- two lanes in each of two groups -- merged
            // in one fixed order by every lane that needs the result
            const float m_o = __shfl_xor(m_run, 32, 64), l_o = __shfl_xor(l_run, 32, 64);
            const float ma = lh ? m_o : m_run, la = lh ? l_o : l_run;
            const float mb = lh ? m_run : m_o, lb = lh ? l_run : l_o;
            const float mg = fmaxf(ma, mb);
            const float lg = ((ma == -INFINITY) ? 0.f : la * M::ex(ma, mg)) + ((mb == -INFINITY) ? 0.f : lb * M::ex(mb, mg));
            if (lh == 0) {
                xs[(g * 2 + 0) * kBM + wid * 32 + l32] = mg;
                xs[(g * 2 + 1) * kBM + wid * 32 + l32] = lg;
            }
            __syncthreads();
            const float m0 = xs[0 * kBM + wid * 32 + l32], l0 = xs[1 * kBM + wid * 32 + l32];
            const float m1 = xs[2 * kBM + wid * 32 + l32], l1 = xs[3 * kBM + wid * 32 + l32];
            m = fmaxf(m0, m1);
            l = ((m0 == -INFINITY) ? 0.f : l0 * M::ex(m0, m)) + ((m1 == -INFINITY) ? 0.f : l1 * M::ex(m1, m));
            if (myrow >= S) { m = 0.f; l = 1.f; }
            if (g == 0 && lh == 0 && myrow < S) {
                p.m[(int64_t)h * S + myrow] = m;
                p.l[(int64_t)h * S + myrow] = l;
            }
        }
        const float y = recip_refined(l);
        const float cs = prob_shift(m, l);

        // ---- pass 2: probabilities and O
        float16_t oacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
        if (!DMA && g < njt) {
            tk.load(tm, K + (int64_t)g * kTileRows * ld, S - g * kTileRows, Ks);
            tv.load(tm, V + (int64_t)g * kTileRows * ld, S - g * kTileRows, Vs);
            tk.store(tm, Ks);
            tv.store(tm, Vs);
        }
        tile_sync<DMA>();
        int it2 = 0;
        if constexpr (FAST && DMA) {
            // The key tiles wholly below the diagonal for every wave, as in pass 1, with the vector arithmetic of a
            // block between the MFMAs of its neighbours: per tile, the scores of its second block are formed while
            // the probabilities of the first are, the first block's P V products run while the second's
            // probabilities are formed, then the second's P V; the first scores of the next tile follow the barrier
            // that publishes it (the P V products read the V tile, which the next iteration's loads overwrite, so
            // they cannot move behind the barrier).  The same operations on the same values in the same order as the
            // general loop below.
            const int nfull = min(qt, niter);
            if (nfull > 0) {
                half2v_t sp[8];
                float pe[16];
                half8_t pk[2][2];                               // packed probabilities of the tile's two blocks
                auto prob_piece = [&](const float16_t &acc, half8_t (&out)[2], auto i_c) __attribute__((always_inline)) {
                    constexpr int i = decltype(i_c)::value;
                    if constexpr (i == 0) {
#pragma unroll
                        for (int e = 0; e < 8; e++)
                            sp[e] = __builtin_convertvector(float2v_t{scaled(p.alpha, acc[2 * e]), scaled(p.alpha, acc[2 * e + 1])}, half2v_t);
                    } else if constexpr (i < 5) {
#pragma unroll
                        for (int e = 4 * (i - 1); e < 4 * i; e++) pe[e] = exp2_mix(sp[e >> 1][e & 1], cs);
                    } else {
                        out[0] = pack8(pe);
                        out[1] = pack8(pe + 8);
                    }
                };
                float16_t accp = prod_direct<KS>(Ks, 0, qf, l32, lh);
                for (int it = 0; it < nfull; it++) {
                    const int jt = 2 * it + g, cur = it & 1;
                    const bool nxt = jt + 2 < njt;
                    if (nxt) {
                        tk.load(tm, K + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Ks + (cur ^ 1) * kTileB);
                        tv.load(tm, V + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Vs + (cur ^ 1) * kTileB);
                    }
                    const float16_t acc2 = prod_direct_with<KS, 6>(Ks + cur * kTileB, 32, qf, l32, lh,
                                                                   [&](auto i_c) { prob_piece(accp, pk[0], i_c); });
                    asm volatile("" : "+v"(pk[0][0]), "+v"(pk[0][1]));
                    prod_tr_with<DT, 6>(oacc, Vs + cur * kTileB, 0, pk[0][0], pk[0][1], lane,
                                        [&](auto i_c) { prob_piece(acc2, pk[1], i_c); });
                    asm volatile("" : "+v"(pk[1][0]), "+v"(pk[1][1]));
                    prod_tr<DT>(oacc, Vs + cur * kTileB, 32, pk[1][0], pk[1][1], lane);
                    tile_sync<DMA>();
                    if (it + 1 < nfull) accp = prod_direct<KS>(Ks + (cur ^ 1) * kTileB, 0, qf, l32, lh);
                }
                it2 = nfull;
            }
        }
        for (int it = it2; it < niter; it++) {
            const int jt = 2 * it + g, cur = it & 1;
            const bool nxt = jt + 2 < njt;
            if (nxt) {
                tk.load(tm, K + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Ks + (cur ^ 1) * kTileB);
                tv.load(tm, V + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Vs + (cur ^ 1) * kTileB);
            }
            if (jt < njt) {
#pragma unroll
                for (int kt = 0; kt < 2; kt++) {
                    const int kb = jt * kTileRows + 32 * kt;
                    if (kb > r0 + 31) continue;
                    const float16_t acc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
                    const bool full = kb + 31 <= r0;
                    float pe[16];
                    if constexpr (FAST) {
                        if (full) {
#pragma unroll
                            for (int e = 0; e < 16; e++) pe[e] = exp2_mix(f2h(scaled(p.alpha, acc[e])), cs);
                        } else {
#pragma unroll
                            for (int e = 0; e < 16; e++) {
                                const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                                pe[e] = key <= myrow ? exp2_mix(f2h(scaled(p.alpha, acc[e])), cs) : 0.f;
                            }
                        }
                    } else if (full) {
#pragma unroll
                        for (int e = 0; e < 16; e++) pe[e] = M::prob(rnd16(scaled(p.alpha, acc[e])), m, l, y);
                    } else {
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            const int key = kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                            const float pr_ = M::prob(rnd16(scaled(p.alpha, acc[e])), m, l, y);
                            pe[e] = key <= myrow ? pr_ : 0.f;
                        }
                    }
                    prod_tr<DT>(oacc, Vs + cur * kTileB, 32 * kt, pack8(pe), pack8(pe + 8), lane);
                }
            }
            if (nxt) {
                tk.store(tm, Ks + (cur ^ 1) * kTileB);
                tv.store(tm, Vs + (cur ^ 1) * kTileB);
            }
            tile_sync<DMA>();
        }
        merge_partials<DT>(oacc, smem + kGroupLds, g, tig);
        if constexpr (DMA) {
            if (g == 0) stage_rows<DT>(smem, oacc, wid * 32 + l32, lh, 1.0f);
            __syncthreads();
            write_rows(smem, p.out + (int64_t)i0 * ld + (int64_t)h * Dh - shift, ld, min(kBM, S - i0), Dh, shift,
                       threadIdx.x, kNT2);
        } else if (g == 0 && myrow < S) {
            half_t *orow = p.out + (int64_t)myrow * ld + (int64_t)h * Dh;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int d0 = 32 * dt + 8 * q + 4 * lh - shift;
                    if (d0 >= 0 && d0 < Dh)
                        store_row4(orow + d0, oacc[dt][4 * q], oacc[dt][4 * q + 1], oacc[dt][4 * q + 2],
                                   oacc[dt][4 * q + 3], 1.0f, 0);
                }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: queries fixed, loop over the key tiles at or before them, work split as in the forward kernel.
// Pass 0 forms sigma = sum_j P' f32(dP16); pass 1 dS16 and dQ.  Leaves y = 1 / l and sigma per row for
// the dK / dV kernel.
template <int KS, int DT, bool FAST, bool DMA>
__global__ void __launch_bounds__(kNT2, 2) attn_bwd_dq_kernel(AttnArgs p)
{
    // the whole argument block in scalar registers at once (read field by field where the control flow first
    // wants it, it costs several dependent round trips to memory before the first tile is requested)
    asm volatile("" ::"s"(p.S), "s"(p.H), "s"(p.Dh), "s"(p.ld), "s"(p.alpha), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.dO),
                 "s"(p.o), "s"(p.out), "s"(p.dq), "s"(p.dk), "s"(p.dv), "s"(p.m), "s"(p.l), "s"(p.y), "s"(p.sig),
                 "s"(p.acc_dq), "s"(p.acc_dk), "s"(p.acc_dv));
    typedef AttnMath<FAST> M;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int g = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8), tig = threadIdx.x & (kNT - 1);
    unsigned char *Ks = smem + g * kGroupLds, *Vs = Ks + 2 * kTileB;
    float *xs = reinterpret_cast<float *>(smem + kXsOff);
    const int lane = tig & 63, wid = __builtin_amdgcn_readfirstlane(tig >> 6), l32 = lane & 31, lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int nqt = (S + kBM - 1) / kBM;
    const int h = blockIdx.x % p.H, qt = nqt - 1 - blockIdx.x / p.H;
    const int64_t hoff = (int64_t)h * Dh;
    const int shift = DMA ? (int)(hoff & 7) : 0;                        // the head's first column in its window
    // the pad columns of the tile buffers: zero from the first barrier on (direct tiles: cleared below, behind
    // the first loads)
    if constexpr (!DMA) zero_lds(smem, 2 * kGroupLds);
    gptr_t K = gp(p.k) + hoff - shift, V = gp(p.v) + hoff - shift;
    {
        const int i0 = qt * kBM, r0 = i0 + wid * 32, myrow = r0 + l32;
        const int kend = min(i0 + kBM, S);
        const int njt = (kend + kTileRows - 1) / kTileRows, niter = (njt + 1) / 2;
        typedef typename std::conditional<DMA, DmaTileMap, TileMap8>::type Map;
        typedef typename std::conditional<DMA, DmaTileLoader, TileLoader8>::type Loader;
        const Map tm(ld, Dh, shift);
        Loader tk, tv;
        auto first_tiles = [&]() __attribute__((always_inline)) {
            if (g < njt) {
                tk.load(tm, K + (int64_t)g * kTileRows * ld, S - g * kTileRows, Ks);
                tv.load(tm, V + (int64_t)g * kTileRows * ld, S - g * kTileRows, Vs);
                tk.store(tm, Ks);
                tv.store(tm, Vs);
            }
        };
        // The fixed operands.  A load in which every lane addresses its own row is served at about one lane
        // per clock and CU (42 such instructions in each of 8 waves: 21 k of the 29 k cycles this kernel used
        // to spend before its first product), so with direct tiles the workgroup's 128 rows of q, dO and the
        // forward output (used by the short form of sigma, decided below from the statistics) come as six
        // tiles straight into LDS, whole row segments per instruction, and each wave picks its fragments out
        // of them; both wave groups hold the same rows and share the tiles.  Then the first key and value
        // tiles go out, into the same buffers, before anything else is computed.
        bool tiles_on_the_way = false;
        float m = ((gfptr_t)p.m)[(int64_t)h * S + min(myrow, S - 1)];
        float l = ((gfptr_t)p.l)[(int64_t)h * S + min(myrow, S - 1)];
        half8_t qf[KS], gf[KS], of[FAST ? KS : 1];
        if constexpr (DMA) {
            const int64_t off = hoff - shift + (int64_t)(i0 + g * kTileRows) * ld;
            const int left = S - (i0 + g * kTileRows);
            const bool want_o = FAST && p.o;
            tk.load(tm, gp(p.q) + off, left, smem + g * kTileB);
            tk.load(tm, gp(p.dO) + off, left, smem + (2 + g) * kTileB);
            if (want_o) tk.load(tm, gp(p.o) + off, left, smem + (4 + g) * kTileB);
            zero_pads(smem, 2 * kGroupLds / kRowB, (Dh + shift + 7) >> 3);
            tile_sync<DMA>();
            const unsigned char *mine = smem + (wid >> 1) * kTileB;
            const int trow = (wid & 1) * 32 + l32;
            frags_from_tile<KS>(qf, mine, trow, Dh, lh, shift);
            frags_from_tile<KS>(gf, mine + 2 * kTileB, trow, Dh, lh, shift);
            if constexpr (FAST) {
                if (want_o) frags_from_tile<KS>(of, mine + 4 * kTileB, trow, Dh, lh, shift);
            }
            __syncthreads();                      // every wave holds its fragments: the buffers are free again
            first_tiles();
            tiles_on_the_way = true;
        } else {
            load_frags<KS>(qf, gp(p.q) + hoff, ld, myrow, S, Dh, lh, shift);
            load_frags<KS>(gf, gp(p.dO) + hoff, ld, myrow, S, Dh, lh, shift);
            if constexpr (FAST) {
                if (p.o) load_frags<KS>(of, gp(p.o) + hoff, ld, myrow, S, Dh, lh, shift);
            }
        }
        float sig = 0.f;
        if (myrow >= S) {
            m = 0.f;
            l = 1.f;
        }
        const float y = recip_refined(l);
        const float cs = prob_shift(m, l);

        float16_t dacc[DT];
        auto run_pass = [&](auto pass_c) __attribute__((always_inline)) {
            constexpr int PASS = decltype(pass_c)::value;
            float part = 0.f;
            if (!tiles_on_the_way) first_tiles();
            tiles_on_the_way = false;
            tile_sync<DMA>();
            for (int it = 0; it < niter; it++) {
                const int jt = 2 * it + g, cur = it & 1;
                const bool nxt = jt + 2 < njt;
                if (nxt) {
                    tk.load(tm, K + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Ks + (cur ^ 1) * kTileB);
                    tv.load(tm, V + (int64_t)(jt + 2) * kTileRows * ld, S - (jt + 2) * kTileRows, Vs + (cur ^ 1) * kTileB);
                }
                if (jt < njt) {
#pragma unroll
                    for (int kt = 0; kt < 2; kt++) {
                        const int kb = jt * kTileRows + 32 * kt;
                        if (kb > r0 + 31) continue;
                        const float16_t sacc = prod_direct<KS>(Ks + cur * kTileB, 32 * kt, qf, l32, lh);
                        const float16_t pacc = prod_direct<KS>(Vs + cur * kTileB, 32 * kt, gf, l32, lh);
                        const bool full = kb + 31 <= r0;
                        float de[16];
                        if constexpr (FAST) {
                            // sigma and dS with the f16 value of dP read by the fused multiply-add
                            half_t dph[16];
                            round16(dph, pacc);
                            if (full) {
#pragma unroll
                                for (int e = 0; e < 16; e++) {
                                    const float pr_ = exp2_mix(f2h(scaled(p.alpha, sacc[e])), cs);
                                    const half_t dp = dph[e];
                                    if (PASS == 0) part = __builtin_fmaf((float)dp, pr_, part);
                                    else de[e] = __builtin_fmaf((float)dp, pr_, -(sig * pr_));
                                }
                            } else {
#pragma unroll
                                for (int e = 0; e < 16; e++) {
                                    const bool live = kb + 8 * (e >> 2) + 4 * lh + (e & 3) <= myrow;
                                    const float pr_ = exp2_mix(f2h(scaled(p.alpha, sacc[e])), cs);
                                    const half_t dp = dph[e];
                                    if (PASS == 0) part += live ? (float)dp * pr_ : 0.f;
                                    else de[e] = live ? __builtin_fmaf((float)dp, pr_, -(sig * pr_)) : 0.f;
                                }
                            }
                        } else if (full) {
#pragma unroll
                            for (int e = 0; e < 16; e++) {
                                const float pr_ = M::prob(rnd16(scaled(p.alpha, sacc[e])), m, l, y);
                                const float tt = pr_ * rnd16(pacc[e]);
                                if (PASS == 0) part += tt;
                                else de[e] = tt - sig * pr_;
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 16; e++) {
                                const bool live = kb + 8 * (e >> 2) + 4 * lh + (e & 3) <= myrow;
                                const float pr_ = M::prob(rnd16(scaled(p.alpha, sacc[e])), m, l, y);
                                const float tt = pr_ * rnd16(pacc[e]);
                                if (PASS == 0) part += live ? tt : 0.f;
                                else de[e] = live ? tt - sig * pr_ : 0.f;
                            }
                        }
                        if (PASS == 1) prod_tr<DT>(dacc, Ks + cur * kTileB, 32 * kt, pack8(de), pack8(de + 8), lane);
                    }
                }
                if (nxt) {
                    tk.store(tm, Ks + (cur ^ 1) * kTileB);
                    tv.store(tm, Vs + (cur ^ 1) * kTileB);
                }
                tile_sync<DMA>();
            }
            return part;
        };
        // sigma_i = sum_j P'_ij f32(dP16_ij).  In exact arithmetic that is sum_d dO_id O_id, which needs no pass
        // over the keys; in the reference's arithmetic the two differ by the f16 roundings of dP16, P16 and O,
        // about 2^-11 |dP| sqrt(sum_j P_ij^2).  Where a row's probability mass is spread that is below the
        // rounding of dS16 itself.  Where it sits on one key it is not: the reference has dP16 - sigma = 0
        // there exactly, and rows 0 and 1 of a sequence failed the element bound with the short form.  So a
        // workgroup takes the short form only if every one of its rows has sum_j exp(S16_ij - m_i) >= kSpread
        // (no probability above 1 / kSpread), else the pass over the keys; the exactly rounded build always
        // takes the pass.
        bool short_sigma = false;
        if constexpr (FAST) {
            if (p.o) short_sigma = __syncthreads_and(myrow >= S || l >= kSpread) != 0;
        }
        if (short_sigma) {
            float part = 0.f;
#pragma unroll
            for (int ks = 0; ks < (FAST ? KS : 1); ks++)
#pragma unroll
                for (int e = 0; e < 8; e++) part = __builtin_fmaf((float)gf[ks][e], (float)of[ks][e], part);
            sig = part + __shfl_xor(part, 32, 64);                     // the two lanes of a row
        } else {
            const float part = run_pass(std::integral_constant<int, 0>{});
            const float pg = part + __shfl_xor(part, 32, 64);         // the two lanes of a row, then the two groups
            if (lh == 0) xs[g * kBM + wid * 32 + l32] = pg;
            __syncthreads();
            sig = xs[wid * 32 + l32] + xs[kBM + wid * 32 + l32];
        }
        if (g == 0 && lh == 0 && myrow < S) {
            p.y[(int64_t)h * S + myrow] = FAST ? cs : y;          // what the dK / dV kernel wants per row
            p.sig[(int64_t)h * S + myrow] = sig;
        }
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) dacc[dt][r] = 0.f;
        run_pass(std::integral_constant<int, 1>{});
        merge_partials<DT>(dacc, smem + kGroupLds, g, tig);
        if (DMA && !p.acc_dq) {
            if (g == 0) stage_rows<DT>(smem, dacc, wid * 32 + l32, lh, p.alpha);
            __syncthreads();
            write_rows(smem, p.dq + (int64_t)i0 * ld + hoff - shift, ld, min(kBM, S - i0), Dh, shift, threadIdx.x, kNT2);
        } else if (g == 0 && myrow < S) {
            half_t *drow = p.dq + (int64_t)myrow * ld + hoff;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int d0 = 32 * dt + 8 * q + 4 * lh - shift;
                    if (d0 >= 0 && d0 < Dh)
                        store_row4(drow + d0, dacc[dt][4 * q], dacc[dt][4 * q + 1], dacc[dt][4 * q + 2],
                                   dacc[dt][4 * q + 3], p.alpha, p.acc_dq);
                }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dK, dV: keys fixed (128 per workgroup of 4 waves, a lane owns one), loop over the query tiles at or
// after them; the key tiles with the most queries first.

constexpr int kDkvBufs = 3;                      // tile buffers per tensor (Q, dO) and sets of row statistics

template <int KS, int DT, bool FAST, bool DMA>
__global__ void __launch_bounds__(kNT, 1) attn_bwd_dkv_kernel(AttnArgs p)
{
    // the whole argument block in scalar registers at once (read field by field where the control flow first
    // wants it, it costs several dependent round trips to memory before the first tile is requested)
    asm volatile("" ::"s"(p.S), "s"(p.H), "s"(p.Dh), "s"(p.ld), "s"(p.alpha), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.dO),
                 "s"(p.o), "s"(p.out), "s"(p.dq), "s"(p.dk), "s"(p.dv), "s"(p.m), "s"(p.l), "s"(p.y), "s"(p.sig),
                 "s"(p.acc_dq), "s"(p.acc_dk), "s"(p.acc_dv));
    typedef AttnMath<FAST> M;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Qs = smem, *Gs = smem + kDkvBufs * kTileB;
    float *St = reinterpret_cast<float *>(smem + 2 * kDkvBufs * kTileB);   // [3][4][64]: m, l, y, sigma of a tile's rows
    const int lane = threadIdx.x & 63, wid = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), l32 = lane & 31,
              lh = lane >> 5;
    const int S = p.S, Dh = p.Dh;
    const int64_t ld = p.ld;
    const int h = blockIdx.x % p.H, pr = blockIdx.x / p.H;
    const int64_t hoff = (int64_t)h * Dh;
    const int shift = DMA ? (int)(hoff & 7) : 0;                        // the head's first column in its window
    gptr_t Q = gp(p.q) + hoff - shift, G = gp(p.dO) + hoff - shift;
    // the pad columns of the tile buffers: zero from the first tile's barrier on (direct tiles: cleared below,
    // behind the first loads)
    if constexpr (!DMA) zero_lds(smem, 2 * kDkvBufs * kTileB);
    // the four per-row statistics of a 64-query tile: lane t of wave w fetches array w, row t
    gfptr_t stat_src = (gfptr_t)(wid == 0 ? p.m : wid == 1 ? p.l : wid == 2 ? p.y : p.sig) + (int64_t)h * S;
    const float stat_pad = (wid == 1 || wid == 2) ? 1.f : 0.f;

    {
        const int kt_ = pr;                                             // low key tiles see the most queries
        const int c00 = kt_ * kBM, c0 = c00 + wid * 32, mykey = c0 + l32;

        // the keys and values of the workgroup: with direct tiles they come as tiles straight into LDS, beside the
        // first query tile (below)
        half8_t kf[KS], vf[KS];
        if constexpr (!DMA) {
            load_frags<KS>(kf, gp(p.k) + hoff, ld, mykey, S, Dh, lh, shift);
            load_frags<KS>(vf, gp(p.v) + hoff, ld, mykey, S, Dh, lh, shift);
        }

        float16_t kacc[DT], vacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                kacc[dt][r] = 0.f;
                vacc[dt][r] = 0.f;
            }
        const int iq0 = c00 / kTileRows, niq = (S + kTileRows - 1) / kTileRows;
        typedef typename std::conditional<DMA, DmaTileMap, FastTileMap>::type Map;
        typedef typename std::conditional<DMA, DmaTileLoader, FastTileLoader>::type Loader;
        const Map tm(ld, Dh, shift);
        Loader tq, tg;
        float st;
        auto load_stat = [&](int iq) __attribute__((always_inline)) {
            const int row = iq * kTileRows + lane;
            const float t = stat_src[row < S ? row : S - 1];
            st = row < S ? t : stat_pad;          // rows beyond S are masked; the pad only has to be finite
        };
        auto buf_of = [&](int iq) __attribute__((always_inline)) { return (iq - iq0) % kDkvBufs; };
        auto fetch = [&](int iq) __attribute__((always_inline)) {        // tile iq on its way (registers or LDS)
            const int bf = buf_of(iq);
            tq.load(tm, Q + (int64_t)iq * kTileRows * ld, S - iq * kTileRows, Qs + bf * kTileB);
            tg.load(tm, G + (int64_t)iq * kTileRows * ld, S - iq * kTileRows, Gs + bf * kTileB);
            if constexpr (DMA) {
                // the statistics the same way (rows beyond S: the last row's, finite like the pad), so that no
                // register load stands between these loads and the point where the kernel waits for them
                const int row = min(iq * kTileRows + lane, S - 1);
                const uint32_t m0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(St + bf * 256 + wid * 64));
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                             :
                             : "s"(m0), "v"((uint32_t)row * 4u), "s"(stat_src)
                             : "memory");
            } else {
                load_stat(iq);
            }
        };
        auto land = [&](int iq) __attribute__((always_inline)) {         // ... into LDS, with its statistics
            const int bf = buf_of(iq);
            tq.store(tm, Qs + bf * kTileB);
            tg.store(tm, Gs + bf * kTileB);
            if constexpr (!DMA) St[bf * 256 + wid * 64 + lane] = st;
        };
        // one 32-query block of a tile, its three stages one after the other
        auto block = [&](int iq, int qb) __attribute__((always_inline)) {
            const int bf = buf_of(iq);
            const float *stc = St + bf * 256;
            const int qb0 = iq * kTileRows + 32 * qb;
            if (qb0 + 31 < c0 || qb0 >= S) return;        // every query of the block is before every key of the wave
            const float16_t sacc = prod_direct<KS, false>(Qs + bf * kTileB, 32 * qb, kf, l32, lh);
            const float16_t pacc = prod_direct<KS, false>(Gs + bf * kTileB, 32 * qb, vf, l32, lh);
            const bool full = qb0 >= c0 + 31 && qb0 + 32 <= S;
            float pe[16], de[16];
            half_t dph[16];
            if constexpr (FAST) round16(dph, pacc);
            auto elems = [&](auto full_c) __attribute__((always_inline)) {
                constexpr bool FULL = decltype(full_c)::value;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int qi = 32 * qb + 8 * q + 4 * lh;
                    float4_t mm, ll;
                    if constexpr (!FAST) {
                        mm = *reinterpret_cast<const float4_t *>(stc + 0 * 64 + qi);
                        ll = *reinterpret_cast<const float4_t *>(stc + 1 * 64 + qi);
                    }
                    const float4_t yy = *reinterpret_cast<const float4_t *>(stc + 2 * 64 + qi);
                    const float4_t sg = *reinterpret_cast<const float4_t *>(stc + 3 * 64 + qi);
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int e = 4 * q + r, query = iq * kTileRows + qi + r;
                        float pr_, ds;
                        if constexpr (FAST) {                 // yy holds the exponent offset of the row
                            pr_ = exp2_mix(f2h(scaled(p.alpha, sacc[e])), yy[r]);
                            ds = __builtin_fmaf((float)dph[e], pr_, -(sg[r] * pr_));
                        } else {
                            pr_ = M::prob(rnd16(scaled(p.alpha, sacc[e])), mm[r], ll[r], yy[r]);
                            const float tt = pr_ * rnd16(pacc[e]);
                            ds = tt - sg[r] * pr_;
                        }
                        const bool live = FULL || (query >= mykey && query < S);
                        pe[e] = live ? pr_ : 0.f;
                        de[e] = live ? ds : 0.f;
                    }
                }
            };
            if (full) elems(std::true_type{});           // no masks on blocks wholly past the diagonal
            else elems(std::false_type{});
            prod_tr<DT>(vacc, Gs + bf * kTileB, 32 * qb, pack8(pe), pack8(pe + 8), lane);
            prod_tr<DT>(kacc, Qs + bf * kTileB, 32 * qb, pack8(de), pack8(de + 8), lane);
        };
        // tiles [a, b), tile a in LDS and published
        auto run_tiles = [&](int a, int b) __attribute__((always_inline)) {
            for (int iq = a; iq < b; iq++) {
                if (iq + 1 < niq) fetch(iq + 1);
                block(iq, 0);
                block(iq, 1);
                if (iq + 1 < niq) land(iq + 1);
                tile_sync<DMA>();
            }
        };

        fetch(iq0);
        land(iq0);
        if constexpr (DMA) {
            // the 128 key and value rows into the second and third buffers, idle until the first tile is worked on
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int64_t off = hoff - shift + (int64_t)(c00 + t * kTileRows) * ld;
                tq.load(tm, gp(p.k) + off, S - (c00 + t * kTileRows), Qs + (1 + t) * kTileB);
                tg.load(tm, gp(p.v) + off, S - (c00 + t * kTileRows), Gs + (1 + t) * kTileB);
            }
            zero_pads(smem, 2 * kDkvBufs * kTileB / kRowB, (Dh + shift + 7) >> 3);
        }
        tile_sync<DMA>();
        if constexpr (DMA) {
            frags_from_tile<KS>(kf, Qs + (1 + (wid >> 1)) * kTileB, (wid & 1) * 32 + l32, Dh, lh, shift);
            frags_from_tile<KS>(vf, Gs + (1 + (wid >> 1)) * kTileB, (wid & 1) * 32 + l32, Dh, lh, shift);
            __syncthreads();                      // every wave holds its fragments: the buffers take query tiles now
        }
        // The tiles that hold the diagonal (two: 128 keys) and a ragged last tile run block by block.  The tiles
        // between them, whose 32-query blocks are whole and past the diagonal for every wave, run as a pipeline
        // (fast arithmetic, tiles loaded straight into LDS): while the vector unit forms P and dS of block b, the
        // matrix unit forms S and dP of block b + 1 and adds block b - 1 to dV and dK.  A wave has its SIMD to
        // itself here, so nothing else would fill the one unit while the other works.
        const int iqB = iq0 + 2, iqE = S / kTileRows;
        if (FAST && DMA && iqE > iqB) {
            run_tiles(iq0, iqB);
            if constexpr (FAST && DMA) {
                const int a4 = (lane >> 2) & 3, b4 = lane & 3, n16 = (lane >> 4) & 1;
                const int colb = 16 * n16 + 4 * b4;
                // blocks alternate between two register sets: SP = the S and dP accumulators (formed in one
                // step, consumed in the next), PD = the packed P and dS of a block (likewise)
                float16_t SPs[2], SPp[2];
                half8_t PD[2][4];                               // P rows 0..15, P rows 16..31, dS likewise
                half8_t xs[KS], xp[KS], xt[2][DT];
                float4_t yy, sg;
                // S1: the fragment reads of k step t of block (tile q1 / g1, qb1)
                auto x_read = [&](auto t_c, const unsigned char *q1, const unsigned char *g1, int qb1) __attribute__((always_inline)) {
                    constexpr int t = decltype(t_c)::value;
                    const int row = 32 * qb1 + l32, o = row * kRowB + (((2 * t + lh) ^ gsw(row)) << 4);
                    xs[t] = *reinterpret_cast<const half8_t *>(q1 + o);
                    xp[t] = *reinterpret_cast<const half8_t *>(g1 + o);
                };
                // S3: the 2 DT transposing reads of group g = 2 which + kk (which: 0 dV from the dO tile, 1 dK from
                // the Q tile; kk: rows 0..15 or 16..31 of the block), and MFMA j = g DT + dt
                auto t_read = [&](auto g_c, const unsigned char *q3, const unsigned char *g3, int qb3) __attribute__((always_inline)) {
                    constexpr int g = decltype(g_c)::value, which = g >> 1, kk = g & 1;
                    const unsigned char *tile = which ? q3 : g3;
                    const int r1 = 32 * qb3 + 16 * kk + 4 * lh + a4, r2 = r1 + 8;
                    const unsigned char *p1 = tile + r1 * kRowB + ((colb & 4) << 1);
                    const unsigned char *p2 = tile + r2 * kRowB + ((colb & 4) << 1);
                    const int g1_ = gsw(r1), g2_ = gsw(r2);
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const int c = (32 * dt + colb) >> 3;
                        xt[g & 1][dt] = as_h8(lds_read_tr(p1 + ((c ^ g1_) << 4)), lds_read_tr(p2 + ((c ^ g2_) << 4)));
                    }
                };
                constexpr int NQ = 32, NM = 2 * KS + 4 * DT;     // quarter pieces of S2 and MFMAs of a step
                // One step.  PAR: parity of the block in S2 (its qb).  S1 forms block (tile1, qb = PAR ^ 1) into
                // set PAR ^ 1, S2 turns set PAR into PD[PAR], S3 adds PD[PAR ^ 1] (block tile3, qb = PAR ^ 1).
                auto step = [&](auto par_c, auto has1_c, auto has3_c, int buf1, int buf2, int buf3) __attribute__((always_inline)) {
                    constexpr int PAR = decltype(par_c)::value, OTH = PAR ^ 1;
                    constexpr bool HAS1 = decltype(has1_c)::value, HAS3 = decltype(has3_c)::value;
                    const unsigned char *q1 = Qs + buf1 * kTileB, *g1 = Gs + buf1 * kTileB;
                    const unsigned char *q3 = Qs + buf3 * kTileB, *g3 = Gs + buf3 * kTileB;
                    const float *stc = St + buf2 * 256;
                    const float16_t &sC = SPs[PAR], &pC = SPp[PAR];
                    // S2 in 32 quarter pieces (8 pairs of elements x 4): the roundings S16 and dP16; the exponentials;
                    // dS; the packed results.  The same operations on the same values as the block-by-block form.
                    half2v_t s2, d2;
                    float pr2[2], ds2[2];
                    auto valu = [&](auto j_c) __attribute__((always_inline)) {
                        constexpr int j = decltype(j_c)::value, pc = j >> 2, qr = j & 3, q = pc >> 1, hf = pc & 1, e0 = 4 * q + 2 * hf;
                        if constexpr (qr == 0) {
                            if constexpr (hf == 0) {
                                const int qi = 32 * PAR + 8 * q + 4 * lh;
                                yy = *reinterpret_cast<const float4_t *>(stc + 2 * 64 + qi);
                                sg = *reinterpret_cast<const float4_t *>(stc + 3 * 64 + qi);
                            }
                            s2 = cvt_pk(scaled(p.alpha, sC[e0]), scaled(p.alpha, sC[e0 + 1]));
                            d2 = cvt_pk(pC[e0], pC[e0 + 1]);
                        } else if constexpr (qr == 1) {
                            pr2[0] = exp2_mix(s2[0], yy[2 * hf]);
                            pr2[1] = exp2_mix(s2[1], yy[2 * hf + 1]);
                        } else if constexpr (qr == 2) {
                            ds2[0] = __builtin_fmaf((float)d2[0], pr2[0], -(sg[2 * hf] * pr2[0]));
                            ds2[1] = __builtin_fmaf((float)d2[1], pr2[1], -(sg[2 * hf + 1] * pr2[1]));
                        } else {
                            half2v_t pn = cvt_pk(pr2[0], pr2[1]), dn = cvt_pk(ds2[0], ds2[1]);
                            // the values are used a step later; without a use here the compiler moves the whole piece there
                            asm volatile("" : "+v"(pn), "+v"(dn));
                            PD[PAR][e0 >> 3][e0 & 7] = pn[0];
                            PD[PAR][e0 >> 3][(e0 & 7) + 1] = pn[1];
                            PD[PAR][2 + (e0 >> 3)][e0 & 7] = dn[0];
                            PD[PAR][2 + (e0 >> 3)][(e0 & 7) + 1] = dn[1];
                        }
                    };
                    if constexpr (HAS1) {
                        x_read(std::integral_constant<int, 0>{}, q1, g1, OTH);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            SPs[OTH][r] = 0.f;
                            SPp[OTH][r] = 0.f;
                        }
                    }
                    if constexpr (HAS3) {
                        t_read(std::integral_constant<int, 0>{}, q3, g3, OTH);
                        t_read(std::integral_constant<int, 1>{}, q3, g3, OTH);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    // One MFMA, its share of the 32 quarter pieces, a scheduling barrier: the matrix unit takes 32
                    // cycles per MFMA and a second one issued behind it stalls the wave -- and with it the vector
                    // instructions behind that -- until the first is through.
                    auto slot_end = [&](auto m_c) __attribute__((always_inline)) {
                        constexpr int m = decltype(m_c)::value;
                        __builtin_amdgcn_sched_barrier(0);
                        static_for<m * NQ / NM, (m + 1) * NQ / NM>([&](auto j_c) __attribute__((always_inline)) { valu(j_c); });
                        __builtin_amdgcn_sched_barrier(0);
                    };
                    static_for<0, KS>([&](auto t_c) __attribute__((always_inline)) {
                        constexpr int t = decltype(t_c)::value;
                        constexpr int j0 = t * 4 * DT / KS, j1 = (t + 1) * 4 * DT / KS, m0 = 2 * t + j0;
                        if constexpr (HAS1) SPs[OTH] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xs[t], kf[t], SPs[OTH], 0, 0, 0);
                        slot_end(std::integral_constant<int, m0>{});
                        if constexpr (HAS1) {
                            SPp[OTH] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xp[t], vf[t], SPp[OTH], 0, 0, 0);
                            if constexpr (t + 1 < KS) x_read(std::integral_constant<int, t + 1>{}, q1, g1, OTH);
                        }
                        slot_end(std::integral_constant<int, m0 + 1>{});
                        static_for<j0, j1>([&](auto j_c) __attribute__((always_inline)) {
                            constexpr int j = decltype(j_c)::value, g = j / DT, dt = j % DT, which = g >> 1, kk = g & 1;
                            if constexpr (HAS3) {
                                const half8_t y = PD[OTH][2 * which + kk];
                                if constexpr (which)
                                    kacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xt[g & 1][dt], y, kacc[dt], 0, 0, 0);
                                else
                                    vacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xt[g & 1][dt], y, vacc[dt], 0, 0, 0);
                                // the reads of group g + 2 (two register sets, g & 1) once the last MFMA of group g is out
                                if constexpr (dt == DT - 1 && g + 2 < 4) t_read(std::integral_constant<int, g + 2>{}, q3, g3, OTH);
                            }
                            slot_end(std::integral_constant<int, 2 * t + 2 + j>{});
                        });
                    });
                };
                const std::integral_constant<int, 0> par0;
                const std::integral_constant<int, 1> par1;
                // the first and the last step stand outside the loop, so that the loop holds one form of each step
                // A tile is fetched two steps before its first use and waited for one step before it (the barrier
                // after every second step), so the latency of the loads has a whole step to pass.
                if (iqB + 1 < niq) fetch(iqB + 1);
                SPs[0] = prod_direct<KS, false>(Qs + buf_of(iqB) * kTileB, 0, kf, l32, lh);
                SPp[0] = prod_direct<KS, false>(Gs + buf_of(iqB) * kTileB, 0, vf, l32, lh);
                {
                    const int bc = buf_of(iqB);
                    step(par0, std::true_type{}, std::false_type{}, bc, bc, bc);       // S1 (iqB, 1), S2 (iqB, 0)
                    tile_sync<DMA>();
                }
                for (int iq = iqB; iq + 1 < iqE; iq++) {
                    const int bc = buf_of(iq), bn = buf_of(iq + 1);
                    // step (iq, 1): S1 (iq + 1, 0), S2 (iq, 1), S3 (iq, 0); tile iq + 2 takes the buffer of tile
                    // iq - 1, which the step before was the last to read
                    if (iq + 2 < niq) fetch(iq + 2);
                    step(par1, std::true_type{}, std::true_type{}, bn, bc, bc);
                    // step (iq + 1, 0): S1 (iq + 1, 1), S2 (iq + 1, 0), S3 (iq, 1)
                    step(par0, std::true_type{}, std::true_type{}, bn, bn, bc);
                    tile_sync<DMA>();
                }
                {
                    const int bc = buf_of(iqE - 1);
                    step(par1, std::false_type{}, std::true_type{}, bc, bc, bc);       // S2 (iqE - 1, 1), S3 (iqE - 1, 0)
                }
                prod_tr<DT>(vacc, Gs + buf_of(iqE - 1) * kTileB, 32, PD[1][0], PD[1][1], lane);
                prod_tr<DT>(kacc, Qs + buf_of(iqE - 1) * kTileB, 32, PD[1][2], PD[1][3], lane);
            }
            run_tiles(iqE, niq);
        } else {
            run_tiles(iq0, niq);
        }
        const bool staged_v = DMA && !p.acc_dv, staged_k = DMA && !p.acc_dk;
        if (staged_v || staged_k) {
            __syncthreads();                              // the last products have read their tiles
            if (staged_k) stage_rows<DT>(Qs, kacc, wid * 32 + l32, lh, p.alpha);
            if (staged_v) stage_rows<DT>(Gs, vacc, wid * 32 + l32, lh, 1.0f);
            __syncthreads();
            const int64_t off = (int64_t)c00 * ld + hoff - shift;
            if (staged_k) write_rows(Qs, p.dk + off, ld, min(kBM, S - c00), Dh, shift, threadIdx.x, kNT);
            if (staged_v) write_rows(Gs, p.dv + off, ld, min(kBM, S - c00), Dh, shift, threadIdx.x, kNT);
        }
        if (mykey < S && !(staged_v && staged_k)) {
            half_t *krow = p.dk + (int64_t)mykey * ld + hoff, *vrow = p.dv + (int64_t)mykey * ld + hoff;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int d0 = 32 * dt + 8 * q + 4 * lh - shift;
                    if (d0 >= 0 && d0 < Dh) {
                        if (!staged_v)
                            store_row4(vrow + d0, vacc[dt][4 * q], vacc[dt][4 * q + 1], vacc[dt][4 * q + 2],
                                       vacc[dt][4 * q + 3], 1.0f, p.acc_dv);
                        if (!staged_k)
                            store_row4(krow + d0, kacc[dt][4 * q], kacc[dt][4 * q + 1], kacc[dt][4 * q + 2],
                                       kacc[dt][4 * q + 3], p.alpha, p.acc_dk);
                    }
                }
        }
    }
}

constexpr size_t kDkvSmem = 2 * kDkvBufs * kTileB + kDkvBufs * 4 * 64 * sizeof(float);

template <class K>
int set_smem(K kern, size_t bytes)
{
    CACTI_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return 0;
}

// Which arithmetic the kernels are launched with (AttnMath).  Measured at 32 heads x 2048 x 100 on MI355X, in a
// hot loop with the register loaders: forward 93 us / adjoint 232 us with the fast form, 123 / 305 us with the exact one; the two
// differ by 3e-5 .. 4e-5 relative L2 in O, dQ, dK, dV, and O, dQ, dK, dV of the fast form agree with
// the CPU restatement of the reference to 4.9e-5 .. 7.1e-5.
std::atomic<int> g_exact{0};             // cacti_hip_attention_set_exact: launch the exactly rounded forms

template <int KS, int DT, bool FAST, bool DMA>
int launch_fwd(const AttnArgs &p, hipStream_t st)
{
    static DeviceOnce ready;
    if (!ready.fresh()) {
        int rc = set_smem(attn_fwd_kernel<KS, DT, FAST, DMA>, kQmSmem);
        if (rc) return rc;
        ready.mark();
    }
    const int nqt = (p.S + kBM - 1) / kBM;
    hipLaunchKernelGGL((attn_fwd_kernel<KS, DT, FAST, DMA>), dim3((unsigned)(nqt * p.H)), dim3(kNT2), kQmSmem, st, p);
    return launch_status("attention_fwd");
}

template <int KS, int DT, bool FAST, bool DMA>
int launch_bwd(const AttnArgs &p, hipStream_t st)
{
    static DeviceOnce ready;
    if (!ready.fresh()) {
        int rc = set_smem(attn_bwd_dq_kernel<KS, DT, FAST, DMA>, kQmSmem);
        if (rc) return rc;
        if ((rc = set_smem(attn_bwd_dkv_kernel<KS, DT, FAST, DMA>, kDkvSmem))) return rc;
        ready.mark();
    }
    const int nqt = (p.S + kBM - 1) / kBM;
    hipLaunchKernelGGL((attn_bwd_dq_kernel<KS, DT, FAST, DMA>), dim3((unsigned)(nqt * p.H)), dim3(kNT2), kQmSmem, st, p);
    int rc = launch_status("attention_bwd_dq");
    if (rc) return rc;
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<KS, DT, FAST, DMA>), dim3((unsigned)(nqt * p.H)), dim3(kNT), kDkvSmem, st, p);
    return launch_status("attention_bwd_dkv");
}

// Whether the tiles of these tensors can be loaded straight into LDS: 16-byte aligned tensors and rows, and
// every head's window (from the 16-byte boundary at or below its start, whole 16-byte chunks) inside its row.
// *span = the window positions a head can occupy (Dh + the largest shift).
bool direct_tiles(int64_t H, int64_t Dh, int64_t ld, std::initializer_list<const void *> tensors, int64_t *span)
{
    *span = Dh;
    if (ld % 8 != 0) return false;
    for (const void *t : tensors)
        if (!aligned(t, 16)) return false;
    int64_t most = 0;
    for (int64_t h = 0; h < H; h++) {
        const int64_t shift = (h * Dh) & 7, start = h * Dh - shift, chunks = (Dh + shift + 7) / 8;
        if (start + 8 * chunks > ld || 8 * chunks > kDP) return false;
        most = std::max(most, Dh + shift);
    }
    *span = most;
    return true;
}

// the instantiation by the window span (16 KS and 32 DT positions must cover it), the arithmetic and the loader
template <template <int, int, bool, bool> class L>
int dispatch(int64_t span, bool exact, bool dma, const AttnArgs &p, hipStream_t st)
{
    auto by_size = [&](auto fast_c, auto dma_c) {
        constexpr bool F = decltype(fast_c)::value, D = decltype(dma_c)::value;
        if (span <= 64) return L<4, 2, F, D>::run(p, st);
        if (span <= 112) return L<7, 4, F, D>::run(p, st);
        return L<8, 4, F, D>::run(p, st);
    };
    if (exact) return dma ? by_size(std::false_type{}, std::true_type{}) : by_size(std::false_type{}, std::false_type{});
    return dma ? by_size(std::true_type{}, std::true_type{}) : by_size(std::true_type{}, std::false_type{});
}
template <int KS, int DT, bool F, bool D> struct Fwd { static int run(const AttnArgs &p, hipStream_t st) { return launch_fwd<KS, DT, F, D>(p, st); } };
template <int KS, int DT, bool F, bool D> struct Bwd { static int run(const AttnArgs &p, hipStream_t st) { return launch_bwd<KS, DT, F, D>(p, st); } };

int check_shape(const char *who, int64_t S, int64_t H, int64_t Dh, int64_t ld)
{
    CACTI_REQUIRE(S > 0 && H > 0 && Dh > 0, CACTI_E_INVALID, "%s: empty shape", who);
    CACTI_REQUIRE(Dh % 4 == 0 && Dh <= kDP, CACTI_E_NOTIMPL, "%s: need Dh %% 4 == 0 and Dh <= %d (Dh=%lld)", who, kDP,
                  (long long)Dh);
    CACTI_REQUIRE(ld >= H * Dh && ld % 4 == 0, CACTI_E_INVALID, "%s: row stride %lld must be a multiple of 4 and >= H*Dh",
                  who, (long long)ld);
    CACTI_REQUIRE(S <= (1 << 24) && S * H < ((int64_t)1 << 31) / 2, CACTI_E_NOTIMPL, "%s: S = %lld is too large", who,
                  (long long)S);
    // the tile loaders keep (row within a tile) * ld + column as a 32-bit offset
    CACTI_REQUIRE(ld <= ((int64_t)1 << 26), CACTI_E_NOTIMPL, "%s: row stride %lld is beyond the 2^26 elements the "
                  "tile loaders address", who, (long long)ld);
    return 0;
}

}  // namespace

CACTI_API int cacti_hip_attention_set_exact(int on)
{
    g_exact.store(on ? 1 : 0, std::memory_order_relaxed);
    return 0;
}

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
    int64_t span;
    const bool dma = direct_tiles(H, Dh, ld, {q, k, v, o}, &span);
    return dispatch<Fwd>(span, g_exact.load(std::memory_order_relaxed) != 0, dma, p, st);
}

CACTI_API int cacti_hip_attention_bwd(int64_t S, int64_t H, int64_t Dh, float alpha, const void *q, const void *k,
                                      const void *v, const void *o, const void *dO, int64_t ld, const void *stats,
                                      void *dq, int dq_acc, void *dk, int dk_acc, void *dv, int dv_acc,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = check_shape("attention_bwd", S, H, Dh, ld);
    if (rc) return rc;
    CACTI_REQUIRE(q && k && v && dO && stats && dq && dk && dv && workspace, CACTI_E_INVALID,
                  "attention_bwd: null pointer");
    CACTI_REQUIRE(aligned(q, 8) && aligned(k, 8) && aligned(v, 8) && aligned(dO, 8) && aligned(o, 8) &&
                      aligned(dq, 8) && aligned(dk, 8) && aligned(dv, 8) && aligned(stats, 4) && aligned(workspace, 4),
                  CACTI_E_INVALID, "attention_bwd: tensors must be 8-byte aligned");
    CACTI_REQUIRE(workspace_bytes >= cacti_hip_attention_bwd_workspace(S, H), CACTI_E_INVALID,
                  "attention_bwd: workspace of %zu bytes is smaller than the %zu needed", workspace_bytes,
                  cacti_hip_attention_bwd_workspace(S, H));
    AttnArgs p = {};
    p.S = (int)S; p.H = (int)H; p.Dh = (int)Dh; p.ld = ld; p.alpha = alpha;
    p.q = (const half_t *)q; p.k = (const half_t *)k; p.v = (const half_t *)v;
    p.dO = (const half_t *)dO;
    p.o = (const half_t *)o;
    p.dq = (half_t *)dq; p.dk = (half_t *)dk; p.dv = (half_t *)dv;
    p.acc_dq = dq_acc; p.acc_dk = dk_acc; p.acc_dv = dv_acc;
    p.m = (float *)const_cast<void *>(stats);
    p.l = p.m + S * H;
    p.y = (float *)workspace;
    p.sig = p.y + S * H;
    hipStream_t st = (hipStream_t)stream;
    int64_t span;
    const bool dma = direct_tiles(H, Dh, ld, {q, k, v, dO, o, dq, dk, dv}, &span);     // o may be null: passes
    return dispatch<Bwd>(span, g_exact.load(std::memory_order_relaxed) != 0, dma, p, st);
}
