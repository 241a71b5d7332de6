// Numerical-health digests over f16 tensors, integer-exact: the NaN count and the histogram of
// floor(log2 |x|) classes that the reference's training example takes of every parameter and
// gradient each cycle (NanCountFutThunkSpec, src/thunk/op.rs:273-349; AbsLog2Hist8FutThunkSpec,
// src/thunk/op.rs:351-441; used at examples/open_llama_3b_train.rs:409-424).
//
// Both stream the tensor once, 16 bytes per lane per step.  The histogram is kept in LDS
// (ds_add_u32).  An f16 tensor of weights or gradients falls into a dozen adjacent bins, so the
// 64 adds of a wave would pile up on a few addresses; every bin therefore has 16 counters, one
// per lane & 15 (16 different banks), which are summed at the end and flushed with one 64-bit
// atomic per non-empty bin and workgroup.  Counts are integers: the order of the adds does not
// matter.
#include "common.h"
#include <vector>

using namespace cacti;

namespace {

constexpr int kThreads = 256;
constexpr int kSub = 16;                   // counters per bin

// bin of one f16 bit pattern: 255 for inf / nan, 0 for +-0, floor(log2 |x|) + 127 otherwise
// (the reference: exponent field - 15 for normal numbers, -24 + floor(log2 mantissa) for
// subnormal ones, shifted by 0x7f into a u8; src/thunk/op.rs:417-432)
__device__ __forceinline__ int abs_log2_bin(uint32_t u)
{
    const uint32_t b = (u >> 10) & 0x1f, m = u & 0x3ff;
    if (b == 0x1f) return 255;
    if (b == 0) return m == 0 ? 0 : 103 + (31 - __builtin_clz(m));   // -24 + log2 m + 127
    return (int)b + 112;                                              // b - 15 + 127
}

__device__ __forceinline__ int is_nan16(uint32_t u) { return (u & 0x7c00) == 0x7c00 && (u & 0x3ff) != 0; }

__global__ void __launch_bounds__(64) zero_i64_kernel(unsigned long long *p, int n)
{
    for (int i = blockIdx.x * 64 + threadIdx.x; i < n; i += gridDim.x * 64) p[i] = 0;
}

// one tensor of a launch: workgroups first_block .. first_block + ceil(n / 8 / chunk) - 1 (at
// least one) read it; out[0..255] += histogram (HIST), out[HIST ? 256 : 0] += NaN count (NANS)
struct DigestSeg {
    const uint16_t *x;
    int64_t n;
    int64_t first_block;
    unsigned long long *out;
};
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kUnroll = 4;                 // 16-byte loads in flight per lane
constexpr int kSweep = kThreads * kUnroll; // 16-byte units a workgroup reads per step
constexpr int kChunk = 8 * kSweep;         // units per workgroup when many tensors share a launch (128 KiB)

inline int64_t seg_blocks(int64_t n, int chunk)
{
    const int64_t b = (n / 8 + chunk - 1) / chunk;
    return b < 1 ? 1 : b;
}

// one tensor alone: 1 to 8 sweeps per workgroup, growing once there are about 1536 workgroups
// (6 per CU; measured on a 205 MB tensor: 8 sweeps 61 us, 3 sweeps 73 us)
inline int chunk_for(int64_t n)
{
    const int64_t sweeps = (n / 8 + 1536 * (int64_t)kSweep - 1) / (1536 * (int64_t)kSweep);
    return (int)(sweeps < 1 ? 1 : sweeps > 8 ? 8 : sweeps) * kSweep;
}

template <bool HIST, bool NANS>
__device__ __forceinline__ void digest_unit(const u32x4 v, uint32_t *wh, uint32_t &nans)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = w[i] & 0xffff, hi = w[i] >> 16;
        if (HIST) {
            atomicAdd(&wh[abs_log2_bin(lo) * kSub], 1u);
            atomicAdd(&wh[abs_log2_bin(hi) * kSub], 1u);
        }
        if (NANS) nans += is_nan16(lo) + is_nan16(hi);
    }
}

// segs == nullptr: the one tensor `one`; otherwise nseg tensors, segs[] sorted by first_block
template <bool HIST, bool NANS>
__global__ void __launch_bounds__(kThreads)
digest_kernel(DigestSeg one, const DigestSeg *__restrict__ segs, int nseg, int chunk)
{
    __shared__ uint32_t hist[HIST ? 256 * kSub : 1];          // [bin][lane & 15]
    const int lane = threadIdx.x & 63;
    if (HIST) {
        for (int i = threadIdx.x; i < 256 * kSub; i += kThreads) hist[i] = 0;
    }
    DigestSeg sg = one;
    if (segs) {
        int lo = 0, hi = nseg - 1;                            // last segment starting at or before this block
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (segs[mid].first_block <= (int64_t)blockIdx.x) lo = mid;
            else hi = mid - 1;
        }
        sg = segs[lo];
    }
    if (HIST) __syncthreads();
    const int64_t lb = (int64_t)blockIdx.x - sg.first_block;
    uint32_t *wh = hist + (HIST ? (lane & (kSub - 1)) : 0);
    uint32_t nans = 0;
    const int64_t n8 = sg.n / 8;                                  // whole 16-byte units (x is 16-byte aligned)
    const int64_t u0 = lb * chunk, u1 = u0 + chunk < n8 ? u0 + chunk : n8;
    const u32x4 *xv = reinterpret_cast<const u32x4 *>(sg.x);
    int64_t u = u0 + threadIdx.x;
    for (; u + (kUnroll - 1) * kThreads < u1; u += kUnroll * kThreads) {
        u32x4 v[kUnroll];
#pragma unroll
        for (int j = 0; j < kUnroll; j++) v[j] = __builtin_nontemporal_load(xv + u + j * kThreads);
#pragma unroll
        for (int j = 0; j < kUnroll; j++) digest_unit<HIST, NANS>(v[j], wh, nans);
    }
    for (; u < u1; u += kThreads) digest_unit<HIST, NANS>(xv[u], wh, nans);
    // the last n % 8 elements: one lane each of the tensor's first workgroup
    if (lb == 0 && threadIdx.x < (int)(sg.n - n8 * 8)) {
        const uint32_t e = sg.x[n8 * 8 + threadIdx.x];
        if (HIST) atomicAdd(&wh[abs_log2_bin(e) * kSub], 1u);
        if (NANS) nans += is_nan16(e);
    }
    if (HIST) {
        __syncthreads();
        uint32_t s = 0;
#pragma unroll
        for (int w = 0; w < kSub; w++) s += hist[threadIdx.x * kSub + ((w + threadIdx.x) & (kSub - 1))];   // kThreads == 256 bins
        if (s) atomicAdd(&sg.out[threadIdx.x], (unsigned long long)s);
    }
    if (NANS) {
        // wave sum of the lane counts, then one atomic per wave
        for (int off = 32; off > 0; off >>= 1) nans += __shfl_down(nans, off, 64);
        if (lane == 0 && nans) atomicAdd(sg.out + (HIST ? 256 : 0), (unsigned long long)nans);
    }
}

template <bool HIST, bool NANS>
int run(int64_t n, const void *x, void *out, hipStream_t st)
{
    hipLaunchKernelGGL(zero_i64_kernel, dim3(1), dim3(64), 0, st, (unsigned long long *)out,
                       (HIST ? 256 : 0) + (NANS ? 1 : 0));
    if (n > 0) {
        const DigestSeg one = {(const uint16_t *)x, n, 0, (unsigned long long *)out};
        const int chunk = chunk_for(n);
        hipLaunchKernelGGL((digest_kernel<HIST, NANS>), dim3((unsigned)seg_blocks(n, chunk)), dim3(kThreads), 0,
                           st, one, (const DigestSeg *)nullptr, 0, chunk);
    }
    return launch_status(HIST ? "abs_log2_hist8" : "nan_count");
}

}  // namespace

namespace cacti {
size_t digest_batch_scratch_bytes(int count);
int digest_batch_f16(int count, const void *const *xs, const int64_t *ns, void *out, void *segs_dev,
                     hipStream_t st);
}  // namespace cacti

CACTI_API int cacti_hip_nan_count_f16(int64_t n, const void *x, void *count_i64, void *stream)
{
    CACTI_REQUIRE(n >= 0 && count_i64 && (x || n == 0), CACTI_E_INVALID, "nan_count: null pointer or negative size");
    CACTI_REQUIRE(aligned(x, 16) && aligned(count_i64, 8), CACTI_E_INVALID,
                  "nan_count: x must be 16-byte aligned, the count 8-byte aligned");
    return run<false, true>(n, x, count_i64, (hipStream_t)stream);
}

CACTI_API int cacti_hip_abs_log2_hist8_f16(int64_t n, const void *x, void *hist_i64_256, void *stream)
{
    CACTI_REQUIRE(n >= 0 && hist_i64_256 && (x || n == 0), CACTI_E_INVALID,
                  "abs_log2_hist8: null pointer or negative size");
    CACTI_REQUIRE(aligned(x, 16) && aligned(hist_i64_256, 8), CACTI_E_INVALID,
                  "abs_log2_hist8: x must be 16-byte aligned, the histogram 8-byte aligned");
    return run<true, false>(n, x, hist_i64_256, (hipStream_t)stream);
}

CACTI_API size_t cacti_hip_digests_scratch_bytes(int count)
{
    return count > 0 ? cacti::digest_batch_scratch_bytes(count) : 0;
}

CACTI_API int cacti_hip_digests_f16_batch(int count, const void *const *xs, const int64_t *ns, void *out_i64,
                                          void *scratch, void *stream)
{
    CACTI_REQUIRE(count >= 0, CACTI_E_INVALID, "digests_batch: negative count");
    if (count == 0) return 0;
    CACTI_REQUIRE(xs && ns && out_i64 && scratch && aligned(out_i64, 8) && aligned(scratch, 8), CACTI_E_INVALID,
                  "digests_batch: null or misaligned argument");
    return cacti::digest_batch_f16(count, xs, ns, out_i64, scratch, (hipStream_t)stream);
}

namespace cacti {

// Both digests of `count` tensors in ONE launch: out[257 * i + 0..255] = histogram and
// out[257 * i + 256] = NaN count of tensor i.  `segs_dev` is device scratch of
// digest_batch_scratch_bytes(count) bytes (8-byte aligned); xs[i] 16-byte aligned, ns[i] >= 0.
size_t digest_batch_scratch_bytes(int count) { return (size_t)count * sizeof(DigestSeg); }

int digest_batch_f16(int count, const void *const *xs, const int64_t *ns, void *out, void *segs_dev,
                     hipStream_t st)
{
    if (count <= 0) return 0;
    std::vector<DigestSeg> segs((size_t)count);
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        CACTI_REQUIRE(ns[i] >= 0 && (xs[i] || ns[i] == 0) && aligned(xs[i], 16), CACTI_E_INVALID,
                      "digest_batch: tensor %d: null, negative size or not 16-byte aligned", i);
        segs[i] = {(const uint16_t *)xs[i], ns[i], blocks, (unsigned long long *)out + (size_t)i * 257};
        blocks += seg_blocks(ns[i], kChunk);
    }
    CACTI_REQUIRE(blocks < (int64_t)1 << 31, CACTI_E_INVALID, "digest_batch: too many workgroups");
    // pageable source: the copy has left the host vector when the call returns
    CACTI_HIP(hipMemcpyAsync(segs_dev, segs.data(), segs.size() * sizeof(DigestSeg), hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(zero_i64_kernel, dim3(64), dim3(64), 0, st, (unsigned long long *)out, count * 257);
    hipLaunchKernelGGL((digest_kernel<true, true>), dim3((unsigned)blocks), dim3(kThreads), 0, st, DigestSeg{},
                       (const DigestSeg *)segs_dev, count, kChunk);
    return launch_status("digest_batch");
}

}  // namespace cacti
