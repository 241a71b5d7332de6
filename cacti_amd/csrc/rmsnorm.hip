// RMSNorm forward and adjoint, one 64-lane wavefront per row.
//
// A row (D halves) lives in registers as CH 16-byte chunks per lane, loaded once
// from HBM; the two row reductions (sum x^2, sum dt*x) are DPP wave reductions, so
// a row needs no barrier.  The adjoint keeps the reference's rounding schedule:
//   du = f32(dy); t = f32(x)/r; dw += f32(f16(du t)); dt = du f32(w);
//   c1 = f16(dt / r); dr = -sum(dt x)/r^2; ds = dr/(r+r); dsq = ds/D;
//   c2 = f16(dsq (x+x)); dx = f16(f16(dx_old + c1) + c2)   (or f16(c1 + c2))
// (rms_norm closure src/librarium/llama.rs:442-451 and its adjoint chain).
#include "common.h"
#include "softmax_math.h"

using namespace cacti;

namespace {

constexpr int kWaves = 8;                 // rows per block
constexpr int kThreads = kWaves * 64;

// x2 != nullptr: the row is first formed as x = f16(x + x2) (the residual add in front of the
// norm, one thunk boundary) and also written to `sum`
template <int CH>
__global__ void __launch_bounds__(kThreads)
rms_norm_fwd_kernel(int64_t N, int D, const half_t *__restrict__ x, const half_t *__restrict__ x2,
                    const half_t *__restrict__ w, float eps, half_t *__restrict__ sum,
                    half_t *__restrict__ y)
{
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * kWaves + wid;
    if (n >= N) return;
    const int nchunk = D / 8;
    const half_t *xr = x + n * D;
    // All loads of the row are issued first and unconditionally (chunks past the row re-read its
    // last chunk): a load inside `if (ch < nchunk)` is waited for at the end of that branch, which
    // makes the CH loads of a lane CH round trips.
    h8 xv[CH], bv[CH], wv[CH];
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int ch = min(c * 64 + lane, nchunk - 1);
        xv[c] = ld8(xr + ch * 8);
        if (x2) bv[c] = ld8(x2 + n * D + ch * 8);         // uniform over the launch
        wv[c] = ld8(w + ch * 8);
    }
    // the squares of f16 values are exact in fp32; summed in fp64 the row sum is the exactly rounded
    // one, whatever the order, so r is the reference's r and not one of its neighbours
    double ss = 0.0;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int ch = c * 64 + lane;
        if (ch < nchunk) {
            if (x2) {
#pragma unroll
                for (int i = 0; i < 8; i++) xv[c].v[i] = f2h(h2f(xv[c].v[i]) + h2f(bv[c].v[i]));
                st8(sum + n * D + ch * 8, xv[c]);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float f = h2f(xv[c].v[i]);
                ss += (double)(f * f);
            }
        }
    }
    ss = wave_sum_f64(ss);
    // t = x / r as the reference divides: a reciprocal and one residual correction give the
    // correctly rounded quotient (x * (1/r) alone is an ulp off for a quarter of the elements, and
    // in a chain of f16-rounded products that ulp grows like any other change of rounding)
    const RowDivide div(sqrtf((float)ss / (float)D + eps));
    half_t *yr = y + n * D;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int ch = c * 64 + lane;
        if (ch < nchunk) {
            h8 o;
#pragma unroll
            for (int i = 0; i < 8; i++) o.v[i] = f2h(h2f(wv[c].v[i]) * div(h2f(xv[c].v[i])));
            st8(yr + ch * 8, o);
        }
    }
}

template <int CH>
__global__ void __launch_bounds__(kThreads)
rms_norm_bwd_kernel(int64_t N, int D, const half_t *__restrict__ x, const half_t *__restrict__ w,
                    float eps, const half_t *__restrict__ dy, half_t *dx, int dx_acc,
                    float *__restrict__ dw_part, int wide_lds)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *sdw = reinterpret_cast<float *>(smem_raw);     // [kWaves][D] (wide_lds) or [D]
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * kWaves + wid;
    const int nchunk = D / 8;
    const bool live = n < N;

    float dwp[CH][8];
#pragma unroll
    for (int c = 0; c < CH; c++)
#pragma unroll
        for (int i = 0; i < 8; i++) dwp[c][i] = 0.f;

    if (live) {
        const half_t *xr = x + n * D, *gr = dy + n * D;
        // every load of the row up front and unconditional (see the forward kernel)
        half_t *or_ = dx + n * D;
        // without accumulation the fourth stream re-reads dy (a cache hit) instead of dx
        const half_t *oldr = dx_acc ? or_ : gr;
        h8 xv[CH], gv[CH], wv[CH], old[CH];
        double ss = 0.0;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = min(c * 64 + lane, nchunk - 1);
            xv[c] = ld8(xr + ch * 8);
            gv[c] = ld8(gr + ch * 8);
            wv[c] = ld8(w + ch * 8);
            old[c] = ld8(oldr + ch * 8);                      // used only when dx accumulates
        }
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * 64 + lane;
            if (ch < nchunk) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float f = h2f(xv[c].v[i]);
                    ss += (double)(f * f);
                }
            }
        }
        ss = wave_sum_f64(ss);                    // as in the forward kernel: the same r, bit for bit
        const float r = sqrtf((float)ss / (float)D + eps);
        const RowDivide div(r), div2(r * r);      // correctly rounded x / r, dt / r and (dt x) / r^2
        double sdx = 0.0;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * 64 + lane;
            if (ch < nchunk) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float xf = h2f(xv[c].v[i]), du = h2f(gv[c].v[i]);
                    float t = div(xf);
                    dwp[c][i] = rnd16(du * t);
                    float dt = du * h2f(wv[c].v[i]);
                    sdx += (double)div2(dt * xf);       // the reference's per-element term of dr
                    gv[c].v[i] = f2h(div(dt));          // c1, kept in place of dy
                    // dt is needed no further: c2 depends only on the row sum
                }
            }
        }
        sdx = wave_sum_f64(sdx);
        const float dr = -(float)sdx;
        const float ds = dr / (r + r);
        const float dsq = ds / (float)D;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * 64 + lane;
            if (ch < nchunk) {
                h8 o;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float xf = h2f(xv[c].v[i]);
                    float c1 = h2f(gv[c].v[i]);
                    float c2 = rnd16(dsq * (xf + xf));
                    float base = dx_acc ? rnd16(h2f(old[c].v[i]) + c1) : c1;
                    o.v[i] = f2h(base + c2);
                }
                st8(or_ + ch * 8, o);
            }
        }
    }

    // block partial of dw (rows summed in wave order either way, so the result does not
    // depend on the LDS mode): with room for one [D] row per wave every wave stores its row
    // at once and the columns are summed after a single barrier ...
    if (wide_lds) {
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int ch = c * 64 + lane;
            if (ch < nchunk) {
                // 16-byte LDS accesses throughout (D % 8 == 0, so every row of sdw starts on 32 bytes):
                // 2 stores per chunk here and 8 loads per 4 columns below, instead of 8 and 32
                float4_t *d4 = reinterpret_cast<float4_t *>(sdw + wid * D + ch * 8);
                d4[0] = float4_t{dwp[c][0], dwp[c][1], dwp[c][2], dwp[c][3]};
                d4[1] = float4_t{dwp[c][4], dwp[c][5], dwp[c][6], dwp[c][7]};
            }
        }
        __syncthreads();
        float *dst = dw_part + (int64_t)blockIdx.x * D;
        for (int i = threadIdx.x * 4; i < D; i += blockDim.x * 4) {
            float4_t a = *reinterpret_cast<const float4_t *>(sdw + i);
#pragma unroll
            for (int wv = 1; wv < kWaves; wv++) a += *reinterpret_cast<const float4_t *>(sdw + wv * D + i);
            *reinterpret_cast<float4_t *>(dst + i) = a;
        }
        return;
    }
    // ... otherwise the waves add their rows into one LDS row one after another
    for (int wv = 0; wv < kWaves; wv++) {
        if (wid == wv) {
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int ch = c * 64 + lane;
                if (ch < nchunk) {
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        if (wv == 0) sdw[ch * 8 + i] = dwp[c][i];
                        else sdw[ch * 8 + i] += dwp[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    float *dst = dw_part + (int64_t)blockIdx.x * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) dst[i] = sdw[i];
}

// dw[d] (+)= f16(sum over block partials): a block owns 32 columns (8 lanes x float4) and
// splits the partial rows over 32 slices, so D / 32 blocks share the read of the partials
constexpr int kFinCols = 32, kFinSlices = 32;
__global__ void __launch_bounds__(kFinCols / 4 * kFinSlices)
rms_norm_dw_finalize_kernel(int G, int D, const float *__restrict__ part, half_t *dw, int acc)
{
    __shared__ float red[kFinSlices][kFinCols];
    const int cg = threadIdx.x & (kFinCols / 4 - 1), slice = threadIdx.x / (kFinCols / 4);
    const int col = blockIdx.x * kFinCols + cg * 4;            // D % 8 == 0: a float4 is whole
    float4_t a = {0.f, 0.f, 0.f, 0.f};
    if (col < D)
        for (int g = slice; g < G; g += kFinSlices)
            a += *reinterpret_cast<const float4_t *>(part + (int64_t)g * D + col);
#pragma unroll
    for (int i = 0; i < 4; i++) red[slice][cg * 4 + i] = a[i];
    __syncthreads();
    const int c = blockIdx.x * kFinCols + threadIdx.x;
    if (threadIdx.x < kFinCols && c < D) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kFinSlices; i++) s += red[i][threadIdx.x];
        dw[c] = acc ? f2h(h2f(dw[c]) + rnd16(s)) : f2h(s);
    }
}

inline int ch_for(int64_t D) { return (int)((D / 8 + 63) / 64); }

template <int CH>
void launch_fwd(int64_t N, int D, const half_t *x, const half_t *x2, const half_t *w, float eps,
                half_t *sum, half_t *y, hipStream_t st)
{
    hipLaunchKernelGGL(rms_norm_fwd_kernel<CH>, dim3((unsigned)((N + kWaves - 1) / kWaves)),
                       dim3(kThreads), 0, st, N, D, x, x2, w, eps, sum, y);
}
template <int CH>
void launch_bwd(int64_t N, int D, const half_t *x, const half_t *w, float eps, const half_t *dy,
                half_t *dx, int dx_acc, float *part, hipStream_t st)
{
    const size_t wide = (size_t)kWaves * D * 4;
    const int wide_lds = wide <= 144 * 1024;
    const size_t smem = wide_lds ? wide : (size_t)D * 4;
    auto kern = rms_norm_bwd_kernel<CH>;
    static DeviceOnce attr_set;                   // one per instantiation
    if (!attr_set.fresh()) {
        (void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  144 * 1024);
        attr_set.mark();
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)((N + kWaves - 1) / kWaves)), dim3(kThreads), smem, st,
                       N, D, x, w, eps, dy, dx, dx_acc, part, wide_lds);
}

}  // namespace

#define CACTI_DISPATCH_CH(ch, CALL)                 \
    switch (ch) {                                   \
        case 1: { constexpr int CH = 1; CALL; } break;   \
        case 2: { constexpr int CH = 2; CALL; } break;   \
        case 3: case 4: { constexpr int CH = 4; CALL; } break;   \
        case 5: case 6: case 7: { constexpr int CH = 7; CALL; } break;   \
        case 8: { constexpr int CH = 8; CALL; } break;   \
        case 9: case 10: case 11: case 12: { constexpr int CH = 12; CALL; } break; \
        default: { constexpr int CH = 16; CALL; } break; \
    }

CACTI_API int cacti_hip_rms_norm_fwd(int64_t N, int64_t D, const void *x, const void *w, float eps,
                                     void *y, void *stream)
{
    CACTI_REQUIRE(N > 0 && D > 0 && x && w && y, CACTI_E_INVALID,
                  "rms_norm_fwd: null pointer or empty shape");
    CACTI_REQUIRE(D % 8 == 0 && D <= 8192, CACTI_E_NOTIMPL,
                  "rms_norm_fwd: need D %% 8 == 0 and D <= 8192 (D=%lld)", (long long)D);
    CACTI_REQUIRE(aligned(x, 16) && aligned(w, 16) && aligned(y, 16), CACTI_E_INVALID,
                  "rms_norm_fwd: tensors must be 16-byte aligned");
    CACTI_DISPATCH_CH(ch_for(D), launch_fwd<CH>(N, (int)D, (const half_t *)x, nullptr, (const half_t *)w,
                                                eps, nullptr, (half_t *)y, (hipStream_t)stream));
    return launch_status("rms_norm_fwd");
}

CACTI_API int cacti_hip_add_rms_norm_fwd(int64_t N, int64_t D, const void *a, const void *b, const void *w,
                                         float eps, void *sum, void *y, void *stream)
{
    CACTI_REQUIRE(N > 0 && D > 0 && a && b && w && sum && y, CACTI_E_INVALID,
                  "add_rms_norm_fwd: null pointer or empty shape");
    CACTI_REQUIRE(D % 8 == 0 && D <= 8192, CACTI_E_NOTIMPL,
                  "add_rms_norm_fwd: need D %% 8 == 0 and D <= 8192 (D=%lld)", (long long)D);
    CACTI_REQUIRE(aligned(a, 16) && aligned(b, 16) && aligned(w, 16) && aligned(sum, 16) && aligned(y, 16),
                  CACTI_E_INVALID, "add_rms_norm_fwd: tensors must be 16-byte aligned");
    CACTI_DISPATCH_CH(ch_for(D), launch_fwd<CH>(N, (int)D, (const half_t *)a, (const half_t *)b,
                                                (const half_t *)w, eps, (half_t *)sum, (half_t *)y,
                                                (hipStream_t)stream));
    return launch_status("add_rms_norm_fwd");
}

CACTI_API size_t cacti_hip_rms_norm_bwd_workspace(int64_t N, int64_t D)
{
    if (N <= 0 || D <= 0) return 0;
    return (size_t)((N + kWaves - 1) / kWaves) * (size_t)D * sizeof(float);
}

CACTI_API int cacti_hip_rms_norm_bwd(int64_t N, int64_t D, const void *x, const void *w, float eps,
                                     const void *dy, void *dx, int dx_acc, void *dw, int dw_acc,
                                     void *workspace, size_t workspace_bytes, void *stream)
{
    CACTI_REQUIRE(N > 0 && D > 0 && x && w && dy && dx && dw && workspace, CACTI_E_INVALID,
                  "rms_norm_bwd: null pointer or empty shape");
    CACTI_REQUIRE(D % 8 == 0 && D <= 8192, CACTI_E_NOTIMPL,
                  "rms_norm_bwd: need D %% 8 == 0 and D <= 8192 (D=%lld)", (long long)D);
    CACTI_REQUIRE(aligned(x, 16) && aligned(w, 16) && aligned(dy, 16) && aligned(dx, 16) &&
                      aligned(workspace, 16),
                  CACTI_E_INVALID, "rms_norm_bwd: tensors must be 16-byte aligned");
    CACTI_REQUIRE(workspace_bytes >= cacti_hip_rms_norm_bwd_workspace(N, D), CACTI_E_INVALID,
                  "rms_norm_bwd: workspace of %zu bytes is smaller than the %zu needed",
                  workspace_bytes, cacti_hip_rms_norm_bwd_workspace(N, D));
    hipStream_t st = (hipStream_t)stream;
    CACTI_DISPATCH_CH(ch_for(D),
                      launch_bwd<CH>(N, (int)D, (const half_t *)x, (const half_t *)w, eps,
                                     (const half_t *)dy, (half_t *)dx, dx_acc, (float *)workspace,
                                     st));
    int rc = launch_status("rms_norm_bwd");
    if (rc) return rc;
    const int G = (int)((N + kWaves - 1) / kWaves);
    hipLaunchKernelGGL(rms_norm_dw_finalize_kernel, dim3((unsigned)((D + kFinCols - 1) / kFinCols)),
                       dim3(kFinCols / 4 * kFinSlices), 0, st, G, (int)D, (const float *)workspace,
                       (half_t *)dw, dw_acc);
    return launch_status("rms_norm_dw_finalize");
}

// ---- the same adjoint for callers that cannot allocate ----------------------------------------
// The fp32 dw partial rows go to a file-scope device array instead of a caller workspace.  The
// array's name is only a host-side stand-in: its device address is looked up once per device and
// that pointer, never the name, is what reaches the kernels.
namespace {
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];          // per device, nullptr until first use on that device
unsigned g_scratch_epoch[kMaxDevices];     // the module epoch each address was taken in
}  // namespace

CACTI_API size_t cacti_hip_rms_norm_bwd_static_max_bytes(void) { return kStaticScratchBytes; }

CACTI_API int cacti_hip_rms_norm_bwd_static(int64_t N, int64_t D, const void *x, const void *w, float eps,
                                            const void *dy, void *dx, int dx_acc, void *dw, int dw_acc,
                                            void *stream)
{
    const size_t need = cacti_hip_rms_norm_bwd_workspace(N, D);
    CACTI_REQUIRE(N > 0 && D > 0 && need <= kStaticScratchBytes, CACTI_E_INVALID,
                  "rms_norm_bwd_static: N=%lld, D=%lld needs %zu bytes of scratch, the built-in buffer "
                  "holds %zu; use cacti_hip_rms_norm_bwd with a workspace",
                  (long long)N, (long long)D, need, kStaticScratchBytes);
    int dev = -1;
    CACTI_HIP(hipGetDevice(&dev));
    CACTI_REQUIRE(dev >= 0 && dev < kMaxDevices, CACTI_E_NOTIMPL,
                  "rms_norm_bwd_static: device %d is beyond the %d this entry point keeps a buffer for",
                  dev, kMaxDevices);
    if (!g_scratch_ptr[dev] || g_scratch_epoch[dev] != module_epoch()) {   // first use, or the modules were reloaded
        void *p = nullptr;
        CACTI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        CACTI_REQUIRE(p != nullptr, CACTI_E_STATE, "rms_norm_bwd_static: no device address for the scratch array");
        g_scratch_ptr[dev] = p;
        g_scratch_epoch[dev] = module_epoch();
    }
    return cacti_hip_rms_norm_bwd(N, D, x, w, eps, dy, dx, dx_acc, dw, dw_acc, g_scratch_ptr[dev],
                                  kStaticScratchBytes, stream);
}
