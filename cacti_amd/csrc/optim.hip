// Optimiser thunks of the reference's AdamW32 (src/librarium/adamw.rs:45-60), Initialize mode: the
// output cell is read and overwritten in place.
//   OnlineAverageScaleInitFutThunkSpec        src/thunk/op.rs:3884-3939   v += rate (s f32(u) - v)
//   OnlineAverageSquareScaleInitFutThunkSpec  src/thunk/op.rs:3941-4002   v += rate ((s f32(u))^2 - v)
//   OnlineAdamWUpdateInitFutThunkSpec         src/thunk/op.rs:4004-4062   w += slr (lru u / (sqrt v + eps) + lam w)
//   CastFutThunkSpec f32 -> f16 / f16 -> f32  src/thunk/op.rs:621-663     (set_lossy_cast / set_cast, src/op.rs:1085-1135)
// and the four of them over a whole list of tensors in one launch (what the example stages per
// minibatch, examples/open_llama_3b_train.rs:252-268): the fused pass reads 14 and writes 14 bytes
// per element instead of 24 + 18 over four launches per tensor, with the same f32 operations in the
// same order, so the results are bit-identical to the separate thunks.
//
// All kernels stream: a lane owns 4 consecutive elements per step (one 8-byte f16 access, one
// 16-byte access per f32 tensor), so every wave instruction covers one contiguous 512-byte or
// 1-KiB run; non-temporal both ways since nothing is read twice.
#include "common.h"
#include <vector>

using namespace cacti;

namespace {

constexpr int kThreads = 256;
constexpr int kUnits = 8;                       // 4-element units per lane
constexpr int kChunk = kThreads * kUnits;       // units per workgroup (8192 elements)

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum Mode : int { M_AVG = 0, M_AVGSQ = 1, M_UPDATE = 2, M_CAST_F32_F16 = 3, M_CAST_F16_F32 = 4, M_STEP = 5 };

// one tensor of a launch; which pointers are used depends on the mode:
//   M_AVG, M_AVGSQ: g (f16 in), a (f32 in/out)        M_UPDATE: a, b (f32 in), w (f32 in/out)
//   M_CAST_F32_F16: w (f32 in), p (f16 out)           M_CAST_F16_F32: g (f16 in), w (f32 out)
//   M_STEP: g (f16 in), a, b, w (f32 in/out), p (f16 out)
struct OptSeg {
    const uint16_t *g;
    float *a, *b, *w;
    uint16_t *p;
    int64_t n;
    int64_t first_block;
};

// {grad_unscale, a1, a2, signed_lr, lr_unbias, lamda, eps}; the single thunks use the slots of
// their own parameters
struct OptScalars {
    float s[7];
};

// every operation rounds to f32 on its own (the file is compiled without contraction), in the
// order the reference's lambdas are written
__device__ __forceinline__ float avg_step(float u, float v, float scale, float rate)
{
    const float su = scale * u;
    const float d = su - v;
    return v + rate * d;
}
__device__ __forceinline__ float avgsq_step(float u, float v, float scale, float rate)
{
    const float su = scale * u;
    const float sq = su * su;
    const float d = sq - v;
    return v + rate * d;
}
__device__ __forceinline__ float update_step(float u, float v, float w, float slr, float lru, float lam, float eps)
{
    // sqrtf and '/' are the correctly rounded ones here (the __fsqrt_rn intrinsic is the
    // approximate root in this toolchain)
    const float den = sqrtf(v) + eps;
    const float q = u / den;
    const float c = lru * q + lam * w;
    return w + slr * c;
}

__device__ __forceinline__ float h2f_bits(uint32_t bits)
{
    return __half2float(__ushort_as_half((unsigned short)bits));
}
__device__ __forceinline__ uint32_t f2h_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

struct Unit {
    float g[4], a[4], b[4], w[4];
};

template <int MODE>
__device__ __forceinline__ void compute(Unit &u, uint32_t (&p)[4], const OptScalars &sc, int cnt)
{
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (i >= cnt) break;
        if (MODE == M_AVG) u.a[i] = avg_step(u.g[i], u.a[i], sc.s[0], sc.s[1]);
        if (MODE == M_AVGSQ) u.a[i] = avgsq_step(u.g[i], u.a[i], sc.s[0], sc.s[2]);
        if (MODE == M_UPDATE) u.w[i] = update_step(u.a[i], u.b[i], u.w[i], sc.s[3], sc.s[4], sc.s[5], sc.s[6]);
        if (MODE == M_CAST_F32_F16) p[i] = f2h_bits(u.w[i]);
        if (MODE == M_CAST_F16_F32) u.w[i] = u.g[i];
        if (MODE == M_STEP) {
            u.a[i] = avg_step(u.g[i], u.a[i], sc.s[0], sc.s[1]);
            u.b[i] = avgsq_step(u.g[i], u.b[i], sc.s[0], sc.s[2]);
            u.w[i] = update_step(u.a[i], u.b[i], u.w[i], sc.s[3], sc.s[4], sc.s[5], sc.s[6]);
            p[i] = f2h_bits(u.w[i]);
        }
    }
}

template <int MODE>
struct Uses {
    static constexpr bool g_in = MODE == M_AVG || MODE == M_AVGSQ || MODE == M_CAST_F16_F32 || MODE == M_STEP;
    static constexpr bool a_in = MODE == M_AVG || MODE == M_AVGSQ || MODE == M_UPDATE || MODE == M_STEP;
    static constexpr bool b_in = MODE == M_UPDATE || MODE == M_STEP;
    static constexpr bool w_in = MODE == M_UPDATE || MODE == M_CAST_F32_F16 || MODE == M_STEP;
    static constexpr bool a_out = MODE == M_AVG || MODE == M_AVGSQ || MODE == M_STEP;
    static constexpr bool b_out = MODE == M_STEP;
    static constexpr bool w_out = MODE == M_UPDATE || MODE == M_CAST_F16_F32 || MODE == M_STEP;
    static constexpr bool p_out = MODE == M_CAST_F32_F16 || MODE == M_STEP;
};

__device__ __forceinline__ void load4(const float *src, float (&d)[4])
{
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src));
#pragma unroll
    for (int i = 0; i < 4; i++) d[i] = v[i];
}
__device__ __forceinline__ void store4(float *dst, const float (&d)[4])
{
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = d[i];
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(dst));
}

// segs == nullptr: the one tensor `one`; otherwise nseg tensors, segs[] sorted by first_block
template <int MODE>
__global__ void __launch_bounds__(kThreads)
optim_kernel(OptSeg one, const OptSeg *__restrict__ segs, int nseg, OptScalars sc)
{
    using U = Uses<MODE>;
    OptSeg sg = one;
    if (segs) {
        int lo = 0, hi = nseg - 1;                            // last segment starting at or before this block
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (segs[mid].first_block <= (int64_t)blockIdx.x) lo = mid;
            else hi = mid - 1;
        }
        sg = segs[lo];
    }
    const int64_t lb = (int64_t)blockIdx.x - sg.first_block;
    const int64_t n4 = sg.n / 4;
    const int64_t u0 = lb * kChunk;
    Unit un[kUnits];
    uint32_t pk[kUnits][4];
    // all loads of the lane first (kUnits x up to 4 loads in flight), then the arithmetic
#pragma unroll
    for (int j = 0; j < kUnits; j++) {
        const int64_t u = u0 + j * kThreads + threadIdx.x;
        if (u >= n4) break;
        if (U::g_in) {
            const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(sg.g) + u);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                un[j].g[2 * i] = h2f_bits(v[i] & 0xffff);
                un[j].g[2 * i + 1] = h2f_bits(v[i] >> 16);
            }
        }
        if (U::a_in) load4(sg.a + u * 4, un[j].a);
        if (U::b_in) load4(sg.b + u * 4, un[j].b);
        if (U::w_in) load4(sg.w + u * 4, un[j].w);
    }
#pragma unroll
    for (int j = 0; j < kUnits; j++) {
        const int64_t u = u0 + j * kThreads + threadIdx.x;
        if (u >= n4) break;
        compute<MODE>(un[j], pk[j], sc, 4);
        if (U::a_out) store4(sg.a + u * 4, un[j].a);
        if (U::b_out) store4(sg.b + u * 4, un[j].b);
        if (U::w_out) store4(sg.w + u * 4, un[j].w);
        if (U::p_out) {
            u32x2 v;
#pragma unroll
            for (int i = 0; i < 2; i++) v[i] = pk[j][2 * i] | (pk[j][2 * i + 1] << 16);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(sg.p) + u);
        }
    }
    // the last n % 4 elements: one lane each of the tensor's first workgroup
    const int rest = (int)(sg.n - n4 * 4);
    if (lb == 0 && (int)threadIdx.x < rest) {
        const int64_t e = n4 * 4 + threadIdx.x;
        Unit t;
        uint32_t p1[4];
        if (U::g_in) t.g[0] = h2f_bits(sg.g[e]);
        if (U::a_in) t.a[0] = sg.a[e];
        if (U::b_in) t.b[0] = sg.b[e];
        if (U::w_in) t.w[0] = sg.w[e];
        compute<MODE>(t, p1, sc, 1);
        if (U::a_out) sg.a[e] = t.a[0];
        if (U::b_out) sg.b[e] = t.b[0];
        if (U::w_out) sg.w[e] = t.w[0];
        if (U::p_out) sg.p[e] = (uint16_t)p1[0];
    }
}

inline int64_t seg_blocks(int64_t n)
{
    const int64_t b = (n / 4 + kChunk - 1) / kChunk;
    return b < 1 ? 1 : b;
}

template <int MODE>
int run_one(const char *what, const OptSeg &sg, const OptScalars &sc, hipStream_t st)
{
    if (sg.n > 0) {
        const int64_t blocks = seg_blocks(sg.n);
        CACTI_REQUIRE(blocks < (int64_t)1 << 31, CACTI_E_INVALID, "%s: tensor too large for one launch", what);
        hipLaunchKernelGGL((optim_kernel<MODE>), dim3((unsigned)blocks), dim3(kThreads), 0, st, sg,
                           (const OptSeg *)nullptr, 0, sc);
    }
    return launch_status(what);
}

}  // namespace

CACTI_API int cacti_hip_online_average_scale_f16_f32(int64_t n, const void *src_f16, void *dst_f32,
                                                     float src_scale, float rate, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((src_f16 && dst_f32) || n == 0), CACTI_E_INVALID,
                  "online_average_scale: null pointer or negative size");
    CACTI_REQUIRE(aligned(src_f16, 16) && aligned(dst_f32, 16), CACTI_E_INVALID,
                  "online_average_scale: operands must be 16-byte aligned");
    OptSeg sg = {(const uint16_t *)src_f16, (float *)dst_f32, nullptr, nullptr, nullptr, n, 0};
    OptScalars sc = {{src_scale, rate, 0, 0, 0, 0, 0}};
    return run_one<M_AVG>("online_average_scale", sg, sc, (hipStream_t)stream);
}

CACTI_API int cacti_hip_online_average_square_scale_f16_f32(int64_t n, const void *src_f16, void *dst_f32,
                                                            float src_scale, float rate, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((src_f16 && dst_f32) || n == 0), CACTI_E_INVALID,
                  "online_average_square_scale: null pointer or negative size");
    CACTI_REQUIRE(aligned(src_f16, 16) && aligned(dst_f32, 16), CACTI_E_INVALID,
                  "online_average_square_scale: operands must be 16-byte aligned");
    OptSeg sg = {(const uint16_t *)src_f16, (float *)dst_f32, nullptr, nullptr, nullptr, n, 0};
    OptScalars sc = {{src_scale, 0, rate, 0, 0, 0, 0}};
    return run_one<M_AVGSQ>("online_average_square_scale", sg, sc, (hipStream_t)stream);
}

CACTI_API int cacti_hip_online_adamw_update_f32(int64_t n, const void *grad1_avg_f32, const void *grad2_avg_f32,
                                                void *master_f32, float signed_lr, float lr_unbias, float lamda,
                                                float eps, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((grad1_avg_f32 && grad2_avg_f32 && master_f32) || n == 0), CACTI_E_INVALID,
                  "online_adamw_update: null pointer or negative size");
    CACTI_REQUIRE(aligned(grad1_avg_f32, 16) && aligned(grad2_avg_f32, 16) && aligned(master_f32, 16),
                  CACTI_E_INVALID, "online_adamw_update: operands must be 16-byte aligned");
    OptSeg sg = {nullptr, (float *)grad1_avg_f32, (float *)grad2_avg_f32, (float *)master_f32, nullptr, n, 0};
    OptScalars sc = {{0, 0, 0, signed_lr, lr_unbias, lamda, eps}};
    return run_one<M_UPDATE>("online_adamw_update", sg, sc, (hipStream_t)stream);
}

CACTI_API int cacti_hip_cast_f32_f16(int64_t n, const void *src_f32, void *dst_f16, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((src_f32 && dst_f16) || n == 0), CACTI_E_INVALID,
                  "cast_f32_f16: null pointer or negative size");
    CACTI_REQUIRE(aligned(src_f32, 16) && aligned(dst_f16, 16), CACTI_E_INVALID,
                  "cast_f32_f16: operands must be 16-byte aligned");
    OptSeg sg = {nullptr, nullptr, nullptr, (float *)src_f32, (uint16_t *)dst_f16, n, 0};
    return run_one<M_CAST_F32_F16>("cast_f32_f16", sg, OptScalars{}, (hipStream_t)stream);
}

CACTI_API int cacti_hip_cast_f16_f32(int64_t n, const void *src_f16, void *dst_f32, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((src_f16 && dst_f32) || n == 0), CACTI_E_INVALID,
                  "cast_f16_f32: null pointer or negative size");
    CACTI_REQUIRE(aligned(src_f16, 16) && aligned(dst_f32, 16), CACTI_E_INVALID,
                  "cast_f16_f32: operands must be 16-byte aligned");
    OptSeg sg = {(const uint16_t *)src_f16, nullptr, nullptr, (float *)dst_f32, nullptr, n, 0};
    return run_one<M_CAST_F16_F32>("cast_f16_f32", sg, OptScalars{}, (hipStream_t)stream);
}

// f32 integer power by square-and-multiply from the low bit, every product rounded to f32: what
// f32::powi computes in the reference's host code (src/op.rs:990, 999)
static float powi_f32(float a, int b)
{
    float r = 1.0f;
    for (;;) {
        if (b & 1) r *= a;
        b /= 2;
        if (b == 0) break;
        a *= a;
    }
    return r;
}

CACTI_API int cacti_adamw32_scalars(int iter_nr, float grad_scale, float lr, float wd, float a1, float a2,
                                    float eps, float *out7)
{
    CACTI_REQUIRE(out7, CACTI_E_INVALID, "adamw32_scalars: null output");
    CACTI_REQUIRE(iter_nr > 0, CACTI_E_INVALID, "adamw32: invalid iter_nr=%d (should be positive)", iter_nr);
    const float unbias1 = iter_nr == 1 ? a1 : 1.0f - powi_f32(1.0f - a1, iter_nr);
    const float unbias2 = iter_nr == 1 ? sqrtf(a2) : sqrtf(1.0f - powi_f32(1.0f - a2, iter_nr));
    out7[0] = grad_scale > 0.0f ? 1.0f / grad_scale : 1.0f;
    out7[1] = a1;
    out7[2] = a2;
    out7[3] = -lr;
    out7[4] = unbias2 / unbias1;
    out7[5] = wd;
    out7[6] = eps * unbias2;
    return 0;
}

CACTI_API size_t cacti_hip_adamw32_scratch_bytes(int count) { return count > 0 ? (size_t)count * sizeof(OptSeg) : 0; }

CACTI_API int cacti_hip_adamw32_step_f16_batch(int count, const void *const *grads_f16, void *const *avgs_f32,
                                               void *const *avg2s_f32, void *const *masters_f32,
                                               void *const *params_f16, const int64_t *ns, const float *scalars7,
                                               void *scratch, void *stream)
{
    CACTI_REQUIRE(count >= 0, CACTI_E_INVALID, "adamw32_step: negative count");
    if (count == 0) return 0;
    CACTI_REQUIRE(grads_f16 && avgs_f32 && avg2s_f32 && masters_f32 && params_f16 && ns && scalars7 && scratch &&
                      aligned(scratch, 8),
                  CACTI_E_INVALID, "adamw32_step: null or misaligned argument");
    std::vector<OptSeg> segs((size_t)count);
    int64_t blocks = 0;
    for (int i = 0; i < count; i++) {
        CACTI_REQUIRE(ns[i] >= 0, CACTI_E_INVALID, "adamw32_step: tensor %d has a negative size", i);
        CACTI_REQUIRE(ns[i] == 0 || (grads_f16[i] && avgs_f32[i] && avg2s_f32[i] && masters_f32[i] && params_f16[i]),
                      CACTI_E_INVALID, "adamw32_step: tensor %d has a null pointer", i);
        CACTI_REQUIRE(aligned(grads_f16[i], 16) && aligned(avgs_f32[i], 16) && aligned(avg2s_f32[i], 16) &&
                          aligned(masters_f32[i], 16) && aligned(params_f16[i], 16),
                      CACTI_E_INVALID, "adamw32_step: tensor %d is not 16-byte aligned", i);
        segs[i] = {(const uint16_t *)grads_f16[i], (float *)avgs_f32[i], (float *)avg2s_f32[i],
                   (float *)masters_f32[i], (uint16_t *)params_f16[i], ns[i], blocks};
        blocks += seg_blocks(ns[i]);
    }
    CACTI_REQUIRE(blocks < (int64_t)1 << 31, CACTI_E_INVALID, "adamw32_step: too many workgroups");
    hipStream_t st = (hipStream_t)stream;
    // pageable source: the copy has left the host vector when the call returns
    CACTI_HIP(hipMemcpyAsync(scratch, segs.data(), segs.size() * sizeof(OptSeg), hipMemcpyHostToDevice, st));
    OptScalars sc;
    for (int k = 0; k < 7; k++) sc.s[k] = scalars7[k];
    hipLaunchKernelGGL((optim_kernel<M_STEP>), dim3((unsigned)blocks), dim3(kThreads), 0, st, OptSeg{},
                       (const OptSeg *)scratch, count, sc);
    return launch_status("adamw32_step");
}
