// Shared device/host helpers for the gfx950 kernels of libcacti_gpu_hip_ffi.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/cacti_gpu_hip_ffi.h"

#define CACTI_API extern "C" __attribute__((visibility("default")))

namespace cacti {

// ---- status plumbing -------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_status(hipError_t e, const char *what);

#define CACTI_HIP(expr)                                        \
    do {                                                       \
        hipError_t e_ = (expr);                                \
        if (e_ != hipSuccess) return ::cacti::hip_status(e_, #expr); \
    } while (0)

#define CACTI_REQUIRE(cond, code, ...)          \
    do {                                        \
        if (!(cond)) {                          \
            ::cacti::set_error(__VA_ARGS__);    \
            return (code);                      \
        }                                       \
    } while (0)

// State a launcher establishes once per device and keeps (a kernel's dynamic-LDS attribute, the device
// address of a file-scope array) belongs to the device's loaded modules.  cacti_hip_primary_ctx_reset
// unloads them, so it advances an epoch, and every such cache is tagged with (device, epoch) and set up
// again when either differs.
unsigned module_epoch();
void module_epoch_advance();
// device contexts (cacti_ctx) alive on a device: a primary-context reset under one would free its pool,
// streams and events behind its back, so the reset entry point refuses while any exists
int live_contexts(int dev);
void live_contexts_add(int dev, int n);
struct DeviceOnce {
    int dev = -1;
    unsigned epoch = 0;
    bool fresh() const
    {
        int d = -2;
        return hipGetDevice(&d) == hipSuccess && d == dev && epoch == module_epoch();
    }
    void mark()
    {
        if (hipGetDevice(&dev) != hipSuccess) dev = -1;
        epoch = module_epoch();
    }
};

inline int launch_status(const char *what) { return hip_status(hipGetLastError(), what); }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---- f16 <-> f32 with IEEE round-to-nearest-even ----------------------------
typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float h2f(half_t h) { return (float)h; }
__device__ __forceinline__ half_t f2h(float f) { return (half_t)f; }   // v_cvt_f16_f32, RNE
// round an fp32 value to the nearest f16 and come back: one reference thunk boundary
__device__ __forceinline__ float rnd16(float f) { return (float)(half_t)f; }

// 16-byte vector of 8 halves moved as one global/LDS transaction
struct __attribute__((aligned(16))) h8 {
    half_t v[8];
};
__device__ __forceinline__ h8 ld8(const half_t *p) { return *reinterpret_cast<const h8 *>(p); }
__device__ __forceinline__ void st8(half_t *p, const h8 &x) { *reinterpret_cast<h8 *>(p) = x; }

// ---- 64-lane wavefront reductions ------------------------------------------
// Lanes exchange through DPP within a row of 16 (quad_perm, row_half_mirror,
// row_mirror), ds_swizzle across rows of a 32-lane half, and a bpermute across
// the two halves; every lane ends with the full result.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float swz_xor16(float v)
{
    // BITMODE swizzle: and_mask 0x1f, or_mask 0, xor_mask 0x10
    return __builtin_bit_cast(float,
                              __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401f));
}
__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

struct OpSum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct OpMax {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

template <class Op>
__device__ __forceinline__ float wave_reduce(float v, Op op)
{
    v = op(v, dpp_f32<0xB1>(v));    // quad_perm [1,0,3,2]  : lane ^ 1
    v = op(v, dpp_f32<0x4E>(v));    // quad_perm [2,3,0,1]  : lane ^ 2
    v = op(v, dpp_f32<0x141>(v));   // row_half_mirror      : other quad of the 8
    v = op(v, dpp_f32<0x140>(v));   // row_mirror           : other half of the 16
    v = op(v, swz_xor16(v));        // lane ^ 16
    v = op(v, xor32(v));            // lane ^ 32
    return v;
}
__device__ __forceinline__ float wave_sum(float v) { return wave_reduce(v, OpSum()); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce(v, OpMax()); }

// fp64 sum over the 64 lanes (two 32-bit exchanges per step); every lane ends with the result
__device__ __forceinline__ double wave_sum_f64(double v)
{
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// Block reduction through LDS: `red` holds one float per wave (<= 16 waves).
template <class Op>
__device__ __forceinline__ float block_reduce(float v, Op op, float ident, float *red)
{
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_reduce(v, op);
    __syncthreads();                // protect `red` against the previous use
    if (lane == 0) red[wid] = v;
    __syncthreads();
    float r = ident;
    for (int i = 0; i < nw; i++) r = op(r, red[i]);
    return r;
}

}  // namespace cacti
