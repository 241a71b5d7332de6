// bf16 <-> f16 / f32 conversions on raw u16 bit patterns, as the reference stages them when a
// checkpoint holds bf16 (set_lossy_cast, src/op.rs:1112-1135):
//   RawCastBf16F16FutThunkSpec  src/thunk/op.rs:665-698   f16.f32 (f32.from_bits (u32 u << 16))
//   RawCastBf16F32FutThunkSpec  src/thunk/op.rs:700-733   f32.from_bits (u32 u << 16)
//   RawCastF32Bf16FutThunkSpec  src/thunk/op.rs:735-768   u16 (f32.to_bits u >> 16)        (truncating)
//   RawCastF16Bf16FutThunkSpec  src/thunk/op.rs:770-803   u16 (f32.to_bits (f32.f16 u) >> 16)
// Streaming kernels: a lane owns 4 consecutive elements per access (8 bytes of a 16-bit tensor, 16
// bytes of an f32 one), every wave instruction covers one contiguous run; non-temporal both ways.
#include "common.h"

using namespace cacti;

namespace {

constexpr int kThreads = 256;
constexpr int kUnits = 8;                       // 4-element units per lane
constexpr int kChunk = kThreads * kUnits;       // units per workgroup

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum Mode : int { BF16_F16 = 0, BF16_F32 = 1, F32_BF16 = 2, F16_BF16 = 3 };

template <int MODE>
__device__ __forceinline__ uint32_t conv(uint32_t in)
{
    if (MODE == BF16_F16) return __half_as_ushort(__float2half_rn(__uint_as_float(in << 16)));
    if (MODE == BF16_F32) return in << 16;
    if (MODE == F32_BF16) return in >> 16;
    return __float_as_uint(__half2float(__ushort_as_half((unsigned short)in))) >> 16;   // F16_BF16
}

template <int MODE>
__global__ void __launch_bounds__(kThreads) rawcast_kernel(int64_t n, const void *__restrict__ src, void *__restrict__ dst)
{
    constexpr bool in32 = MODE == F32_BF16, out32 = MODE == BF16_F32;
    const int64_t n4 = n / 4;
    const int64_t u0 = (int64_t)blockIdx.x * kChunk;
    uint32_t v[kUnits][4];
#pragma unroll
    for (int j = 0; j < kUnits; j++) {
        const int64_t u = u0 + j * kThreads + threadIdx.x;
        if (u >= n4) break;
        if (in32) {
            const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + u);
#pragma unroll
            for (int i = 0; i < 4; i++) v[j][i] = __float_as_uint(x[i]);
        } else {
            const u32x2 x = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(src) + u);
            v[j][0] = x[0] & 0xffff;
            v[j][1] = x[0] >> 16;
            v[j][2] = x[1] & 0xffff;
            v[j][3] = x[1] >> 16;
        }
    }
#pragma unroll
    for (int j = 0; j < kUnits; j++) {
        const int64_t u = u0 + j * kThreads + threadIdx.x;
        if (u >= n4) break;
        uint32_t r[4];
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = conv<MODE>(v[j][i]);
        if (out32) {
            f32x4 y;
#pragma unroll
            for (int i = 0; i < 4; i++) y[i] = __uint_as_float(r[i]);
            __builtin_nontemporal_store(y, reinterpret_cast<f32x4 *>(dst) + u);
        } else {
            u32x2 y;
            y[0] = r[0] | (r[1] << 16);
            y[1] = r[2] | (r[3] << 16);
            __builtin_nontemporal_store(y, reinterpret_cast<u32x2 *>(dst) + u);
        }
    }
    // the last n % 4 elements: one lane each of the first workgroup
    if (blockIdx.x == 0 && (int64_t)threadIdx.x < n - n4 * 4) {
        const int64_t e = n4 * 4 + threadIdx.x;
        const uint32_t in = in32 ? reinterpret_cast<const uint32_t *>(src)[e] : reinterpret_cast<const uint16_t *>(src)[e];
        const uint32_t r = conv<MODE>(in);
        if (out32) reinterpret_cast<uint32_t *>(dst)[e] = r;
        else reinterpret_cast<uint16_t *>(dst)[e] = (uint16_t)r;
    }
}

template <int MODE>
int run(const char *what, int64_t n, const void *src, void *dst, void *stream)
{
    CACTI_REQUIRE(n >= 0 && ((src && dst) || n == 0), CACTI_E_INVALID, "%s: null pointer or negative size", what);
    CACTI_REQUIRE(aligned(src, 16) && aligned(dst, 16), CACTI_E_INVALID, "%s: operands must be 16-byte aligned", what);
    if (n > 0) {
        int64_t blocks = (n / 4 + kChunk - 1) / kChunk;
        if (blocks < 1) blocks = 1;
        CACTI_REQUIRE(blocks < (int64_t)1 << 31, CACTI_E_INVALID, "%s: tensor too large for one launch", what);
        hipLaunchKernelGGL((rawcast_kernel<MODE>), dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, n, src,
                           dst);
    }
    return launch_status(what);
}

}  // namespace

CACTI_API int cacti_hip_raw_cast_bf16_f16(int64_t n, const void *src_u16, void *dst_f16, void *stream)
{
    return run<BF16_F16>("raw_cast_bf16_f16", n, src_u16, dst_f16, stream);
}
CACTI_API int cacti_hip_raw_cast_bf16_f32(int64_t n, const void *src_u16, void *dst_f32, void *stream)
{
    return run<BF16_F32>("raw_cast_bf16_f32", n, src_u16, dst_f32, stream);
}
CACTI_API int cacti_hip_raw_cast_f32_bf16(int64_t n, const void *src_f32, void *dst_u16, void *stream)
{
    return run<F32_BF16>("raw_cast_f32_bf16", n, src_f32, dst_u16, stream);
}
CACTI_API int cacti_hip_raw_cast_f16_bf16(int64_t n, const void *src_f16, void *dst_u16, void *stream)
{
    return run<F16_BF16>("raw_cast_f16_bf16", n, src_f16, dst_u16, stream);
}
