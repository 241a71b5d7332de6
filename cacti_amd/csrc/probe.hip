// Measurement aid, not part of the path: what rate of MFMAs the device SUSTAINS, as a function of the
// operand values, the instruction shape and the fragment traffic from LDS.  A step of this library keeps
// the matrix pipes busy for tens of milliseconds, and over such a stretch the device is limited by
// power: the same instruction stream runs at 2400 TFLOP/s on zero operands and at 1600 - 1800 on random
// ones.  bench.py --workload mfma-power runs the variants below for a second or two each; their ratios
// are what the choice of v_mfma_f32_16x16x32_f16 for the large products rests on.
#include "common.h"

using namespace cacti;

namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

// 512 lanes per workgroup, one workgroup per CU.  Per iteration and wave: 8 products 32 x 32 x 16 or 16
// products 16 x 16 x 32 (the same flops) on fragments held in registers, READS of which (0, 4 or 6 of the 6
// a 128 x 64 wave patch needs per k step) are refreshed from LDS with ds_read_b128 each iteration.
template <int SHAPE, int READS>
__global__ void __launch_bounds__(512) mfma_probe_kernel(float *out, int64_t iters, uint32_t seed, int random_operands)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
    for (int i = threadIdx.x; i < 16384; i += 512) {
        uint32_t h = (i * 2654435761u) ^ seed;
        h ^= h >> 15;
        h *= 2246822519u;
        h ^= h >> 13;
        // two halves of random sign and mantissa with exponents 13 .. 15 (magnitudes 0.25 .. 2)
        const uint32_t a = (h & 0x8000u) | ((13u + ((h >> 10) & 3u) % 3u) << 10) | (h & 0x3ffu);
        const uint32_t b = ((h >> 16) & 0x8000u) | ((13u + ((h >> 26) & 3u) % 3u) << 10) | ((h >> 16) & 0x3ffu);
        reinterpret_cast<uint32_t *>(lds)[i] = random_operands ? (a | (b << 16)) : 0u;
    }
    __syncthreads();
    const half8_t *L = reinterpret_cast<const half8_t *>(lds);
    float16v acc[8];
    float4_t acc4[16];
#pragma unroll
    for (int n = 0; n < 8; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[n][r] = 0.f;
#pragma unroll
    for (int n = 0; n < 16; n++) acc4[n] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t af[2][4], bf[2][2];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        af[0][i] = L[(threadIdx.x + i * 512) & 4095];
        af[1][i] = L[(threadIdx.x + i * 512 + 77) & 4095];
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        bf[0][j] = L[(threadIdx.x + j * 512 + 256) & 4095];
        bf[1][j] = L[(threadIdx.x + j * 512 + 300) & 4095];
    }
    constexpr int NRA = READS >= 6 ? 4 : READS >= 4 ? 2 : 0, NRB = READS >= 4 ? 2 : 0;
    for (int64_t it = 0; it < iters; it += 2) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int i = 0; i < NRA; i++) af[h ^ 1][i] = L[(threadIdx.x + i * 512 + (int)(it + h) * 64) & 4095];
#pragma unroll
            for (int j = 0; j < NRB; j++) bf[h ^ 1][j] = L[(threadIdx.x + j * 512 + 256 + (int)(it + h) * 64) & 4095];
            if (SHAPE == 1) {
#pragma unroll
                for (int m = 0; m < 16; m++)
                    acc4[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[h][m & 1], af[h][(m >> 1) & 3], acc4[m], 0, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[h][j], af[h][i], acc[i * 2 + j], 0, 0, 0);
            }
        }
        if ((it & 127) == 126) {              // keep the sums in range
#pragma unroll
            for (int n = 0; n < 8; n++) acc[n] *= 0.0001f;
#pragma unroll
            for (int n = 0; n < 16; n++) acc4[n] *= 0.0001f;
        }
    }
    float f = 0.f;
#pragma unroll
    for (int n = 0; n < 8; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) f += acc[n][r];
#pragma unroll
    for (int n = 0; n < 16; n++)
#pragma unroll
        for (int r = 0; r < 4; r++) f += acc4[n][r];
    out[(int64_t)blockIdx.x * 512 + threadIdx.x] = f;
}

template <int SHAPE>
int launch(int reads, int blocks, float *out, int64_t iters, uint32_t seed, int random_operands, hipStream_t st)
{
    if (reads >= 6) hipLaunchKernelGGL((mfma_probe_kernel<SHAPE, 6>), dim3(blocks), dim3(512), 0, st, out, iters, seed, random_operands);
    else if (reads >= 4) hipLaunchKernelGGL((mfma_probe_kernel<SHAPE, 4>), dim3(blocks), dim3(512), 0, st, out, iters, seed, random_operands);
    else hipLaunchKernelGGL((mfma_probe_kernel<SHAPE, 0>), dim3(blocks), dim3(512), 0, st, out, iters, seed, random_operands);
    return launch_status("mfma_probe");
}

}  // namespace

// One launch of the probe: `blocks` workgroups of 8 waves, each wave `iters` (even) iterations of 262144 flops.
// shape 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_16x16x32_f16; lds_reads 0, 4 or 6 fragment reads per
// iteration; random_operands 0: all operands zero.  out: blocks * 512 floats of device memory.
CACTI_API int cacti_hip_mfma_probe(int shape, int lds_reads, int random_operands, int blocks, int64_t iters,
                                   unsigned seed, void *out, void *stream)
{
    CACTI_REQUIRE(out && blocks > 0 && iters > 0 && iters % 2 == 0 && (shape == 0 || shape == 1), CACTI_E_INVALID,
                  "mfma_probe: bad argument");
    hipStream_t st = (hipStream_t)stream;
    return shape == 1 ? launch<1>(lds_reads, blocks, (float *)out, iters, seed, random_operands, st)
                      : launch<0>(lds_reads, blocks, (float *)out, iters, seed, random_operands, st);
}
