// Measurement aid: a pure stream of bf16 MFMA instructions, used to find the rate the chip
// sustains under its power limit (the published peak assumes the full clock, which real
// operand data does not hold).  Not on any product path.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ksa_api_internal.h"

namespace {

typedef float probe_f16 __attribute__((ext_vector_type(16)));
typedef __bf16 probe_b8 __attribute__((ext_vector_type(8)));

__device__ inline uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

// 16 MFMA 32x32x16 per iteration and wave, four independent accumulator chains, operands taken
// from four register sets in rotation (random values in (-0.1, 0.1), or zeros).
__global__ __launch_bounds__(512) void ksa_mfma_stream_kernel(float* out, int iters, int zero) {
    probe_b8 a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t h = probe_hash(threadIdx.x * 64 + j * 8 + i + blockIdx.x * 77777);
            const float fa = ((h & 0xffff) / 65536.f - 0.5f) * 0.2f;
            const float fb = ((h >> 16) / 65536.f - 0.5f) * 0.2f;
            a[j][i] = (__bf16)(zero ? 0.f : fa);
            b[j][i] = (__bf16)(zero ? 0.f : fb);
        }
    probe_f16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b[(r + 1) & 3], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(r + 1) & 3], b[r], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(r + 2) & 3], b[(r + 3) & 3], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(r + 3) & 3], b[(r + 2) & 3], acc[3], 0, 0, 0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[c][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace

extern "C" int ksa_probe_mfma_stream(void* out, int blocks, int waves_per_block, int iters,
                                     int zero_operands, double* flop, void* stream) {
    if (!out || blocks <= 0 || waves_per_block <= 0 || waves_per_block > 8 || iters <= 0)
        return KSA_ERR_INVALID;
    hipLaunchKernelGGL(ksa_mfma_stream_kernel, dim3(blocks), dim3(waves_per_block * 64), 0,
                       (hipStream_t)stream, (float*)out, iters, zero_operands);
    if (flop) *flop = (double)blocks * waves_per_block * iters * 16.0 * (2.0 * 32 * 32 * 16);
    return hipGetLastError() == hipSuccess ? KSA_OK : KSA_ERR_LAUNCH;
}
