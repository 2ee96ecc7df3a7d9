// Measurement aid: what the i8 matrix pipe of this GPU sustains on a loop of nothing but MFMAs,
// with operands that are all zero and with random operands, and the shader clock it runs at while
// doing so.  The nominal peak (5.0 POP/s dense int8) assumes the boost clock; under the power limit
// the clock a kernel actually gets depends on how much its data toggles, so the rate measured here
// with random operands is the practical ceiling for a GEMM on real data.
#include "ti8_common.h"

namespace ti8 {

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

// 8 waves per workgroup (2 per SIMD), each with a 2 x 2 grid of 32 x 32 accumulators: 16 MFMAs
// per iteration and wave, 4 independent chains.  PROMOTE adds the block-channel promotion of every
// 4th MFMA's result (convert + fma per accumulator element, 2 vector ops per element per 128-deep
// K block) to show what that vector work costs beside the MFMAs.
template <bool PROMOTE>
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* sink, long long* clocks, int iters, int random_operands, float f) {
    v4i a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a[i][c] = random_operands ? (int)probe_hash(threadIdx.x * 131u + i * 17u + c * 3u + blockIdx.x * 7919u) : 0;
            b[i][c] = random_operands ? (int)probe_hash(threadIdx.x * 977u + i * 29u + c * 5u + blockIdx.x * 104729u) : 0;
        }
    const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16i acc[2][2] = {{z, z}, {z, z}};
    float accf[2][2][16];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[i][j][r] = 0.0f;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], (PROMOTE && ks == 0) ? z : acc[i][j], 0, 0, 0);
        if (PROMOTE) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) accf[i][j][r] = __builtin_fmaf(static_cast<float>(acc[i][j][r]), f, accf[i][j][r]);
        }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += accf[i][j][r] + static_cast<float>(acc[i][j][r]);
    sink[blockIdx.x * 512 + threadIdx.x] = s;   // keeps the loop alive
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = c1 - c0;   // shader clock cycles
        clocks[1] = w1 - w0;   // ticks of the constant 100 MHz counter
    }
}

}  // namespace ti8

using namespace ti8;

extern "C" int ti8_probe_mfma(float* sink, int64_t sink_elems, int64_t* clocks, int workgroups, int iters, int random_operands,
                              int with_promotion, ti8_stream_t stream) {
    if (!sink || !clocks) return fail(TI8_ERR_NULL, "ti8_probe_mfma: sink and clocks are required");
    if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || sink_elems < (int64_t)workgroups * 512)
        return fail(TI8_ERR_SHAPE, "ti8_probe_mfma: need 0 < workgroups <= 65536, iters > 0 and 512 sink elements per workgroup");
    hipStream_t st = static_cast<hipStream_t>(stream);
    long long* ck = reinterpret_cast<long long*>(clocks);
    if (with_promotion)
        hipLaunchKernelGGL(probe_mfma_kernel<true>, dim3((unsigned)workgroups), dim3(512), 0, st, sink, ck, iters, random_operands, 0.5f);
    else
        hipLaunchKernelGGL(probe_mfma_kernel<false>, dim3((unsigned)workgroups), dim3(512), 0, st, sink, ck, iters, random_operands, 0.5f);
    return check_launch("ti8_probe_mfma");
}
