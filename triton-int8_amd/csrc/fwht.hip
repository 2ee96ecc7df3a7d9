// Walsh-Hadamard transform along rows (Sylvester order, un-normalised), bf16 in/out,
// fp32 butterflies in the fixed order stride 1, 2, 4, ..., n/2.  The order is part of
// the contract: fp32 sums are order dependent and the CPU checker uses the same one.
//
// A workgroup of 256 threads owns L consecutive elements of one row: L = n when
// n >= 2048, else gcd(cols, 2048) (several length-n groups), staged in LDS as fp32.  The log2(n) stages
// run in passes of up to 4 stages: in a pass over index bits [p, p+r) a thread gathers
// the 2^r elements that differ only in those bits, does the butterflies in registers
// and writes them back.  Compile with -ffp-contract=off (the optional scale multiply
// must not fuse with a butterfly).
#include "ti8_common.h"

namespace ti8 {

template <int RB>
__device__ __forceinline__ void pass_in_lds(float* lds, int L, int p, int tid) {
    constexpr int RAD = 1 << RB;
    const int ngroups = L >> RB;
    for (int vt = tid; vt < ngroups; vt += 256) {
        const int lo = vt & ((1 << p) - 1);
        const int hi = vt >> p;
        const int base = (hi << (p + RB)) | lo;
        float a[RAD];
#pragma unroll
        for (int e = 0; e < RAD; ++e) a[e] = lds[base + (e << p)];
#pragma unroll
        for (int h = 1; h < RAD; h <<= 1)
#pragma unroll
            for (int e = 0; e < RAD; ++e)
                if ((e & h) == 0) {
                    const float u = a[e], w = a[e + h];
                    a[e] = u + w;
                    a[e + h] = u - w;
                }
#pragma unroll
        for (int e = 0; e < RAD; ++e) lds[base + (e << p)] = a[e];
    }
}

__global__ __launch_bounds__(256) void fwht_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                   uint16_t* __restrict__ y, int64_t ldy, int cols, int logn,
                                                   int L, float scale) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int segs_per_row = cols / L;
    const int64_t row = blockIdx.x / segs_per_row;
    const int seg = blockIdx.x % segs_per_row;
    const uint16_t* xr = x + row * ldx + (int64_t)seg * L;
    uint16_t* yr = y + row * ldy + (int64_t)seg * L;

    for (int c = tid; c < (L >> 3); c += 256) {
        const uint4 v = *reinterpret_cast<const uint4*>(xr + c * 8);
        float4 a = make_float4(bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y));
        float4 b = make_float4(bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w));
        *reinterpret_cast<float4*>(lds + c * 8) = a;
        *reinterpret_cast<float4*>(lds + c * 8 + 4) = b;
    }
    __syncthreads();
    int p = 0;
    while (p < logn) {
        const int rb = (logn - p) >= 4 ? 4 : (logn - p);
        switch (rb) {
            case 4: pass_in_lds<4>(lds, L, p, tid); break;
            case 3: pass_in_lds<3>(lds, L, p, tid); break;
            case 2: pass_in_lds<2>(lds, L, p, tid); break;
            default: pass_in_lds<1>(lds, L, p, tid); break;
        }
        p += rb;
        __syncthreads();
    }
    for (int c = tid; c < (L >> 3); c += 256) {
        const float4 a = *reinterpret_cast<const float4*>(lds + c * 8);
        const float4 b = *reinterpret_cast<const float4*>(lds + c * 8 + 4);
        uint4 o;
        if (scale != 1.0f) {
            o.x = f32_to_bf16_bits(a.x * scale) | (f32_to_bf16_bits(a.y * scale) << 16);
            o.y = f32_to_bf16_bits(a.z * scale) | (f32_to_bf16_bits(a.w * scale) << 16);
            o.z = f32_to_bf16_bits(b.x * scale) | (f32_to_bf16_bits(b.y * scale) << 16);
            o.w = f32_to_bf16_bits(b.z * scale) | (f32_to_bf16_bits(b.w * scale) << 16);
        } else {
            o.x = f32_to_bf16_bits(a.x) | (f32_to_bf16_bits(a.y) << 16);
            o.y = f32_to_bf16_bits(a.z) | (f32_to_bf16_bits(a.w) << 16);
            o.z = f32_to_bf16_bits(b.x) | (f32_to_bf16_bits(b.y) << 16);
            o.w = f32_to_bf16_bits(b.z) | (f32_to_bf16_bits(b.w) << 16);
        }
        *reinterpret_cast<uint4*>(yr + c * 8) = o;
    }
}

}  // namespace ti8

using namespace ti8;

extern "C" int ti8_fwht(const void* x, int64_t ldx, void* y, int64_t ldy, int64_t rows, int64_t cols, int64_t n,
                        float scale, ti8_stream_t stream) {
    if (!x || !y) return fail(TI8_ERR_NULL, "ti8_fwht: x and y are required");
    if (n < 128 || n > 32768 || (n & (n - 1))) return fail(TI8_ERR_SHAPE, "ti8_fwht: n must be a power of two in [128, 32768], got %lld", (long long)n);
    if (rows <= 0 || cols <= 0 || cols % n) return fail(TI8_ERR_SHAPE, "ti8_fwht: need rows>0 and cols%%n==0; got rows=%lld cols=%lld n=%lld", (long long)rows, (long long)cols, (long long)n);
    // elements per workgroup: a whole group when n >= 2048, else as many groups as divide
    // both the row and 2048
    int64_t L = n;
    if (n < 2048) {
        int64_t a = cols, b = 2048;
        while (b) { const int64_t t = a % b; a = b; b = t; }
        L = a;  // gcd(cols, 2048), a multiple of n because n divides both
    }
    if (ldx < cols || ldy < cols) return fail(TI8_ERR_SHAPE, "ti8_fwht: leading dimension smaller than cols");
    if (!aligned16(x) || !aligned16(y) || (ldx % 8) || (ldy % 8)) return fail(TI8_ERR_ALIGN, "ti8_fwht: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    const int64_t nblocks = rows * (cols / L);
    if (nblocks > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "ti8_fwht: too many segments");
    int logn = 0;
    while ((1LL << logn) < n) ++logn;
    const size_t shmem = (size_t)L * sizeof(float);
    static thread_local int attr_set_for = -1;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (shmem > 64 * 1024 && attr_set_for != dev) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fwht_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        if (e != hipSuccess) return fail(TI8_ERR_HIP, "ti8_fwht: cannot raise the LDS limit: %s", hipGetErrorString(e));
        attr_set_for = dev;
    }
    hipLaunchKernelGGL(fwht_kernel, dim3((unsigned)nblocks), dim3(256), shmem, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(y), ldy, (int)cols, logn, (int)L, scale);
    return check_launch("ti8_fwht");
}
