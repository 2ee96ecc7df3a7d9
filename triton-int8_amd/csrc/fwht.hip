// Walsh-Hadamard transform along rows (Sylvester order, un-normalised), bf16 in/out,
// fp32 butterflies in the fixed order stride 1, 2, 4, ..., n/2.  The order is part of
// the contract: fp32 sums are order dependent and the CPU checker uses the same one.
//
// A workgroup owns L consecutive elements of one row: L = n when
// n >= 2048, else gcd(cols, 2048) (several length-n groups).  The log2(n) stages run in
// passes: in a pass over index bits [p, p+r) a thread gathers the 2^r elements that
// differ only in those bits, does the butterflies in registers and hands them on through
// LDS (fp32).  The first pass (bits 0..3) takes its 16 consecutive elements straight from
// global memory; the passes are bits 0..3, 4..7 and then the remaining bits in one pass
// (up to 5 bits) or two.
//
// LDS index i lives at word i + i/16.  With that padding a wave's 64 accesses of one
// instruction fall into 64 different banks in every pass: stride 17 in the first pass,
// four runs of 16 words at offsets 0, 16, 32, 48 (mod 64) in the second, consecutive
// words afterwards.  Without it the first two passes serialise 16- and 4-fold.
// Compile with -ffp-contract=off (the optional scale multiply must not fuse with a
// butterfly).
#include "ti8_common.h"
#include "index_math.h"

namespace ti8 {

__device__ __forceinline__ int padded(int i) { return idx::fwht_padded(i); }

template <int RB>
__device__ __forceinline__ void butterflies(float (&a)[1 << RB]) {
    constexpr int RAD = 1 << RB;
#pragma unroll
    for (int h = 1; h < RAD; h <<= 1)
#pragma unroll
        for (int e = 0; e < RAD; ++e)
            if ((e & h) == 0) {
                const float u = a[e], w = a[e + h];
                a[e] = u + w;
                a[e + h] = u - w;
            }
}

template <int RB, int NT>
__device__ __forceinline__ void pass_in_lds(float* lds, int L, int p, int tid) {
    constexpr int RAD = 1 << RB;
    const int ngroups = L >> RB;
    for (int vt = tid; vt < ngroups; vt += NT) {
        const int base = idx::fwht_group_base(vt, p, RB);
        float a[RAD];
#pragma unroll
        for (int e = 0; e < RAD; ++e) a[e] = lds[padded(base + (e << p))];
        butterflies<RB>(a);
#pragma unroll
        for (int e = 0; e < RAD; ++e) lds[padded(base + (e << p))] = a[e];
    }
}

template <int NT>
__device__ __forceinline__ void pass_dispatch(float* lds, int L, int p, int rb, int tid) {
    switch (rb) {
        case 5: pass_in_lds<5, NT>(lds, L, p, tid); break;
        case 4: pass_in_lds<4, NT>(lds, L, p, tid); break;
        case 3: pass_in_lds<3, NT>(lds, L, p, tid); break;
        case 2: pass_in_lds<2, NT>(lds, L, p, tid); break;
        default: pass_in_lds<1, NT>(lds, L, p, tid); break;
    }
}

// NT threads per workgroup: 256, or 1024 for segments of 16384 elements and more (their LDS
// footprint allows only one or two workgroups per CU, which 256 threads would leave idle)
template <int NT>
__global__ __launch_bounds__(NT) void fwht_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                   uint16_t* __restrict__ y, int64_t ldy, int cols, int logn,
                                                   int L, float scale) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int segs_per_row = cols / L;
    const uint16_t* xr = x + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldx, L);
    uint16_t* yr = y + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldy, L);

    // pass over bits 0..3 (n >= 128, so all four stages belong to every group)
    for (int vt = tid; vt < (L >> 4); vt += NT) {
        const uint4 v0 = *reinterpret_cast<const uint4*>(xr + vt * 16);
        const uint4 v1 = *reinterpret_cast<const uint4*>(xr + vt * 16 + 8);
        float a[16] = {bf16_lo(v0.x), bf16_hi(v0.x), bf16_lo(v0.y), bf16_hi(v0.y), bf16_lo(v0.z), bf16_hi(v0.z),
                       bf16_lo(v0.w), bf16_hi(v0.w), bf16_lo(v1.x), bf16_hi(v1.x), bf16_lo(v1.y), bf16_hi(v1.y),
                       bf16_lo(v1.z), bf16_hi(v1.z), bf16_lo(v1.w), bf16_hi(v1.w)};
        butterflies<4>(a);
#pragma unroll
        for (int e = 0; e < 16; ++e) lds[vt * 17 + e] = a[e];   // = padded(16 vt + e)
    }
    __syncthreads();
    // bits 4..7 (4..6 when n = 128)
    const int rb1 = min(4, logn - 4);
    pass_dispatch<NT>(lds, L, 4, rb1, tid);
    __syncthreads();
    int rem = logn - 8;
    if (rem > 0) {
        const int rb2 = rem <= 5 ? rem : (rem + 1) / 2;
        pass_dispatch<NT>(lds, L, 8, rb2, tid);
        __syncthreads();
        rem -= rb2;
        if (rem > 0) {
            pass_dispatch<NT>(lds, L, 8 + rb2, rem, tid);
            __syncthreads();
        }
    }
    for (int c = tid; c < (L >> 3); c += NT) {
        const float* src = lds + padded(c * 8);   // 8 words of one 16-word run: contiguous
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = src[e];
        if (scale != 1.0f) {
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = f[e] * scale;
        }
        uint4 o;
        o.x = pack_bf16x2(f[0], f[1]);
        o.y = pack_bf16x2(f[2], f[3]);
        o.z = pack_bf16x2(f[4], f[5]);
        o.w = pack_bf16x2(f[6], f[7]);
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
    const int64_t L = idx::fwht_segment_len(cols, n);   // elements per workgroup
    if (ldx < cols || ldy < cols) return fail(TI8_ERR_SHAPE, "ti8_fwht: leading dimension smaller than cols");
    if (!aligned16(x) || !aligned16(y) || (ldx % 8) || (ldy % 8)) return fail(TI8_ERR_ALIGN, "ti8_fwht: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    const int64_t nblocks = rows * (cols / L);
    if (nblocks > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "ti8_fwht: too many segments");
    int logn = 0;
    while ((1LL << logn) < n) ++logn;
    const size_t shmem = (size_t)idx::fwht_lds_words(L) * sizeof(float);
    static thread_local int attr_set_for = -1;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (attr_set_for != dev) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fwht_kernel<1024>), hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024);
        if (e != hipSuccess) return fail(TI8_ERR_HIP, "ti8_fwht: cannot raise the LDS limit: %s", hipGetErrorString(e));
        attr_set_for = dev;
    }
    if (idx::fwht_threads(L) == 1024)
        hipLaunchKernelGGL(fwht_kernel<1024>, dim3((unsigned)nblocks), dim3(1024), shmem, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(y), ldy, (int)cols, logn, (int)L, scale);
    else
        hipLaunchKernelGGL(fwht_kernel<256>, dim3((unsigned)nblocks), dim3(256), shmem, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(y), ldy, (int)cols, logn, (int)L, scale);
    return check_launch("ti8_fwht");
}
