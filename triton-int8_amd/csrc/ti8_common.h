// Shared host/device helpers of libti8 (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>

#include "../../include/ti8.h"

namespace ti8 {

// ---- error reporting (host) ------------------------------------------------------
char* err_buf();  // thread-local buffer behind ti8_last_error()

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TI8_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return TI8_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- per-device one-time set-up (host) ---------------------------------------------
inline int current_device() {
    int dev = 0;
    (void)hipGetDevice(&dev);
    return dev;
}

// One bit per device index: whether a kernel's dynamic LDS limit has been raised there.  The call is idempotent,
// so two threads that race through it only repeat it.  ti8_init() goes through every kernel that needs it, so that
// nothing of the kind is left for the first launch.
struct OncePerDevice {
    std::atomic<uint64_t> done{0};
};
inline hipError_t raise_lds_limit(OncePerDevice& once, const void* kern, int bytes) {
    const uint64_t bit = 1ull << (current_device() & 63);
    if (once.done.load(std::memory_order_acquire) & bit) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) once.done.fetch_or(bit, std::memory_order_release);
    else (void)hipGetLastError();
    return e;
}

// Compute units of the current device (looked up once per device).
int device_cu_count();

// What ti8_init() calls: the per-device set-up of each source file's kernels (LDS limits, device symbols).
int init_gemm_kernels();
int init_chain_kernel();
int init_skinny_kernels();
int init_fwht_kernels();
int init_quant_scratch();

// ---- pieces of quant.hip that the one-call step (step.hip) uses --------------------
// ti8_quant_block_multi that also zeroes `clear_words` 32-bit words at `clear` (NULL: nothing) in the same launch
int quant_block_multi_and_clear(const ti8_qblock_operand* operands, int count, int qflags, int inv_mode,
                                unsigned int* clear, int64_t clear_words, ti8_stream_t stream);
int fill_words(unsigned int* p, int64_t words, unsigned int value, hipStream_t st);

// ---- which kernel served the last GEMM call of this thread (ti8_last_gemm_kernel) ---
void note_gemm_kernel(int kind, int bm, int bn, int epi);

// ---- device helpers --------------------------------------------------------------
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> bf16 bits, round to nearest even (finite values; NaN stays NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// two fp32 -> two bf16 in one dword (`lo` in the low half), round to nearest even: gfx950's
// v_cvt_pk_bf16_f32, same results as f32_to_bf16_bits for every finite value and infinity
typedef __bf16 ti8_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ti8_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const ti8_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ti8_bf16x2));
}

// Reductions over lanes with DPP moves (no LDS traffic).
// max(v, v of the lane that DPP control CTRL names) in the rows of ROW_MASK; other lanes keep v
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_max(float v) {
    const int i = __float_as_int(v);
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(i, i, CTRL, ROW_MASK, 0xf, false)));
}

// max over each half-wave of 32 lanes without LDS traffic; valid in lanes 16-31 and 48-63.
// quad_perm lane^1, lane^2, then row_half_mirror and row_mirror (all 16 lanes of a row agree),
// then row_bcast:15 into rows 1 and 3 (lane 15 of the row before).
__device__ __forceinline__ float half_wave_max_hi(float v) {
    v = dpp_max<0xB1>(v);
    v = dpp_max<0x4E>(v);
    v = dpp_max<0x141>(v);
    v = dpp_max<0x140>(v);
    return dpp_max<0x142, 0xA>(v);
}

// max over the 16 lanes of a DPP row, in all of them
__device__ __forceinline__ float row16_max(float v) {
    v = dpp_max<0xB1>(v);
    v = dpp_max<0x4E>(v);
    v = dpp_max<0x141>(v);
    return dpp_max<0x140>(v);
}

// max over the wave, in every lane: half_wave_max_hi, row_bcast:31 into rows 2 and 3 (lane 63 then
// holds the maximum), and a read of lane 63
__device__ __forceinline__ float wave_max(float v) {
    v = dpp_max<0x143, 0xC>(half_wave_max_hi(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

}  // namespace ti8
