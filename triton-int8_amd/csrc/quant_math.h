// Arithmetic shared by every kernel that quantises to int8 (quant.hip, fwht.hip): the quantisation mode, the group
// multiplier and the stored scale, rounding and the saturating int8 conversion, absmax of 8 packed bf16.
// Translation units that include this MUST be compiled with -ffp-contract=off: `x*scale + 0.5f` has to round twice
// (multiply, then add) to reproduce the reference arithmetic bit for bit.
#pragma once
#include "ti8_common.h"

namespace ti8 {

struct QMode {
    int clamp;       // TI8_Q_CLAMP (recorded; the byte conversion saturates either way, see qbiased)
    int eps_add;     // TI8_Q_EPS_ADD
    int scale_bf16;  // TI8_Q_SCALE_BF16
    int inv_mode;    // ti8_inv_mode
};

// Arithmetic of the conversion.  ARITH_KERNEL is that of the reference's Triton kernels.  The
// other two are those of its pure-torch quantisers per_token_cast_to_int8 / per_block_cast_to_int8
// (tilelang/block_channel_fwd.py:215-230, tilelang/block_channel_bwd.py:96-104), evaluated the way
// torch evaluates them: `127.0 / amax` is reciprocal(amax) * 127 (two roundings), round() is
// half-to-even, the clamp is [-127, 127], the returned scale is reciprocal(scale); in the bf16
// variant (bf16 input, no .float() anywhere) every intermediate is rounded to bf16, the product
// x * scale included.
enum { ARITH_KERNEL = 0, ARITH_TORCH_F32 = 1, ARITH_TORCH_BF16 = 2 };

__device__ __forceinline__ float round_bf16(float f) { return __uint_as_float(f32_to_bf16_bits(f) << 16); }

template <int ARITH>
__device__ __forceinline__ float group_multiplier(float amax) {   // amax already floored
    if (ARITH == ARITH_KERNEL) return 127.0f / amax;
    float r = 1.0f / amax;
    if (ARITH == ARITH_TORCH_BF16) r = round_bf16(r);
    r = r * 127.0f;
    return ARITH == ARITH_TORCH_BF16 ? round_bf16(r) : r;
}
template <int ARITH>
__device__ __forceinline__ float amax_floor_arith(float amax, int eps_add) {
    if (ARITH == ARITH_KERNEL) return eps_add ? (amax + 1e-5f) : (amax > 1e-4f ? amax : 1e-4f);
    // torch clamp(min=1e-4) compares in the tensor's dtype: the constant is rounded to bf16 there
    const float e = ARITH == ARITH_TORCH_BF16 ? round_bf16(1e-4f) : 1e-4f;
    return amax > e ? amax : e;
}

__device__ __forceinline__ float amax_floor(float amax, int eps_add) {
    // triton/block_channel_fwd32.py:182 `where(amax > 1e-4, amax, 1e-4)`;
    // triton/fused_triton_fwd32.py:49 `max|x| + 1e-5`
    return eps_add ? (amax + 1e-5f) : (amax > 1e-4f ? amax : 1e-4f);
}

__device__ __forceinline__ float stored_scale(float amax, float scale, const QMode& m) {
    float s;
    switch (m.inv_mode) {
        case TI8_INV_RCP_OF_SCALE: s = 1.0f / scale; break;
        case TI8_INV_AMAX_DIV_127: s = amax / 127.0f; break;
        case TI8_INV_AMAX_MUL_RCP127: s = amax * (1.0f / 127.0f); break;
        default: s = scale; break;
    }
    if (m.scale_bf16) s = __uint_as_float(f32_to_bf16_bits(s) << 16);
    return s;
}
template <int ARITH>
__device__ __forceinline__ float stored_scale_arith(float amax, float scale, const QMode& m) {
    if (ARITH == ARITH_KERNEL) return stored_scale(amax, scale, m);
    const float s = 1.0f / scale;   // torch: (1.0 / scale) = reciprocal(scale) * 1.0
    return ARITH == ARITH_TORCH_BF16 ? round_bf16(s) : s;
}

// Rounding and int8 conversion.  r = floor(x*scale + 0.5) with two roundings (contraction is
// off), then r + 128 (exact: r is integral) goes through the saturating float -> u8 conversion
// v_cvt_pk_u8_f32, which also places the byte in a chosen position of a dword; xor 0x80 per byte
// turns the biased byte into two's complement.  The saturation IS the [-128, 127] clamp; without
// TI8_Q_CLAMP the reference applies no clamp, which gives the same bytes for every finite input
// because |x*scale| <= 127 when scale = 127 / absmax of the same data.
template <int ARITH = ARITH_KERNEL>
__device__ __forceinline__ float qbiased(float x, float scale) {
    if (ARITH == ARITH_KERNEL) return floorf(x * scale + 0.5f) + 128.0f;
    float t = x * scale;
    if (ARITH == ARITH_TORCH_BF16) t = round_bf16(t);
    t = rintf(t);                                       // half to even
    t = fminf(fmaxf(t, -127.0f), 127.0f);
    return t + 128.0f;
}
__device__ __forceinline__ uint32_t put_u8(float t, uint32_t byte, uint32_t old) {
    return __builtin_amdgcn_cvt_pk_u8_f32(t, byte, old);
}
constexpr uint32_t UNBIAS4 = 0x80808080u;

// 8 bf16 (one 16-byte load) -> 8 int8 in two dwords, element 0 in the low byte
template <int ARITH = ARITH_KERNEL>
__device__ __forceinline__ uint2 quant8(const uint4& v, float scale) {
    uint32_t a = put_u8(qbiased<ARITH>(bf16_lo(v.x), scale), 0, 0u), b = put_u8(qbiased<ARITH>(bf16_lo(v.z), scale), 0, 0u);
    a = put_u8(qbiased<ARITH>(bf16_hi(v.x), scale), 1, a);
    b = put_u8(qbiased<ARITH>(bf16_hi(v.z), scale), 1, b);
    a = put_u8(qbiased<ARITH>(bf16_lo(v.y), scale), 2, a);
    b = put_u8(qbiased<ARITH>(bf16_lo(v.w), scale), 2, b);
    a = put_u8(qbiased<ARITH>(bf16_hi(v.y), scale), 3, a);
    b = put_u8(qbiased<ARITH>(bf16_hi(v.w), scale), 3, b);
    uint2 o;
    o.x = a ^ UNBIAS4;
    o.y = b ^ UNBIAS4;
    return o;
}

// the 8 elements of row j (j < 4) of a 4-row patch, each with its own column scale, into byte j of
// w[0..7] (biased: xor UNBIAS4 once all four rows are in)
__device__ __forceinline__ void put_row_by_cols(const uint4& v, const float (&scale)[8], uint32_t j, uint32_t (&w)[8]) {
    w[0] = put_u8(qbiased(bf16_lo(v.x), scale[0]), j, w[0]);
    w[1] = put_u8(qbiased(bf16_hi(v.x), scale[1]), j, w[1]);
    w[2] = put_u8(qbiased(bf16_lo(v.y), scale[2]), j, w[2]);
    w[3] = put_u8(qbiased(bf16_hi(v.y), scale[3]), j, w[3]);
    w[4] = put_u8(qbiased(bf16_lo(v.z), scale[4]), j, w[4]);
    w[5] = put_u8(qbiased(bf16_hi(v.z), scale[5]), j, w[5]);
    w[6] = put_u8(qbiased(bf16_lo(v.w), scale[6]), j, w[6]);
    w[7] = put_u8(qbiased(bf16_hi(v.w), scale[7]), j, w[7]);
}

__device__ __forceinline__ float absmax8(const uint4& v, float m) {
    m = fmaxf(m, fabsf(bf16_lo(v.x)));
    m = fmaxf(m, fabsf(bf16_hi(v.x)));
    m = fmaxf(m, fabsf(bf16_lo(v.y)));
    m = fmaxf(m, fabsf(bf16_hi(v.y)));
    m = fmaxf(m, fabsf(bf16_lo(v.z)));
    m = fmaxf(m, fabsf(bf16_hi(v.z)));
    m = fmaxf(m, fabsf(bf16_lo(v.w)));
    m = fmaxf(m, fabsf(bf16_hi(v.w)));
    return m;
}

// max over the 256 threads of a workgroup (4 waves), result in every thread
__device__ __forceinline__ float block_max_256(float v, float* red4) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red4[wave] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red4[0], red4[1]), fmaxf(red4[2], red4[3]));
    return v;
}

inline int parse_mode(int qflags, int inv_mode, QMode* m) {
    if (qflags & ~(TI8_Q_CLAMP | TI8_Q_EPS_ADD | TI8_Q_SCALE_BF16 | TI8_Q_HAD128)) return fail(TI8_ERR_MODE, "unknown quantiser flag 0x%x", qflags);
    if (inv_mode < 0 || inv_mode > 3) return fail(TI8_ERR_MODE, "unknown inv_mode %d", inv_mode);
    m->clamp = (qflags & TI8_Q_CLAMP) ? 1 : 0;
    m->eps_add = (qflags & TI8_Q_EPS_ADD) ? 1 : 0;
    m->scale_bf16 = (qflags & TI8_Q_SCALE_BF16) ? 1 : 0;
    m->inv_mode = inv_mode;
    return TI8_OK;
}

}  // namespace ti8
