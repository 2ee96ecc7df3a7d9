// Walsh-Hadamard transform along rows (Sylvester order, un-normalised), bf16 in/out,
// fp32 butterflies in the fixed order stride 1, 2, 4, ..., n/2.  The order is part of
// the contract: fp32 sums are order dependent and the CPU checker uses the same one.
//
// Lengths from 4096 on: fwht_row_kernel (described there): registers, lanes, one exchange through LDS per 4096 elements.
// Shorter lengths: fwht_kernel.  A workgroup owns L consecutive elements of one row: L = n when
// n >= 2048, else gcd(cols, 2048) (several length-n groups).  The log2(n) stages run in
// passes: in a pass over index bits [p, p+r) a thread gathers the 2^r elements that
// differ only in those bits, does the butterflies in registers and hands them on through
// LDS (fp32).  The first pass (bits 0..3) takes its 16 consecutive elements straight from
// global memory.  Segments of 1024 elements and more then run bits 4..9 across the 64 lanes of
// a wave (DPP and lane-swap instructions, no LDS) and what is left (up to 5 bits) in one pass
// through LDS: two LDS round trips and three barriers per row instead of three or four and
// four or five.  Shorter segments go through LDS after bits 0..3: bits 4..7, then the rest.
// The kernel is bound by the vector unit, not by HBM: 13 butterfly stages at n = 8192 are 13
// fp32 adds per element before any conversion or addressing (packed fp32 is not used).
//
// LDS index i lives at word i + i/16.  With that padding a wave's 64 accesses of one
// instruction fall into 64 different banks in every pass: stride 17 in the first pass,
// four runs of 16 words at offsets 0, 16, 32, 48 (mod 64) in the second, consecutive
// words afterwards.  Without it the first two passes serialise 16- and 4-fold.
// Compile with -ffp-contract=off (the optional scale multiply must not fuse with a
// butterfly).
#include "ti8_common.h"
#include "index_math.h"
#include "quant_math.h"

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

// ---- stages over index bits 4..9 without LDS: the 16-element chunks of 1024 consecutive elements sit in the 64 lanes
// of a wave.  Bits 4..7 pair lanes of one row of 16: with chunk idx::had_chunk(l) in lane l of its row the partners are
// lanes l ^ 1, l ^ 2, l ^ 7, l ^ 8, one DPP pattern each, and a stage is own + sigma * partner (sigma = -1 where the
// chunk has the bit set: an fma whose product is exact, rounded once like the add or subtract it stands for).  That
// leaves the upper lane of a pair with the negative of its result; both partners of every later stage carry the same
// number of such flips, so nothing else changes and the lane multiplies by its sign (-1 for an odd number of set bits
// among the stages that ran) at the end.  Bits 8 and 9 pair lanes 16 and 32 apart, through v_permlane16_swap /
// v_permlane32_swap (described where they are used).
struct LaneStages {
    float sigma[4];   // per DPP stage: -1 in lanes whose chunk has the stage's bit set
    float sign;       // what the DPP stages that ran have multiplied the lane's values by
};
__device__ __forceinline__ LaneStages lane_stages(int lane, int nstages) {
    const int c = idx::had_chunk(lane & 15) | (lane & 48);
    LaneStages st;
#pragma unroll
    for (int k = 0; k < 4; ++k) st.sigma[k] = ((c >> k) & 1) ? -1.0f : 1.0f;
    const int ran = c & 15 & ((1 << (nstages < 4 ? nstages : 4)) - 1);
    st.sign = (__builtin_popcount(ran) & 1) ? -1.0f : 1.0f;
    return st;
}
// A[e] += (A[e] of the partner lane) * SIGMA for 16 registers.  A DPP operand must not be read within two instructions of
// the vector instruction that wrote it: inside the block every register was written 16 instructions earlier, and the
// s_nop covers whatever the compiler placed in front.  All 64 lanes are active where this is used.
#define TI8_FWHT_FMAC(N, PATTERN) "v_fmac_f32_dpp %" #N ", %" #N ", %16 " PATTERN " row_mask:0xf bank_mask:0xf\n\t"
#define TI8_FWHT_DPP_STAGE(A, SIGMA, PATTERN)                                                                                   \
    asm("s_nop 1\n\t" TI8_FWHT_FMAC(0, PATTERN) TI8_FWHT_FMAC(1, PATTERN) TI8_FWHT_FMAC(2, PATTERN) TI8_FWHT_FMAC(3, PATTERN)    \
        TI8_FWHT_FMAC(4, PATTERN) TI8_FWHT_FMAC(5, PATTERN) TI8_FWHT_FMAC(6, PATTERN) TI8_FWHT_FMAC(7, PATTERN)                 \
        TI8_FWHT_FMAC(8, PATTERN) TI8_FWHT_FMAC(9, PATTERN) TI8_FWHT_FMAC(10, PATTERN) TI8_FWHT_FMAC(11, PATTERN)               \
        TI8_FWHT_FMAC(12, PATTERN) TI8_FWHT_FMAC(13, PATTERN) TI8_FWHT_FMAC(14, PATTERN) TI8_FWHT_FMAC(15, PATTERN)             \
        : "+v"(A[0]), "+v"(A[1]), "+v"(A[2]), "+v"(A[3]), "+v"(A[4]), "+v"(A[5]), "+v"(A[6]), "+v"(A[7]), "+v"(A[8]),           \
          "+v"(A[9]), "+v"(A[10]), "+v"(A[11]), "+v"(A[12]), "+v"(A[13]), "+v"(A[14]), "+v"(A[15])                              \
        : "v"(SIGMA))

// One DPP stage with the sign of every zero as the plain butterfly leaves it: own + sigma * partner computes b - a in the
// upper lane, and where a == b that is +0 although it stands for -(a - b) = -0, so a result that is exactly zero could
// come out as -0 at the end.  Nothing that is quantised afterwards can tell, but the bf16 output of the transform itself
// is compared bit for bit (zero-padded rows are all-zero rows).  Here the upper lane negates its own value first (exact)
// and adds: partner + (-own) = a - b, the lower lane partner + own; two instructions per element instead of one.
template <int CTRL>
__device__ __forceinline__ void exact_dpp_stage(float (&a)[16], float sigma) {
    const uint32_t flip = __float_as_uint(sigma) & 0x80000000u;   // sign bit set in the upper lane
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const float own = __uint_as_float(__float_as_uint(a[e]) ^ flip);
        a[e] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(a[e]), CTRL, 0xf, 0xf, true)) + own;
    }
}

// the stages over bits 4 .. 4 + nstages - 1 (nstages <= 6) on the 16 elements of this lane's chunk.  EXACT_ZEROS: see
// exact_dpp_stage (the bf16 output path); otherwise one instruction per element and stage (the quantising path)
// APPLY_SIGN = false leaves the values of the one-instruction form multiplied by st.sign for a caller that multiplies
// them by something else anyway (every later stage of this file pairs values of the same chunk position, i.e. sign)
template <bool EXACT_ZEROS, bool APPLY_SIGN = true>
__device__ __forceinline__ void lane_butterflies(float (&a)[16], const LaneStages& st, int nstages) {
#if defined(__HIP_DEVICE_COMPILE__)
    if (EXACT_ZEROS) {
        if (nstages > 0) exact_dpp_stage<0xB1>(a, st.sigma[0]);
        if (nstages > 1) exact_dpp_stage<0x4E>(a, st.sigma[1]);
        if (nstages > 2) exact_dpp_stage<0x141>(a, st.sigma[2]);
        if (nstages > 3) exact_dpp_stage<0x128>(a, st.sigma[3]);
    } else {
        if (nstages > 0) TI8_FWHT_DPP_STAGE(a, st.sigma[0], "quad_perm:[1,0,3,2]");
        if (nstages > 1) TI8_FWHT_DPP_STAGE(a, st.sigma[1], "quad_perm:[2,3,0,1]");
        if (nstages > 2) TI8_FWHT_DPP_STAGE(a, st.sigma[2], "row_half_mirror");
        if (nstages > 3) TI8_FWHT_DPP_STAGE(a, st.sigma[3], "row_ror:8");
        if (APPLY_SIGN) {
#pragma unroll
            for (int e = 0; e < 16; ++e) a[e] = a[e] * st.sign;
        }
    }
    // Bits 8 and 9 pair lanes 16 and 32 apart, two elements at a time: a lane swap of the two registers brings both values
    // of every pair into ONE lane (element e in the even rows / lower half, element e + 1 in the others), the butterfly is
    // an ordinary add and subtract there, and the same swap takes sums and differences back to where they belong -- four
    // instructions for two elements, true signs.
    if (nstages > 4) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const auto r = __builtin_amdgcn_permlane16_swap(__float_as_int(a[e]), __float_as_int(a[e + 1]), false, false);
            const float u = __int_as_float(r[0]), v = __int_as_float(r[1]);
            const auto t = __builtin_amdgcn_permlane16_swap(__float_as_int(u + v), __float_as_int(u - v), false, false);
            a[e] = __int_as_float(t[0]);
            a[e + 1] = __int_as_float(t[1]);
        }
    }
    if (nstages > 5) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            const auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(a[e]), __float_as_int(a[e + 1]), false, false);
            const float u = __int_as_float(r[0]), v = __int_as_float(r[1]);
            const auto t = __builtin_amdgcn_permlane32_swap(__float_as_int(u + v), __float_as_int(u - v), false, false);
            a[e] = __int_as_float(t[0]);
            a[e + 1] = __int_as_float(t[1]);
        }
    }
#endif
}

// Segments of up to 2048 elements (lengths below 4096), NT = 256 threads per workgroup.
// QUANT: the workgroup's segment is a whole row (L >= cols), and instead of the rotated bf16 row the
// kernel writes what the per-row quantiser makes of it -- int8 q[row][cols] and the row's scale --
// with the quantiser's own arithmetic on the same bf16-rounded values: the rotated operand never
// goes to HBM (3 bytes per element instead of 4 + 3).
template <int NT, bool QUANT>
__global__ __launch_bounds__(NT) void fwht_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                   uint16_t* __restrict__ y, int64_t ldy, int cols, int logn,
                                                   int L, float scale, int8_t* __restrict__ q, int64_t ldq,
                                                   float* __restrict__ s, QMode mode) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    // cols < L: one zero-extended row per workgroup (a length that is no power of two, transformed as the next power of
    // two and cut back): elements from `valid` on read as zero and are not stored
    const int valid = cols < L ? cols : L;
    const int segs_per_row = cols < L ? 1 : cols / L;
    const uint16_t* xr = x + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldx, L);
    uint16_t* yr = y + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldy, L);

    // Segments of 1024 elements and more: bits 0..3 in registers and bits 4..9 across the lanes of a wave, whose 64 lanes
    // hold 64 consecutive chunks (in the order lane_stages wants), then one pass through LDS for what is left.
    const bool by_lanes = L >= 1024;
    if (by_lanes) {
        const int nstages = min(6, logn - 4);
        const LaneStages st = lane_stages(tid & 63, nstages);
        for (int v0 = tid; v0 < (L >> 4); v0 += NT) {   // L / 16 is a multiple of 64: whole waves
            const int vt = (v0 & ~15) | idx::had_chunk(v0 & 15);
            const bool in = idx::fwht_chunk_valid(vt * 16, 16, valid);
            const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
            const uint4 v0q = in ? *reinterpret_cast<const uint4*>(xr + vt * 16) : zero4;
            const uint4 v1q = in ? *reinterpret_cast<const uint4*>(xr + vt * 16 + 8) : zero4;
            float a[16] = {bf16_lo(v0q.x), bf16_hi(v0q.x), bf16_lo(v0q.y), bf16_hi(v0q.y), bf16_lo(v0q.z), bf16_hi(v0q.z),
                           bf16_lo(v0q.w), bf16_hi(v0q.w), bf16_lo(v1q.x), bf16_hi(v1q.x), bf16_lo(v1q.y), bf16_hi(v1q.y),
                           bf16_lo(v1q.z), bf16_hi(v1q.z), bf16_lo(v1q.w), bf16_hi(v1q.w)};
            butterflies<4>(a);
            lane_butterflies<!QUANT>(a, st, nstages);
#pragma unroll
            for (int e = 0; e < 16; ++e) lds[vt * 17 + e] = a[e];   // = padded(16 vt + e)
        }
        __syncthreads();
        const int rem = logn - 10;
        if (rem > 0) {
            pass_dispatch<NT>(lds, L, 10, rem, tid);
            __syncthreads();
        }
    }
    // pass over bits 0..3 (n >= 128, so all four stages belong to every group)
    for (int vt = tid; vt < (by_lanes ? 0 : (L >> 4)); vt += NT) {
        const bool in = idx::fwht_chunk_valid(vt * 16, 16, valid);   // valid is a multiple of 16: a chunk is inside or outside
        const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
        const uint4 v0 = in ? *reinterpret_cast<const uint4*>(xr + vt * 16) : zero4;
        const uint4 v1 = in ? *reinterpret_cast<const uint4*>(xr + vt * 16 + 8) : zero4;
        float a[16] = {bf16_lo(v0.x), bf16_hi(v0.x), bf16_lo(v0.y), bf16_hi(v0.y), bf16_lo(v0.z), bf16_hi(v0.z),
                       bf16_lo(v0.w), bf16_hi(v0.w), bf16_lo(v1.x), bf16_hi(v1.x), bf16_lo(v1.y), bf16_hi(v1.y),
                       bf16_lo(v1.z), bf16_hi(v1.z), bf16_lo(v1.w), bf16_hi(v1.w)};
        butterflies<4>(a);
#pragma unroll
        for (int e = 0; e < 16; ++e) lds[vt * 17 + e] = a[e];   // = padded(16 vt + e)
    }
    if (!by_lanes) __syncthreads();
    // bits 4..7 (4..6 when n = 128)
    const int rb1 = min(4, logn - 4);
    if (!by_lanes) {
        pass_dispatch<NT>(lds, L, 4, rb1, tid);
        __syncthreads();
    }
    int rem = by_lanes ? 0 : logn - 8;
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
    if (QUANT) {
        // a thread's chunks stay in registers (bf16, as they would have been stored) while the row's absmax is reduced
        constexpr int MAXC = 1;          // L / 8 / NT: at most 2048 elements on 256 threads
        uint4 o[MAXC];
        float amax = 0.0f;
#pragma unroll
        for (int k = 0; k < MAXC; ++k) {
            const int c = tid + k * NT;
            o[k] = make_uint4(0u, 0u, 0u, 0u);
            if (c < (L >> 3) && idx::fwht_chunk_valid(c * 8, 8, valid)) {
                const float* src = lds + padded(c * 8);
                float f[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) f[e] = src[e];
                if (scale != 1.0f) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[e] = f[e] * scale;
                }
                o[k] = make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
                amax = absmax8(o[k], amax);
            }
        }
        __syncthreads();                 // everybody has taken its values out of LDS: its first words now serve the reduction
        amax = wave_max(amax);
        if ((tid & 63) == 0) lds[tid >> 6] = amax;
        __syncthreads();
        amax = lds[0];
#pragma unroll
        for (int w = 1; w < NT / 64; ++w) amax = fmaxf(amax, lds[w]);
        amax = amax_floor(amax, mode.eps_add);
        const float mult = 127.0f / amax;
        const int64_t row = blockIdx.x;
        if (tid == 0) s[row] = stored_scale(amax, mult, mode);
        int8_t* qr = q + row * ldq;
#pragma unroll
        for (int k = 0; k < MAXC; ++k) {
            const int c = tid + k * NT;
            if (c < (L >> 3) && idx::fwht_chunk_valid(c * 8, 8, valid)) *reinterpret_cast<uint2*>(qr + c * 8) = quant8(o[k], mult);
        }
        return;
    }
    for (int c = tid; c < (L >> 3); c += NT) {
        if (!idx::fwht_chunk_valid(c * 8, 8, valid)) continue;
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

// ---- segments of 4096 * CH elements (CH = 1, 2, 4, 8), one per workgroup of 4 waves, with a single trip through LDS.
// Slice k of the segment (4096 elements) is 4 x 1024: wave w transforms elements [1024 (4k + w), + 1024) over bits 0..9
// in registers and across its lanes (16 elements per lane, lane_butterflies).  Bits 10 and 11 pair the four waves of a
// slice: every lane writes its 16 values to LDS and takes back elements 4w .. 4w + 3 of its chunk position from all four
// waves (a radix-4 butterfly on each of the four elements).  Bits 12 and up pair the slices, which by then sit in the same
// thread's registers.  A thread ends with 4 consecutive elements of 4 CH chunks and stores them from registers (8 bytes of
// bf16, or 4 bytes of int8 behind the row's absmax when QUANT): there is no read-back pass, and the exchange buffer is
// 16 KiB (two of them, so that one barrier per slice is enough) whatever the length.  Same stage order, same roundings as
// fwht_kernel: bit-identical.
template <int CH, bool QUANT>
__global__ __launch_bounds__(256) void fwht_row_kernel(const uint16_t* __restrict__ x, int64_t ldx, uint16_t* __restrict__ y,
                                                       int64_t ldy, int cols, float scale, int8_t* __restrict__ q, int64_t ldq,
                                                       float* __restrict__ s, QMode mode) {
    constexpr int L = 4096 * CH;
    constexpr int BUF = 4 * 64 * 16;                      // one slice: 4 waves x 64 chunk positions x 16 values (idx::fwht_row_lds)
    __shared__ __attribute__((aligned(16))) float xbuf[(CH > 1 ? 2 : 1) * BUF];   // (one buffer and a second barrier per slice measured the same)
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int valid = cols < L ? cols : L;                // cols < L: one zero-extended row per workgroup
    const int segs_per_row = cols < L ? 1 : cols / L;
    const uint16_t* xr = x + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldx, L);
    const LaneStages st = lane_stages(lane, 6);
    const int lp = (lane & ~15) | idx::had_chunk(lane & 15);   // this lane's chunk among the 64 of its wave's 1024 elements

    float b[CH][16];
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    // a chunk beyond the row's end (zero-extended rows) reads the row's first chunk instead and is then replaced by zeros:
    // the load stays an ordinary global load (a select between the load and a constant becomes a select of addresses)
    auto load_slice = [&](int k, uint4& lo, uint4& hi) {
        const int first = idx::fwht_row_chunk_first(k, w, lp);
        const bool in = idx::fwht_chunk_valid(first, 16, valid);
        const uint16_t* p = xr + (in ? first : 0);
        lo = *reinterpret_cast<const uint4*>(p);
        hi = *reinterpret_cast<const uint4*>(p + 8);
        if (!in) lo = hi = zero4;
    };
    uint4 lo, hi, nlo = zero4, nhi = zero4;
    load_slice(0, lo, hi);
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        if (k + 1 < CH) load_slice(k + 1, nlo, nhi);
        float a[16] = {bf16_lo(lo.x), bf16_hi(lo.x), bf16_lo(lo.y), bf16_hi(lo.y), bf16_lo(lo.z), bf16_hi(lo.z), bf16_lo(lo.w), bf16_hi(lo.w),
                       bf16_lo(hi.x), bf16_hi(hi.x), bf16_lo(hi.y), bf16_hi(hi.y), bf16_lo(hi.z), bf16_hi(hi.z), bf16_lo(hi.w), bf16_hi(hi.w)};
        butterflies<4>(a);
        lane_butterflies<!QUANT, false>(a, st, 6);   // QUANT: the lane's sign goes into its quantisation multiplier below
        float* buf = xbuf + (k & 1) * BUF;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<float4*>(buf + idx::fwht_row_lds(w, lp, 4 * j)) = make_float4(a[4 * j], a[4 * j + 1], a[4 * j + 2], a[4 * j + 3]);
        __syncthreads();   // with two buffers this also orders the reads of slice k - 1 before the writes of slice k + 1
        float c[4][4];
#pragma unroll
        for (int ws = 0; ws < 4; ++ws) {
            const float4 v = *reinterpret_cast<const float4*>(buf + idx::fwht_row_lds(ws, lp, 4 * w));
            c[ws][0] = v.x;
            c[ws][1] = v.y;
            c[ws][2] = v.z;
            c[ws][3] = v.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {   // bit 10: waves 0|1 and 2|3
            const float u0 = c[0][e], v0 = c[1][e], u1 = c[2][e], v1 = c[3][e];
            c[0][e] = u0 + v0;
            c[1][e] = u0 - v0;
            c[2][e] = u1 + v1;
            c[3][e] = u1 - v1;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {   // bit 11: waves 0|2 and 1|3
            const float u0 = c[0][e], v0 = c[2][e], u1 = c[1][e], v1 = c[3][e];
            c[0][e] = u0 + v0;
            c[2][e] = u0 - v0;
            c[1][e] = u1 + v1;
            c[3][e] = u1 - v1;
        }
#pragma unroll
        for (int ws = 0; ws < 4; ++ws)
#pragma unroll
            for (int e = 0; e < 4; ++e) b[k][ws * 4 + e] = c[ws][e];
        lo = nlo;
        hi = nhi;
    }
    // bits 12 and up: the slices
#pragma unroll
    for (int h = 1; h < CH; h <<= 1)
#pragma unroll
        for (int k = 0; k < CH; ++k)
            if ((k & h) == 0) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float u = b[k][j], v = b[k + h][j];
                    b[k][j] = u + v;
                    b[k + h][j] = u - v;
                }
            }
    // the thread's results as bf16: element idx::fwht_row_out(k, ws, lp, w) + e  <-  b[k][4 ws + e]
    uint2 o[CH][4];
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int ws = 0; ws < 4; ++ws) {
            float f[4] = {b[k][ws * 4], b[k][ws * 4 + 1], b[k][ws * 4 + 2], b[k][ws * 4 + 3]};
            if (scale != 1.0f) {
#pragma unroll
                for (int e = 0; e < 4; ++e) f[e] = f[e] * scale;
            }
            o[k][ws] = make_uint2(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]));
        }
    if (!QUANT) {
        uint16_t* yr = y + idx::fwht_segment_offset(blockIdx.x, segs_per_row, ldy, L);
#pragma unroll
        for (int k = 0; k < CH; ++k)
#pragma unroll
            for (int ws = 0; ws < 4; ++ws) {
                const int first = idx::fwht_row_out(k, ws, lp, w);
                if (idx::fwht_chunk_valid(first, 4, valid)) *reinterpret_cast<uint2*>(yr + first) = o[k][ws];
            }
        return;
    }
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int ws = 0; ws < 4; ++ws)
            if (idx::fwht_chunk_valid(idx::fwht_row_out(k, ws, lp, w), 4, valid)) {   // a chain, so that pairs become v_max3_f32
                amax = fmaxf(amax, fabsf(bf16_lo(o[k][ws].x)));
                amax = fmaxf(amax, fabsf(bf16_hi(o[k][ws].x)));
                amax = fmaxf(amax, fabsf(bf16_lo(o[k][ws].y)));
                amax = fmaxf(amax, fabsf(bf16_hi(o[k][ws].y)));
            }
    amax = wave_max(amax);
    __syncthreads();                 // the last slice's exchange has been read: the buffer's first words serve the reduction
    if (lane == 0) xbuf[w] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(xbuf[0], xbuf[1]), fmaxf(xbuf[2], xbuf[3]));
    amax = amax_floor(amax, mode.eps_add);
    const float mult = 127.0f / amax;
    const int64_t row = blockIdx.x;
    if (tid == 0) s[row] = stored_scale(amax, mult, mode);
    // everything this thread holds came from chunk position lp of some wave and slice, so it carries this lane's sign
    const float lane_mult = mult * st.sign;
    int8_t* qr = q + row * ldq;
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int ws = 0; ws < 4; ++ws) {
            const int first = idx::fwht_row_out(k, ws, lp, w);
            if (!idx::fwht_chunk_valid(first, 4, valid)) continue;
            uint32_t v = put_u8(qbiased(bf16_lo(o[k][ws].x), lane_mult), 0, 0u);
            v = put_u8(qbiased(bf16_hi(o[k][ws].x), lane_mult), 1, v);
            v = put_u8(qbiased(bf16_lo(o[k][ws].y), lane_mult), 2, v);
            v = put_u8(qbiased(bf16_hi(o[k][ws].y), lane_mult), 3, v);
            *reinterpret_cast<uint32_t*>(qr + first) = v ^ UNBIAS4;
        }
}

// ---- transposed input: y[c][r] = sum_r' H[r][r'] x[r'][c], i.e. the transform of x^T along its
// rows without materialising x^T.  A workgroup owns W columns of x (W = 8, 4, 2, 1 as the length R
// grows: W * R fp32 elements must fit in LDS), reads them row by row -- W bf16 = 2 W bytes per row;
// the other columns of the same 128-byte lines belong to the sibling workgroups that the block map
// keeps together on one XCD -- and lays them out in LDS as W segments of R elements in the padded
// layout of the kernel above, after which the butterfly passes are those of the kernel above
// applied to every segment (bits 0..3 first, from LDS here), and each segment leaves as one
// contiguous row of y.  Same butterfly order, same single rounding: bit-identical to
// ti8_fwht(transpose(x)).
template <int RB, int NT>
__device__ __forceinline__ void pass_in_lds_segments(float* lds, int L, int Lp, int W, int p, int tid) {
    constexpr int RAD = 1 << RB;
    const int per_seg = L >> RB;
    for (int vt = tid; vt < W * per_seg; vt += NT) {
        float* seg = lds + (vt / per_seg) * Lp;
        const int base = idx::fwht_group_base(vt % per_seg, p, RB);
        float a[RAD];
#pragma unroll
        for (int e = 0; e < RAD; ++e) a[e] = seg[padded(base + (e << p))];
        butterflies<RB>(a);
#pragma unroll
        for (int e = 0; e < RAD; ++e) seg[padded(base + (e << p))] = a[e];
    }
}

template <int NT>
__device__ __forceinline__ void pass_dispatch_segments(float* lds, int L, int Lp, int W, int p, int rb, int tid) {
    switch (rb) {
        case 5: pass_in_lds_segments<5, NT>(lds, L, Lp, W, p, tid); break;
        case 4: pass_in_lds_segments<4, NT>(lds, L, Lp, W, p, tid); break;
        case 3: pass_in_lds_segments<3, NT>(lds, L, Lp, W, p, tid); break;
        case 2: pass_in_lds_segments<2, NT>(lds, L, Lp, W, p, tid); break;
        default: pass_in_lds_segments<1, NT>(lds, L, Lp, W, p, tid); break;
    }
}

template <int W> struct ColumnLoad;
template <> struct ColumnLoad<8> { typedef uint4 type; };
template <> struct ColumnLoad<4> { typedef uint2 type; };
template <> struct ColumnLoad<2> { typedef uint32_t type; };
template <> struct ColumnLoad<1> { typedef uint16_t type; };

template <int NT, int W>
__global__ __launch_bounds__(NT) void fwht_t_kernel(const uint16_t* __restrict__ x, int64_t ldx, uint16_t* __restrict__ y,
                                                     int64_t ldy, int R, int logn, int64_t nblocks, float scale) {
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int L = R, Lp = (int)idx::fwht_lds_words(R);
    const int64_t c0 = idx::fwht_t_colblock(blockIdx.x, nblocks, W) * W;
    typedef typename ColumnLoad<W>::type load_t;
    for (int r = tid; r < R; r += NT) {
        const load_t v = *reinterpret_cast<const load_t*>(x + (int64_t)r * ldx + c0);
        uint16_t h[W];
        __builtin_memcpy(h, &v, sizeof(v));
#pragma unroll
        for (int w = 0; w < W; ++w) lds[w * Lp + padded(r)] = __uint_as_float((uint32_t)h[w] << 16);
    }
    __syncthreads();
    pass_in_lds_segments<4, NT>(lds, L, Lp, W, 0, tid);   // bits 0..3 (R >= 128)
    __syncthreads();
    const int rb1 = min(4, logn - 4);
    pass_dispatch_segments<NT>(lds, L, Lp, W, 4, rb1, tid);
    __syncthreads();
    int rem = logn - 8;
    if (rem > 0) {
        const int rb2 = rem <= 5 ? rem : (rem + 1) / 2;
        pass_dispatch_segments<NT>(lds, L, Lp, W, 8, rb2, tid);
        __syncthreads();
        rem -= rb2;
        if (rem > 0) {
            pass_dispatch_segments<NT>(lds, L, Lp, W, 8 + rb2, rem, tid);
            __syncthreads();
        }
    }
    const int per_seg = L >> 3;
    for (int i = tid; i < W * per_seg; i += NT) {
        const int w = i / per_seg, c = i % per_seg;
        const float* src = lds + w * Lp + padded(c * 8);   // 8 words of one 16-word run: contiguous
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
        *reinterpret_cast<uint4*>(y + (c0 + w) * ldy + c * 8) = o;
    }
}

// bf16 transpose, 64 x 64 tiles through LDS: x [R][C] -> y [C][R], 16-byte loads and stores.
// Thread t reads 8 consecutive columns of row (t / 8) + 32 h; the tile is kept as 32-bit words of
// two ROWS' elements so that a thread later picks up 8 consecutive rows of one column with 4 reads.
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const uint16_t* __restrict__ x, int64_t ldx, uint16_t* __restrict__ y,
                                                             int64_t ldy, int tiles_c) {
    __shared__ uint16_t tile[64][64 + 2];   // +2: rows 4 bytes apart modulo the banks
    const int tc = blockIdx.x % tiles_c, tr = blockIdx.x / tiles_c;
    const int tid = threadIdx.x;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int r = (tid >> 3) + 32 * h, c = (tid & 7) * 8;
        const uint4 v = *reinterpret_cast<const uint4*>(x + ((int64_t)tr * 64 + r) * ldx + (int64_t)tc * 64 + c);
        uint16_t e[8];
        __builtin_memcpy(e, &v, 16);
#pragma unroll
        for (int k = 0; k < 8; ++k) tile[c + k][r] = e[k];   // transposed in LDS: tile[column][row]
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int c = (tid >> 3) + 32 * h, r = (tid & 7) * 8;   // row c of y's tile = column c of x's tile
        uint16_t e[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] = tile[c][r + k];
        uint4 v;
        __builtin_memcpy(&v, e, 16);
        *reinterpret_cast<uint4*>(y + ((int64_t)tc * 64 + c) * ldy + (int64_t)tr * 64 + r) = v;
    }
}

}  // namespace ti8

using namespace ti8;

constexpr int FWHT_LDS_LIMIT = 136 * 1024;

template <int NT, int W>
static int prepare_fwht_t() {
    static OncePerDevice once;
    const hipError_t e = raise_lds_limit(once, reinterpret_cast<const void*>(fwht_t_kernel<NT, W>), FWHT_LDS_LIMIT);
    if (e != hipSuccess) return fail(TI8_ERR_HIP, "ti8_fwht_t: cannot raise the LDS limit: %s", hipGetErrorString(e));
    return TI8_OK;
}

// segments of 4096 elements and more: the kernel with one trip through LDS
template <bool QUANT>
static void launch_fwht_rows(int64_t n, int64_t nblocks, const uint16_t* x, int64_t ldx, uint16_t* y, int64_t ldy, int cols, float scale,
                             int8_t* q, int64_t ldq, float* s, const QMode& mode, hipStream_t st) {
    const dim3 grid((unsigned)nblocks), block(256);
    switch (n) {
        case 4096: hipLaunchKernelGGL((fwht_row_kernel<1, QUANT>), grid, block, 0, st, x, ldx, y, ldy, cols, scale, q, ldq, s, mode); break;
        case 8192: hipLaunchKernelGGL((fwht_row_kernel<2, QUANT>), grid, block, 0, st, x, ldx, y, ldy, cols, scale, q, ldq, s, mode); break;
        case 16384: hipLaunchKernelGGL((fwht_row_kernel<4, QUANT>), grid, block, 0, st, x, ldx, y, ldy, cols, scale, q, ldq, s, mode); break;
        default: hipLaunchKernelGGL((fwht_row_kernel<8, QUANT>), grid, block, 0, st, x, ldx, y, ldy, cols, scale, q, ldq, s, mode); break;
    }
}

namespace ti8 {
int init_fwht_kernels() {
    if (int e = prepare_fwht_t<1024, 8>()) return e;
    if (int e = prepare_fwht_t<1024, 4>()) return e;
    if (int e = prepare_fwht_t<1024, 2>()) return e;
    return prepare_fwht_t<1024, 1>();
}
}  // namespace ti8

template <int NT, int W>
static int launch_fwht_t(const void* x, int64_t ldx, void* y, int64_t ldy, int64_t R, int64_t C, int logn, float scale, hipStream_t st) {
    const size_t shmem = (size_t)W * idx::fwht_lds_words(R) * sizeof(float);
    auto kern = fwht_t_kernel<NT, W>;
    if (shmem > 64 * 1024)
        if (int e = prepare_fwht_t<NT, W>()) return e;
    const int64_t nblocks = C / W;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(NT), shmem, st, static_cast<const uint16_t*>(x), ldx,
                       static_cast<uint16_t*>(y), ldy, (int)R, logn, nblocks, scale);
    return check_launch("ti8_fwht_t");
}

extern "C" int ti8_fwht_t(const void* x, int64_t ldx, void* y, int64_t ldy, int64_t R, int64_t C, float scale, ti8_stream_t stream) {
    if (!x || !y) return fail(TI8_ERR_NULL, "ti8_fwht_t: x and y are required");
    if (R < 128 || R > 32768 || (R & (R - 1))) return fail(TI8_ERR_SHAPE, "ti8_fwht_t: R must be a power of two in [128, 32768], got %lld", (long long)R);
    if (C <= 0 || C % 8) return fail(TI8_ERR_SHAPE, "ti8_fwht_t: need C > 0 and C %% 8 == 0; got C=%lld", (long long)C);
    if (x == y) return fail(TI8_ERR_MODE, "ti8_fwht_t: the transform cannot run in place");
    if (ldx < C || ldy < R) return fail(TI8_ERR_SHAPE, "ti8_fwht_t: leading dimension smaller than the row length");
    if (!aligned16(x) || !aligned16(y) || (ldx % 8) || (ldy % 8)) return fail(TI8_ERR_ALIGN, "ti8_fwht_t: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    if (C / 1 > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "ti8_fwht_t: too many columns");
    int logn = 0;
    while ((1LL << logn) < R) ++logn;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (idx::fwht_t_direct(R, C)) {
        switch (idx::fwht_t_cols_per_wg(R)) {
            case 8: return R * 8 >= 16384 ? launch_fwht_t<1024, 8>(x, ldx, y, ldy, R, C, logn, scale, st)
                                          : launch_fwht_t<256, 8>(x, ldx, y, ldy, R, C, logn, scale, st);
            case 4: return launch_fwht_t<1024, 4>(x, ldx, y, ldy, R, C, logn, scale, st);
            case 2: return launch_fwht_t<1024, 2>(x, ldx, y, ldy, R, C, logn, scale, st);
            default: return launch_fwht_t<1024, 1>(x, ldx, y, ldy, R, C, logn, scale, st);
        }
    }
    // long columns: one or two columns per workgroup would be read 2 or 4 bytes per row and lane; transpose
    // into y with 16-byte accesses instead and transform y in place (the output is the only scratch)
    hipLaunchKernelGGL(transpose_bf16_kernel, dim3((unsigned)((R / 64) * (C / 64))), dim3(256), 0, st, static_cast<const uint16_t*>(x), ldx,
                       static_cast<uint16_t*>(y), ldy, (int)(C / 64));
    if (int e = check_launch("ti8_fwht_t")) return e;
    return ti8_fwht(y, ldy, y, ldy, C, R, R, scale, stream);
}

extern "C" int ti8_fwht(const void* x, int64_t ldx, void* y, int64_t ldy, int64_t rows, int64_t cols, int64_t n,
                        float scale, ti8_stream_t stream) {
    if (!x || !y) return fail(TI8_ERR_NULL, "ti8_fwht: x and y are required");
    if (n < 128 || n > 32768 || (n & (n - 1))) return fail(TI8_ERR_SHAPE, "ti8_fwht: n must be a power of two in [128, 32768], got %lld", (long long)n);
    // cols a multiple of n, or a row shorter than n (n the next power of two: n / 2 < cols < n) that is transformed zero-extended
    const bool extended = cols > n / 2 && cols < n;
    if (rows <= 0 || cols <= 0 || (cols % n && !extended) || (extended && cols % 16))
        return fail(TI8_ERR_SHAPE, "ti8_fwht: need rows>0 and cols%%n==0, or n/2 < cols < n with cols%%16==0; got rows=%lld cols=%lld n=%lld", (long long)rows, (long long)cols, (long long)n);
    if (extended && x == y && ldx != ldy) return fail(TI8_ERR_MODE, "ti8_fwht: in place needs ldx == ldy");
    const int64_t L = idx::fwht_segment_len(cols, n);   // elements per workgroup
    if (ldx < cols || ldy < cols) return fail(TI8_ERR_SHAPE, "ti8_fwht: leading dimension smaller than cols");
    if (!aligned16(x) || !aligned16(y) || (ldx % 8) || (ldy % 8)) return fail(TI8_ERR_ALIGN, "ti8_fwht: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    const int64_t nblocks = rows * (extended ? 1 : cols / L);
    if (nblocks > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "ti8_fwht: too many segments");
    int logn = 0;
    while ((1LL << logn) < n) ++logn;
    const size_t shmem = (size_t)idx::fwht_lds_words(L) * sizeof(float);   // at most 8.5 KiB: L <= 2048 here
    const QMode none = {0, 0, 0, 0};
    if (n >= 4096)
        launch_fwht_rows<false>(n, nblocks, static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(y), ldy, (int)cols, scale, nullptr, 0, nullptr,
                                none, static_cast<hipStream_t>(stream));
    else
        hipLaunchKernelGGL((fwht_kernel<256, false>), dim3((unsigned)nblocks), dim3(256), shmem, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(y), ldy, (int)cols, logn, (int)L, scale,
                           (int8_t*)nullptr, (int64_t)0, (float*)nullptr, none);
    return check_launch("ti8_fwht");
}

extern "C" int ti8_fwht_quant_row(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s, int64_t rows, int64_t cols, int64_t n,
                                  int qflags, int inv_mode, ti8_stream_t stream) {
    const char* fn = "ti8_fwht_quant_row";
    if (!x || !q || !s) return fail(TI8_ERR_NULL, "%s: x, q and s are required", fn);
    if (n < 128 || n > 32768 || (n & (n - 1))) return fail(TI8_ERR_SHAPE, "%s: n must be a power of two in [128, 32768], got %lld", fn, (long long)n);
    // the rotation runs over the whole row: cols = n, or a row shorter than n (n / 2 < cols < n) that is transformed zero-extended
    const bool extended = cols > n / 2 && cols < n;
    if (rows <= 0 || rows > 0x7fffffffLL || (cols != n && !extended) || cols % 16)
        return fail(TI8_ERR_SHAPE, "%s: need rows>0 and cols==n, or n/2 < cols < n, with cols%%16==0; got rows=%lld cols=%lld n=%lld", fn, (long long)rows,
                    (long long)cols, (long long)n);
    QMode mode;
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (qflags & (TI8_Q_HAD128 | TI8_Q_SCALE_BF16)) return fail(TI8_ERR_MODE, "%s: only TI8_Q_CLAMP and TI8_Q_EPS_ADD apply here", fn);
    if (ldx < cols || ldq < cols) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than cols", fn);
    if (!aligned16(x) || !aligned16(q) || (ldx % 8) || (ldq % 16)) return fail(TI8_ERR_ALIGN, "%s: pointers must be 16-byte aligned and strides multiples of 16 bytes", fn);
    int logn = 0;
    while ((1LL << logn) < n) ++logn;
    const int64_t L = n;   // one workgroup per row
    const size_t shmem = (size_t)idx::fwht_lds_words(L) * sizeof(float);
    if (n >= 4096)
        launch_fwht_rows<true>(n, rows, static_cast<const uint16_t*>(x), ldx, nullptr, 0, (int)cols, 1.0f, q, ldq, s, mode, static_cast<hipStream_t>(stream));
    else
        hipLaunchKernelGGL((fwht_kernel<256, true>), dim3((unsigned)rows), dim3(256), shmem, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(x), ldx, (uint16_t*)nullptr, (int64_t)0, (int)cols, logn, (int)L, 1.0f, q, ldq, s, mode);
    return check_launch(fn);
}

extern "C" int ti8_fwht_t_quant_row(const void* x, int64_t ldx, void* scratch, int8_t* q, int64_t ldq, float* s, int64_t R, int64_t C,
                                    int qflags, int inv_mode, ti8_stream_t stream) {
    const char* fn = "ti8_fwht_t_quant_row";
    if (!x || !scratch || !q || !s) return fail(TI8_ERR_NULL, "%s: x, scratch, q and s are required", fn);
    if (R < 128 || R > 32768 || R % 64 || C <= 0 || C % 64)
        return fail(TI8_ERR_SHAPE, "%s: need 128 <= R <= 32768, R %% 64 == 0 and C %% 64 == 0; got R=%lld C=%lld", fn, (long long)R, (long long)C);
    if ((R / 64) * (C / 64) > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "%s: too many tiles", fn);
    if (ldx < C) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than the row length", fn);
    if (!aligned16(x) || !aligned16(scratch) || (ldx % 8)) return fail(TI8_ERR_ALIGN, "%s: pointers must be 16-byte aligned and strides multiples of 16 bytes", fn);
    if (x == scratch) return fail(TI8_ERR_MODE, "%s: the scratch buffer must not be the input", fn);
    int64_t n = 128;
    while (n < R) n <<= 1;
    // n = the next power of two: R itself, or R is transformed zero-extended (n / 2 < R < n, R % 16 == 0 holds).
    // The other checks of the second launch, made before the first one is queued:
    if (ldq < R) return fail(TI8_ERR_SHAPE, "%s: leading dimension of q smaller than R", fn);
    if (!aligned16(q) || (ldq % 16)) return fail(TI8_ERR_ALIGN, "%s: q must be 16-byte aligned with a stride that is a multiple of 16", fn);
    QMode mode;
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (qflags & (TI8_Q_HAD128 | TI8_Q_SCALE_BF16)) return fail(TI8_ERR_MODE, "%s: only TI8_Q_CLAMP and TI8_Q_EPS_ADD apply here", fn);
    hipLaunchKernelGGL(transpose_bf16_kernel, dim3((unsigned)((R / 64) * (C / 64))), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(x), ldx, static_cast<uint16_t*>(scratch), R, (int)(C / 64));
    if (int e = check_launch(fn)) return e;
    return ti8_fwht_quant_row(scratch, R, q, ldq, s, C, R, n, qflags, inv_mode, stream);
}
