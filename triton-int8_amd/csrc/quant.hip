// Absmax -> int8 quantisers for gfx950.  All are HBM-bound: each reads every bf16
// element once with 16-byte loads, keeps it in registers while the group's absmax is
// reduced (wave shuffles + a few LDS words), and writes packed int8.
//
// This file MUST be compiled with -ffp-contract=off: `x*scale + 0.5f` has to round
// twice (multiply, then add) to reproduce the reference arithmetic bit for bit.
#include <mutex>

#include "ti8_common.h"
#include "index_math.h"
#include "quant_math.h"

namespace ti8 {

// 128-point Walsh-Hadamard transform of a row segment held as 8 consecutive bf16 per lane by 16
// consecutive lanes: butterflies in the fixed order stride 1, 2, 4 (in registers), 8, 16, 32, 64
// (across lanes), fp32, un-normalised; one rounding to bf16.
//
// Which lane holds which 16-byte chunk is chosen so that every cross-lane stage is ONE instruction.
// Lane l (of its row of 16) holds chunk idx::had_chunk(l) = l ^ (l & 4 ? 3 : 0); then the partners
// of the four stages (chunk ^ 1, ^ 2, ^ 4, ^ 8) sit in lanes l ^ 1, l ^ 2, l ^ 7, l ^ 8, each a single
// DPP pattern (two quad_perms, row_half_mirror, row_ror:8; there is none for l ^ 4).  A stage is
// (a, b) -> (a + b, a - b) with a in the lane whose chunk bit is clear; here every lane computes
// own + sigma * partner with sigma = +1 / -1 for a clear / set chunk bit (an fma with a DPP operand:
// the product with +-1 is exact, so the one rounding is that of the add or subtract).  The upper
// lane thereby gets b - a, the NEGATIVE of its result; as both partners of a later stage carry the
// same number of such flips, the stages stay as they are and a lane ends with all its values
// multiplied by had_sign(lane) = -1 if its chunk index has an odd number of bits set.  The callers
// quantise with the scale multiplied by the same sign (exact; absmax does not see signs).
struct HadLane {
    float sigma[4];   // per stage: -1 where the lane's chunk has that bit set
    float sign;       // what the lane's results are multiplied by
};
__device__ __forceinline__ HadLane had_lane(int lane) {
    const int c = idx::had_chunk(lane & 15);
    HadLane h;
#pragma unroll
    for (int k = 0; k < 4; ++k) h.sigma[k] = ((c >> k) & 1) ? -1.0f : 1.0f;
    h.sign = (__builtin_popcount(c) & 1) ? -1.0f : 1.0f;
    return h;
}
// One cross-lane stage for the 8 values of a lane: A[e] += partner's A[e] * SIGMA, the partner chosen by
// the DPP pattern.  Written out because the compiler keeps a separate v_mov_b32_dpp in front of an fma.
// A DPP operand must not be read within two instructions of the vector instruction that wrote it: inside
// a stage the eight chains are independent (each register was written eight instructions earlier), and
// the s_nop covers whatever the compiler placed in front of the stage.  All 64 lanes are active here.
#define TI8_HAD_FMAC(N, PATTERN) "v_fmac_f32_dpp %" #N ", %" #N ", %8 " PATTERN " row_mask:0xf bank_mask:0xf\n\t"
#define TI8_HAD_STAGE(A, SIGMA, PATTERN)                                                                                     \
    asm("s_nop 1\n\t" TI8_HAD_FMAC(0, PATTERN) TI8_HAD_FMAC(1, PATTERN) TI8_HAD_FMAC(2, PATTERN) TI8_HAD_FMAC(3, PATTERN)     \
        TI8_HAD_FMAC(4, PATTERN) TI8_HAD_FMAC(5, PATTERN) TI8_HAD_FMAC(6, PATTERN) TI8_HAD_FMAC(7, PATTERN)                  \
        : "+v"(A[0]), "+v"(A[1]), "+v"(A[2]), "+v"(A[3]), "+v"(A[4]), "+v"(A[5]), "+v"(A[6]), "+v"(A[7])                     \
        : "v"(SIGMA))

__device__ __forceinline__ uint4 fwht128_bf16_signed(const uint4& v, const HadLane& hl) {
    float a[8] = {bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y), bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w)};
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if ((e & h) == 0) {
                const float u = a[e], w = a[e + h];
                a[e] = u + w;
                a[e + h] = u - w;
            }
    TI8_HAD_STAGE(a, hl.sigma[0], "quad_perm:[1,0,3,2]");
    TI8_HAD_STAGE(a, hl.sigma[1], "quad_perm:[2,3,0,1]");
    TI8_HAD_STAGE(a, hl.sigma[2], "row_half_mirror");
    TI8_HAD_STAGE(a, hl.sigma[3], "row_ror:8");
    uint4 o;
    o.x = pack_bf16x2(a[0], a[1]);
    o.y = pack_bf16x2(a[2], a[3]);
    o.z = pack_bf16x2(a[4], a[5]);
    o.w = pack_bf16x2(a[6], a[7]);
    return o;
}

// 4 x 4 byte transpose: out[e] = byte e of r0, r1, r2, r3 (r0 in the low byte), two rounds of
// v_perm_b32 (selector values 0-3 pick bytes of the second operand, 4-7 of the first)
__device__ __forceinline__ void transpose4x4_bytes(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t* out) {
    const uint32_t t01l = __builtin_amdgcn_perm(r1, r0, 0x05010400u), t01h = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    const uint32_t t23l = __builtin_amdgcn_perm(r3, r2, 0x05010400u), t23h = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    out[0] = __builtin_amdgcn_perm(t23l, t01l, 0x05040100u);
    out[1] = __builtin_amdgcn_perm(t23l, t01l, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(t23h, t01h, 0x05040100u);
    out[3] = __builtin_amdgcn_perm(t23h, t01h, 0x07060302u);
}

// ---------------------------------------------------------------------------------
// 128 x (128*NSUB) tile per workgroup of 256 threads.  Thread t owns, in every
// 128x128 sub-tile, rows {64h + 4*(t/16) + j : h<2, j<4} x columns [8*(t%16), +8):
// a wave load instruction covers whole 256-byte row segments, and the 4-row patches
// transpose in registers for the optional transposed output (staged through LDS so
// that the global writes of qT are 128-byte rows too).
template <int NSUB, bool WRITE_Q, bool WRITE_QT, int ARITH = ARITH_KERNEL>
__device__ __forceinline__ void quant_block_tile(
    const uint16_t* __restrict__ x, int64_t bsx, int64_t ldx, int8_t* __restrict__ q, int64_t bsq, int64_t ldq,
    int8_t* __restrict__ qT, int64_t bsqt, int64_t ldqt, float* __restrict__ s, int64_t ssb, int64_t ssr,
    int64_t ssc, int nrb, int ncb, const QMode& mode, int tile_index, float* red4, uint32_t* tileT) {
    const idx::TileId tl = idx::qblock_tile(tile_index, nrb, ncb);
    const int b = tl.b, rb = tl.rb, cb = tl.cb;

    const int tid = threadIdx.x;
    const int cc = tid & 15;   // 8-column chunk
    const int rg = tid >> 4;   // 4-row group

    // Addresses: a uniform tile origin (scalar registers) plus a 32-bit per-thread byte offset -- the thread's first row times
    // the leading dimension, once, then uniform multiples of the leading dimension -- instead of a 64-bit product per access
    // (two quarter-rate multiply-adds each, a fifth of this kernel's vector time); the host checks that 128 rows fit 32 bits.
    const char* xt = reinterpret_cast<const char*>(x + idx::qblock_origin(b, bsx, rb, ldx, cb, 128 * NSUB));
    const uint32_t ldx_b = (uint32_t)ldx * 2u;
    const uint32_t x_first = (uint32_t)idx::qblock_row(tid, 0, 0) * ldx_b + (uint32_t)idx::qblock_col(tid) * 2u;
    uint4 v[NSUB][2][4];
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j)   // row = idx::qblock_row(tid, h, j) = the first row + 64 h + j
                v[u][h][j] = *reinterpret_cast<const uint4*>(xt + (x_first + (uint32_t)(idx::qblock_row(0, h, j)) * ldx_b + (uint32_t)(u * 256)));

    float amax = 0.0f;
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) amax = absmax8(v[u][h][j], amax);
    amax = block_max_256(amax, red4);
    amax = amax_floor_arith<ARITH>(amax, mode.eps_add);
    const float scale = group_multiplier<ARITH>(amax);
    if (tid == 0) s[b * ssb + rb * ssr + cb * ssc] = stored_scale_arith<ARITH>(amax, scale, mode);

#pragma unroll
    for (int u = 0; u < NSUB; ++u) {
        uint2 o[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[h][j] = quant8<ARITH>(v[u][h][j], scale);

        if (WRITE_Q) {
            char* qt = reinterpret_cast<char*>(q + idx::qblock_origin(b, bsq, rb, ldq, cb, 128 * NSUB));
            const uint32_t q_first = (uint32_t)idx::qblock_row(tid, 0, 0) * (uint32_t)ldq + (uint32_t)idx::qblock_col(tid) + (uint32_t)(u * 128);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *reinterpret_cast<uint2*>(qt + (q_first + (uint32_t)idx::qblock_row(0, h, j) * (uint32_t)ldq)) = o[h][j];
        }
        if (WRITE_QT) {  // NSUB == 1 only (checked on the host)
#pragma unroll
            for (int h = 0; h < 2; ++h)
            {
                uint32_t w[8];
                transpose4x4_bytes(o[h][0].x, o[h][1].x, o[h][2].x, o[h][3].x, w);
                transpose4x4_bytes(o[h][0].y, o[h][1].y, o[h][2].y, o[h][3].y, w + 4);
#pragma unroll
                for (int e = 0; e < 8; ++e) tileT[(cc * 8 + e) * 33 + h * 16 + rg] = w[e];  // [column of x][4-row group]
            }
            __syncthreads();
            char* qtt = reinterpret_cast<char*>(qT + idx::qblock_origin(b, bsqt, cb, ldqt, rb, 128));   // tile (cb, rb) of the transposed tensor
            const uint32_t t_first = (uint32_t)idx::qblock_t_row(tid, 0) * (uint32_t)ldqt + (uint32_t)idx::qblock_t_col(tid);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int tr = idx::qblock_t_row(tid, p);  // row of the transposed tile = column of x
                const int tc = tid & 7;                    // 16-byte chunk along the original rows
                uint4 w;
                w.x = tileT[tr * 33 + tc * 4 + 0];
                w.y = tileT[tr * 33 + tc * 4 + 1];
                w.z = tileT[tr * 33 + tc * 4 + 2];
                w.w = tileT[tr * 33 + tc * 4 + 3];
                *reinterpret_cast<uint4*>(qtt + (t_first + (uint32_t)idx::qblock_t_row(0, p) * (uint32_t)ldqt)) = w;
            }
        }
    }
}


template <int NSUB, bool WRITE_Q, bool WRITE_QT, int ARITH = ARITH_KERNEL>
__global__ __launch_bounds__(256) void quant_block_kernel(
    const uint16_t* __restrict__ x, int64_t bsx, int64_t ldx, int8_t* __restrict__ q, int64_t bsq, int64_t ldq,
    int8_t* __restrict__ qT, int64_t bsqt, int64_t ldqt, float* __restrict__ s, int64_t ssb, int64_t ssr,
    int64_t ssc, int nrb, int ncb, QMode mode) {
    __shared__ float red4[4];
    __shared__ uint32_t tileT[WRITE_QT ? 128 * 33 : 1];
    quant_block_tile<NSUB, WRITE_Q, WRITE_QT, ARITH>(x, bsx, ldx, q, bsq, ldq, qT, bsqt, ldqt, s, ssb, ssr, ssc, nrb, ncb, mode,
                                                     blockIdx.x, red4, tileT);
}

// Several operands in one launch (a training step quantises X and dY the same way: one launch
// instead of two saves a kernel boundary and fills the tail of one operand with tiles of the next).
// Workgroup w works on tile w - first[i] of the operand i whose range holds w.
constexpr int QBLOCK_MULTI_MAX = 4;
struct QBlockOperand {
    const uint16_t* x;
    int64_t bsx, ldx;
    int8_t* q;
    int64_t bsq, ldq;
    int8_t* qT;
    int64_t bsqt, ldqt;
    float* s;
    int64_t ssb, ssr, ssc;
    int nrb, ncb;
};
struct QBlockMulti {
    QBlockOperand op[QBLOCK_MULTI_MAX];
    int first[QBLOCK_MULTI_MAX + 1];   // first workgroup of operand i; first[count] = grid size
    int count;
    unsigned int* clear;               // words that the launch zeroes on the side (thread i of the grid clears word i), or NULL
    int clear_words;
};

template <bool WRITE_Q, bool WRITE_QT>
__global__ __launch_bounds__(256) void quant_block_multi_kernel(const QBlockMulti m, QMode mode) {
    __shared__ float red4[4];
    __shared__ uint32_t tileT[WRITE_QT ? 128 * 33 : 1];
    {   // the next launch's maxima workspace, cleared here so that no launch exists only to clear it
        const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (w < m.clear_words) m.clear[w] = 0u;
    }
    int i = 0;
#pragma unroll
    for (int k = 1; k < QBLOCK_MULTI_MAX; ++k)
        if (k < m.count && (int)blockIdx.x >= m.first[k]) i = k;
    const QBlockOperand& o = m.op[i];
    const int local = (int)blockIdx.x - m.first[i];
    quant_block_tile<1, WRITE_Q, WRITE_QT, ARITH_KERNEL>(o.x, o.bsx, o.ldx, o.q, o.bsq, o.ldq, o.qT, o.bsqt, o.ldqt, o.s, o.ssb, o.ssr,
                                                         o.ssc, o.nrb, o.ncb, mode, local, red4, tileT);
}


// ---------------------------------------------------------------------------------
// Block quantiser with the 128-point Hadamard rotation fused in (one read of x, no bf16
// intermediate in HBM).  ALONG_ROWS = false: rotate every 128-column row segment of the tile
// and write q in the orientation of x.  ALONG_ROWS = true: rotate every 128-row column segment;
// the tile goes through LDS once (16-byte chunks swizzled by row group) so that each thread
// picks up 8 consecutive ROWS of one column, after which the same code runs on the transposed
// tile and q comes out transposed, [C][R] -- the K-contiguous operand of a GEMM that contracts
// over the rows (tokens).
// SCALE selects the quantisation group: HAD_BLOCK = the 128 x 128 tile (one scale per tile);
// HAD_COLMAX / HAD_COL (ALONG_ROWS only) = a whole column of the rotated operand, i.e. a whole row
// of the transposed output, in two launches: HAD_COLMAX only merges the tile's column maxima
// into ws[C] (atomic max on the float bits), HAD_COL quantises with the scales that ws then
// holds and writes them to s[C].
enum { HAD_BLOCK = 0, HAD_COLMAX = 1, HAD_COL = 2 };

template <bool ALONG_ROWS, int SCALE = HAD_BLOCK>
__global__ __launch_bounds__(256) void quant_block_had_kernel(
    const uint16_t* __restrict__ x, int64_t bsx, int64_t ldx, int8_t* __restrict__ q, int64_t bsq, int64_t ldq,
    float* __restrict__ s, int64_t ssb, int64_t ssr, int64_t ssc, int nrb, int ncb, QMode mode,
    unsigned int* __restrict__ ws = nullptr) {
    static_assert(SCALE == HAD_BLOCK || ALONG_ROWS, "column-wise scales go with the rotation along rows");
    __shared__ float red4[4];
    __shared__ __attribute__((aligned(16))) uint16_t tile[ALONG_ROWS ? 128 * 128 : 8];

    int t = blockIdx.x;
    const int cb = t % ncb;
    t /= ncb;
    const int rb = t % nrb;
    const int b = t / nrb;
    const int tid = threadIdx.x;
    // chunk of 8 elements along the rotated direction that this lane holds (see fwht128_bf16_signed)
    const int cc = idx::had_chunk(tid & 15), rg = tid >> 4;
    const int lc = ALONG_ROWS ? (tid & 15) : cc;   // chunk of the row that this lane loads

    const uint16_t* xt = x + b * bsx + (int64_t)rb * 128 * ldx + (int64_t)cb * 128;
    uint4 v[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[h][j] = *reinterpret_cast<const uint4*>(xt + (int64_t)(h * 64 + rg * 4 + j) * ldx + lc * 8);

    if (ALONG_ROWS) {
        // tile[row][chunk ^ (row >> 3)]: the 16 lanes that later read one column from 16 different
        // row groups hit 16 different chunks
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = h * 64 + rg * 4 + j;
                *reinterpret_cast<uint4*>(tile + row * 128 + ((lc ^ (row >> 3)) & 15) * 8) = v[h][j];
            }
        __syncthreads();
        // now this thread is (transposed row = original column h*64 + rg*4 + j, transposed columns = original rows 8cc..8cc+7)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = h * 64 + rg * 4 + j;
                uint32_t e[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int row = cc * 8 + k;   // row >> 3 == cc
                    e[k] = tile[row * 128 + (((col >> 3) ^ cc) & 15) * 8 + (col & 7)];
                }
                v[h][j] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
            }
    }
    const HadLane hl = had_lane(tid);
    if (SCALE != HAD_BLOCK) {
        // this thread holds, per (h, j), 8 consecutive rows of column h*64 + rg*4 + j of the tile;
        // the 16 lanes with the same rg hold the other rows of that column
        int8_t* qcol = q + (int64_t)cb * 128 * ldq + (int64_t)rb * 128 + cc * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = cb * 128 + h * 64 + rg * 4 + j;
                const uint4 r = fwht128_bf16_signed(v[h][j], hl);
                if (SCALE == HAD_COLMAX) {
                    const float m = row16_max(absmax8(r, 0.0f));
                    if (cc == 0) atomicMax(ws + col, __float_as_uint(m));
                } else {
                    const float amax = amax_floor(__uint_as_float(ws[col]), mode.eps_add);
                    const float scale = 127.0f / amax;
                    if (rb == 0 && cc == 0) s[col] = stored_scale(amax, scale, mode);
                    *reinterpret_cast<uint2*>(qcol + (int64_t)(h * 64 + rg * 4 + j) * ldq) = quant8(r, scale * hl.sign);
                }
            }
        return;
    }
    float amax = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[h][j] = fwht128_bf16_signed(v[h][j], hl);
            amax = absmax8(v[h][j], amax);
        }
    amax = block_max_256(amax, red4);
    amax = amax_floor(amax, mode.eps_add);
    const float scale = 127.0f / amax;
    if (tid == 0) s[b * ssb + rb * ssr + cb * ssc] = stored_scale(amax, scale, mode);
    const float lane_scale = scale * hl.sign;
    // output tile origin: same orientation as x, or transposed
    int8_t* qt = ALONG_ROWS ? q + b * bsq + (int64_t)cb * 128 * ldq + (int64_t)rb * 128
                            : q + b * bsq + (int64_t)rb * 128 * ldq + (int64_t)cb * 128;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<uint2*>(qt + (int64_t)(h * 64 + rg * 4 + j) * ldq + cc * 8) = quant8(v[h][j], lane_scale);
}

// ---------------------------------------------------------------------------------
// Per-row quantiser, one pass.  WG_ROW = false: one wavefront per row (4 rows per
// workgroup); WG_ROW = true: one 256-thread workgroup per row.  Each thread keeps
// NLOAD 16-byte chunks of its row in registers.  GROUP16: one scale per 16 chunks
// (128 columns) instead of per row.
template <int NLOAD, bool WG_ROW, bool GROUP16, bool HAD, int ARITH = ARITH_KERNEL>
__global__ __launch_bounds__(256) void quant_row_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                        int8_t* __restrict__ q, int64_t ldq,
                                                        float* __restrict__ s, int64_t rows, int cols,
                                                        QMode mode) {
    __shared__ float red4[4];
    constexpr int T = WG_ROW ? 256 : 64;
    const int t = WG_ROW ? threadIdx.x : (threadIdx.x & 63);
    const int64_t row = idx::qrow_row(blockIdx.x, threadIdx.x >> 6, WG_ROW);
    if (row >= rows) return;  // whole wave (or workgroup) leaves together
    const int nchunk = cols >> 3;
    const uint16_t* xr = x + row * ldx;

    uint4 v[NLOAD];
    HadLane hl;
    if (HAD) hl = had_lane(threadIdx.x);
    const float lane_sign = HAD ? hl.sign : 1.0f;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
        // the 16 chunks of a 128-column group sit in 16 consecutive lanes (T % 16 == 0), with the
        // rotation in the order that fwht128_bf16_signed wants (cols % 128 == 0 then: the permuted
        // chunk is inside the row whenever the plain one is)
        const int c = HAD ? idx::had_chunk(idx::qrow_chunk(t, i, T)) : idx::qrow_chunk(t, i, T);
        v[i] = (c < nchunk) ? *reinterpret_cast<const uint4*>(xr + c * 8) : make_uint4(0, 0, 0, 0);
        if (HAD) v[i] = fwht128_bf16_signed(v[i], hl);
    }
    int8_t* qr = q + row * ldq;
    if (GROUP16) {
        const int ngrp = cols >> 7;
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int c = HAD ? idx::had_chunk(idx::qrow_chunk(t, i, T)) : idx::qrow_chunk(t, i, T);
            const float amax = amax_floor(row16_max(absmax8(v[i], 0.0f)), mode.eps_add);
            const float scale = 127.0f / amax;
            if (c < nchunk) {
                *reinterpret_cast<uint2*>(qr + c * 8) = quant8(v[i], scale * lane_sign);
                if ((c & 15) == 0) s[row * ngrp + (c >> 4)] = stored_scale(amax, scale, mode);
            }
        }
        return;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) amax = absmax8(v[i], amax);
    if (WG_ROW)
        amax = block_max_256(amax, red4);
    else
        amax = wave_max(amax);
    amax = amax_floor_arith<ARITH>(amax, mode.eps_add);
    const float scale = group_multiplier<ARITH>(amax);
    if (t == 0) s[row] = stored_scale_arith<ARITH>(amax, scale, mode);
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
        const int c = HAD ? idx::had_chunk(idx::qrow_chunk(t, i, T)) : idx::qrow_chunk(t, i, T);
        if (c < nchunk) *reinterpret_cast<uint2*>(qr + c * 8) = quant8<ARITH>(v[i], scale * lane_sign);
    }
}

__global__ void fill_u32_kernel(unsigned int* p, int n, unsigned int v) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Quantise a 128x128 tile of x with one scale PER COLUMN (from ws[]) and write it
// transposed: qT[c][r].  Same thread <-> element map as quant_block_kernel.
__global__ __launch_bounds__(256) void quant_col_t_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                          int8_t* __restrict__ qT, int64_t ldqt,
                                                          float* __restrict__ s, const float* __restrict__ ws,
                                                          int ncb, QMode mode) {
    __shared__ uint32_t tileT[128 * 33];
    __shared__ __attribute__((aligned(16))) float sc[128];
    const int cb = blockIdx.x % ncb;
    const int rb = blockIdx.x / ncb;
    const int tid = threadIdx.x;
    const int cc = tid & 15, rg = tid >> 4;
    const uint16_t* xt = x + (int64_t)rb * 128 * ldx + (int64_t)cb * 128;

    uint4 v[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[h][j] = *reinterpret_cast<const uint4*>(xt + (int64_t)(h * 64 + rg * 4 + j) * ldx + cc * 8);

    // the tile's 128 column scales: one division each, shared through LDS
    if (tid < 128) {
        const float amax = amax_floor(ws[cb * 128 + tid], mode.eps_add);
        const float sv = 127.0f / amax;
        sc[tid] = sv;
        if (rb == 0) s[cb * 128 + tid] = stored_scale(amax, sv, mode);
    }
    __syncthreads();
    float scale[8];
    {
        const float4 c0 = *reinterpret_cast<const float4*>(&sc[cc * 8]), c1 = *reinterpret_cast<const float4*>(&sc[cc * 8 + 4]);
        scale[0] = c0.x; scale[1] = c0.y; scale[2] = c0.z; scale[3] = c0.w;
        scale[4] = c1.x; scale[5] = c1.y; scale[6] = c1.z; scale[7] = c1.w;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) put_row_by_cols(v[h][j], scale, j, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) tileT[(cc * 8 + e) * 33 + h * 16 + rg] = w[e] ^ UNBIAS4;
    }
    __syncthreads();
    int8_t* qtt = qT + (int64_t)cb * 128 * ldqt + (int64_t)rb * 128;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int tr = p * 32 + (tid >> 3);
        const int tc = tid & 7;
        uint4 w;
        w.x = tileT[tr * 33 + tc * 4 + 0];
        w.y = tileT[tr * 33 + tc * 4 + 1];
        w.z = tileT[tr * 33 + tc * 4 + 2];
        w.w = tileT[tr * 33 + tc * 4 + 3];
        *reinterpret_cast<uint4*>(qtt + (int64_t)tr * ldqt + tc * 16) = w;
    }
}

// ---------------------------------------------------------------------------------
// Column absmax, and optionally row absmax, of x in one read (WITH_ROWS: both quantisations of
// an operand that a training step needs, by rows for one GEMM, by columns -- transposed -- for
// another).  Workgroup = TR rows x 256 columns; thread t reads the 16-byte chunk t%32 of rows
// t/32 + 8i.  |x| of a bf16 is its bit pattern without the sign, and non-negative bf16 order
// like their 16-bit patterns, so the maxima are taken on packed pairs of 16-bit integers (no
// unpacking, two elements per instruction) and widened to fp32 bit patterns (<< 16) at the end,
// where they are merged into ws[] with an unsigned atomic max.
// NaN elements are left out of the maxima, as the float maxima of the other quantisers (v_max_f32)
// and the reference's tl.max leave them out: the patterns are biased by 0x7f, which moves the NaN
// patterns 0x7f81 .. 0x7fff -- and only those -- to 0x8000 and above, and compared as SIGNED
// 16-bit values (v_pk_max_i16), where those are negative and lose against every number, infinity
// included; a group of nothing but NaN ends below the biased zero and counts as zero.
// Row maxima meet over the 32
// lanes of a half-wave through DPP moves; column maxima over the two half-waves by a lane swap
// and over the four waves through LDS.  Short tiles win although they issue more atomics: 32
// rows measured 6 % faster than 128 on 4096 x 4096 and on 8192 x 4096 (more workgroups per CU,
// so the loads of one overlap the reductions of another); 16 and 64 rows are 1-2 % slower than 32.
constexpr int ABSMAX_ROWS = 32;
constexpr uint32_t ABS_BIAS2 = 0x007f007fu;   // the bias of both halves = the biased zero

typedef short ti8_i16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_i16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(ti8_i16x2, a), __builtin_bit_cast(ti8_i16x2, b)));
}
// |x| patterns of two bf16, biased
__device__ __forceinline__ uint32_t abs_biased2(uint32_t w) { return (w & 0x7fff7fffu) + ABS_BIAS2; }
// biased maxima of both halves -> the larger |x| pattern (0 if everything was NaN)
__device__ __forceinline__ uint32_t unbias_max2(uint32_t m) {
    const int lo = static_cast<short>(m & 0xffffu), hi = static_cast<short>(m >> 16);
    return static_cast<uint32_t>(max(max(lo, hi), 0x7f) - 0x7f);
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ uint32_t dpp_pk_max_i16(uint32_t v) {
    return pk_max_i16(v, (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false));
}

template <int TR, bool WITH_ROWS>  // TR: rows of x per workgroup (8, 16, ... 128)
__global__ __launch_bounds__(256) void absmax_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                     unsigned int* __restrict__ ws_row,
                                                     unsigned int* __restrict__ ws_col, int64_t R, int C) {
    constexpr int NR = TR / 8;
    __shared__ uint4 part[4][32];  // [wave][chunk]: 8 biased column maxima per chunk
    __shared__ uint32_t rowpart[WITH_ROWS ? TR : 1];  // row maxima of the tile (fp32 bit patterns)
    const int tid = threadIdx.x;
    const int cc = tid & 31, rg = tid >> 5;
    const int c0 = blockIdx.x * 256 + cc * 8;
    const int64_t r0 = (int64_t)blockIdx.y * TR;
    uint32_t m[4] = {ABS_BIAS2, ABS_BIAS2, ABS_BIAS2, ABS_BIAS2};  // columns c0 + 2k (low half) and c0 + 2k + 1 (high half)
    uint32_t rmax[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) rmax[i] = ABS_BIAS2;
    if (c0 < C) {
        uint4 v[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i)
            v[i] = *reinterpret_cast<const uint4*>(x + (r0 + rg + 8 * i) * ldx + c0);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const uint32_t a0 = abs_biased2(v[i].x), a1 = abs_biased2(v[i].y), a2 = abs_biased2(v[i].z), a3 = abs_biased2(v[i].w);
            m[0] = pk_max_i16(m[0], a0);
            m[1] = pk_max_i16(m[1], a1);
            m[2] = pk_max_i16(m[2], a2);
            m[3] = pk_max_i16(m[3], a3);
            if (WITH_ROWS) rmax[i] = pk_max_i16(pk_max_i16(a0, a1), pk_max_i16(a2, a3));
        }
    }
    if (WITH_ROWS) {
        // over the 32 lanes (tid % 32) that hold the same rows: quad_perm lane^1, lane^2,
        // row_half_mirror, row_mirror, row_bcast:15 into rows 1 and 3 -> valid in lanes 16-31, 48-63
        // (one step for all rows at a time: the chains are independent and interleave)
#pragma unroll
        for (int i = 0; i < NR; ++i) rmax[i] = dpp_pk_max_i16<0xB1>(rmax[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) rmax[i] = dpp_pk_max_i16<0x4E>(rmax[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) rmax[i] = dpp_pk_max_i16<0x141>(rmax[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) rmax[i] = dpp_pk_max_i16<0x140>(rmax[i]);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const uint32_t a = dpp_pk_max_i16<0x142, 0xA>(rmax[i]);
            if (cc == 16 + i) rowpart[rg + 8 * i] = unbias_max2(a) << 16;
        }
    }
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int k = 0; k < 4; ++k) {  // lanes l and l ^ 32 hold the same columns
        const auto r = __builtin_amdgcn_permlane32_swap(m[k], m[k], false, false);
        m[k] = pk_max_i16(r[0], r[1]);
    }
#endif
    if ((tid & 32) == 0) part[tid >> 6][cc] = make_uint4(m[0], m[1], m[2], m[3]);
    __syncthreads();
    // the tile's rows are consecutive words of ws_row: one atomic instruction for all of them
    // (an instruction per row and half-wave, two lanes each, measured 2.5 us slower on 8192 x 4096)
    if (WITH_ROWS && tid < TR) atomicMax(ws_row + r0 + tid, rowpart[tid]);
    const uint32_t* pw = reinterpret_cast<const uint32_t*>(part);  // dword j of a wave's row: columns 2j, 2j + 1
    const uint32_t u = pk_max_i16(pk_max_i16(pw[tid >> 1], pw[128 + (tid >> 1)]),
                                  pk_max_i16(pw[256 + (tid >> 1)], pw[384 + (tid >> 1)]));
    const int b = static_cast<short>((tid & 1) ? (u >> 16) : (u & 0xffffu));   // biased, signed
    const uint32_t a = static_cast<uint32_t>(max(b, 0x7f) - 0x7f);
    const int c = blockIdx.x * 256 + tid;
    if (c < C) atomicMax(ws_col + c, a << 16);
}

// Quantise a 128x128 tile of x twice: with one scale per ROW into q (same orientation) and
// with one scale per COLUMN into qT (transposed).  Thread <-> element map of quant_block_kernel.
__global__ __launch_bounds__(256) void quant_rowcol_kernel(const uint16_t* __restrict__ x, int64_t ldx,
                                                           int8_t* __restrict__ q, int64_t ldq,
                                                           float* __restrict__ s_row, int8_t* __restrict__ qT,
                                                           int64_t ldqt, float* __restrict__ s_col,
                                                           const float* __restrict__ ws_row,
                                                           const float* __restrict__ ws_col,
                                                           float* __restrict__ ws_next, int64_t R, int ncb, QMode mode) {
    __shared__ uint32_t tileT[128 * 33];
    __shared__ __attribute__((aligned(16))) float sc[256];  // [0,128): row scales, [128,256): column scales
    const int cb = blockIdx.x % ncb;
    const int rb = blockIdx.x / ncb;
    const int tid = threadIdx.x;
    const int cc = tid & 15, rg = tid >> 4;
    const uint16_t* xt = x + (int64_t)rb * 128 * ldx + (int64_t)cb * 128;

    uint4 v[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[h][j] = *reinterpret_cast<const uint4*>(xt + (int64_t)(h * 64 + rg * 4 + j) * ldx + cc * 8);

    // the tile's 128 row scales and 128 column scales: one division per thread, shared through LDS
    {
        const bool is_row = tid < 128;
        const int idx = tid & 127;
        const int64_t at = is_row ? (int64_t)rb * 128 + idx : (int64_t)cb * 128 + idx;
        // two-part workspace: clear the part that the next call will collect its maxima in
        if (ws_next && (is_row ? cb == 0 : rb == 0)) ws_next[is_row ? at : R + at] = 0.0f;
        const float amax = amax_floor(is_row ? ws_row[at] : ws_col[at], mode.eps_add);
        const float scale = 127.0f / amax;
        sc[tid] = scale;
        if (is_row ? cb == 0 : rb == 0) (is_row ? s_row : s_col)[at] = stored_scale(amax, scale, mode);
    }
    __syncthreads();
    float cscale[8];
    {
        const float4 c0 = *reinterpret_cast<const float4*>(&sc[128 + cc * 8]), c1 = *reinterpret_cast<const float4*>(&sc[132 + cc * 8]);
        cscale[0] = c0.x; cscale[1] = c0.y; cscale[2] = c0.z; cscale[3] = c0.w;
        cscale[4] = c1.x; cscale[5] = c1.y; cscale[6] = c1.z; cscale[7] = c1.w;
    }
    int8_t* qt = q + (int64_t)rb * 128 * ldq + (int64_t)cb * 128 + cc * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = h * 64 + rg * 4 + j;
            *reinterpret_cast<uint2*>(qt + (int64_t)row * ldq) = quant8(v[h][j], sc[row]);
            put_row_by_cols(v[h][j], cscale, j, w);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) tileT[(cc * 8 + e) * 33 + h * 16 + rg] = w[e] ^ UNBIAS4;
    }
    __syncthreads();
    int8_t* qtt = qT + (int64_t)cb * 128 * ldqt + (int64_t)rb * 128;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int tr = p * 32 + (tid >> 3);
        const int tc = tid & 7;
        uint4 w;
        w.x = tileT[tr * 33 + tc * 4 + 0];
        w.y = tileT[tr * 33 + tc * 4 + 1];
        w.z = tileT[tr * 33 + tc * 4 + 2];
        w.w = tileT[tr * 33 + tc * 4 + 3];
        *reinterpret_cast<uint4*>(qtt + (int64_t)tr * ldqt + tc * 16) = w;
    }
}

// arithmetic variant a flag set asks for (only ti8_quant_block and ti8_quant_row take the flags)
static int arith_of(int qflags) {
    return (qflags & TI8_Q_TORCH_BF16) ? ARITH_TORCH_BF16 : ((qflags & TI8_Q_TORCH_ROUND) ? ARITH_TORCH_F32 : ARITH_KERNEL);
}

}  // namespace ti8

using namespace ti8;

// argument checks of one block-quantiser operand (shared by ti8_quant_block and ti8_quant_block_multi)
static int check_qblock_operand(const char* fn, const void* x, int64_t bsx, int64_t ldx, const int8_t* q, int64_t bsq, int64_t ldq,
                                const int8_t* qT, int64_t bsqt, int64_t ldqt, const float* s, int64_t B, int64_t R, int64_t C, int group_c) {
    if (!x || !s || (!q && !qT)) return fail(TI8_ERR_NULL, "%s: x, s and one of q/qT are required", fn);
    if (group_c != 128 && group_c != 256) return fail(TI8_ERR_MODE, "%s: group_c must be 128 or 256, got %d", fn, group_c);
    if (qT && group_c != 128) return fail(TI8_ERR_MODE, "%s: the transposed output needs group_c = 128", fn);
    if (B <= 0 || R <= 0 || C <= 0 || R % 128 || C % group_c)
        return fail(TI8_ERR_SHAPE, "%s: need B>0, R%%128==0, C%%%d==0; got B=%lld R=%lld C=%lld", fn, group_c,
                    (long long)B, (long long)R, (long long)C);
    if (ldx < C || (q && ldq < C) || (qT && ldqt < R)) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than the row length", fn);
    if (!aligned16(x) || (ldx % 8) || (bsx % 8) || (q && (!aligned16(q) || (ldq % 16) || (bsq % 16))) ||
        (qT && (!aligned16(qT) || (ldqt % 16) || (bsqt % 16))))
        return fail(TI8_ERR_ALIGN, "%s: pointers must be 16-byte aligned and strides multiples of 16 bytes", fn);
    if (B * (R / 128) * (C / group_c) > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "%s: too many tiles", fn);
    // the kernels address a tile's 128 rows with 32-bit byte offsets from the tile's origin
    if (ldx > 0x00ffffff || (q && ldq > 0x00ffffff) || (qT && ldqt > 0x00ffffff)) return fail(TI8_ERR_SHAPE, "%s: leading dimension beyond 2^24 - 1", fn);
    return TI8_OK;
}

extern "C" int ti8_quant_block(const void* x, int64_t bsx, int64_t ldx, int8_t* q, int64_t bsq, int64_t ldq,
                               int8_t* qT, int64_t bsqt, int64_t ldqt, float* s, int64_t ssb, int64_t ssr,
                               int64_t ssc, int64_t B, int64_t R, int64_t C, int group_c, int qflags,
                               int inv_mode, ti8_stream_t stream) {
    QMode mode;
    const int arith = arith_of(qflags);
    qflags &= ~(TI8_Q_TORCH_ROUND | TI8_Q_TORCH_BF16);
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (arith != ARITH_KERNEL && (group_c != 128 || qT || (qflags & (TI8_Q_EPS_ADD | TI8_Q_SCALE_BF16)) || inv_mode != TI8_INV_RCP_OF_SCALE))
        return fail(TI8_ERR_MODE, "ti8_quant_block: the torch arithmetic goes with group_c = 128, q only, no other flag and TI8_INV_RCP_OF_SCALE");
    if (qflags & TI8_Q_HAD128) return fail(TI8_ERR_MODE, "ti8_quant_block: use ti8_quant_block_had128 for the Hadamard rotation");
    if (int e = check_qblock_operand("ti8_quant_block", x, bsx, ldx, q, bsq, ldq, qT, bsqt, ldqt, s, B, R, C, group_c)) return e;
    const int64_t ntiles = B * (R / 128) * (C / group_c);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const int nrb = (int)(R / 128), ncb = (int)(C / group_c);
    dim3 grid((unsigned)ntiles), block(256);
#define TI8_LAUNCH_QB(NSUB, WQ, WQT)                                                                          \
    hipLaunchKernelGGL((quant_block_kernel<NSUB, WQ, WQT>), grid, block, 0, st, xp, bsx, ldx, q, bsq, ldq, qT, \
                       bsqt, ldqt, s, ssb, ssr, ssc, nrb, ncb, mode)
    if (arith == ARITH_TORCH_F32)
        hipLaunchKernelGGL((quant_block_kernel<1, true, false, ARITH_TORCH_F32>), grid, block, 0, st, xp, bsx, ldx, q, bsq, ldq, qT, bsqt, ldqt, s, ssb, ssr, ssc, nrb, ncb, mode);
    else if (arith == ARITH_TORCH_BF16)
        hipLaunchKernelGGL((quant_block_kernel<1, true, false, ARITH_TORCH_BF16>), grid, block, 0, st, xp, bsx, ldx, q, bsq, ldq, qT, bsqt, ldqt, s, ssb, ssr, ssc, nrb, ncb, mode);
    else if (group_c == 256) TI8_LAUNCH_QB(2, true, false);
    else if (q && qT) TI8_LAUNCH_QB(1, true, true);
    else if (q) TI8_LAUNCH_QB(1, true, false);
    else TI8_LAUNCH_QB(1, false, true);
#undef TI8_LAUNCH_QB
    return check_launch("ti8_quant_block");
}

extern "C" int ti8_quant_block_multi(const ti8_qblock_operand* operands, int count, int qflags, int inv_mode, ti8_stream_t stream) {
    return ti8::quant_block_multi_and_clear(operands, count, qflags, inv_mode, nullptr, 0, stream);
}

int ti8::fill_words(unsigned int* p, int64_t words, unsigned int value, hipStream_t st) {
    if (words <= 0) return TI8_OK;
    if (!p || words > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "fill: bad buffer");
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, p, (int)words, value);
    return check_launch("fill");
}

int ti8::quant_block_multi_and_clear(const ti8_qblock_operand* operands, int count, int qflags, int inv_mode,
                                     unsigned int* clear, int64_t clear_words, ti8_stream_t stream) {
    const char* fn = "ti8_quant_block_multi";
    QMode mode;
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (qflags & TI8_Q_HAD128) return fail(TI8_ERR_MODE, "%s: the Hadamard rotation is not offered here", fn);
    if (!operands) return fail(TI8_ERR_NULL, "%s: operands is required", fn);
    if (count < 1 || count > QBLOCK_MULTI_MAX) return fail(TI8_ERR_SHAPE, "%s: between 1 and %d operands, got %d", fn, QBLOCK_MULTI_MAX, count);
    QBlockMulti m;
    int64_t total = 0;
    for (int i = 0; i < count; ++i) {
        const ti8_qblock_operand& o = operands[i];
        if (int e = check_qblock_operand(fn, o.x, o.bsx, o.ldx, o.q, o.bsq, o.ldq, o.qT, o.bsqt, o.ldqt, o.s, o.B, o.R, o.C, 128)) return e;
        if ((o.q != nullptr) != (operands[0].q != nullptr) || (o.qT != nullptr) != (operands[0].qT != nullptr))
            return fail(TI8_ERR_MODE, "%s: every operand must ask for the same outputs (q, qT or both)", fn);
        m.op[i] = QBlockOperand{static_cast<const uint16_t*>(o.x), o.bsx, o.ldx, o.q, o.bsq, o.ldq, o.qT, o.bsqt, o.ldqt, o.s,
                                o.ssb, o.ssr, o.ssc, (int)(o.R / 128), (int)(o.C / 128)};
        m.first[i] = (int)total;
        total += o.B * (o.R / 128) * (o.C / 128);
        if (total > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "%s: too many tiles", fn);
    }
    for (int i = count; i < QBLOCK_MULTI_MAX; ++i) { m.op[i] = m.op[0]; m.first[i] = (int)total; }
    m.first[QBLOCK_MULTI_MAX] = (int)total;
    m.count = count;
    hipStream_t st = static_cast<hipStream_t>(stream);
    m.clear = nullptr;
    m.clear_words = 0;
    if (clear && clear_words > 0) {
        if (clear_words <= total * 256) {
            m.clear = clear;
            m.clear_words = (int)clear_words;
        } else if (int e = fill_words(clear, clear_words, 0u, st)) {   // more words than threads: a launch of its own
            return e;
        }
    }
    dim3 grid((unsigned)total), block(256);
    const bool wq = operands[0].q != nullptr, wqt = operands[0].qT != nullptr;
    if (wq && wqt) hipLaunchKernelGGL((quant_block_multi_kernel<true, true>), grid, block, 0, st, m, mode);
    else if (wq) hipLaunchKernelGGL((quant_block_multi_kernel<true, false>), grid, block, 0, st, m, mode);
    else hipLaunchKernelGGL((quant_block_multi_kernel<false, true>), grid, block, 0, st, m, mode);
    return check_launch(fn);
}

extern "C" int ti8_quant_row(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s, int64_t rows,
                             int64_t cols, int group, int qflags, int inv_mode, ti8_stream_t stream) {
    QMode mode;
    const int arith = arith_of(qflags);
    qflags &= ~(TI8_Q_TORCH_ROUND | TI8_Q_TORCH_BF16);
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (arith != ARITH_KERNEL && (group != 0 || (qflags & (TI8_Q_EPS_ADD | TI8_Q_SCALE_BF16 | TI8_Q_HAD128)) || inv_mode != TI8_INV_RCP_OF_SCALE))
        return fail(TI8_ERR_MODE, "ti8_quant_row: the torch arithmetic goes with group = 0, no other flag and TI8_INV_RCP_OF_SCALE");
    if (!x || !q || !s) return fail(TI8_ERR_NULL, "ti8_quant_row: x, q and s are required");
    if (group != 0 && group != 128) return fail(TI8_ERR_MODE, "ti8_quant_row: group must be 0 or 128, got %d", group);
    if (rows <= 0 || cols <= 0 || cols % 128 || cols > 32768 || rows > 0x7fffffffLL)
        return fail(TI8_ERR_SHAPE, "ti8_quant_row: need rows>0, cols%%128==0, cols<=32768; got rows=%lld cols=%lld",
                    (long long)rows, (long long)cols);
    if (ldx < cols || ldq < cols) return fail(TI8_ERR_SHAPE, "ti8_quant_row: leading dimension smaller than cols");
    if (!aligned16(x) || !aligned16(q) || (ldx % 8) || (ldq % 16))
        return fail(TI8_ERR_ALIGN, "ti8_quant_row: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const int nchunk = (int)(cols / 8);
    const int c = (int)cols;
    const bool had = (qflags & TI8_Q_HAD128) != 0;
#define TI8_LAUNCH_QR(NL, WG, G16, GRID) \
    do { if (!G16 && arith == ARITH_TORCH_F32) hipLaunchKernelGGL((quant_row_kernel<NL, WG, false, false, ARITH_TORCH_F32>), dim3((unsigned)(GRID)), dim3(256), 0, st, xp, ldx, q, ldq, s, rows, c, mode); \
         else if (!G16 && arith == ARITH_TORCH_BF16) hipLaunchKernelGGL((quant_row_kernel<NL, WG, false, false, ARITH_TORCH_BF16>), dim3((unsigned)(GRID)), dim3(256), 0, st, xp, ldx, q, ldq, s, rows, c, mode); \
         else if (had) hipLaunchKernelGGL((quant_row_kernel<NL, WG, G16, true>), dim3((unsigned)(GRID)), dim3(256), 0, st, xp, ldx, q, ldq, s, rows, c, mode); \
         else hipLaunchKernelGGL((quant_row_kernel<NL, WG, G16, false>), dim3((unsigned)(GRID)), dim3(256), 0, st, xp, ldx, q, ldq, s, rows, c, mode); } while (0)
    const idx::QRowConfig cfg = idx::qrow_config(nchunk, group == 128);
    const int64_t grid = cfg.wg_row ? rows : (rows + 3) / 4;
    if (group == 128) {
        if (!cfg.wg_row) TI8_LAUNCH_QR(8, false, true, grid);
        else if (cfg.nload == 8) TI8_LAUNCH_QR(8, true, true, grid);
        else TI8_LAUNCH_QR(16, true, true, grid);
    } else if (!cfg.wg_row) {
        if (cfg.nload == 2) TI8_LAUNCH_QR(2, false, false, grid);
        else if (cfg.nload == 4) TI8_LAUNCH_QR(4, false, false, grid);
        else TI8_LAUNCH_QR(8, false, false, grid);
    } else if (cfg.nload == 4) TI8_LAUNCH_QR(4, true, false, grid);
    else if (cfg.nload == 8) TI8_LAUNCH_QR(8, true, false, grid);
    else TI8_LAUNCH_QR(16, true, false, grid);
#undef TI8_LAUNCH_QR
    return check_launch("ti8_quant_row");
}

extern "C" int ti8_quant_col_t(const void* x, int64_t ldx, int8_t* qT, int64_t ldqt, float* s, float* ws,
                               int64_t R, int64_t C, int qflags, int inv_mode, ti8_stream_t stream) {
    QMode mode;
    if (int e = parse_mode(qflags, inv_mode, &mode)) return e;
    if (!x || !qT || !s || !ws) return fail(TI8_ERR_NULL, "ti8_quant_col_t: x, qT, s and ws are required");
    if (R <= 0 || C <= 0 || R % 128 || C % 128 || C > 0x7fffffffLL)
        return fail(TI8_ERR_SHAPE, "ti8_quant_col_t: need R%%128==0 and C%%128==0; got R=%lld C=%lld", (long long)R, (long long)C);
    if (ldx < C || ldqt < R) return fail(TI8_ERR_SHAPE, "ti8_quant_col_t: leading dimension smaller than the row length");
    if (!aligned16(x) || !aligned16(qT) || (ldx % 8) || (ldqt % 16))
        return fail(TI8_ERR_ALIGN, "ti8_quant_col_t: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    const int64_t ntiles = (R / 128) * (C / 128);
    if (ntiles > 0x7fffffffLL || R / ABSMAX_ROWS > 65535) return fail(TI8_ERR_SHAPE, "ti8_quant_col_t: too many tiles");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    unsigned int* wsu = reinterpret_cast<unsigned int*>(ws);
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((C + 255) / 256)), dim3(256), 0, st, wsu, (int)C, 0u);
    if (qflags & TI8_Q_HAD128) {
        // rotate every 128-row segment of every column first (x^T rotated along its contraction
        // dim): both passes redo the rotation on the tile they read instead of storing it
        const int nrb = (int)(R / 128), ncb = (int)(C / 128);
        hipLaunchKernelGGL((quant_block_had_kernel<true, HAD_COLMAX>), dim3((unsigned)ntiles), dim3(256), 0, st, xp, (int64_t)0, ldx,
                           qT, (int64_t)0, ldqt, s, (int64_t)0, (int64_t)0, (int64_t)0, nrb, ncb, mode, wsu);
        hipLaunchKernelGGL((quant_block_had_kernel<true, HAD_COL>), dim3((unsigned)ntiles), dim3(256), 0, st, xp, (int64_t)0, ldx,
                           qT, (int64_t)0, ldqt, s, (int64_t)0, (int64_t)0, (int64_t)0, nrb, ncb, mode, wsu);
        return check_launch("ti8_quant_col_t");
    }
    hipLaunchKernelGGL((absmax_kernel<ABSMAX_ROWS, false>), dim3((unsigned)((C + 255) / 256), (unsigned)(R / ABSMAX_ROWS)),
                       dim3(256), 0, st, xp, ldx, (unsigned int*)nullptr, wsu, R, (int)C);
    hipLaunchKernelGGL(quant_col_t_kernel, dim3((unsigned)ntiles), dim3(256), 0, st, xp, ldx, qT, ldqt, s, ws,
                       (int)(C / 128), mode);
    return check_launch("ti8_quant_col_t");
}

// The launches of ti8_quant_row_col_t on a workspace the caller of this function has settled on
static int quant_row_col_t_impl(const char* fn, const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s_row, int8_t* qT,
                                int64_t ldqt, float* s_col, float* ws, int64_t R, int64_t C, int qflags, int inv_mode,
                                ti8_stream_t stream) {
    const bool pingpong = (qflags & TI8_Q_WS_PINGPONG) != 0, second = (qflags & TI8_Q_WS_SECOND) != 0;
    const bool is_zero = (qflags & TI8_Q_WS_IS_ZERO) != 0;
    if (second && !pingpong) return fail(TI8_ERR_MODE, "%s: TI8_Q_WS_SECOND needs TI8_Q_WS_PINGPONG", fn);
    if (is_zero && pingpong) return fail(TI8_ERR_MODE, "%s: TI8_Q_WS_IS_ZERO and TI8_Q_WS_PINGPONG exclude each other", fn);
    QMode mode;
    if (int e = parse_mode(qflags & ~(TI8_Q_WS_PINGPONG | TI8_Q_WS_SECOND | TI8_Q_WS_IS_ZERO), inv_mode, &mode)) return e;
    if (qflags & TI8_Q_HAD128) return fail(TI8_ERR_MODE, "%s: the Hadamard rotation is not offered here", fn);
    if (!x || !q || !s_row || !qT || !s_col || !ws) return fail(TI8_ERR_NULL, "%s: x, q, s_row, qT, s_col and ws are required", fn);
    if (R <= 0 || C <= 0 || R % 128 || C % 128 || C > 0x7fffffffLL)
        return fail(TI8_ERR_SHAPE, "%s: need R%%128==0 and C%%128==0; got R=%lld C=%lld", fn, (long long)R, (long long)C);
    if (ldx < C || ldq < C || ldqt < R) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than the row length", fn);
    if (!aligned16(x) || !aligned16(q) || !aligned16(qT) || (ldx % 8) || (ldq % 16) || (ldqt % 16))
        return fail(TI8_ERR_ALIGN, "%s: pointers must be 16-byte aligned and strides multiples of 16 bytes", fn);
    const int64_t ntiles = (R / 128) * (C / 128);
    if (ntiles > 0x7fffffffLL || R / ABSMAX_ROWS > 65535 || R + C > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "%s: too many tiles", fn);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    float* ws_next = nullptr;  // [R row maxima][C column maxima], once or twice
    if (pingpong) {
        ws_next = second ? ws : ws + R + C;
        ws = second ? ws + R + C : ws;
    }
    unsigned int* wsu = reinterpret_cast<unsigned int*>(ws);
    if (!pingpong && !is_zero)
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((R + C + 255) / 256)), dim3(256), 0, st, wsu, (int)(R + C), 0u);
    hipLaunchKernelGGL((absmax_kernel<ABSMAX_ROWS, true>), dim3((unsigned)((C + 255) / 256), (unsigned)(R / ABSMAX_ROWS)),
                       dim3(256), 0, st, xp, ldx, wsu, wsu + R, R, (int)C);
    hipLaunchKernelGGL(quant_rowcol_kernel, dim3((unsigned)ntiles), dim3(256), 0, st, xp, ldx, q, ldq, s_row, qT, ldqt,
                       s_col, ws, ws + R, ws_next, R, (int)(C / 128), mode);
    return check_launch(fn);
}

extern "C" int ti8_quant_row_col_t(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s_row, int8_t* qT,
                                   int64_t ldqt, float* s_col, float* ws, int64_t R, int64_t C, int qflags,
                                   int inv_mode, ti8_stream_t stream) {
    return quant_row_col_t_impl("ti8_quant_row_col_t", x, ldx, q, ldq, s_row, qT, ldqt, s_col, ws, R, C, qflags, inv_mode, stream);
}

// ---------------------------------------------------------------------------------
// The same operation for callers that cannot allocate: the row and column maxima are collected in
// a fixed array in device memory that belongs to the library (one copy per GPU, held until the
// process ends) instead of a workspace argument.
namespace ti8 {
static __device__ __align__(256) unsigned int scratch[TI8_NOALLOC_MAX_ROWS_PLUS_COLS];

// Device address of `scratch` on the current device.  In host code the array's name is only a
// handle for hipGetSymbolAddress, never an address a kernel can use; each GPU has its own copy at
// its own address, looked up once per device (with that device current) and kept.
static int scratch_address(const char* fn, float** out) {
    constexpr int MAX_DEV = 64;
    static std::mutex mu;
    static float* addr[MAX_DEV] = {nullptr};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(TI8_ERR_HIP, "%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEV) return fail(TI8_ERR_HIP, "%s: device index %d out of range", fn, dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(TI8_ERR_HIP, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
        addr[dev] = static_cast<float*>(p);
    }
    *out = addr[dev];
    return TI8_OK;
}

int init_quant_scratch() {
    float* p = nullptr;
    return scratch_address("ti8_init", &p);
}
}  // namespace ti8

extern "C" int ti8_quant_row_col_t_noalloc(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s_row, int8_t* qT,
                                           int64_t ldqt, float* s_col, int64_t R, int64_t C, int qflags,
                                           int inv_mode, ti8_stream_t stream) {
    const char* fn = "ti8_quant_row_col_t_noalloc";
    if (qflags & (TI8_Q_WS_PINGPONG | TI8_Q_WS_SECOND | TI8_Q_WS_IS_ZERO))
        return fail(TI8_ERR_MODE, "%s: the workspace flags belong to ti8_quant_row_col_t (there is no workspace argument here)", fn);
    if (R > 0 && C > 0 && R + C > TI8_NOALLOC_MAX_ROWS_PLUS_COLS)
        return fail(TI8_ERR_SHAPE, "%s: R + C = %lld exceeds the library's fixed scratch of %d floats; use ti8_quant_row_col_t with a workspace",
                    fn, (long long)(R + C), TI8_NOALLOC_MAX_ROWS_PLUS_COLS);
    float* ws = nullptr;
    if (int e = scratch_address(fn, &ws)) return e;
    // the array keeps the last call's maxima: the shared launch sequence starts with the fill kernel
    // that zeroes the R + C words this call uses (a kernel, not a memset, so the call can be captured)
    return quant_row_col_t_impl(fn, x, ldx, q, ldq, s_row, qT, ldqt, s_col, ws, R, C, qflags, inv_mode, stream);
}

extern "C" int ti8_quant_block_had128(const void* x, int64_t bsx, int64_t ldx, int8_t* q, int64_t bsq, int64_t ldq,
                                      float* s, int64_t ssb, int64_t ssr, int64_t ssc, int64_t B, int64_t R, int64_t C,
                                      int along_rows, int qflags, int inv_mode, ti8_stream_t stream) {
    QMode mode;
    if (int e = parse_mode(qflags & ~TI8_Q_HAD128, inv_mode, &mode)) return e;
    if (!x || !q || !s) return fail(TI8_ERR_NULL, "ti8_quant_block_had128: x, q and s are required");
    if (B <= 0 || R <= 0 || C <= 0 || R % 128 || C % 128)
        return fail(TI8_ERR_SHAPE, "ti8_quant_block_had128: need B>0, R%%128==0, C%%128==0; got B=%lld R=%lld C=%lld", (long long)B, (long long)R, (long long)C);
    if (ldx < C || ldq < (along_rows ? R : C)) return fail(TI8_ERR_SHAPE, "ti8_quant_block_had128: leading dimension smaller than the row length");
    if (!aligned16(x) || !aligned16(q) || (ldx % 8) || (bsx % 8) || (ldq % 16) || (bsq % 16))
        return fail(TI8_ERR_ALIGN, "ti8_quant_block_had128: pointers must be 16-byte aligned and strides multiples of 16 bytes");
    const int64_t ntiles = B * (R / 128) * (C / 128);
    if (ntiles > 0x7fffffffLL) return fail(TI8_ERR_SHAPE, "ti8_quant_block_had128: too many tiles");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    if (along_rows)
        hipLaunchKernelGGL(quant_block_had_kernel<true>, dim3((unsigned)ntiles), dim3(256), 0, st, xp, bsx, ldx, q, bsq, ldq, s, ssb, ssr, ssc, (int)(R / 128), (int)(C / 128), mode);
    else
        hipLaunchKernelGGL(quant_block_had_kernel<false>, dim3((unsigned)ntiles), dim3(256), 0, st, xp, bsx, ldx, q, bsq, ldq, s, ssb, ssr, ssc, (int)(R / 128), (int)(C / 128), mode);
    return check_launch("ti8_quant_block_had128");
}
