// INT8 NT GEMM for few rows (decode-like shapes: up to 256 rows, in steps of 32).
//
// With so few rows the tiled kernel of gemm.hip has only N/128 workgroups, and each walks the
// whole K behind a two-stage LDS pipeline: its time is load latency, not MFMA.  Here C is cut
// into 32 x 32 blocks, one per workgroup, (N/32) * (M/32) of them, and K is split over the four
// waves of the workgroup, each of which runs its own load -> LDS -> MFMA pipeline with no
// barrier in the loop.
//
// The arithmetic and the epilogue are those of the tiled kernel's int32 and fast-promotion paths,
// operation for operation; only the order in which K tiles are added differs (four partial sums
// per output, K tiles walked from a workgroup-dependent start).  The int32 path is therefore
// bit-identical to the tiled kernel, the promoted path differs by fp32 association only.
#include "gemm_args.h"

namespace ti8 {

// s_waitcnt vmcnt(n) (gfx9 encoding: vmcnt in bits 3:0 and 15:14) and lgkmcnt(0) (bits 11:8),
// expcnt untouched (bits 6:4)
#define TI8_WAIT_VMCNT_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | 0x0070)

// A workgroup owns 32 x 32 of C and its four waves split K into quarters.  Every wave streams ITS
// quarter of both operands through a private LDS ring (WS_STAGES stages of [A 32 rows][B 32 rows]
// = 8 KiB, filled by global_load_lds in the swizzled layout of the tiled kernel), waits only
// for its own loads and never for another wave; the four partial results meet in LDS at the end
// and are added in the fixed order q0 + q1 + q2 + q3 (int32: exact; fp32: deterministic).
// Independent streams hide the per-tile latency chain (load -> LDS -> MFMA -> convert) that one
// stream per workgroup behind a barrier exposes: a version with 64 x 32 blocks, an 8-stage ring
// shared by the workgroup and one barrier per K tile took 14.4 us where this one takes 11.2 us
// (128 rows, K = N = 4096).  Two stages = 64 KiB per workgroup, so two workgroups share a CU.
constexpr int WS_STAGES = 2;
constexpr int WS_STAGE_BYTES = 2 * 32 * 128;
constexpr int WS_LOADS = 8;  // global->LDS instructions per wave and stage

template <bool I32FULL>
__global__ __launch_bounds__(256) void gemm_i8_wavering_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];  // 4 waves x WS_STAGES x 8 KiB

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int batch = blockIdx.y;
    const int mtiles = g.M >> 5, nstrips = g.N >> 5;
    int strip, mt;
    if ((nstrips & 7) == 0) {   // workgroups that share a strip of B on one XCD (ids 8 apart)
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        strip = (idx / mtiles) * 8 + xcd;
        mt = idx % mtiles;
    } else {
        strip = blockIdx.x / mtiles;
        mt = blockIdx.x % mtiles;
    }
    const int n0 = strip * 32, m0 = mt * 32;
    const int nk = g.K >> 7;
    const int kbeg = (wave * nk) >> 2, kend = ((wave + 1) * nk) >> 2;
    const int nq = kend - kbeg;

    // ---- global -> LDS (same slab layout and swizzle as the other kernels): 4 instructions of A
    // (rows 8i .. 8i+7) and 4 of B per stage, all issued by the wave that consumes them
    const int ld_row = lane >> 3;
    uint32_t voffA[2], voffB[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int ch = (lane & 7) ^ ld_row ^ p;
        voffA[p] = (uint32_t)(ld_row * (int)g.lda + ch * 16);
        voffB[p] = (uint32_t)(ld_row * (int)g.ldb + ch * 16);
    }
    const int8_t* baseA = g.A + (int64_t)batch * g.bsa + (int64_t)m0 * g.lda;
    const int8_t* baseB = g.B + (int64_t)batch * g.bsb + (int64_t)n0 * g.ldb;
    const int64_t strideA8 = 8 * g.lda, strideB8 = 8 * g.ldb;
    int8_t* const ring = smem + wave * (WS_STAGES * WS_STAGE_BYTES);
    // step i of this wave's walk is K tile kbeg + (i + rot) mod nq: workgroups start at different
    // tiles so that they do not ask the same memory channels for their lines at the same time
    const int rot = nq > 0 ? (int)(((blockIdx.x >> 3) * 3u + blockIdx.y) % (unsigned)nq) : 0;
    auto tile_of_step = [&](int i) {
        int j = min(i, max(nq - 1, 0)) + rot;   // past the end: the last one again, into a free stage
        if (j >= nq) j -= nq;
        return min(kbeg + max(j, 0), nk - 1);
    };
    auto issue_stage = [&](int i) {
        int8_t* st = ring + (i & (WS_STAGES - 1)) * WS_STAGE_BYTES;
        const int koff = tile_of_step(i) * 128;
        issue_tile_loads<4>(baseA + koff, strideA8, voffA, 0, st);
        issue_tile_loads<4>(baseB + koff, strideB8, voffB, 0, st + 4096);
    };

    // ---- scales: unconditional loads (an operand that contributes no in-loop factor is read with
    // stride 0 and dropped; a load under a branch would be waited for on the spot), issued before
    // the tile loads
    const bool divide = !I32FULL && g.combine == TI8_COMBINE_DIV_PROD;
    const bool a_in = !I32FULL && g.sa.mode != TI8_SCALE_ROW, b_in = !I32FULL && g.sb.mode != TI8_SCALE_ROW;
    float fvec[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (!I32FULL) {
        const int sha = g.sa.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0, shb = g.sb.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0;
        const float* pa = g.sa.p + (int64_t)batch * g.sa.bs + (a_in ? (int64_t)(m0 >> 7) * g.sa.rs : 0);
        const float* pb = g.sb.p + (int64_t)batch * g.sb.bs + (b_in ? (int64_t)(n0 >> 7) * g.sb.rs : 0);
        const int64_t ska = a_in ? g.sa.ks : 0, skb = b_in ? g.sb.ks : 0;
        float fa[4], fb[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int kt = min(c * 64 + lane, nk - 1);
            fa[c] = pa[(int64_t)(kt >> sha) * ska];
            fb[c] = pb[(int64_t)(kt >> shb) * skb];
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float f = (a_in ? fa[c] : 1.0f) * (b_in ? fb[c] : 1.0f);
            if (divide) f = 1.0f / f;
            fvec[c] = f;
        }
    }
    // epilogue scales of the 4 outputs this thread will finish: row t/8, columns 4*(t%8) .. +3
    const int e_row = threadIdx.x >> 3, e_col = (threadIdx.x & 7) * 4;
    const bool row_part = I32FULL || g.sa.mode == TI8_SCALE_ROW, col_part = I32FULL || g.sb.mode == TI8_SCALE_ROW;
    float rowm = g.sa.p[(int64_t)batch * g.sa.bs + (row_part ? (int64_t)(m0 + e_row) * g.sa.rs : 0)];
    float coln[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) coln[c] = g.sb.p[(int64_t)batch * g.sb.bs + (col_part ? (int64_t)(n0 + e_col + c) * g.sb.rs : 0)];
    if (divide) {
        rowm = 1.0f / rowm;
#pragma unroll
        for (int c = 0; c < 4; ++c) coln[c] = 1.0f / coln[c];
    }

    const int fr_row = lane & 31, fr_half = lane >> 5;
    const int sw = (lane & 7) ^ ((lane >> 3) & 1);
    int choff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) choff[ks] = ((ks * 2 + fr_half) ^ sw) * 16;
    const int a_off = fr_row * 128, b_off = 4096 + fr_row * 128;

    const v16i vzero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16i acc = vzero;
    float accf[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) accf[i] = 0.0f;

#pragma unroll
    for (int s = 0; s < WS_STAGES - 1; ++s) issue_stage(s);
    // pin the scale vectors to registers here (they are older than the tile loads, so this waits
    // for nothing else): a load still pending at the loop's entry makes the compiler drain the
    // whole load queue at the top of every iteration
    asm volatile("" : "+v"(rowm));
#pragma unroll
    for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(coln[c]));

    auto factor_of_step = [&](int i) -> float {
        const int kt = tile_of_step(i);
        const int l = kt & 63, c = kt >> 6;
        const float v0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[0]), l));
        const float v1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[1]), l));
        const float v2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[2]), l));
        const float v3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[3]), l));
        return c == 0 ? v0 : (c == 1 ? v1 : (c == 2 ? v2 : v3));
    };
    v16i d = vzero;
    float f_prev = 0.0f;
    for (int i = 0; i < nq; ++i) {
        // own loads of step i landed (at most the WS_STAGES - 2 younger steps outstanding); own
        // LDS reads of step i - 1 returned, so its stage can be refilled.  No barrier: nobody
        // else touches this wave's ring.
        TI8_WAIT_VMCNT_LGKM0((WS_STAGES - 2) * WS_LOADS);
        issue_stage(i + WS_STAGES - 1);
        const int8_t* st = ring + (i & (WS_STAGES - 1)) * WS_STAGE_BYTES;
        v4i fa[4], fb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            fa[ks] = *reinterpret_cast<const v4i*>(st + a_off + choff[ks]);
            fb[ks] = *reinterpret_cast<const v4i*>(st + b_off + choff[ks]);
        }
        __builtin_amdgcn_sched_barrier(0);   // all eight reads go out before anything else
        if (I32FULL) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks], fb[ks], acc, 0, 0, 0);
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[r] = __builtin_fmaf(static_cast<float>(d[r]), f_prev, accf[r]);
            __builtin_amdgcn_sched_barrier(0);
            d = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0], fb[0], vzero, 0, 0, 0);
#pragma unroll
            for (int ks = 1; ks < 4; ++ks) d = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks], fb[ks], d, 0, 0, 0);
            f_prev = factor_of_step(i);
        }
    }
    if (!I32FULL) {
#pragma unroll
        for (int r = 0; r < 16; ++r) accf[r] = __builtin_fmaf(static_cast<float>(d[r]), f_prev, accf[r]);
    }
    // every load (the redundant ones of the last steps included) has landed and every wave is
    // done with its ring before the rings are reused for the partial results
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    uint32_t* part = reinterpret_cast<uint32_t*>(smem);   // [K quarter][32 rows][32 columns]
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int row = 8 * (i >> 2) + 4 * fr_half + (i & 3);
        part[(wave * 32 + row) * 32 + fr_row] = I32FULL ? static_cast<uint32_t>(acc[i]) : __float_as_uint(accf[i]);
    }
    __syncthreads();
    uint4 pq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) pq[q] = *reinterpret_cast<const uint4*>(part + (q * 32 + e_row) * 32 + e_col);
    const uint32_t w0[4] = {pq[0].x, pq[0].y, pq[0].z, pq[0].w}, w1[4] = {pq[1].x, pq[1].y, pq[1].z, pq[1].w};
    const uint32_t w2[4] = {pq[2].x, pq[2].y, pq[2].z, pq[2].w}, w3[4] = {pq[3].x, pq[3].y, pq[3].z, pq[3].w};
    float t[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float v;
        if (I32FULL) {
            v = static_cast<float>(static_cast<int32_t>(w0[c] + w1[c] + w2[c] + w3[c])) * rowm;
            v = v * coln[c];
            if (g.post_scale != 0.0f) v = __uint_as_float(f32_to_bf16_bits(v) << 16) * g.post_scale;
        } else {
            v = __uint_as_float(w0[c]) + __uint_as_float(w1[c]);
            v = v + __uint_as_float(w2[c]);
            v = v + __uint_as_float(w3[c]);
            if (row_part) v = v * rowm;
            if (col_part) v = v * coln[c];
            if (g.out_scale != 1.0f) v = v * g.out_scale;
        }
        t[c] = v;
    }
    uint2 o;
    o.x = pack_bf16x2(t[0], t[1]);
    o.y = pack_bf16x2(t[2], t[3]);
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(g.C) + (int64_t)batch * g.bsc + (int64_t)(m0 + e_row) * g.ldc + n0 + e_col) = o;
}

bool skinny_supported(const GemmArgs& a) {
    // factors that vary inside a 32 x 32 block (one scale per row or column AND K tile) and more
    // than 256 K tiles are left to the tiled kernels
    if (a.sa.mode == TI8_SCALE_ROW_K128 || a.sb.mode == TI8_SCALE_ROW_K128) return false;
    if (a.K > 256 * 128) return false;
    return (int64_t)(a.N / 32) * (a.M / 32) <= 0x7fffffffLL;
}

constexpr size_t WAVERING_LDS_BYTES = (size_t)4 * WS_STAGES * WS_STAGE_BYTES;

int init_skinny_kernels() {
    static OncePerDevice once_i32, once_promote;
    hipError_t e = raise_lds_limit(once_i32, reinterpret_cast<const void*>(gemm_i8_wavering_kernel<true>), (int)WAVERING_LDS_BYTES);
    if (e == hipSuccess) e = raise_lds_limit(once_promote, reinterpret_cast<const void*>(gemm_i8_wavering_kernel<false>), (int)WAVERING_LDS_BYTES);
    if (e != hipSuccess) return fail(TI8_ERR_HIP, "gemm: cannot raise the LDS limit to %zu: %s", WAVERING_LDS_BYTES, hipGetErrorString(e));
    return TI8_OK;
}

static int launch_wavering(const GemmArgs& a, int64_t batch, bool i32_full, hipStream_t st) {
    constexpr size_t shmem = WAVERING_LDS_BYTES;
    if (int e = init_skinny_kernels()) return e;
    dim3 grid((unsigned)((a.N / 32) * (a.M / 32)), (unsigned)batch), block(256);
    if (i32_full)
        hipLaunchKernelGGL(gemm_i8_wavering_kernel<true>, grid, block, shmem, st, a);
    else
        hipLaunchKernelGGL(gemm_i8_wavering_kernel<false>, grid, block, shmem, st, a);
    note_gemm_kernel(TI8_KERNEL_FEW_ROWS, 32, 32, i32_full ? EPI_ROWS : EPI_PROMOTE);
    return check_launch("ti8_gemm_i8_nt");
}

int launch_skinny(const GemmArgs& a, int64_t batch, bool i32_full, hipStream_t st) {
    return launch_wavering(a, batch, i32_full, st);
}

}  // namespace ti8
