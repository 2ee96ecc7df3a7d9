// INT8 NT GEMM for few rows (decode-like shapes: up to 256 tokens after padding).
//
// With so few rows the tiled kernel of gemm.hip has only N/128 workgroups, and each walks the
// whole K behind a two-stage LDS pipeline: its time is load latency, not MFMA.  Here C is cut
// into 64 x 32 blocks, one per workgroup of 4 waves, (N/32) * (M/64) of them, and each workgroup
// streams its operands through an 8-stage LDS ring (one 128-byte K tile per stage: 64 rows of A +
// 32 rows of B = 12 KiB), so that seven K tiles of loads are in flight per CU at any time:
//   * all four waves issue the loads of a stage (global_load_lds_dwordx4, whole 128-byte row
//     segments, the same swizzled LDS layout as the tiled kernel): two instructions of A and one
//     of B per wave and stage;
//   * waves 0 and 1 own one 32 x 32 block of C each and run the 4 MFMAs of a K tile on it; waves
//     2 and 3 only load;
//   * one barrier per K tile: it publishes the tile that has landed and frees the stage that was
//     consumed in the previous iteration, which is refilled at once.
// The arithmetic and the epilogue are those of the tiled kernel's int32 and fast-promotion paths,
// operation for operation; only the order of the K tiles is rotated per workgroup.  The int32
// path is therefore bit-identical to the tiled kernel, the promoted path differs by fp32
// association only.
#include "gemm_args.h"

namespace ti8 {

constexpr int SK_STAGES = 8;
constexpr int SK_A_BYTES = 64 * 128, SK_B_BYTES = 32 * 128, SK_STAGE_BYTES = SK_A_BYTES + SK_B_BYTES;
constexpr int SK_LOADS = 3;  // global->LDS instructions per wave and stage

// s_waitcnt vmcnt(n) (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
// and lgkmcnt(0) (bits 11:8), expcnt untouched (bits 6:4)
#define TI8_WAIT_VMCNT_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | 0x0070)

template <bool I32FULL>
__global__ __launch_bounds__(256) void gemm_i8_skinny_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];  // SK_STAGES x [A 64 rows][B 32 rows]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int batch = blockIdx.y;
    // Workgroup -> block of C.  Consecutive workgroup ids go round-robin over the 8 XCDs, each with
    // its own L2: the M/64 workgroups that share a 32-column strip of B are given ids 8 apart, so
    // that they meet in one L2 and the strip comes out of HBM once.
    const int mtiles = g.M >> 6, nstrips = g.N >> 5;
    int strip, mt;
    if ((nstrips & 7) == 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        strip = (idx / mtiles) * 8 + xcd;
        mt = idx % mtiles;
    } else {
        strip = blockIdx.x / mtiles;
        mt = blockIdx.x % mtiles;
    }
    const int n0 = strip * 32, m0 = mt * 64;
    const int nk = g.K >> 7;

    // ---- global -> LDS: wave w brings A rows 16w .. 16w+15 and B rows 8w .. 8w+7 of every K tile.
    // An instruction covers 8 rows: lane l lands at byte 16*l of its 1 KiB slab = (row l/8,
    // physical chunk l%8), and fetches the logical chunk that belongs there:
    // physical chunk p of row r holds logical chunk p ^ (r & 7) ^ ((r >> 3) & 1).
    const int ld_row = lane >> 3;
    uint32_t voffA[2], voffB[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int ch = (lane & 7) ^ ld_row ^ p;
        voffA[p] = (uint32_t)(ld_row * (int)g.lda + ch * 16);
        voffB[p] = (uint32_t)(ld_row * (int)g.ldb + ch * 16);
    }
    const int8_t* baseA = g.A + (int64_t)batch * g.bsa + (int64_t)(m0 + wave * 16) * g.lda;
    const int8_t* baseB = g.B + (int64_t)batch * g.bsb + (int64_t)(n0 + wave * 8) * g.ldb;
    const int64_t strideA8 = 8 * g.lda;
    // Workgroup-dependent starting tile: step i of the walk is K tile (i + rot) mod nk.  Rows are a
    // multiple of 4 KiB apart, so workgroups walking K in step would ask the same few L2 channels
    // for all their lines at the same time; rotated, the requests of the workgroups of an XCD
    // spread over the whole row.
    const int rot = (int)(((blockIdx.x >> 3) * 5u + blockIdx.y) % (unsigned)nk);
    auto issue_stage = [&](int i) {   // step i (clamped: past the end the last tile is re-read into a free stage)
        int8_t* st = smem + (i & (SK_STAGES - 1)) * SK_STAGE_BYTES;
        int kt = min(i, nk - 1) + rot;
        if (kt >= nk) kt -= nk;
        const int koff = kt * 128;
        issue_tile_loads<2>(baseA + koff, strideA8, voffA, 2 * wave, st + wave * 2048);
        issue_tile_loads<1>(baseB + koff, 0, voffB, wave, st + SK_A_BYTES + wave * 1024);
    };

    // ---- per-K-tile factors of the fast promotion, as in the tiled kernel: block scales are
    // uniform over a 32 x 32 block, all nk (<= 256) products are fetched once (lane l of fvec[c] =
    // K tile 64c + l) and picked with v_readlane; per-row scale vectors wait for the epilogue
    const bool divide = !I32FULL && g.combine == TI8_COMBINE_DIV_PROD;
    const bool a_in = !I32FULL && g.sa.mode != TI8_SCALE_ROW, b_in = !I32FULL && g.sb.mode != TI8_SCALE_ROW;
    const int cw = wave & 1;   // the 32-row block this wave computes (waves 2, 3 mirror 0, 1 and compute nothing)
    // All scale loads are unconditional (an operand that contributes nothing to a factor is read
    // with stride 0 and its value dropped): a load inside a branch is waited for on the spot, and
    // a dozen of those in a row cost more than the whole K loop.
    float fvec[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (!I32FULL) {
        const int sha = g.sa.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0, shb = g.sb.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0;
        const float* pa = g.sa.p + (int64_t)batch * g.sa.bs + (a_in ? (int64_t)((m0 + cw * 32) >> 7) * g.sa.rs : 0);
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
    // per-row scale vectors of the epilogue, fetched now so that nothing waits for them later
    const int fr_row = lane & 31, fr_half = lane >> 5;
    const bool row_part = I32FULL || g.sa.mode == TI8_SCALE_ROW, col_part = I32FULL || g.sb.mode == TI8_SCALE_ROW;
    float rowm[16];
    {
        const float* prow = g.sa.p + (int64_t)batch * g.sa.bs;
        const int64_t rs = row_part ? g.sa.rs : 0;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            rowm[i] = prow[(int64_t)(m0 + cw * 32 + 8 * (i >> 2) + 4 * fr_half + (i & 3)) * rs];
    }
    float coln = g.sb.p[(int64_t)batch * g.sb.bs + (col_part ? (int64_t)(n0 + fr_row) * g.sb.rs : 0)];
    if (divide) {
        coln = 1.0f / coln;
#pragma unroll
        for (int i = 0; i < 16; ++i) rowm[i] = 1.0f / rowm[i];
    }

    // ---- LDS -> MFMA operands (lane l: row l % 32, bytes 16*(l / 32) .. +15 of each 32-deep k-step)
    const int sw = (lane & 7) ^ ((lane >> 3) & 1);
    int choff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) choff[ks] = ((ks * 2 + fr_half) ^ sw) * 16;
    const int a_off = (cw * 32 + fr_row) * 128, b_off = SK_A_BYTES + fr_row * 128;

    const v16i vzero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16i acc = vzero;
    float accf[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) accf[i] = 0.0f;

#pragma unroll
    for (int s = 0; s < SK_STAGES - 1; ++s) issue_stage(s);
    // Pin the scale vectors to registers here (they are older than the tile loads just issued, so
    // this waits for nothing else): a load still pending at the loop's entry makes the compiler
    // drain the whole load queue at the top of every iteration.
#pragma unroll
    for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(rowm[i]));
    asm volatile("" : "+v"(coln));

    // Step i of a computing wave: read the operands of step i from LDS and, while they travel, fold
    // the finished dot products of step i - 1 (`d`) into the float accumulators; then the 4 MFMAs
    // of step i, whose result is picked up in the next step.
    auto factor_of_step = [&](int i) -> float {
        int kt = i + rot;
        if (kt >= nk) kt -= nk;
        const int l = kt & 63, c = kt >> 6;
        const float v0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[0]), l));
        const float v1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[1]), l));
        const float v2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[2]), l));
        const float v3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[3]), l));
        return c == 0 ? v0 : (c == 1 ? v1 : (c == 2 ? v2 : v3));
    };
    v16i d = vzero;
    float f_prev = 0.0f;
    for (int i = 0; i < nk; ++i) {
        // own loads of step i have landed once at most those of the SK_STAGES - 2 younger steps
        // are outstanding; own LDS reads of step i - 1 have returned (its stage is refilled below)
        TI8_WAIT_VMCNT_LGKM0((SK_STAGES - 2) * SK_LOADS);
        __syncthreads();
        issue_stage(i + SK_STAGES - 1);  // into the stage of step i - 1
        if (wave < 2) {
            const int8_t* st = smem + (i & (SK_STAGES - 1)) * SK_STAGE_BYTES;
            v4i fa[4], fb[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                fa[ks] = *reinterpret_cast<const v4i*>(st + a_off + choff[ks]);
                fb[ks] = *reinterpret_cast<const v4i*>(st + b_off + choff[ks]);
            }
            // all eight reads go out before anything else: left alone the scheduler pairs each
            // MFMA with its own two reads and waits for them four times in a row
            __builtin_amdgcn_sched_barrier(0);
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
    }
    if (!I32FULL) {
#pragma unroll
        for (int r = 0; r < 16; ++r) accf[r] = __builtin_fmaf(static_cast<float>(d[r]), f_prev, accf[r]);
    }
    // the redundant loads of the last iterations still target LDS: let them land before the
    // workgroup's LDS can be handed to another one
    __builtin_amdgcn_s_waitcnt(0);
    if (wave >= 2) return;

    // ---- epilogue: straight from the MFMA result layout (register i of lane l is row
    // 8*(i/4) + 4*(l/32) + i%4, column l%32 of the block); the block is only 2 KiB of bf16
    const int n = n0 + fr_row;
    uint16_t* crow = reinterpret_cast<uint16_t*>(g.C) + (int64_t)batch * g.bsc + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int m = m0 + cw * 32 + 8 * (i >> 2) + 4 * fr_half + (i & 3);
        float v;
        if (I32FULL) {
            v = static_cast<float>(acc[i]) * rowm[i];
            v = v * coln;
            if (g.post_scale != 0.0f) v = __uint_as_float(f32_to_bf16_bits(v) << 16) * g.post_scale;
        } else {
            v = accf[i];
            if (row_part) v = v * rowm[i];
            if (col_part) v = v * coln;
            if (g.out_scale != 1.0f) v = v * g.out_scale;
        }
        crow[(int64_t)m * g.ldc] = static_cast<uint16_t>(pack_bf16x2(v, 0.0f));
    }
}

bool skinny_supported(const GemmArgs& a) {
    // factors that vary inside a 32 x 32 block (one scale per row or column AND K tile) and more
    // than 256 K tiles are left to the tiled kernels
    if (a.sa.mode == TI8_SCALE_ROW_K128 || a.sb.mode == TI8_SCALE_ROW_K128) return false;
    if (a.K > 256 * 128) return false;
    return (int64_t)(a.N / 32) * (a.M / 64) <= 0x7fffffffLL;
}

int launch_skinny(const GemmArgs& a, int64_t batch, bool i32_full, hipStream_t st) {
    // M and N are multiples of 128 (checked by the caller), so 64 x 32 blocks tile C exactly
    constexpr size_t shmem = (size_t)SK_STAGES * SK_STAGE_BYTES;
    static thread_local int attr_dev = -1;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (attr_dev != dev) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_i8_skinny_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_i8_skinny_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return fail(TI8_ERR_HIP, "gemm: cannot raise the LDS limit to %zu: %s", shmem, hipGetErrorString(e));
        attr_dev = dev;
    }
    dim3 grid((unsigned)((a.N / 32) * (a.M / 64)), (unsigned)batch), block(256);
    if (i32_full)
        hipLaunchKernelGGL(gemm_i8_skinny_kernel<true>, grid, block, shmem, st, a);
    else
        hipLaunchKernelGGL(gemm_i8_skinny_kernel<false>, grid, block, shmem, st, a);
    return check_launch("ti8_gemm_i8_nt");
}

}  // namespace ti8
