// INT8 NT GEMM on CDNA4 i8 MFMA (v_mfma_i32_32x32x32_i8) with fused dequantisation.
//
// C[b][m][n] = dequant( sum_k A[b][m][k] * B[b][n][k] ), both operands K-contiguous.
//
// Data flow per workgroup (BM x BN output tile, K walked in tiles of 128 bytes):
//   HBM --global_load_lds_dwordx4--> LDS (double buffered, 16-byte chunks XOR-swizzled
//   by row so that the 32 rows a wave reads at one k offset fall in distinct banks)
//   --ds_read_b128--> MFMA operand registers --> int32 accumulators.
// A K tile is exactly one 128-deep quantisation block, so the block-channel variants
// convert and scale the int32 partial into an fp32 accumulator once per K tile.  Large
// block-channel shapes use a variant of the main loop (EPI_PROMOTE_CHAIN, described where it
// starts) that keeps no int32 accumulator from one K tile to the next.
//
// MFMA operand/result layout used (32x32x32 i8): lane l supplies row (l % 32) of its
// operand and the 16 bytes k = 16*(l / 32) .. +15 of the 32-deep slice (the same map
// for both operands, which is all an NT dot product needs); result register r of lane
// l is C[8*(r/4) + 4*(l/32) + r%4][l % 32] with rows from A and columns from B.
#include <type_traits>
#include "gemm_args.h"

namespace ti8 {

// Interleaving hint for one k-step: TM*TN MFMAs, with up to NDS LDS reads, NVM global->LDS
// loads and NVA*TM*TN VALU ops slotted one group per MFMA so that the matrix pipe never waits
// behind a burst of memory or vector instructions.
template <int NMFMA, int NDS, int NVM, int NVA>
__device__ __forceinline__ void interleave_hint() {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int q = 0; q < NMFMA; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                   // 1 MFMA
        if (NVA > 0) __builtin_amdgcn_sched_group_barrier(0x002, NVA, 0);    // NVA VALU
        if (q < NDS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // 1 DS read
        if (q < NVM) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);      // 1 VMEM read
    }
#endif
}

// Software pipeline of the main loop (per workgroup, K tile kt, LDS buffers cur = kt & 1):
//   k-step 0: MFMA on fragments(kt, 0) | read fragments(kt, 1)
//   k-step 1: MFMA on fragments(kt, 1) | read fragments(kt, 2)
//   k-step 2: MFMA on fragments(kt, 2) | read fragments(kt, 3)
//             wait: own loads of tile kt+1 landed, own LDS reads of buffer cur returned; BARRIER
//   k-step 3: MFMA on fragments(kt, 3) | read fragments(kt+1, 0) | issue tile kt+2 (one K tile of lead)
//             into buffer cur (every wave is past its last read of it)
// so there is one barrier per K tile, it sits where the next fragments are already in
// registers, and a tile's loads have a full K tile of MFMA time to land.
// One output tile of one GEMM: the whole kernel body.  `block_x` = index of the workgroup among the
// tiles of this GEMM, `batch` = batch index.
template <int BM, int BN, int WM, int WN, int EPI>
__device__ __forceinline__ void gemm_i8_tile(const GemmArgs& g, const int block_x, const int batch) {
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM / 32;  // 32x32 blocks per wave along M
    constexpr int TN = BN / WN / 32;
    constexpr int A_INSTR = BM / 8 / NW;  // global->LDS wave instructions per K tile per wave
    constexpr int B_INSTR = BN / 8 / NW;
    constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
    constexpr bool CHAIN = (EPI == EPI_PROMOTE_CHAIN || EPI == EPI_PROMOTE_CHAIN_LANE);
    constexpr bool FAST = (EPI == EPI_PROMOTE || EPI == EPI_PROMOTE_LANE || CHAIN);
    constexpr bool LANEB = (EPI == EPI_PROMOTE_LANE || EPI == EPI_PROMOTE_CHAIN_LANE);
    constexpr bool PROMOTE = (FAST || EPI == EPI_STRICT);
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile/wave mismatch");

    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    // layout: [A buf0][A buf1][B buf0][B buf1]
    int8_t* const ldsA = smem;
    int8_t* const ldsB = smem + 2 * A_BYTES;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keep it in an SGPR
    const int wm = wave / WN, wn = wave % WN;

    // ---- tile assignment: XCD-aware remap, then groups of GROUP tile rows -------------
    // one contiguous range of tiles per XCD, then groups of GROUP tile rows: the 32 workgroups one
    // XCD runs at a time then cover GROUP x 32/GROUP tiles, chosen so that the A and B panels they
    // share are about the same size (256-row tiles: 4 measured 0.4 % faster than 8 and 1 % faster
    // than 16 on 8192 x 4096 x 4096)
    constexpr int GROUP = idx::gemm_group_rows(BM);
    const idx::TileCoord tc = idx::gemm_tile_of(block_x, g.tiles_m, g.tiles_n, GROUP);
    const int m0 = tc.tile_m * BM, n0 = tc.tile_n * BN;

    const int8_t* Ab = g.A + (int64_t)batch * g.bsa;
    const int8_t* Bb = g.B + (int64_t)batch * g.bsb;

    // ---- global -> LDS mapping --------------------------------------------------------
    // wave instruction t covers tile rows 8t..8t+7; lane l lands at byte 16*l of that 1 KiB
    // slab = (row 8t + l/8, physical chunk l%8).  Physical chunk p of row r holds logical
    // chunk p ^ (r & 7) ^ ((r >> 3) & 1): the 16 rows a quarter-wave reads at one k offset
    // then sit in 16 distinct 16-byte bank groups.
    // Address = (uniform row base of the instruction, SGPRs) + (per-lane 32-bit offset, one
    // VGPR per parity of t): keeps the loop's address registers to four VGPRs.
    uint32_t voffA[2], voffB[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        voffA[p] = idx::gemm_lane_offset_bytes(lane, p, (int)g.lda);
        voffB[p] = idx::gemm_lane_offset_bytes(lane, p, (int)g.ldb);
    }
    // a wave's instructions cover A_INSTR*8 consecutive tile rows (a divisor of 128): if they
    // start past M (a multiple of 128) they re-read the valid half; those results are masked
    static_assert(128 % (A_INSTR * 8) == 0 && 128 % (B_INSTR * 8) == 0, "a wave's rows must not straddle a 128-row boundary");
    const int rA0 = idx::gemm_wave_first_row(m0, wave, A_INSTR, g.M), rB0 = idx::gemm_wave_first_row(n0, wave, B_INSTR, g.N);
    const int8_t* const baseA = Ab + (int64_t)rA0 * g.lda;  // wave-uniform
    const int8_t* const baseB = Bb + (int64_t)rB0 * g.ldb;
    const int64_t strideA8 = 8 * g.lda, strideB8 = 8 * g.ldb;
    int8_t* const wA = ldsA + wave * A_INSTR * 1024;  // this wave's share of the A buffer
    int8_t* const wB = ldsB + wave * B_INSTR * 1024;

    // ---- LDS -> register mapping ------------------------------------------------------
    const int fr_row = lane & 31;
    const int fr_half = lane >> 5;
    const int sw = (lane & 7) ^ ((lane >> 3) & 1);
    const int a_row_off = (wm * TM * 32 + fr_row) * 128;
    const int b_row_off = (wn * TN * 32 + fr_row) * 128;
    int choff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) choff[ks] = ((ks * 2 + fr_half) ^ sw) * 16;

    v16i acc[TM][TN];
    float accf[PROMOTE ? TM : 1][PROMOTE ? TN : 1][16];
    const v16i vzero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = vzero;
    if (PROMOTE) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) accf[i][j][r] = 0.0f;
    }

    // ---- per-K-tile factors of the fast promotion ---------------------------------------
    // accf += f32(dot_kt) * f_kt with f_kt = fa_kt * fb_kt (or its reciprocal for the fused
    // kernels' division).  Operands scaled per row contribute 1 here and their row / column
    // vector in the epilogue.  A wave's tile (128 rows x 64 columns) lies inside one 128 x 128
    // scale block, so with block scales f_kt is wave-uniform: all nk (<= 256) values are
    // fetched once before the loop, lane l of fvec[c] holding tile kt = 64 c + l, and the loop
    // picks them with v_readlane -- no memory instruction for scales inside the loop.
    const bool divide = FAST && g.combine == TI8_COMBINE_DIV_PROD;
    const bool a_in = FAST && g.sa.mode != TI8_SCALE_ROW, b_in = FAST && g.sb.mode != TI8_SCALE_ROW;
    const int sha = g.sa.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0, shb = g.sb.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0;
    float fvec[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    float fraw_a[4] = {1.0f, 1.0f, 1.0f, 1.0f}, fraw_b[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    const float* pfb[TN];  // LANEB: this lane's column of B's scale grid
    if (FAST) {
        static_assert(!FAST || (128 % (TM * 32) == 0 && 128 % (TN * 32) == 0), "a wave tile must lie inside one 128 x 128 scale block");
        const int rowblk = idx::gemm_factor_block(m0 + wm * TM * 32, g.M);
        const int colblk = idx::gemm_factor_block(n0 + wn * TN * 32, g.N);
        const int nkt = g.K >> 7;
        // unconditional loads (an operand without in-loop factors is read with stride 0 and its
        // value dropped): a load under a branch is waited for on the spot, one after the other
        const int64_t ska = a_in ? g.sa.ks : 0, skb = (b_in && !LANEB) ? g.sb.ks : 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int kt = idx::gemm_factor_kt(c, lane, nkt);
            fraw_a[c] = g.sa.p[idx::gemm_factor_index(batch, g.sa.bs, rowblk, g.sa.rs, kt, sha, ska)];
            fraw_b[c] = g.sb.p[idx::gemm_factor_index(batch, g.sb.bs, colblk, g.sb.rs, kt, shb, skb)];
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            pfb[j] = g.sb.p + idx::epi_col_scale_index(batch, g.sb.bs, n0 + (wn * TN + j) * 32 + fr_row, g.N, g.sb.rs);
        }
    }
    // column scale vector of the epilogue (4 columns per lane there), fetched now for the same reason
    constexpr int WCOLS = TN * 32;                       // columns of the wave tile
    constexpr int LPR = WCOLS / 8;                       // lanes per row in the epilogue's read-back (8 columns each)
    constexpr int RPI = 64 / LPR;                        // rows per wave instruction there
    const int rb_col = idx::epi_col_of_lane(lane, WCOLS);
    const int rb_row = idx::epi_row_of_lane(lane, WCOLS);
    // the column scales are fetched here, 4 per lane (16 lanes cover the wave tile's columns, every
    // group of 16 lanes alike), and handed to the lanes that store those columns in the epilogue
    const int ncol0 = n0 + wn * WCOLS + idx::epi_scale_col_of_lane(lane);
    const bool col_part = EPI == EPI_ROWS || (FAST && g.sb.mode == TI8_SCALE_ROW);
    const bool row_part = EPI == EPI_ROWS || (FAST && g.sa.mode == TI8_SCALE_ROW);
    float coln[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (EPI == EPI_ROWS || FAST) {
        const int64_t cs = col_part ? g.sb.rs : 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) coln[c] = g.sb.p[idx::epi_col_scale_index(batch, g.sb.bs, ncol0 + c, g.N, cs)];
    }
    float f_cur = 1.0f;   // wave-uniform factor of the K tile being accumulated
    float fb[TN];         // LANEB only: per-lane factors of that tile
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = 1.0f;
    auto load_factors = [&](int kt) {
        const int l = kt & 63, c = kt >> 6;
        if (g.K <= 64 * 128) {   // the usual case: one register holds every tile's factor
            f_cur = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[0]), l));
        } else {
            const float v0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[0]), l));
            const float v1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[1]), l));
            const float v2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[2]), l));
            const float v3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec[3]), l));
            f_cur = c == 0 ? v0 : (c == 1 ? v1 : (c == 2 ? v2 : v3));
        }
        if (LANEB && !CHAIN) {  // issued before this tile's loads; consumed after its barrier (which waits for them)
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = pfb[j][(int64_t)kt * g.sb.ks];
        }
    };

    v4i a[2][TM], b[2][TN];
    auto load_frags = [&](int set, const int8_t* sA, const int8_t* sB, int ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i) a[set][i] = *reinterpret_cast<const v4i*>(sA + i * 4096 + choff[ks]);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[set][j] = *reinterpret_cast<const v4i*>(sB + j * 4096 + choff[ks]);
    };
    auto mfmas = [&](int fset, bool first) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[fset][i], b[fset][j], first ? vzero : acc[i][j], 0, 0, 0);
    };
    // Last k-step of a K tile in the fast promotion: the MFMA that completes a block's 128-deep
    // dot product writes it to ordinary VGPRs (its accumulator input still comes from the
    // accumulation registers), where convert + fma can consume it directly; the accumulation
    // registers restart from zero in the next tile, so nothing is copied or cleared.
    auto mfmas_promote = [&](int fset) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[fset][i], b[fset][j], acc[i][j], 0, 0, 0);
                float f = f_cur;
                if (LANEB) {
                    f = f_cur * fb[j];
                    const float rf = 1.0f / f;
                    f = divide ? rf : f;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) accf[i][j][r] = __builtin_fmaf(static_cast<float>(d[r]), f, accf[i][j][r]);
            }
    };

    const int nk = g.K >> 7;
    // prologue: tile 0 complete, tile 1 in flight, fragments (0, 0) in registers
    const int tA0 = wave * A_INSTR, tB0 = wave * B_INSTR;
    issue_tile_loads<A_INSTR>(baseA, strideA8, voffA, tA0, wA);
    issue_tile_loads<B_INSTR>(baseB, strideB8, voffB, tB0, wB);
    if (FAST) {   // the scale loads have been in flight since before the tile loads
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float f = a_in ? fraw_a[c] : 1.0f;
            if (!LANEB && b_in) f = f * fraw_b[c];
            if (!LANEB && divide) f = 1.0f / f;
            fvec[c] = f;
        }
    }
    if (divide) {
#pragma unroll
        for (int c = 0; c < 4; ++c) coln[c] = 1.0f / coln[c];
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const int klast = (nk - 1) * 128;  // loads past the last K tile re-read it into a free buffer: no branches in the loop
    issue_tile_loads<A_INSTR>(baseA + idx::gemm_k_offset(1, klast), strideA8, voffA, tA0, wA + A_BYTES);
    // (the chained kernel issues the B half of tile kt+1 at the top of iteration kt instead: with
    // both halves behind its barrier it measured 1 % slower, the other kernels 2.5 % faster)
    if constexpr (!CHAIN) issue_tile_loads<B_INSTR>(baseB + idx::gemm_k_offset(1, klast), strideB8, voffB, tB0, wB + B_BYTES);
    if constexpr (CHAIN) {
        // Promotion without int32 accumulators that outlive a K tile: a 32 x 32 block's four MFMAs of
        // a K tile chain into a temporary (two blocks of one block row interleaved, so that
        // dependent MFMAs are two issues apart), which is folded into the float accumulators
        // right away.  Only the float accumulators persist, which is what lets a wave own
        // 128 x 64 (8 blocks = 128 VGPRs) instead of 64 x 64: a third fewer LDS reads and L2->LDS
        // bytes per MFMA.  Registers: A fragments of one block row (4 k-steps) + the next row's
        // being read, B fragments of both block columns for the whole K tile, two temporaries.
        v4i fa[2][4], fbv[TN][4];
        static_assert(!CHAIN || TN == 2, "two block columns per wave");
        auto read_a = [&](int buf, const int8_t* stage_a, int i) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) fa[buf][ks] = *reinterpret_cast<const v4i*>(stage_a + a_row_off + i * 4096 + choff[ks]);
        };
        auto read_b = [&](const int8_t* stage_b, int ks) {
#pragma unroll
            for (int j = 0; j < TN; ++j) fbv[j][ks] = *reinterpret_cast<const v4i*>(stage_b + b_row_off + j * 4096 + choff[ks]);
        };
        // factors of the K tile being folded, per block column: the wave-uniform one, or with operand B scaled per
        // (column, K tile) this lane's column's (fb[] holds tile kt's values, fbn[] tile kt + 1's, requested one tile
        // ahead so that the wait in front of the barrier has long covered them)
        float f0 = 1.0f, f1 = 1.0f;
        float fbn[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) fbn[j] = 1.0f;
        auto tile_factors = [&](int kt) {
            load_factors(kt);   // f_cur (and nothing else: the per-lane values are handled here)
            if (LANEB) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    fb[j] = fbn[j];
                    fbn[j] = pfb[j][(int64_t)min(kt + 1, nk - 1) * g.sb.ks];
                }
                f0 = f_cur * fb[0];
                f1 = f_cur * fb[1];
                if (divide) {
                    f0 = 1.0f / f0;
                    f1 = 1.0f / f1;
                }
            } else {
                f0 = f1 = f_cur;
            }
        };
        auto fold = [&](int i, const v16i& d0, const v16i& d1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[PROMOTE ? i : 0][0][r] = __builtin_fmaf(static_cast<float>(d0[r]), f0, accf[PROMOTE ? i : 0][0][r]);
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[PROMOTE ? i : 0][PROMOTE ? 1 : 0][r] = __builtin_fmaf(static_cast<float>(d1[r]), f1, accf[PROMOTE ? i : 0][PROMOTE ? 1 : 0][r]);
        };
        if (LANEB) {
#pragma unroll
            for (int j = 0; j < TN; ++j) fbn[j] = pfb[j][0];
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) read_b(ldsB, ks);
        read_a(0, ldsA, 0);
        for (int kt = 0; kt < nk; ++kt) {
            const int cur = kt & 1;
            const int8_t* stA = ldsA + cur * A_BYTES;
            const int8_t* stAn = ldsA + (cur ^ 1) * A_BYTES;
            const int8_t* stBn = ldsB + (cur ^ 1) * B_BYTES;
            tile_factors(kt);
            issue_tile_loads<B_INSTR>(baseB + idx::gemm_k_offset(kt + 1, klast), strideB8, voffB, tB0, wB + (cur ^ 1) * B_BYTES);
#pragma unroll
            for (int i = 0; i < TM - 1; ++i) {
                read_a((i + 1) & 1, stA, i + 1);
                __builtin_amdgcn_sched_barrier(0);
                v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i & 1][0], fbv[0][0], vzero, 0, 0, 0);
                v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i & 1][0], fbv[1][0], vzero, 0, 0, 0);
#pragma unroll
                for (int ks = 1; ks < 4; ++ks) {
                    d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i & 1][ks], fbv[0][ks], d0, 0, 0, 0);
                    d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i & 1][ks], fbv[1][ks], d1, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                fold(i, d0, d1);
                __builtin_amdgcn_sched_barrier(0);
            }
            // last block row: tile kt+1 has landed, its fragments replace those of tile kt as they retire
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            issue_tile_loads<A_INSTR>(baseA + idx::gemm_k_offset(kt + 2, klast), strideA8, voffA, tA0, wA + cur * A_BYTES);
            constexpr int LB = (TM - 1) & 1;   // buffer that holds the last block row
            read_a(LB ^ 1, stAn, 0);
            __builtin_amdgcn_sched_barrier(0);
            v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][0], fbv[0][0], vzero, 0, 0, 0);
            v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][0], fbv[1][0], vzero, 0, 0, 0);
            d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][1], fbv[0][1], d0, 0, 0, 0);
            d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][1], fbv[1][1], d1, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_b(stBn, 0);
            read_b(stBn, 1);
            __builtin_amdgcn_sched_barrier(0);
            d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][2], fbv[0][2], d0, 0, 0, 0);
            d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][2], fbv[1][2], d1, 0, 0, 0);
            d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][3], fbv[0][3], d0, 0, 0, 0);
            d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[LB][3], fbv[1][3], d1, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_b(stBn, 2);
            read_b(stBn, 3);
            __builtin_amdgcn_sched_barrier(0);
            fold(TM - 1, d0, d1);
            __builtin_amdgcn_sched_barrier(0);
            // the next tile starts with block row 0 in buffer LB ^ 1; with an even number of block
            // rows per wave that is buffer 0 again
            static_assert(!CHAIN || ((TM - 1) & 1) == 1, "an even number of block rows keeps the A buffers in phase");
        }
    } else {
    load_frags(0, ldsA + a_row_off, ldsB + b_row_off, 0);

    auto ktile = [&](int kt) {
        const int cur = kt & 1;
        const int8_t* sA = ldsA + cur * A_BYTES + a_row_off;
        const int8_t* sB = ldsB + cur * B_BYTES + b_row_off;
        if (FAST) load_factors(kt);
        // k-step 0
        load_frags(1, sA, sB, 1);
        mfmas(0, FAST);
        interleave_hint<TM * TN, TM + TN, 0, 0>();
        // k-step 1
        load_frags(0, sA, sB, 2);
        mfmas(1, false);
        interleave_hint<TM * TN, TM + TN, 0, 0>();
        // k-step 2
        load_frags(1, sA, sB, 3);
        mfmas(0, false);
        interleave_hint<TM * TN, TM + TN, 0, 0>();
        __builtin_amdgcn_s_waitcnt(0);  // tile kt+1 landed; every read of buffer `cur` returned
        __syncthreads();
        // k-step 3
        issue_tile_loads<A_INSTR>(baseA + idx::gemm_k_offset(kt + 2, klast), strideA8, voffA, tA0, wA + cur * A_BYTES);
        issue_tile_loads<B_INSTR>(baseB + idx::gemm_k_offset(kt + 2, klast), strideB8, voffB, tB0, wB + cur * B_BYTES);
        load_frags(0, ldsA + (cur ^ 1) * A_BYTES + a_row_off, ldsB + (cur ^ 1) * B_BYTES + b_row_off, 0);
        if (FAST) {
            mfmas_promote(1);
            interleave_hint<TM * TN, TM + TN, A_INSTR + B_INSTR, 32>();
        } else {
            mfmas(1, false);
            interleave_hint<TM * TN, TM + TN, A_INSTR + B_INSTR, 0>();
        }
    };
    {
        for (int kt = 0; kt < nk; ++kt) {
            ktile(kt);
            if (EPI == EPI_STRICT) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const float sb = scale_at(g.sb, batch, min(n0 + (wn * TN + j) * 32 + fr_row, g.N - 1), kt);
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int mrow = min(m0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * fr_half + (r & 3), g.M - 1);
                            const float sa = scale_at(g.sa, batch, mrow, kt);
                            const float d = static_cast<float>(acc[i][j][r]);
                            float t;
                            if (g.combine == TI8_COMBINE_MUL_MUL) {
                                t = d * sa;
                                t = t * sb;
                            } else if (g.combine == TI8_COMBINE_MUL_PROD) {
                                t = d * (sa * sb);
                            } else {
                                t = d / (sa * sb);
                            }
                            accf[i][j][r] = accf[i][j][r] + t;  // separate rounding: contraction is off
                            acc[i][j][r] = 0;
                        }
                    }
            }
        }
    }
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // ---- epilogue ---------------------------------------------------------------------
    // Each wave moves its accumulators through a private LDS slab, 32 tile rows at a time, so
    // that the global stores are whole row segments (8 columns per lane, 8 rows per instruction)
    // instead of one column per lane.  The main loop ended with a workgroup barrier, so the
    // operand buffers are free.  Slab rows are padded by 4 words: the two rows that 16 lanes read
    // together then sit in different banks.
    // A wave's tile lies inside one 128-row and one 128-column block, and M and N are multiples of
    // 128: the tile is all inside the output or all outside, so nothing below is checked per lane.
    if (m0 + wm * TM * 32 >= g.M || n0 + wn * WCOLS >= g.N) return;
    constexpr int SLAB_LD = idx::EPI_SLAB_LD(WCOLS);
    static_assert(SLAB_LD * 32 * 4 * NW <= 2 * (A_BYTES + B_BYTES), "epilogue slab does not fit");
    uint32_t* slab = reinterpret_cast<uint32_t*>(smem) + wave * (32 * SLAB_LD);
    constexpr int NRR = 32 / RPI;                        // rows of a 32-row block per lane
    static_assert(NRR * RPI == 32, "a block row advances the output by 32 rows");
    // column factors of this lane's 8 columns: lanes 2q and 2q + 1 fetched them (q = lane % 8)
    float cm[8];
#pragma unroll
    for (int c = 0; c < 8; ++c)
        cm[c] = __int_as_float(__builtin_amdgcn_ds_bpermute(idx::epi_scale_lane(lane, c) * 4, __float_as_int(coln[c & 3])));
    const int row0 = m0 + wm * TM * 32 + rb_row;          // this lane's first output row
    const int64_t c_off = idx::epi_out_offset(batch, g.bsc, row0, g.ldc, n0 + wn * WCOLS + rb_col);
    const int64_t c_step = (int64_t)RPI * g.ldc;          // uniform: the output address advances by scalar adds
    const float* prow0 = g.sa.p + idx::epi_row_scale_base(batch, g.sa.bs, row0, g.sa.rs);
    auto store_tile = [&](auto extra_tag, auto mrow_tag, auto mcol_tag) {
        constexpr bool EXTRA = decltype(extra_tag)::value;  // EPI_ROWS: post_scale, promotion: out_scale
        constexpr bool MROW = decltype(mrow_tag)::value;    // a per-row scale vector of A multiplies the rows
        constexpr bool MCOL = decltype(mcol_tag)::value;    // a per-row scale vector of B multiplies the columns
        int64_t off = c_off;
        // every row scale of the tile is fetched before the first store: loads and stores share
        // one in-order counter, so a load issued behind a block row's stores could only be waited
        // for together with those stores
        float rm_all[MROW ? TM : 1][MROW ? NRR : 1];
        if (MROW) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int k = 0; k < NRR; ++k) rm_all[i][k] = prow0[(int64_t)(i * 32 + k * RPI) * g.sa.rs];
            if (FAST && divide) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int k = 0; k < NRR; ++k) rm_all[i][k] = 1.0f / rm_all[i][k];
            }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int rr = 8 * (r >> 2) + 4 * fr_half + (r & 3);
                    const uint32_t bits = PROMOTE ? __float_as_uint(accf[PROMOTE ? i : 0][PROMOTE ? j : 0][r])
                                                  : static_cast<uint32_t>(acc[i][j][r]);
                    slab[rr * SLAB_LD + j * 32 + fr_row] = bits;
                }
            // same wave reads what it wrote: an LDS counter wait is enough, no barrier
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
            __builtin_amdgcn_wave_barrier();
            uint4 w[NRR][2];
#pragma unroll
            for (int k = 0; k < NRR; ++k) {
                const uint32_t* src = slab + (rb_row + k * RPI) * SLAB_LD + rb_col;
                w[k][0] = *reinterpret_cast<const uint4*>(src);
                w[k][1] = *reinterpret_cast<const uint4*>(src + 4);
            }
#pragma unroll
            for (int k = 0; k < NRR; ++k, off += c_step) {
                const uint32_t wb[8] = {w[k][0].x, w[k][0].y, w[k][0].z, w[k][0].w, w[k][1].x, w[k][1].y, w[k][1].z, w[k][1].w};
                if (EPI == EPI_I32) {
                    int32_t* dst = reinterpret_cast<int32_t*>(g.C) + off;
                    *reinterpret_cast<uint4*>(dst) = w[k][0];
                    *reinterpret_cast<uint4*>(dst + 4) = w[k][1];
                    continue;
                }
                float t[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    float v;
                    if (EPI == EPI_ROWS) {
                        v = static_cast<float>(static_cast<int32_t>(wb[c])) * rm_all[MROW ? i : 0][MROW ? k : 0];
                        v = v * cm[c];
                        if (EXTRA) v = __uint_as_float(pack_bf16x2(v, 0.0f) << 16) * g.post_scale;
                    } else {
                        v = __uint_as_float(wb[c]);
                        if (MROW) v = v * rm_all[MROW ? i : 0][MROW ? k : 0];
                        if (MCOL) v = v * cm[c];
                        if (EXTRA) v = v * g.out_scale;
                    }
                    t[c] = v;
                }
                uint4 o;
                o.x = pack_bf16x2(t[0], t[1]);
                o.y = pack_bf16x2(t[2], t[3]);
                o.z = pack_bf16x2(t[4], t[5]);
                o.w = pack_bf16x2(t[6], t[7]);
                uint16_t* dst = reinterpret_cast<uint16_t*>(g.C) + off;
                // two 8-byte stores: measured 3 us per 256 x 256 tile faster than one of 16 bytes
                *reinterpret_cast<uint2*>(dst) = make_uint2(o.x, o.y);
                *reinterpret_cast<uint2*>(dst + 4) = make_uint2(o.z, o.w);
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_wave_barrier();
        }
    };
    const bool extra = (EPI == EPI_ROWS) ? (g.post_scale != 0.0f) : (EPI != EPI_I32 && g.out_scale != 1.0f);
    using T_ = std::true_type;
    using F_ = std::false_type;
    if (EPI == EPI_ROWS) {
        if (extra) store_tile(T_{}, T_{}, T_{});
        else store_tile(F_{}, T_{}, T_{});
    } else if (FAST) {
        // block scales on both operands leave nothing to multiply; a scale vector multiplies only where there is one
        if (extra) {
            if (row_part && col_part) store_tile(T_{}, T_{}, T_{});
            else if (row_part) store_tile(T_{}, T_{}, F_{});
            else if (col_part) store_tile(T_{}, F_{}, T_{});
            else store_tile(T_{}, F_{}, F_{});
        } else {
            if (row_part && col_part) store_tile(F_{}, T_{}, T_{});
            else if (row_part) store_tile(F_{}, T_{}, F_{});
            else if (col_part) store_tile(F_{}, F_{}, T_{});
            else store_tile(F_{}, F_{}, F_{});
        }
    } else {
        if (extra) store_tile(T_{}, F_{}, F_{});
        else store_tile(F_{}, F_{}, F_{});
    }
}

template <int BM, int BN, int WM, int WN, int EPI>
__global__ __launch_bounds__(64 * WM * WN) void gemm_i8_kernel(const GemmArgs g) {
    gemm_i8_tile<BM, BN, WM, WN, EPI>(g, blockIdx.x, blockIdx.y);
}

// Several GEMMs (batch of one each) in ONE launch: workgroup w computes tile w - first[i] of the
// GEMM i whose range holds w.  The three GEMMs of a training step (Y, dX, dW) run this way when all
// their operands are at hand: no kernel boundary between them, and the last tiles of one GEMM run
// beside the first tiles of the next instead of beside idle CUs.
template <int BM, int BN, int WM, int WN, int EPI>
__global__ __launch_bounds__(64 * WM * WN) void gemm_i8_multi_kernel(const GemmMulti m) {
    static_assert(GEMM_MULTI_MAX == 3, "gemm_multi_pick knows three ranges");
    const int i = idx::gemm_multi_pick((int)blockIdx.x, m.first[1], m.first[2], m.count);
    gemm_i8_tile<BM, BN, WM, WN, EPI>(m.g[i], (int)blockIdx.x - m.first[i], 0);
}

constexpr size_t tile_lds_bytes(int bm, int bn) { return 2 * (size_t)(bm + bn) * 128; }

// Per-device set-up of one kernel instance (MULTI: the several-GEMMs form): its dynamic LDS limit where the
// double-buffered operand tiles exceed the 64 KiB a kernel gets by default.
template <int BM, int BN, int WM, int WN, int EPI, bool MULTI>
static int prepare_kernel() {
    constexpr size_t shmem = tile_lds_bytes(BM, BN);
    if (shmem <= 64 * 1024) return TI8_OK;
    static OncePerDevice once;
    const void* kern = MULTI ? reinterpret_cast<const void*>(gemm_i8_multi_kernel<BM, BN, WM, WN, EPI>)
                             : reinterpret_cast<const void*>(gemm_i8_kernel<BM, BN, WM, WN, EPI>);
    const hipError_t e = raise_lds_limit(once, kern, (int)shmem);
    if (e != hipSuccess) return fail(TI8_ERR_HIP, "gemm: cannot raise the LDS limit to %zu: %s", shmem, hipGetErrorString(e));
    return TI8_OK;
}

template <int BM, int BN, int WM, int WN, int EPI>
static int launch_multi(GemmMulti& m, hipStream_t st) {
    int total = 0;
    for (int i = 0; i < m.count; ++i) {
        m.g[i].tiles_m = (m.g[i].M + BM - 1) / BM;
        m.g[i].tiles_n = (m.g[i].N + BN - 1) / BN;
        m.first[i] = total;
        total += m.g[i].tiles_m * m.g[i].tiles_n;
    }
    for (int i = m.count; i <= GEMM_MULTI_MAX; ++i) m.first[i] = total;
    for (int i = m.count; i < GEMM_MULTI_MAX; ++i) m.g[i] = m.g[0];
    if (int e = prepare_kernel<BM, BN, WM, WN, EPI, true>()) return e;
    hipLaunchKernelGGL((gemm_i8_multi_kernel<BM, BN, WM, WN, EPI>), dim3((unsigned)total), dim3(64 * WM * WN), tile_lds_bytes(BM, BN), st, m);
    note_gemm_kernel(TI8_KERNEL_ONE_TILE_MULTI, BM, BN, EPI);
    return check_launch("ti8_gemm_i8_nt_multi");
}

template <int BM, int BN, int WM, int WN, int EPI>
static int launch(const GemmArgs& a0, int64_t batch, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.N + BN - 1) / BN;
    if (int e = prepare_kernel<BM, BN, WM, WN, EPI, false>()) return e;
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)batch), block(64 * WM * WN);
    hipLaunchKernelGGL((gemm_i8_kernel<BM, BN, WM, WN, EPI>), grid, block, tile_lds_bytes(BM, BN), st, a);
    note_gemm_kernel(TI8_KERNEL_ONE_TILE, BM, BN, EPI);
    return check_launch("ti8_gemm_i8_nt");
}

static int check_operands(const char* fn, const void* A, int64_t bsa, int64_t lda, const void* B, int64_t bsb, int64_t ldb,
                          const void* C, int64_t ldc, int64_t batch, int64_t M, int64_t N, int64_t K, int m_step = 128) {
    if (!A || !B || !C) return fail(TI8_ERR_NULL, "%s: A, B and C are required", fn);
    if (batch <= 0 || M <= 0 || N <= 0 || K <= 0 || K % 128 || M % m_step || N % 128)
        return fail(TI8_ERR_SHAPE, "%s: need batch>0 and M, N, K positive multiples of 128 (M: of 32 up to 256 rows); got batch=%lld M=%lld N=%lld K=%lld",
                    fn, (long long)batch, (long long)M, (long long)N, (long long)K);
    if (M > 0x3fffffff || N > 0x3fffffff || K > 0x3fffffff || batch > 65535)
        return fail(TI8_ERR_SHAPE, "%s: dimension too large", fn);
    if (lda < K || ldb < K || ldc < N) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than the row length", fn);
    // the kernels keep 8 * ld in 32-bit lane offsets
    if (lda > 0x0fffffff || ldb > 0x0fffffff) return fail(TI8_ERR_SHAPE, "%s: leading dimension of A or B too large", fn);
    if (!aligned16(A) || !aligned16(B) || (lda % 16) || (ldb % 16) || (bsa % 16) || (bsb % 16))
        return fail(TI8_ERR_ALIGN, "%s: A and B must be 16-byte aligned with strides multiples of 16", fn);
    return TI8_OK;
}

static int check_scale(const char* fn, const char* which, const float* p, int mode) {
    if (!p) return fail(TI8_ERR_NULL, "%s: scale pointer of %s is NULL", fn, which);
    if (mode < 0 || mode > 3) return fail(TI8_ERR_MODE, "%s: unknown scale mode %d for %s", fn, mode, which);
    return TI8_OK;
}

// Argument checks of one dequantising GEMM and its argument block (shared by ti8_gemm_i8_nt and
// ti8_gemm_i8_nt_multi)
static int prepare_gemm(const char* fn, const ti8_gemm_problem& p, int gemm_flags, GemmArgs* out) {
    // up to 256 rows M may be any multiple of 32 (decode shapes): only the few-rows kernel takes those
    if (int e = check_operands(fn, p.A, p.bsa, p.lda, p.B, p.bsb, p.ldb, p.C, p.ldc, p.batch, p.M, p.N, p.K, p.M <= 256 ? 32 : 128)) return e;
    if (int e = check_scale(fn, "A", p.sA, p.modeA)) return e;
    if (int e = check_scale(fn, "B", p.sB, p.modeB)) return e;
    // the epilogue keeps (row within a tile) * (row stride of A's scales) in 32 bits
    if (p.modeA == TI8_SCALE_ROW && (p.sa_rs < 0 || p.sa_rs > 0x00ffffff))
        return fail(TI8_ERR_SHAPE, "%s: row stride of A's scales must be in [0, 2^24)", fn);
    if (p.combine < 0 || p.combine > 2) return fail(TI8_ERR_MODE, "%s: unknown combine %d", fn, p.combine);
    if (gemm_flags & ~(TI8_GEMM_STRICT | TI8_GEMM_TILED | TI8_GEMM_SKINNY | TI8_GEMM_LARGE_TILES | TI8_GEMM_ONE_TILE)) return fail(TI8_ERR_MODE, "%s: unknown flag 0x%x", fn, gemm_flags);
    if ((gemm_flags & TI8_GEMM_SKINNY) && (gemm_flags & (TI8_GEMM_TILED | TI8_GEMM_LARGE_TILES)))
        return fail(TI8_ERR_MODE, "%s: TI8_GEMM_SKINNY excludes TI8_GEMM_TILED and TI8_GEMM_LARGE_TILES", fn);
    if (p.acc_i32_full && (p.modeA != TI8_SCALE_ROW || p.modeB != TI8_SCALE_ROW))
        return fail(TI8_ERR_MODE, "%s: int32 accumulation over the whole K needs per-row scales on both operands", fn);
    if ((p.modeA == TI8_SCALE_BLOCK_K256 || p.modeB == TI8_SCALE_BLOCK_K256) && (p.K % 256))
        return fail(TI8_ERR_SHAPE, "%s: 256-wide scale groups need K %% 256 == 0", fn);
    if ((reinterpret_cast<uintptr_t>(p.C) & 7) || (p.ldc % 4) || (p.bsc % 4)) return fail(TI8_ERR_ALIGN, "%s: C must be 8-byte aligned with strides multiples of 4", fn);
    GemmArgs a;
    a.A = p.A; a.B = p.B; a.C = p.C;
    a.bsa = p.bsa; a.lda = p.lda; a.bsb = p.bsb; a.ldb = p.ldb; a.bsc = p.bsc; a.ldc = p.ldc;
    a.sa = ScaleDesc{p.sA, p.modeA, p.sa_bs, p.sa_rs, p.sa_ks};
    a.sb = ScaleDesc{p.sB, p.modeB, p.sb_bs, p.sb_rs, p.sb_ks};
    a.M = (int)p.M; a.N = (int)p.N; a.K = (int)p.K;
    a.tiles_m = a.tiles_n = 0;
    a.combine = p.combine;
    a.strict = (gemm_flags & TI8_GEMM_STRICT) ? 1 : 0;
    a.out_scale = p.out_scale; a.post_scale = p.post_scale;
    *out = a;
    return TI8_OK;
}

// every kernel instance that the launchers below can select, for ti8_init()
int init_gemm_kernels() {
#define TI8_GEMM_CASE(BM, BN, WM, WN, EPI) \
    if (int e = prepare_kernel<BM, BN, WM, WN, EPI, false>()) return e
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_ROWS);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_I32);
    TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE_LANE);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN_LANE);
    TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE);
#undef TI8_GEMM_CASE
#define TI8_GEMM_CASE(BM, BN, WM, WN, EPI) \
    if (int e = prepare_kernel<BM, BN, WM, WN, EPI, true>()) return e
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_ROWS);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN);
    TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE);
#undef TI8_GEMM_CASE
    return TI8_OK;
}

// The chained promotion on persistent workgroups where its limits allow (gemm_chain.hip); CHAIN_UNAVAILABLE otherwise
static int try_chain_persistent(GemmMulti& m, const int64_t* batch, hipStream_t st) {
    if (!chain_persistent_supported(m)) return CHAIN_UNAVAILABLE;
    int64_t total = 0;
    for (int i = 0; i < m.count; ++i) {
        m.g[i].tiles_m = (m.g[i].M + 255) / 256;
        m.g[i].tiles_n = (m.g[i].N + 255) / 256;
        m.first[i] = (int)total;
        total += (int64_t)m.g[i].tiles_m * m.g[i].tiles_n * batch[i];
    }
    if (total > 0x3fffffff) return CHAIN_UNAVAILABLE;
    for (int i = m.count; i <= GEMM_MULTI_MAX; ++i) m.first[i] = (int)total;
    for (int i = m.count; i < GEMM_MULTI_MAX; ++i) m.g[i] = m.g[0];
    return launch_chain_persistent(m, (int)total, device_cu_count(), st);
}

// One GEMM on the LDS-tiled kernel that `c` names
static int launch_tiled(const char* fn, const GemmArgs& a, int64_t batch, const idx::GemmConfig& c, bool persistent, hipStream_t st) {
    if (c.epi == EPI_PROMOTE_CHAIN && persistent) {
        GemmMulti m;
        m.count = 1;
        m.g[0] = a;
        const int rc = try_chain_persistent(m, &batch, st);
        if (rc != CHAIN_UNAVAILABLE) return rc;
    }
#define TI8_GEMM_CASE(BM, BN, WM, WN, EPI) \
    if (c.bm == BM && c.bn == BN && c.epi == EPI) return launch<BM, BN, WM, WN, EPI>(a, batch, st)
    TI8_GEMM_CASE(128, 128, 2, 2, EPI_ROWS);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_ROWS);
    TI8_GEMM_CASE(128, 128, 2, 2, EPI_STRICT);
    TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE_LANE);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN);
    TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN_LANE);
    TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE);
    TI8_GEMM_CASE(128, 128, 2, 2, EPI_PROMOTE);
#undef TI8_GEMM_CASE
    return fail(TI8_ERR_MODE, "%s: no kernel for tile %d x %d, epilogue %d", fn, c.bm, c.bn, c.epi);
}

}  // namespace ti8

using namespace ti8;

extern "C" int ti8_gemm_i8_nt(const int8_t* A, int64_t bsa, int64_t lda, const int8_t* B, int64_t bsb, int64_t ldb,
                              void* C, int64_t bsc, int64_t ldc, const float* sA, int modeA, int64_t sa_bs,
                              int64_t sa_rs, int64_t sa_ks, const float* sB, int modeB, int64_t sb_bs, int64_t sb_rs,
                              int64_t sb_ks, int64_t batch, int64_t M, int64_t N, int64_t K, int acc_i32_full,
                              int combine, float out_scale, float post_scale, int gemm_flags, ti8_stream_t stream) {
    const char* fn = "ti8_gemm_i8_nt";
    const ti8_gemm_problem p = {A, bsa, lda, B, bsb, ldb, C, bsc, ldc, sA, modeA, sa_bs, sa_rs, sa_ks, sB, modeB, sb_bs, sb_rs, sb_ks,
                                batch, M, N, K, acc_i32_full, combine, out_scale, post_scale};
    GemmArgs a;
    if (int e = prepare_gemm(fn, p, gemm_flags, &a)) return e;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // few rows: too few 256-row tiles to fill the machine, take the kernel that splits N and K finer
    const bool large = (gemm_flags & TI8_GEMM_LARGE_TILES) != 0;
    const bool want_skinny = (gemm_flags & TI8_GEMM_SKINNY) || (!(gemm_flags & (TI8_GEMM_TILED | TI8_GEMM_LARGE_TILES)) && M <= 256);
    if (want_skinny && !a.strict && skinny_supported(a)) return launch_skinny(a, batch, acc_i32_full != 0, st);
    if (M % 128)
        return fail(TI8_ERR_SHAPE, "%s: M = %lld is not a multiple of 128, which only the few-rows kernel accepts "
                    "(not with TI8_GEMM_STRICT / TI8_GEMM_TILED, per-(row, K tile) scales or K > 32768)", fn, (long long)M);
    return launch_tiled(fn, a, batch, idx::gemm_config(M, N, K, batch, acc_i32_full != 0, a.strict != 0, modeA, modeB, large, device_cu_count()),
                        !(gemm_flags & TI8_GEMM_ONE_TILE), st);
}

extern "C" int ti8_gemm_i8_nt_multi(const ti8_gemm_problem* problems, int count, int gemm_flags, ti8_stream_t stream) {
    const char* fn = "ti8_gemm_i8_nt_multi";
    if (!problems) return fail(TI8_ERR_NULL, "%s: problems is required", fn);
    if (count < 1 || count > GEMM_MULTI_MAX) return fail(TI8_ERR_SHAPE, "%s: between 1 and %d GEMMs, got %d", fn, GEMM_MULTI_MAX, count);
    if (gemm_flags & TI8_GEMM_SKINNY) return fail(TI8_ERR_MODE, "%s: the few-rows kernel is not offered here", fn);
    GemmMulti m;
    m.count = count;
    idx::GemmConfig c[GEMM_MULTI_MAX];
    // every GEMM runs the kernel its own shape selects; one launch serves them when they all agree on it
    bool one_launch = true;
    for (int i = 0; i < count; ++i) {
        const ti8_gemm_problem& p = problems[i];
        if (int e = prepare_gemm(fn, p, gemm_flags, &m.g[i])) return e;
        if (p.batch != 1) return fail(TI8_ERR_SHAPE, "%s: every GEMM must have batch = 1, GEMM %d has %lld", fn, i, (long long)p.batch);
        if (p.M % 128) return fail(TI8_ERR_SHAPE, "%s: M must be a multiple of 128, GEMM %d has %lld", fn, i, (long long)p.M);
        c[i] = idx::gemm_config(p.M, p.N, p.K, 1, p.acc_i32_full != 0, m.g[i].strict != 0, p.modeA, p.modeB,
                                (gemm_flags & TI8_GEMM_LARGE_TILES) != 0, device_cu_count());
        one_launch = one_launch && c[i].bm == c[0].bm && c[i].bn == c[0].bn && c[i].epi == c[0].epi;
    }
    one_launch = one_launch && c[0].epi != EPI_STRICT && c[0].epi != EPI_PROMOTE_LANE && c[0].epi != EPI_PROMOTE_CHAIN_LANE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool persistent = !(gemm_flags & TI8_GEMM_ONE_TILE);
    if (one_launch && c[0].epi == EPI_PROMOTE_CHAIN && persistent) {
        const int64_t ones[GEMM_MULTI_MAX] = {1, 1, 1};
        const int rc = try_chain_persistent(m, ones, st);
        if (rc != CHAIN_UNAVAILABLE) return rc;
    }
    if (one_launch) {
#define TI8_GEMM_CASE(BM, BN, WM, WN, EPI) \
        if (c[0].bm == BM && c[0].bn == BN && c[0].epi == EPI) return launch_multi<BM, BN, WM, WN, EPI>(m, st)
        TI8_GEMM_CASE(128, 128, 2, 2, EPI_ROWS);
        TI8_GEMM_CASE(256, 256, 2, 4, EPI_ROWS);
        TI8_GEMM_CASE(256, 256, 2, 4, EPI_PROMOTE_CHAIN);
        TI8_GEMM_CASE(256, 128, 4, 2, EPI_PROMOTE);
        TI8_GEMM_CASE(128, 128, 2, 2, EPI_PROMOTE);
#undef TI8_GEMM_CASE
    }
    for (int i = 0; i < count; ++i)
        if (int e = launch_tiled(fn, m.g[i], 1, c[i], persistent, st)) return e;
    return TI8_OK;
}

extern "C" int ti8_gemm_i8_nt_i32(const int8_t* A, int64_t bsa, int64_t lda, const int8_t* B, int64_t bsb, int64_t ldb,
                                  int32_t* C, int64_t bsc, int64_t ldc, int64_t batch, int64_t M, int64_t N, int64_t K,
                                  ti8_stream_t stream) {
    const char* fn = "ti8_gemm_i8_nt_i32";
    if (int e = check_operands(fn, A, bsa, lda, B, bsb, ldb, C, ldc, batch, M, N, K)) return e;
    GemmArgs a;
    a.A = A; a.B = B; a.C = C;
    a.bsa = bsa; a.lda = lda; a.bsb = bsb; a.ldb = ldb; a.bsc = bsc; a.ldc = ldc;
    a.sa = ScaleDesc{nullptr, 0, 0, 0, 0};
    a.sb = a.sa;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.tiles_m = a.tiles_n = 0;
    a.combine = 0; a.strict = 0; a.out_scale = 1.0f; a.post_scale = 0.0f;
    return launch<256, 256, 2, 4, EPI_I32>(a, batch, static_cast<hipStream_t>(stream));
}
