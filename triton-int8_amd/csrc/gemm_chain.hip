// Block-channel promotion GEMM (EPI_PROMOTE_CHAIN arithmetic of gemm.hip) with PERSISTENT workgroups:
// one workgroup per CU walks its output tiles (256 x 256, 8 waves of 128 x 64) one after the other,
// and the K loop never stops at a tile boundary:
//   * the loads that the one-tile kernel spends on re-reading the last K tile (it fetches one to two K
//     tiles ahead without a branch) fetch the NEXT output tile's K tiles 0 and 1 instead, and the last
//     iteration reads that tile's first fragments as it would read the next K tile's: a tile starts with
//     its operands in LDS and in registers, no prologue;
//   * the epilogue goes through an LDS slab of its own (32 KiB beyond the operand buffers, 16 tile rows
//     at a time), so that it does not wait for, or disturb, the operand loads in flight;
//   * its global stores drain while the next tile's first K tile is multiplied.
// Per tile this leaves the epilogue's own instructions; measured against one workgroup per tile: the
// prologue, the workgroup turn-over and most of the store drain.
// Arithmetic, operand layout in LDS, fragment reads and accumulator layout are those of the chained loop
// in gemm.hip; results are bit-identical.  Limits: K / 128 even and in [2, 256] for every GEMM of the launch (a
// tile's K tiles alternate between the two LDS buffers from a fixed start, which makes every LDS address a register
// plus an immediate; one register holds the per-K-tile factors of 64 K tiles and is refilled every 64; the launcher
// sends other shapes to the one-tile kernel).
#include <type_traits>
#include "gemm_args.h"

namespace ti8 {

namespace {

constexpr int BM = 256, BN = 256, WM = 2, WN = 4, NW = WM * WN, TM = 4, TN = 2;
constexpr int A_INSTR = BM / 8 / NW, B_INSTR = BN / 8 / NW;
constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
constexpr int WCOLS = TN * 32;
constexpr int SLAB_ROWS = 16;                                   // tile rows per pass through the slab
constexpr int SLAB_BYTES = NW * SLAB_ROWS * WCOLS * 4;          // 32 KiB
constexpr int LDS_BYTES = 2 * (A_BYTES + B_BYTES) + SLAB_BYTES; // 160 KiB
// Epilogue stores and the waits that count them.  A wave whose tile lies inside the output stores it row by row:
// every lane writes its 8 bf16 columns of a row with ONE 16-byte store, 8 rows (RPI) per instruction, so a wave
// issues exactly ROWS_PER_WAVE / RPI of them.  Rows of C are ldc apart, so no compiler can merge two of them, and a
// store that a compiler split in two would only make the waits below stronger: the count is a LOWER bound on the
// vector-memory operations a wave issues in its epilogue, which is what `s_waitcnt vmcnt(count)` needs to be safe
// (vector-memory operations complete in issue order: once at most `count` are outstanding, everything issued before
// the stores has completed).  The store loop in `store_tile` runs over the same constants.
constexpr int RPI = 64 / (WCOLS / 8);                  // rows per store instruction: 64 lanes, 8 columns per lane
constexpr int STORE_PASSES = TM * 2;                  // slab passes per tile (16 rows each)
constexpr int STORES_PER_PASS = SLAB_ROWS / RPI;      // store instructions per pass
constexpr int EPILOGUE_STORES = STORE_PASSES * STORES_PER_PASS;
constexpr int waitcnt_vm(int vm, int other) { return ((vm >> 4) << 14) | (vm & 15) | other; }   // vmcnt[3:0] | expcnt << 4 | lgkmcnt << 8 | vmcnt[5:4] << 14
// vmcnt(EPILOGUE_STORES) lgkmcnt(0)
constexpr int WAIT_ALL_BUT_STORES = waitcnt_vm(EPILOGUE_STORES, 0x70);
// vmcnt(B_INSTR) / vmcnt(B_INSTR + EPILOGUE_STORES) with the other counters left alone
constexpr int WAIT_FACTORS = waitcnt_vm(B_INSTR, 0x70 | 0xF00);
constexpr int WAIT_FACTORS_BEHIND_STORES = waitcnt_vm(B_INSTR + EPILOGUE_STORES, 0x70 | 0xF00);
static_assert(RPI == 8 && STORES_PER_PASS == 2 && EPILOGUE_STORES == 16 && EPILOGUE_STORES * RPI == TM * 32, "one 16-byte store per lane and row of the 128-row wave tile");
static_assert(B_INSTR == 4 && WAIT_FACTORS == 0xF74 && WAIT_FACTORS_BEHIND_STORES == 0x4F74 && WAIT_ALL_BUT_STORES == 0x4070, "s_waitcnt encoding");

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// What a wave needs to know about one output tile; every member is wave-uniform.
struct Tile {
    int gi;                  // GEMM of the launch
    int batch;
    int m0, n0;              // first row / column of the tile
    int nk;                  // K tiles
    const int8_t* baseA;     // first row of this wave's share of the tile's A (B) rows, K offset 0
    const int8_t* baseB;
    int lda, ldb;
    // scale values that a wave fetches with one register of per-lane offset each (32-bit: checked on the host)
    const float* fa_p;       // A's scale grid at this wave tile's row block, K block 0
    const float* fb_p;       // B's, at its column block
    uint32_t fa_ks, fb_ks;   // stride between K blocks (0 for an operand whose factor is not applied inside the loop)
    int wide;                // bit 0 / bit 1: A / B has 256-wide scale groups (two K tiles per scale)
    const float* col_p;      // B's per-row scales at the wave tile's first column (the operand's own first row when it has none)
    uint32_t col_s;          // their stride (0 when B has none)
};

}  // namespace

__global__ __launch_bounds__(64 * NW) void gemm_i8_chain_kernel(const GemmMulti m, const int total_tiles) {
    extern __shared__ __attribute__((aligned(1024))) int8_t smem[];
    // layout: [A buf0][A buf1][B buf0][B buf1][epilogue slab]
    int8_t* const ldsA = smem;
    int8_t* const ldsB = smem + 2 * A_BYTES;
    uint32_t* const slab = reinterpret_cast<uint32_t*>(smem + 2 * (A_BYTES + B_BYTES)) +
                           __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * (SLAB_ROWS * WCOLS);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int tA0 = wave * A_INSTR, tB0 = wave * B_INSTR;
    int8_t* const wA = ldsA + wave * A_INSTR * 1024;  // this wave's share of an A buffer
    int8_t* const wB = ldsB + wave * B_INSTR * 1024;

    // LDS -> register mapping (as in gemm.hip)
    const int fr_row = lane & 31;
    const int fr_half = lane >> 5;
    const int sw = (lane & 7) ^ ((lane >> 3) & 1);
    const int a_row_off = (wm * TM * 32 + fr_row) * 128;
    const int b_row_off = (wn * TN * 32 + fr_row) * 128;
    // byte address in LDS of this lane's 16 bytes of k-step ks in row 0 of its wave's A (B) rows of buffer 0: the ONLY
    // registers fragment reads are addressed with (made opaque so that every read is one of them plus an immediate)
    uint32_t abase[4], bbase[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int choff = ((ks * 2 + fr_half) ^ sw) * 16;
        abase[ks] = (uint32_t)(a_row_off + choff);
        bbase[ks] = (uint32_t)(2 * A_BYTES + b_row_off + choff);
        asm volatile("" : "+v"(abase[ks]), "+v"(bbase[ks]));
    }

    constexpr int GROUP = idx::gemm_group_rows(BM);
    const int stride_t = gridDim.x;

    // ---- tile T of the launch -> what the loops need --------------------------------------
    auto locate = [&](int T) {
        Tile t;
        t.gi = idx::gemm_multi_pick(T, m.first[1], m.first[2], m.count);
        const GemmArgs& g = m.g[t.gi];
        const int local = T - m.first[t.gi];
        const int per_batch = g.tiles_m * g.tiles_n;
        // (divisions of uniform values come out of the vector unit: back into scalar registers)
        t.batch = __builtin_amdgcn_readfirstlane(local / per_batch);
        const idx::TileCoord tc = idx::gemm_tile_of(local - t.batch * per_batch, g.tiles_m, g.tiles_n, GROUP);
        t.m0 = __builtin_amdgcn_readfirstlane(tc.tile_m) * BM;
        t.n0 = __builtin_amdgcn_readfirstlane(tc.tile_n) * BN;
        t.nk = g.K >> 7;
        t.lda = (int)g.lda;
        t.ldb = (int)g.ldb;
        const int rA0 = idx::gemm_wave_first_row(t.m0, wave, A_INSTR, g.M), rB0 = idx::gemm_wave_first_row(t.n0, wave, B_INSTR, g.N);
        t.baseA = g.A + (int64_t)t.batch * g.bsa + (int64_t)rA0 * g.lda;   // scalar arithmetic: every term is wave-uniform
        t.baseB = g.B + (int64_t)t.batch * g.bsb + (int64_t)rB0 * g.ldb;
        const bool a_in = g.sa.mode != TI8_SCALE_ROW, b_in = g.sb.mode != TI8_SCALE_ROW;
        t.fa_p = g.sa.p + idx::gemm_factor_index(t.batch, g.sa.bs, idx::gemm_factor_block(t.m0 + wm * TM * 32, g.M), g.sa.rs, 0, 0, 0);
        t.fb_p = g.sb.p + idx::gemm_factor_index(t.batch, g.sb.bs, idx::gemm_factor_block(t.n0 + wn * TN * 32, g.N), g.sb.rs, 0, 0, 0);
        t.fa_ks = a_in ? (uint32_t)g.sa.ks : 0u;
        t.fb_ks = b_in ? (uint32_t)g.sb.ks : 0u;
        t.wide = __builtin_amdgcn_readfirstlane((g.sa.mode == TI8_SCALE_BLOCK_K256 ? 1 : 0) | (g.sb.mode == TI8_SCALE_BLOCK_K256 ? 2 : 0));
        t.col_s = b_in ? 0u : (uint32_t)g.sb.rs;
        t.col_p = g.sb.p + idx::epi_col_scale_index(t.batch, g.sb.bs, idx::chain_col_scale_first(t.n0 + wn * WCOLS, g.N), g.N, t.col_s);
        return t;
    };
    // one wave's global -> LDS loads of one K tile of an operand (per-lane offsets rebuilt from the leading
    // dimension each time: one multiply-add per parity instead of registers held across the loop)
    auto load_a = [&](const Tile& t, int koff, int8_t* dst) {
        const uint32_t vo[2] = {idx::gemm_lane_offset_bytes(lane, 0, t.lda), idx::gemm_lane_offset_bytes(lane, 1, t.lda)};
        issue_tile_loads<A_INSTR>(t.baseA + koff, (int64_t)8 * t.lda, vo, tA0, dst);
    };
    auto load_b = [&](const Tile& t, int koff, int8_t* dst) {
        const uint32_t vo[2] = {idx::gemm_lane_offset_bytes(lane, 0, t.ldb), idx::gemm_lane_offset_bytes(lane, 1, t.ldb)};
        issue_tile_loads<B_INSTR>(t.baseB + koff, (int64_t)8 * t.ldb, vo, tB0, dst);
    };
    // per-K-tile factors of a tile, K tile 64 `block64` + lane in each lane (raw scale values; `finish_factors` combines them).
    // Unconditional loads: an operand without in-loop factors is read with stride 0 and its value dropped.
    // (lane-derived values of the once-per-tile code are rebuilt from an opaque copy of the lane number: hoisted out
    // of the tile loop they would sit in registers that the K loop has no room for)
    auto opaque_lane = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    auto load_raw_factors = [&](const Tile& t, int block64, float& ra, float& rb) {
        const uint32_t kt = (uint32_t)idx::gemm_factor_kt(block64, opaque_lane(), t.nk);
        ra = t.fa_p[(kt >> (t.wide & 1)) * t.fa_ks];
        rb = t.fb_p[(kt >> ((t.wide >> 1) & 1)) * t.fb_ks];
    };
    // the same two loads written out, for the place where the compiler must not count them: it would wait for the
    // epilogue's stores along with them (the caller waits with the counts it knows, then calls `landed`)
    auto load_raw_factors_uncounted = [&](const Tile& t, float& ra, float& rb) {
        const uint32_t kt = (uint32_t)idx::gemm_factor_kt(0, opaque_lane(), t.nk);
        const float* pa = t.fa_p + (kt >> (t.wide & 1)) * t.fa_ks;
        const float* pb = t.fb_p + (kt >> ((t.wide >> 1) & 1)) * t.fb_ks;
        asm volatile("global_load_dword %0, %1, off" : "=v"(ra) : "v"(pa) : "memory");
        asm volatile("global_load_dword %0, %1, off" : "=v"(rb) : "v"(pb) : "memory");
    };
    auto landed = [&](float& ra, float& rb) { asm volatile("" : "+v"(ra), "+v"(rb)); };
    // 16 bytes from LDS that the compiler does not count (the caller waits for lgkmcnt itself)
    auto lds_read_uncounted = [&](const uint32_t* p) {
        u32x4 v;
        const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint32_t*)p;
        asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
        return v;
    };
    auto finish_factors = [&](const Tile& t, float ra, float rb) {
        const GemmArgs& g = m.g[t.gi];
        float f = g.sa.mode != TI8_SCALE_ROW ? ra : 1.0f;
        if (g.sb.mode != TI8_SCALE_ROW) f = f * rb;
        if (g.combine == TI8_COMBINE_DIV_PROD) f = 1.0f / f;
        return f;
    };
    // the 4 column scales this lane fetches for the epilogue (16 lanes cover the wave tile's 64 columns)
    auto load_col_scales = [&](const Tile& t, float (&cn)[4]) {
        const uint32_t c0 = (uint32_t)idx::epi_scale_col_of_lane(opaque_lane());
#pragma unroll
        for (int c = 0; c < 4; ++c) cn[c] = t.col_p[(c0 + c) * t.col_s];
    };

    float accf[TM][TN][16];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) accf[i][j][r] = 0.0f;
    const v16i vzero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // A fragments of ONE block row: the next row's are read behind the MFMAs that use the registers and in front of the convert + fma
    // that follows, which covers the LDS latency (a second set, read one row ahead, measured 1 % slower and costs 16 registers)
    v4i fa[1][4], fbv[TN][4];
    // block row i of the A rows (block column j of the B rows) of LDS buffer `stage`
    auto read_a = [&](int buf, int stage, int i) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) fa[buf][ks] = *reinterpret_cast<const v4i*>(smem + abase[ks] + (stage * A_BYTES + i * 4096));
    };
    auto read_b = [&](int stage, int ks) {
#pragma unroll
        for (int j = 0; j < TN; ++j) fbv[j][ks] = *reinterpret_cast<const v4i*>(smem + bbase[ks] + (stage * B_BYTES + j * 4096));
    };
    float f_cur = 1.0f;
    auto fold = [&](int i, const v16i& d0, const v16i& d1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) accf[i][0][r] = __builtin_fmaf(static_cast<float>(d0[r]), f_cur, accf[i][0][r]);
#pragma unroll
        for (int r = 0; r < 16; ++r) accf[i][1][r] = __builtin_fmaf(static_cast<float>(d1[r]), f_cur, accf[i][1][r]);
    };

    // One K tile in LDS buffer `parity` (a tile's K tile kt sits in buffer kt & 1); the B half of the K tile
    // after this one is issued at the top, the A half of the one after that behind the barrier: `nb` / `na` say where
    // those come from (this tile or the next output tile).
    // `read_next`: whether the last block row also reads the next K tile's first fragments (not across a tile
    // boundary: the epilogue needs the registers, and reads them afterwards)
    // `first`: the first K tile of an output tile.  The B half of its successor is already on its way (issued before the
    // previous tile's epilogue), and it waits only for the loads issued before that epilogue's stores: the stores
    // (`stores_pending` of them at most, the youngest operations of this wave) drain while this K tile is multiplied.
    // `parity` is a compile-time value, so that every LDS address of the K tile is a register plus an immediate
    // (with the buffer chosen at run time each fragment read costs a vector add: 17 per K tile and wave).
    auto ktile_p = [&](auto first_tag, auto read_next_tag, auto parity_tag, bool stores_pending, float fvec, int kt, const Tile& nb, int koff_b,
                       const Tile& na, int koff_a) {
        constexpr bool FIRST = decltype(first_tag)::value;
        constexpr bool READ_NEXT = decltype(read_next_tag)::value;
        constexpr int cur = decltype(parity_tag)::value;
        constexpr int stA = cur, stAn = cur ^ 1, stBn = cur ^ 1;
        f_cur = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fvec), kt & 63));
        if (!FIRST) load_b(nb, koff_b, wB + (cur ^ 1) * B_BYTES);
#pragma unroll
        for (int i = 0; i < TM - 1; ++i) {
            __builtin_amdgcn_sched_barrier(0);
            v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][0], fbv[0][0], vzero, 0, 0, 0);
            v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][0], fbv[1][0], vzero, 0, 0, 0);
#pragma unroll
            for (int ks = 1; ks < 4; ++ks) {
                d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][ks], fbv[0][ks], d0, 0, 0, 0);
                d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][ks], fbv[1][ks], d1, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            read_a(0, stA, i + 1);   // behind the MFMAs that read the registers, in front of the fold that covers the latency
            __builtin_amdgcn_sched_barrier(0);
            fold(i, d0, d1);
            __builtin_amdgcn_sched_barrier(0);
        }
        // last block row: the next K tile has landed, its fragments replace this one's as they retire
        if (FIRST) {
            // what this barrier orders is in LDS: this wave's operand loads have landed and its fragment reads have returned once
            // the counters below are down.  The barrier instruction is written out because the compiler puts a wait for ALL
            // vector-memory operations in front of the one it knows, which would wait for the stores after all.
            if (stores_pending) __builtin_amdgcn_s_waitcnt(WAIT_ALL_BUT_STORES);
            else __builtin_amdgcn_s_waitcnt(0);
            asm volatile("s_barrier" ::: "memory");
        } else {
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
        load_a(na, koff_a, wA + cur * A_BYTES);
        __builtin_amdgcn_sched_barrier(0);
        v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][0], fbv[0][0], vzero, 0, 0, 0);
        v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][0], fbv[1][0], vzero, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][1], fbv[0][1], d0, 0, 0, 0);
        d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][1], fbv[1][1], d1, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (READ_NEXT) {
            read_b(stBn, 0);
            read_b(stBn, 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][2], fbv[0][2], d0, 0, 0, 0);
        d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][2], fbv[1][2], d1, 0, 0, 0);
        d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][3], fbv[0][3], d0, 0, 0, 0);
        d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0][3], fbv[1][3], d1, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (READ_NEXT) {
            read_b(stBn, 2);
            read_b(stBn, 3);
            read_a(0, stAn, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        fold(TM - 1, d0, d1);
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- epilogue of one tile: accumulators -> slab (16 rows at a time) -> bf16 rows in C -----------------
    // Slab word (row, col) of a wave sits at row * 64 + (col ^ 4 (row & 1)): the two rows that 16 lanes read
    // together then fall in different banks.  A wave's tile lies inside one 128-row and one 128-column block and
    // M, N are multiples of 128, so a wave either stores its whole tile or nothing.
    auto epilogue = [&](const Tile& t, const float (&coln)[4]) {
        const GemmArgs& g = m.g[t.gi];
        if (t.m0 + wm * TM * 32 >= g.M || t.n0 + wn * WCOLS >= g.N) return false;
        const int el = opaque_lane();
        const int rb_col = idx::epi_col_of_lane(el, WCOLS), rb_row = idx::epi_row_of_lane(el, WCOLS);
        const int e_row = el & 31, e_half = el >> 5;
        const bool divide = g.combine == TI8_COMBINE_DIV_PROD;
        const bool row_part = g.sa.mode == TI8_SCALE_ROW, col_part = g.sb.mode == TI8_SCALE_ROW;
        float cm[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float v = __int_as_float(__builtin_amdgcn_ds_bpermute(idx::epi_scale_lane(el, c) * 4, __float_as_int(coln[c & 3])));
            cm[c] = divide ? 1.0f / v : v;
        }
        const int row0 = t.m0 + wm * TM * 32 + rb_row;
        const int64_t c_off = idx::epi_out_offset(t.batch, g.bsc, row0, g.ldc, t.n0 + wn * WCOLS + rb_col);
        const int64_t c_step = (int64_t)RPI * g.ldc;
        const float* prow0 = g.sa.p + idx::epi_row_scale_base(t.batch, g.sa.bs, row0, g.sa.rs);
        auto store_tile = [&](auto extra_tag, auto mrow_tag, auto mcol_tag) {
            constexpr bool EXTRA = decltype(extra_tag)::value;
            constexpr bool MROW = decltype(mrow_tag)::value;
            constexpr bool MCOL = decltype(mcol_tag)::value;
            int64_t off = c_off;
            float rm_all[MROW ? EPILOGUE_STORES : 1];   // one row scale per store instruction
            if (MROW) {   // every row scale of the tile before the first store (loads and stores share one in-order counter)
#pragma unroll
                for (int q = 0; q < EPILOGUE_STORES; ++q) rm_all[q] = prow0[(int64_t)(q * RPI) * g.sa.rs];
                if (divide) {
#pragma unroll
                    for (int q = 0; q < EPILOGUE_STORES; ++q) rm_all[q] = 1.0f / rm_all[q];
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int h = 0; h < STORE_PASSES / TM; ++h) {   // rows 16 h .. 16 h + 15 of block row i: accumulator registers 8 h .. 8 h + 7
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const int rr = idx::epi_chain_slab_row(e, e_half);
                            slab[idx::epi_chain_slab_word(rr, j * 32 + e_row)] = __float_as_uint(accf[i][j][8 * h + e]);
                        }
                    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): same wave reads what it wrote, no barrier
                    __builtin_amdgcn_wave_barrier();
                    // the read-back is written out: before an LDS read that it knows, the compiler waits for the operand loads
                    // in flight (they write LDS too), i.e. for the next tile's K tile 1 issued a moment ago
                    u32x4 w[STORES_PER_PASS][2];
#pragma unroll
                    for (int k = 0; k < STORES_PER_PASS; ++k) {
                        const int rr = rb_row + k * RPI;
                        w[k][0] = lds_read_uncounted(slab + idx::epi_chain_slab_word(rr, rb_col));
                        w[k][1] = lds_read_uncounted(slab + idx::epi_chain_slab_word(rr, rb_col + 4));
                    }
                    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
#pragma unroll
                    for (int k = 0; k < STORES_PER_PASS; ++k) asm volatile("" : "+v"(w[k][0]), "+v"(w[k][1]));
#pragma unroll
                    for (int k = 0; k < STORES_PER_PASS; ++k, off += c_step) {
                        const uint32_t wb[8] = {w[k][0].x, w[k][0].y, w[k][0].z, w[k][0].w, w[k][1].x, w[k][1].y, w[k][1].z, w[k][1].w};
                        float v[8];
#pragma unroll
                        for (int c = 0; c < 8; ++c) {
                            v[c] = __uint_as_float(wb[c]);
                            if (MROW) v[c] = v[c] * rm_all[MROW ? (i * (STORE_PASSES / TM) + h) * STORES_PER_PASS + k : 0];
                            if (MCOL) v[c] = v[c] * cm[c];
                            if (EXTRA) v[c] = v[c] * g.out_scale;
                        }
                        // the ONE store of this (pass, k): EPILOGUE_STORES counts these
                        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(g.C) + off) =
                            make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
                    }
                    __builtin_amdgcn_s_waitcnt(0xc07f);
                    __builtin_amdgcn_wave_barrier();
                }
        };
        using T_ = std::true_type;
        using F_ = std::false_type;
        if (g.out_scale != 1.0f) {
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
        return true;
    };

    // ---- first tile: operands of K tile 0 into LDS and registers, K tile 1's A half in flight ------------
    int T = blockIdx.x;
    Tile cur = locate(T);
    // without a next tile the loads that run ahead fetch this tile's K tiles 0 and 1 again (nobody reads them)
    bool more = T + stride_t < total_tiles;
    Tile nxt = more ? locate(T + stride_t) : cur;
    float fvec;
    {
        load_a(cur, 0, wA);
        load_b(cur, 0, wB);
        float ra, rb;
        load_raw_factors(cur, 0, ra, rb);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        fvec = finish_factors(cur, ra, rb);
        load_a(cur, 128, wA + A_BYTES);
        load_b(cur, 128, wB + B_BYTES);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) read_b(0, ks);
        read_a(0, 0, 0);
    }
    bool stored = false;   // whether this wave's previous epilogue left stores behind
    while (true) {
        const int nk = cur.nk;
        // all but the last K tile: B of kt + 1 from this tile (for kt = 0 it is under way already); A of kt + 2 from this tile,
        // in the last of them K tile 0 of the next
        using T_ = std::true_type;
        using F_ = std::false_type;
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        // K / 128 is even: a tile starts in LDS buffer 0 and its K tiles alternate 0, 1, 0, 1, ...
        {
            const bool a_next = 2 >= nk;
            ktile_p(T_{}, T_{}, P0{}, stored, fvec, 0, cur, 128, a_next ? nxt : cur, a_next ? 0 : 256);
        }
        // K tiles 1 .. nk - 2 in pairs (buffer 1, buffer 0).  The register `fvec` holds the factors of 64 K tiles: the pair that
        // straddles a multiple of 64 sits outside the inner loop and refills it in between (waited for on the spot: once per 64 K tiles)
        for (int kt = 1; kt < nk - 1;) {
            const int last = (kt | 63) - 2 < nk - 3 ? (kt | 63) - 2 : nk - 3;   // last odd K tile whose pair lies inside this block of 64
            for (; kt <= last; kt += 2) {
                ktile_p(F_{}, T_{}, P1{}, false, fvec, kt, cur, (kt + 1) * 128, cur, (kt + 2) * 128);
                const bool a_next = kt + 3 >= nk;
                ktile_p(F_{}, T_{}, P0{}, false, fvec, kt + 1, cur, (kt + 2) * 128, a_next ? nxt : cur, a_next ? 0 : (kt + 3) * 128);
            }
            if (kt >= nk - 1) break;
            ktile_p(F_{}, T_{}, P1{}, false, fvec, kt, cur, (kt + 1) * 128, cur, (kt + 2) * 128);
            {
                float ra, rb;
                load_raw_factors(cur, (kt + 1) >> 6, ra, rb);
                fvec = finish_factors(cur, ra, rb);
            }
            const bool a_next = kt + 3 >= nk;
            ktile_p(F_{}, T_{}, P0{}, false, fvec, kt + 1, cur, (kt + 2) * 128, a_next ? nxt : cur, a_next ? 0 : (kt + 3) * 128);
            kt += 2;
        }
        // last K tile: the column scales of this tile's epilogue travel beside it
        float coln[4];
        load_col_scales(cur, coln);
        __builtin_amdgcn_sched_barrier(0);
        ktile_p(F_{}, F_{}, P1{}, false, fvec, nk - 1, nxt, 0, nxt, 128);
        // the accumulators are complete HERE: without this the optimiser moves the last K tile's convert + fma behind
        // the epilogue's branches and keeps that tile's 128 int32 results alive until then
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                float* a = accf[i][j];
                asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                                  "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
            }
        // the next tile's factors: fetched here, ahead of the stores, and combined behind the epilogue (operations complete in
        // issue order, so waiting for them does not wait for the stores)
        float ra, rb;
        load_raw_factors_uncounted(nxt, ra, rb);
        // the B half of the next tile's K tile 1, into the buffer the last K tile's B has left: issued before the epilogue's
        // stores, so that the next tile's first K tile need not wait for them
        load_b(nxt, 128, wB + B_BYTES);
        stored = epilogue(cur, coln);
        if (!more) break;
        // the factor loads were issued before the 4 loads of the B half and the stores: done once at most that many operations are
        // outstanding (said explicitly: the compiler would wait for everything, stores included, at the head of the tile loop)
        if (stored) __builtin_amdgcn_s_waitcnt(WAIT_FACTORS_BEHIND_STORES);
        else __builtin_amdgcn_s_waitcnt(WAIT_FACTORS);
        landed(ra, rb);
        fvec = finish_factors(nxt, ra, rb);
        // the next tile's K tile 0 has been in LDS since the barrier of the last K tile: its first fragments
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) read_b(0, ks);
        read_a(0, 0, 0);
        // the accumulators are free: the place for the integer divisions that find the tile after the next
        T += stride_t;
        cur = nxt;
        more = T + stride_t < total_tiles;
        if (more) nxt = locate(T + stride_t);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) accf[i][j][r] = 0.0f;
    }
    // loads that ran ahead of the last tile are still landing in this workgroup's LDS
    __builtin_amdgcn_s_waitcnt(0);
}

bool chain_persistent_supported(const GemmMulti& m) {
    for (int i = 0; i < m.count; ++i) {
        const int nk = m.g[i].K >> 7;
        if (nk < 2 || nk > 256 || (nk & 1) || m.g[i].strict) return false;
        if (m.g[i].sa.mode == TI8_SCALE_ROW_K128 || m.g[i].sb.mode == TI8_SCALE_ROW_K128) return false;
        // the epilogue stores 16 bytes per lane and row (the one-tile kernels store 8)
        if ((reinterpret_cast<uintptr_t>(m.g[i].C) & 15) || (m.g[i].ldc % 8) || (m.g[i].bsc % 8)) return false;
        // per-lane offsets into the scale arrays are kept in 32 bits: 64 K blocks x stride, 64 columns x stride
        const int64_t lim = (int64_t)1 << 24;
        if (m.g[i].sa.ks < 0 || m.g[i].sa.ks >= lim || m.g[i].sb.ks < 0 || m.g[i].sb.ks >= lim || m.g[i].sb.rs < 0 || m.g[i].sb.rs >= lim) return false;
    }
    return true;
}

// `m` with tiles_m / tiles_n / first[] filled for 256 x 256 tiles and first[i + 1] - first[i] = tiles of GEMM i times
// its batch count; one workgroup per CU (fewer when there are fewer tiles)
// Whether the current device grants the kernel its 160 KiB of LDS (asked once per device).  A refusal is remembered
// and reported through ti8_last_error() by the call that met it; callers then take the one-tile kernel.
static bool chain_kernel_available() {
    static OncePerDevice granted, refused;
    const uint64_t bit = 1ull << (current_device() & 63);
    if (refused.done.load(std::memory_order_acquire) & bit) return false;
    const hipError_t e = raise_lds_limit(granted, reinterpret_cast<const void*>(gemm_i8_chain_kernel), LDS_BYTES);
    if (e == hipSuccess) return true;
    refused.done.fetch_or(bit, std::memory_order_release);
    (void)fail(TI8_OK, "gemm: device %d refuses %d bytes of LDS for the persistent kernel (%s); one workgroup per tile serves its shapes",
               current_device(), LDS_BYTES, hipGetErrorString(e));
    return false;
}

int init_chain_kernel() {
    (void)chain_kernel_available();
    return TI8_OK;
}

int launch_chain_persistent(const GemmMulti& m, int total_tiles, int num_cu, hipStream_t st) {
    if (!chain_kernel_available()) return CHAIN_UNAVAILABLE;
    const int grid = total_tiles < num_cu ? total_tiles : num_cu;
    hipLaunchKernelGGL(gemm_i8_chain_kernel, dim3((unsigned)grid), dim3(64 * NW), LDS_BYTES, st, m, total_tiles);
    note_gemm_kernel(TI8_KERNEL_PERSISTENT_CHAIN, BM, BN, EPI_PROMOTE_CHAIN);
    return check_launch("ti8_gemm_i8_nt");
}

}  // namespace ti8
