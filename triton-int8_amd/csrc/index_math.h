// Index arithmetic of the kernels, as functions that compile for the device AND for the host.
//
// The kernels compute every global-memory offset (and the LDS offsets that depend on the launch
// geometry) through these functions; a host program can therefore walk (workgroup, wave, lane,
// iteration) tuples of a launch and check each access against the size of the buffer it goes to,
// without a GPU (tests/kernel_bounds/).  Offsets are in ELEMENTS of the tensor they index unless a
// name says bytes.  No HIP types here: the file is also compiled by g++.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define TI8_HD __host__ __device__ __forceinline__
#else
#define TI8_HD inline
#endif

namespace ti8 {
namespace idx {

TI8_HD int imin(int a, int b) { return a < b ? a : b; }
TI8_HD int imax(int a, int b) { return a > b ? a : b; }

// ---- LDS-tiled GEMM (gemm.hip) -------------------------------------------------------------

// workgroup id -> (tile_m, tile_n): one contiguous range of tiles per XCD (ids 8 apart share an
// XCD) when the tile count is a multiple of 8, then groups of `group` tile rows walked column by
// column inside a group
struct TileCoord {
    int tile_m, tile_n;
};
TI8_HD TileCoord gemm_tile_of(int block_id, int tiles_m, int tiles_n, int group) {
    const int ntiles = tiles_m * tiles_n;
    int pid = block_id;
    if ((ntiles & 7) == 0) pid = (pid & 7) * (ntiles >> 3) + (pid >> 3);
    const int per_group = group * tiles_n;
    const int group_id = pid / per_group;
    const int first_m = group_id * group;
    const int gsz = imin(tiles_m - first_m, group);
    TileCoord t;
    t.tile_m = first_m + (pid % per_group) % gsz;
    t.tile_n = (pid % per_group) / gsz;
    return t;
}

// GEMM of a several-GEMM launch that workgroup `block` works for: GEMM i owns the workgroups
// [first[i], first[i + 1]), first[0] = 0; only first[1] and first[2] are needed for up to 3 GEMMs
TI8_HD int gemm_multi_pick(int block, int first1, int first2, int count) {
    int i = 0;
    if (count > 1 && block >= first1) i = 1;
    if (count > 2 && block >= first2) i = 2;
    return i;
}

// tile rows per group of the map above for tiles of bm rows
constexpr int gemm_group_rows(int bm) { return bm >= 256 ? 4 : 8; }

// index of the scale of operand row `row` at K block `kb` for a scale descriptor (mode = ti8_scale_mode:
// 0 per row, 1 per 128 x 128 block, 2 per (row, K block), 3 per 128 rows x 256 columns)
TI8_HD int64_t scale_index(int mode, int64_t bs, int64_t rs, int64_t ks, int64_t batch, int row, int kb) {
    switch (mode) {
        case 0: return batch * bs + (int64_t)row * rs;
        case 1: return batch * bs + (int64_t)(row >> 7) * rs + (int64_t)kb * ks;
        case 2: return batch * bs + (int64_t)row * rs + (int64_t)kb * ks;
        default: return batch * bs + (int64_t)(row >> 7) * rs + (int64_t)(kb >> 1) * ks;
    }
}

// first operand row of the rows that `wave` copies into LDS: its n_instr instructions cover
// n_instr * 8 consecutive rows of the tile starting at tile_row0; a span that starts past the
// operand's last row (rows is a multiple of 128, and so is the span's distance to the valid
// half) re-reads the 128 rows before it, whose results nobody stores
TI8_HD int gemm_wave_first_row(int tile_row0, int wave, int n_instr, int rows) {
    const int r = tile_row0 + wave * n_instr * 8;
    return r >= rows ? r - 128 : r;
}

// per-lane byte offset inside the 8-row slab one global->LDS instruction copies: lane l lands at
// byte 16 l of the 1 KiB LDS slab = (row l/8, physical chunk l%8), and fetches the logical chunk
// that the XOR swizzle puts there; `parity` = (index of the instruction within the tile) & 1
TI8_HD uint32_t gemm_lane_offset_bytes(int lane, int parity, int ld) {
    const int ld_row = lane >> 3;
    const int ch = (lane & 7) ^ ld_row ^ parity;
    return (uint32_t)(ld_row * ld + ch * 16);
}

// K offset (bytes = elements) of the tile fetched for K tile `kt`: tiles past the last one fetch
// the last one again (into a buffer nobody reads) so that the loop has no branch
TI8_HD int gemm_k_offset(int kt, int klast) { return imin(kt * 128, klast); }

// byte offset, from the operand's batch base, of the 16 bytes that `lane` fetches in instruction
// `i` (of the wave's n_instr) of a tile: the composition issue_tile_loads performs
TI8_HD int64_t gemm_load_offset_bytes(int first_row, int64_t ld, int koff, int i, uint32_t lane_off) {
    return (int64_t)first_row * ld + koff + (int64_t)i * (8 * ld) + lane_off;
}

// index into a block-scale grid for the per-K-tile factor that lane `lane` keeps in register c
// (K tile 64 c + lane, clamped): (row block) * rs + (kt >> shift) * ks, with ks = 0 for an operand
// whose factor is not applied inside the loop
TI8_HD int gemm_factor_kt(int c, int lane, int nkt) { return imin(c * 64 + lane, nkt - 1); }
TI8_HD int gemm_factor_block(int first_row_of_wave_tile, int rows) { return imin(first_row_of_wave_tile, rows - 1) >> 7; }
TI8_HD int64_t gemm_factor_index(int64_t batch, int64_t bs, int block, int64_t rs, int kt, int shift, int64_t ks) {
    return batch * bs + (int64_t)block * rs + (int64_t)(kt >> shift) * ks;
}

// epilogue: a wave stores its tile 32 rows at a time through an LDS slab; with wcols columns per
// wave tile a row of the tile takes lpr = wcols / 8 lanes (8 columns each) and one instruction
// covers rpi = 64 / lpr rows.  Slab rows are padded by 4 words.
constexpr int EPI_SLAB_LD(int wcols) { return wcols + 4; }
TI8_HD int epi_col_of_lane(int lane, int wcols) { return (lane % (wcols / 8)) * 8; }
TI8_HD int epi_row_of_lane(int lane, int wcols) { return lane / (wcols / 8); }
// the column scales are fetched before the main loop, 4 per lane: lane l those of the wave tile's
// columns 4 (l % 16) .. + 3; in the epilogue the lane that stores columns 8 q .. 8 q + 7 (q = lane % 8)
// takes scale c of them from lane 2 q + c / 4 (register c % 4 there)
TI8_HD int epi_scale_col_of_lane(int lane) { return (lane % 16) * 4; }
TI8_HD int epi_scale_lane(int lane, int c) { return 2 * (lane % 8) + (c >> 2); }
// persistent chained kernel (gemm_chain.hip): its slab holds 16 tile rows of 64 words per wave; accumulator
// register 8 h + e (e < 8) of a 32 x 32 block is row 16 h + epi_chain_slab_row(e, lane / 32) of the block, and
// word (row, col) sits at row * 64 + (col ^ 4 (row & 1))
// first column whose per-row scale of B a wave of the persistent kernel fetches: its tile's first column, or, for a
// tile outside the operand (N is a multiple of 128, the wave tile has 64 columns), the operand's last 64 columns
TI8_HD int chain_col_scale_first(int first_col_of_wave_tile, int ncols) { return imin(first_col_of_wave_tile, ncols - 64); }
TI8_HD int epi_chain_slab_row(int e, int fr_half) { return 8 * (e >> 2) + 4 * fr_half + (e & 3); }
TI8_HD int epi_chain_slab_word(int row, int col) { return row * 64 + (col ^ (4 * (row & 1))); }
// index of the column scale of column `col` (clamped to the last column; stride 0 when absent)
TI8_HD int64_t epi_col_scale_index(int64_t batch, int64_t bs, int col, int ncols, int64_t cs) {
    return batch * bs + (int64_t)imin(col, ncols - 1) * cs;
}
// per-row scale of A of this lane's first output row (only waves whose tile lies inside the output get here)
TI8_HD int64_t epi_row_scale_base(int64_t batch, int64_t bs, int row0, int64_t rs) {
    return batch * bs + (int64_t)row0 * rs;
}
// output element offset of (batch, row0, col0) and the step between the rows one lane stores
TI8_HD int64_t epi_out_offset(int64_t batch, int64_t bsc, int row0, int64_t ldc, int col0) {
    return batch * bsc + (int64_t)row0 * ldc + col0;
}

// ---- Walsh-Hadamard transform (fwht.hip) ----------------------------------------------------
TI8_HD int fwht_padded(int i) { return i + (i >> 4); }
// element offset of segment `seg` (of L elements) of row `row`
TI8_HD int64_t fwht_segment_offset(int64_t block, int segs_per_row, int64_t ld, int L) {
    const int64_t row = block / segs_per_row;
    const int seg = (int)(block % segs_per_row);
    return row * ld + (int64_t)seg * L;
}
// whether the `len` elements from `first` of a segment exist in memory (`valid` elements do; the rest of a zero-extended
// row reads as zero and is not stored); valid is a multiple of len
TI8_HD bool fwht_chunk_valid(int first, int len, int valid) { return first + len <= valid; }
// LDS words a workgroup needs for L elements
TI8_HD int64_t fwht_lds_words(int64_t L) { return L + L / 16; }
// fwht_row_kernel (segments of 4096 * CH elements on 4 waves): first element of the 16-element chunk that the lane at chunk
// position `lp` of wave `w` takes from slice `k`; the word of its value `e` in the exchange buffer; and the first of the 4
// consecutive elements of (slice k, wave ws, chunk position lp) that wave `w` ends up with
TI8_HD int fwht_row_chunk_first(int k, int w, int lp) { return ((k * 4 + w) * 64 + lp) * 16; }
// (laid out so that a lane's elements 4j .. 4j + 3 are one aligned 16-byte unit and consecutive chunk positions are
// consecutive units: both the writes -- four units per lane -- and the reads -- unit j = w of all four waves -- are
// 16-byte LDS accesses without bank conflicts)
TI8_HD int fwht_row_lds(int w, int lp, int e) { return (((e >> 2) * 4 + w) * 64 + lp) * 4 + (e & 3); }
TI8_HD int fwht_row_out(int k, int ws, int lp, int w) { return ((k * 4 + ws) * 64 + lp) * 16 + 4 * w; }
// base LDS index of the radix-2^rb group `vt` in the pass over index bits [p, p + rb)
TI8_HD int fwht_group_base(int vt, int p, int rb) {
    const int lo = vt & ((1 << p) - 1);
    const int hi = vt >> p;
    return (hi << (p + rb)) | lo;
}

// transposed-input transform (y = FWHT of x^T along its rows = along the ROWS of x, length R):
// columns of x per workgroup (as many as fit the LDS budget of 32768 fp32 elements, at most the 8
// that one 16-byte load brings) and the column block of workgroup `id`: the G = 64 / W workgroups
// whose columns share one 128-byte line of every row get consecutive places on ONE XCD (workgroup
// ids 8 apart share an XCD), so that the line is fetched from HBM once; identity when the number of
// such groups is not a multiple of 8
TI8_HD int fwht_t_cols_per_wg(int64_t R) { return R <= 4096 ? 8 : (int)(32768 / R); }
// whether the one-kernel transposed transform is used: up to 2048 rows; longer columns go through a
// transposing copy into the output and an in-place transform there (lengths from 4096 on have the
// faster row kernel: 8192 x 4096 in 58 instead of 78 us, 8192 x 8192 in 105 instead of 146 us,
// 4096 x 4096 the same either way), which needs whole 64 x 64 tiles
TI8_HD bool fwht_t_direct(int64_t R, int64_t C) { return R <= 2048 || (C % 64) != 0; }
TI8_HD int64_t fwht_t_colblock(int64_t id, int64_t nblocks, int W) {
    const int G = 64 / W;
    if (nblocks % (8 * (int64_t)G) != 0) return id;
    const int64_t xcd = id & 7, j = id >> 3;
    return ((j / G) * 8 + xcd) * G + (j % G);
}

// ---- per-row quantiser (quant.hip) -----------------------------------------------------------
// row handled by (workgroup, wave): one workgroup per row, or one wave per row (4 rows per workgroup)
TI8_HD int64_t qrow_row(int64_t block, int wave, bool wg_row) { return wg_row ? block : block * 4 + wave; }
// 16-byte chunk index of load i of thread t (T threads per row)
TI8_HD int qrow_chunk(int t, int i, int T) { return t + i * T; }
// The quantisers that rotate 128-element segments first (H128 across 16 lanes x 8 elements) give chunk
// c ^ (c & 4 ? 3 : 0) of a segment to the lane that would otherwise hold chunk c: a permutation within
// every aligned group of 16 chunks (its own inverse), under which the partners of all four cross-lane
// stages are one DPP pattern away.
TI8_HD int had_chunk(int c) { return c ^ ((c & 4) ? 3 : 0); }

// ---- 128 x 128 tile quantisers (quant.hip) ---------------------------------------------------
struct TileId {
    int b, rb, cb;
};
TI8_HD TileId qblock_tile(int block, int nrb, int ncb) {
    TileId t;
    t.cb = block % ncb;
    block /= ncb;
    t.rb = block % nrb;
    t.b = block / nrb;
    return t;
}
// element offset of a tile's origin in a [B][R][C] tensor with tiles of 128 x tile_c
TI8_HD int64_t qblock_origin(int b, int64_t bs, int rb, int64_t ld, int cb, int tile_c) {
    return b * bs + (int64_t)rb * 128 * ld + (int64_t)cb * tile_c;
}
// thread t of 256 owns rows {64 h + 4 (t / 16) + j : h < 2, j < 4} x columns [8 (t % 16), + 8)
TI8_HD int qblock_row(int t, int h, int j) { return h * 64 + (t >> 4) * 4 + j; }
TI8_HD int qblock_col(int t) { return (t & 15) * 8; }
// the transposed tile leaves LDS as 128-byte rows: pass p of thread t writes row p * 32 + t / 8
// (= column of x), bytes 16 (t % 8) .. + 15 (= rows of x)
TI8_HD int qblock_t_row(int t, int p) { return p * 32 + (t >> 3); }
TI8_HD int qblock_t_col(int t) { return (t & 7) * 16; }

// ---- which kernel an entry point launches (decided on the host) ------------------------------

// per-row quantiser: NLOAD 16-byte chunks per thread, one wave (4 rows per workgroup) or one
// 256-thread workgroup per row, by the number of 16-byte chunks in a row
struct QRowConfig {
    int nload;
    bool wg_row;
};
TI8_HD QRowConfig qrow_config(int nchunk, bool group128) {
    QRowConfig c;
    if (group128) {
        c.nload = nchunk <= 256 * 8 ? 8 : 16;
        c.wg_row = nchunk > 64 * 8;
    } else if (nchunk <= 64 * 8) {
        c.nload = nchunk <= 64 * 2 ? 2 : (nchunk <= 64 * 4 ? 4 : 8);
        c.wg_row = false;
    } else {
        c.nload = nchunk <= 256 * 4 ? 4 : (nchunk <= 256 * 8 ? 8 : 16);
        c.wg_row = true;
    }
    return c;
}

// Walsh-Hadamard transform: elements per workgroup (a whole group of n when n >= 2048, else as
// many groups as divide both the row and 2048) and threads per workgroup
TI8_HD int64_t fwht_segment_len(int64_t cols, int64_t n) {
    if (n >= 2048 || cols < n) return n;    // cols < n: a zero-extended row of n elements per workgroup
    int64_t a = cols, b = 2048;
    while (b) {
        const int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;  // gcd(cols, 2048), a multiple of n because n divides both
}
TI8_HD int fwht_threads(int64_t) { return 256; }   // fwht_kernel: segments of up to 2048 elements (longer ones: fwht_row_kernel)

// LDS-tiled GEMM: tile shape, waves and epilogue kind by shape and scale modes.  `epi` values are
// the EPI_* constants of gemm_args.h.
struct GemmConfig {
    int bm, bn, wm, wn, epi;
};
TI8_HD GemmConfig gemm_config(int64_t M, int64_t N, int64_t K, int64_t batch, bool acc_i32_full, bool strict, int modeA,
                              int modeB, bool large, int num_cu) {
    const int64_t tiles_256x256 = ((M + 255) / 256) * ((N + 255) / 256) * batch;
    const int64_t tiles_256x128 = ((M + 255) / 256) * (N / 128) * batch;
    if (acc_i32_full) {
        // medium sizes: when the large tiles would leave CUs without a workgroup, 128 x 128 tiles
        // (4 waves of 64 x 64, two workgroups per CU)
        if (!large && tiles_256x256 < num_cu) return GemmConfig{128, 128, 2, 2, 1};
        return GemmConfig{256, 256, 2, 4, 1};
    }
    // the fast promotion keeps at most 256 per-K-tile factors in registers and cannot apply a
    // factor that varies per row of A inside the loop: those cases take the literal kernel
    if (strict || modeA == 2 || K > 256 * 128) return GemmConfig{128, 128, 2, 2, 3};
    // operand B scaled per (row, K block): 256 x 256 tiles with the chained promotion where they fill the machine
    if (modeB == 2) return (large || tiles_256x256 >= num_cu) ? GemmConfig{256, 256, 2, 4, 6} : GemmConfig{256, 128, 4, 2, 4};
    // 256 x 256 tiles (128 x 64 per wave, float accumulators only) where they fill the machine, else
    // 256 x 128 (64 x 64 per wave, int32 + float accumulators), else 128 x 128
    if (large || tiles_256x256 >= num_cu) return GemmConfig{256, 256, 2, 4, 5};
    if (tiles_256x128 >= num_cu) return GemmConfig{256, 128, 4, 2, 2};
    return GemmConfig{128, 128, 2, 2, 2};
}

}  // namespace idx
}  // namespace ti8
