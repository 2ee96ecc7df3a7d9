// Host-side walk over the launches of libti8's kernels: for the geometry an entry point would
// launch, visit every (workgroup, wave, lane, iteration) and check each global-memory access
// against the number of elements that lie between the pointer the caller passed and the end of
// its allocation.  The offsets come from triton-int8_amd/csrc/index_math.h, the same functions the
// kernels call; what is mirrored by hand here is only the order in which a kernel combines them
// (each such place cites the kernel's lines).  Built with g++ by tests/test_kernel_bounds.py: no
// GPU, no HIP.
//
// Every walk_* function returns 0 when all accesses are in bounds (and, for the GEMM, when every
// element of C is stored exactly once), else 1 with a description of the first violation in msg.
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "index_math.h"

using namespace ti8::idx;

namespace {

struct Report {
    char* msg;
    int len;
    bool bad = false;
    int64_t checked = 0;
    void fail(const char* fmt, ...) {
        if (bad) return;
        bad = true;
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(msg, len, fmt, ap);
        va_end(ap);
    }
    // access of `n` elements at element offset `off` of a buffer with `size` elements
    bool access(const char* what, int64_t off, int64_t n, int64_t size, int64_t a = -1, int64_t b = -1, int64_t c = -1, int64_t d = -1) {
        ++checked;
        if (off < 0 || off + n > size) {
            fail("%s: elements [%lld, %lld) outside the buffer of %lld (at %lld, %lld, %lld, %lld)", what, (long long)off,
                 (long long)(off + n), (long long)size, (long long)a, (long long)b, (long long)c, (long long)d);
            return false;
        }
        return true;
    }
};

}  // namespace

extern "C" {

// ti8_fwht -> fwht_kernel<NT, false> (fwht.hip): bf16 x [rows][cols] (ldx) -> y (ldy).
// quant: ti8_fwht_quant_row -> fwht_kernel<NT, true>: one workgroup per row (L = n), int8 q [rows][cols] (ldy = ldq, y_elems
// = bytes of q) and one fp32 scale per row (s_elems) instead of y
static int walk_fwht_impl(bool quant, int64_t ldx, int64_t ldy, int64_t rows, int64_t cols, int64_t n, int64_t x_elems, int64_t y_elems,
                          int64_t s_elems, int64_t lds_bytes_limit, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    const int64_t L = quant ? n : fwht_segment_len(cols, n);
    if (quant && cols > n) r.fail("fwht_quant_row: %lld columns exceed the transform length %lld", (long long)cols, (long long)n);
    if (n >= 4096) {
        // fwht_row_kernel<CH, QUANT>: 4 waves, slice by slice through a 2 x 4096-word exchange buffer, results stored from registers
        const int CH = (int)(n / 4096);
        const bool extended = cols < L;
        const int valid = (int)(extended ? cols : L);
        const int segs_per_row = extended ? 1 : (int)(cols / L);
        const int64_t nblocks = rows * segs_per_row;
        const int64_t lds_words = (CH > 1 ? 2 : 1) * 4 * 64 * 16;
        if (lds_words * 4 > 65536) r.fail("fwht rows: %lld bytes of static LDS", (long long)(lds_words * 4));
        if (quant && segs_per_row != 1) r.fail("fwht_quant_row: %d segments per row", segs_per_row);
        std::vector<uint8_t> taken((size_t)L / 4, 0);   // every group of 4 output elements belongs to exactly one thread
        for (int tid = 0; tid < 256 && !r.bad; ++tid) {
            const int lane = tid & 63, w = tid >> 6, lp = (lane & ~15) | had_chunk(lane & 15);
            for (int k = 0; k < CH; ++k) {
                const int64_t base = (int64_t)(k & 1) * 4 * 64 * 16;
                for (int e = 0; e < 16; ++e) r.access("fwht rows lds write", base + fwht_row_lds(w, lp, e), 1, lds_words, tid, k, e);
                for (int ws = 0; ws < 4; ++ws) {
                    for (int e = 0; e < 4; ++e) r.access("fwht rows lds read", base + fwht_row_lds(ws, lp, 4 * w + e), 1, lds_words, tid, k, ws, e);
                    const int first = fwht_row_out(k, ws, lp, w);
                    if (first < 0 || first + 4 > L || first % 4) { r.fail("fwht rows: thread %d owns elements from %d of %lld", tid, first, (long long)L); break; }
                    ++taken[(size_t)first / 4];
                }
            }
            if (quant) r.access("fwht rows lds wave maxima", w, 1, lds_words, tid);
        }
        for (size_t i = 0; i < taken.size() && !r.bad; ++i)
            if (taken[i] != 1) r.fail("fwht rows: elements %lld.. are stored by %d threads", (long long)(i * 4), (int)taken[i]);
        for (int64_t block = 0; block < nblocks && !r.bad; ++block) {
            const int64_t xo = fwht_segment_offset(block, segs_per_row, ldx, (int)L);
            const int64_t yo = fwht_segment_offset(block, segs_per_row, ldy, (int)L);
            for (int tid = 0; tid < 256; ++tid) {
                const int lane = tid & 63, w = tid >> 6, lp = (lane & ~15) | had_chunk(lane & 15);
                for (int k = 0; k < CH; ++k) {
                    const int first = fwht_row_chunk_first(k, w, lp);
                    const int from = fwht_chunk_valid(first, 16, valid) ? first : 0;   // a chunk past the end re-reads the first one
                    r.access("fwht x", xo + from, 8, x_elems, block, tid, k);
                    r.access("fwht x", xo + from + 8, 8, x_elems, block, tid, k);
                    for (int ws = 0; ws < 4; ++ws) {
                        const int out = fwht_row_out(k, ws, lp, w);
                        if (fwht_chunk_valid(out, 4, valid)) r.access(quant ? "fwht q" : "fwht y", yo + out, 4, y_elems, block, tid, k, ws);
                    }
                }
                if (quant && tid == 0) r.access("fwht s", block, 1, s_elems, block);
            }
        }
        *n_checked = r.checked;
        return r.bad;
    }
    const int NT = fwht_threads(L);
    const bool extended = cols < L;             // a zero-extended row per workgroup
    const int valid = (int)(extended ? cols : L);
    const int64_t nblocks = rows * (extended ? 1 : cols / L);
    const int64_t lds_words = fwht_lds_words(L);
    if (lds_words * 4 > lds_bytes_limit) r.fail("fwht: %lld bytes of LDS requested, limit %lld", (long long)(lds_words * 4), (long long)lds_bytes_limit);
    int logn = 0;
    while ((1LL << logn) < n) ++logn;
    const int segs_per_row = extended ? 1 : (int)(cols / L);
    // LDS indices do not depend on the workgroup: walk them once
    // segments of 1024 elements and more run bits 4..9 across the lanes of a wave (lane l of a row of 16 takes chunk
    // had_chunk(l)); that needs whole waves of chunks
    const bool by_lanes = L >= 1024;
    if (by_lanes && ((L >> 4) % 64)) r.fail("fwht: %lld chunks are not whole waves", (long long)(L >> 4));
    for (int tid = 0; tid < NT && !r.bad; ++tid) {
        for (int v0 = tid; v0 < (L >> 4); v0 += NT) {
            const int vt = by_lanes ? ((v0 & ~15) | had_chunk(v0 & 15)) : v0;
            for (int e = 0; e < 16; ++e) r.access("fwht lds first pass", vt * 17 + e, 1, lds_words, tid, vt, e);
        }
        auto pass = [&](int p, int rb) {   // pass_in_lds<RB, NT>
            const int ngroups = (int)(L >> rb);
            for (int vt = tid; vt < ngroups; vt += NT) {
                const int base = fwht_group_base(vt, p, rb);
                for (int e = 0; e < (1 << rb); ++e) r.access("fwht lds pass", fwht_padded(base + (e << p)), 1, lds_words, tid, vt, e, p);
            }
        };
        if (by_lanes) {
            if (logn - 10 > 0) pass(10, logn - 10);
        } else {
            const int rb1 = imin(4, logn - 4);
            pass(4, rb1);
            int rem = logn - 8;
            if (rem > 0) {
                const int rb2 = rem <= 5 ? rem : (rem + 1) / 2;
                pass(8, rb2);
                rem -= rb2;
                if (rem > 0) pass(8 + rb2, rem);
            }
        }
        if (quant) {   // one chunk per thread is kept in registers; the first words of LDS then hold one maximum per wave
            if (tid < (L >> 3)) r.access("fwht lds read-back", fwht_padded(tid * 8), 8, lds_words, tid);
            r.access("fwht lds wave maxima", tid >> 6, 1, lds_words, tid);
        } else {
            for (int c = tid; c < (L >> 3); c += NT) r.access("fwht lds read-back", fwht_padded(c * 8), 8, lds_words, tid, c);
        }
    }
    if (quant && (L >> 3) > NT) r.fail("fwht_quant_row: %lld chunks do not fit one per thread on %d threads", (long long)(L >> 3), NT);
    for (int64_t block = 0; block < nblocks && !r.bad; ++block) {
        const int64_t xo = fwht_segment_offset(block, segs_per_row, ldx, (int)L);
        const int64_t yo = fwht_segment_offset(block, segs_per_row, ldy, (int)L);
        for (int tid = 0; tid < NT; ++tid) {
            for (int v0 = tid; v0 < (L >> 4); v0 += NT) {   // two 16-byte loads: elements vt*16 .. +16
                const int vt = by_lanes ? ((v0 & ~15) | had_chunk(v0 & 15)) : v0;
                if (!fwht_chunk_valid(vt * 16, 16, valid)) continue;
                r.access("fwht x", xo + vt * 16, 8, x_elems, block, tid, vt);
                r.access("fwht x", xo + vt * 16 + 8, 8, x_elems, block, tid, vt);
            }
            for (int c = tid; c < (L >> 3); c += NT)
                if (fwht_chunk_valid(c * 8, 8, valid)) r.access(quant ? "fwht q" : "fwht y", yo + c * 8, 8, y_elems, block, tid, c);
            if (quant && tid == 0) r.access("fwht s", block, 1, s_elems, block);
        }
    }
    *n_checked = r.checked;
    return r.bad;
}
int walk_fwht(int64_t ldx, int64_t ldy, int64_t rows, int64_t cols, int64_t n, int64_t x_elems, int64_t y_elems,
              int64_t lds_bytes_limit, int64_t* n_checked, char* msg, int msglen) {
    return walk_fwht_impl(false, ldx, ldy, rows, cols, n, x_elems, y_elems, 0, lds_bytes_limit, n_checked, msg, msglen);
}
int walk_fwht_quant_row(int64_t ldx, int64_t ldq, int64_t rows, int64_t cols, int64_t n, int64_t x_elems, int64_t q_elems, int64_t s_elems,
                        int64_t lds_bytes_limit, int64_t* n_checked, char* msg, int msglen) {
    return walk_fwht_impl(true, ldx, ldq, rows, cols, n, x_elems, q_elems, s_elems, lds_bytes_limit, n_checked, msg, msglen);
}

// transpose_bf16_kernel (fwht.hip): x bf16 [R][C] (ldx) -> y bf16 [C][R] (ldy), 64 x 64 tiles
static void walk_transpose_tiles(Report& r, int64_t ldx, int64_t ldy, int64_t R, int64_t C, int64_t x_elems, int64_t y_elems) {
    if (R % 64 || C % 64) { r.fail("transpose: %lld x %lld is not made of 64 x 64 tiles", (long long)R, (long long)C); return; }
    const int tiles_c = (int)(C / 64);
    for (int64_t block = 0; block < (R / 64) * (C / 64) && !r.bad; ++block) {
        const int64_t tc = block % tiles_c, tr = block / tiles_c;
        for (int tid = 0; tid < 256; ++tid)
            for (int h = 0; h < 2; ++h) {
                const int a = (tid >> 3) + 32 * h, b = (tid & 7) * 8;
                r.access("fwht_t transpose x", (tr * 64 + a) * ldx + tc * 64 + b, 8, x_elems, block, tid, h);
                r.access("fwht_t transpose y", (tc * 64 + a) * ldy + tr * 64 + b, 8, y_elems, block, tid, h);
            }
    }
}
int walk_transpose_bf16(int64_t ldx, int64_t ldy, int64_t R, int64_t C, int64_t x_elems, int64_t y_elems, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    walk_transpose_tiles(r, ldx, ldy, R, C, x_elems, y_elems);
    *n_checked = r.checked;
    return r.bad;
}

// ti8_fwht_t -> fwht_t_kernel<NT, W> (fwht.hip): x bf16 [R][C] (ldx) -> y bf16 [C][R] (ldy)
int walk_fwht_t(int64_t ldx, int64_t ldy, int64_t R, int64_t C, int64_t x_elems, int64_t y_elems, int64_t lds_bytes_limit,
                int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    if (!fwht_t_direct(R, C)) {
        // transpose_bf16_kernel: 64 x 64 tiles, thread t reads 8 columns of rows t/8 and t/8 + 32 and writes 8 rows
        // of columns t/8 and t/8 + 32; then fwht_kernel in place on y [C][R]
        walk_transpose_tiles(r, ldx, ldy, R, C, x_elems, y_elems);
        int64_t n2 = 0;
        const int bad = r.bad ? 1 : walk_fwht(ldy, ldy, C, R, R, y_elems, y_elems, lds_bytes_limit, &n2, msg, msglen);
        *n_checked = r.checked + n2;
        return bad;
    }
    const int W = fwht_t_cols_per_wg(R);
    const int NT = (int64_t)W * R >= 16384 ? 1024 : 256;
    const int64_t nblocks = C / W;
    const int64_t Lp = fwht_lds_words(R), lds_words = (int64_t)W * Lp;
    if (C % W) r.fail("fwht_t: %lld columns are not a multiple of %d per workgroup", (long long)C, W);
    if (lds_words * 4 > lds_bytes_limit) r.fail("fwht_t: %lld bytes of LDS requested, limit %lld", (long long)(lds_words * 4), (long long)lds_bytes_limit);
    int logn = 0;
    while ((1LL << logn) < R) ++logn;
    // LDS indices (the same for every workgroup)
    for (int tid = 0; tid < NT && !r.bad; ++tid) {
        for (int row = tid; row < R; row += NT)
            for (int w = 0; w < W; ++w) r.access("fwht_t lds fill", w * Lp + fwht_padded(row), 1, lds_words, tid, row, w);
        auto pass = [&](int p, int rb) {   // pass_in_lds_segments<RB, NT>
            const int per_seg = (int)(R >> rb);
            for (int vt = tid; vt < W * per_seg; vt += NT) {
                const int base = fwht_group_base(vt % per_seg, p, rb);
                for (int e = 0; e < (1 << rb); ++e)
                    r.access("fwht_t lds pass", (vt / per_seg) * Lp + fwht_padded(base + (e << p)), 1, lds_words, tid, vt, e, p);
            }
        };
        pass(0, 4);
        pass(4, imin(4, logn - 4));
        int rem = logn - 8;
        if (rem > 0) {
            const int rb2 = rem <= 5 ? rem : (rem + 1) / 2;
            pass(8, rb2);
            rem -= rb2;
            if (rem > 0) pass(8 + rb2, rem);
        }
        const int per_seg = (int)(R >> 3);
        for (int i = tid; i < W * per_seg; i += NT) r.access("fwht_t lds read-back", (i / per_seg) * Lp + fwht_padded((i % per_seg) * 8), 8, lds_words, tid, i);
    }
    std::vector<uint8_t> seen((size_t)nblocks, 0);
    for (int64_t block = 0; block < nblocks && !r.bad; ++block) {
        const int64_t cb = fwht_t_colblock(block, nblocks, W);
        if (cb < 0 || cb >= nblocks) { r.fail("fwht_t: workgroup %lld maps to column block %lld of %lld", (long long)block, (long long)cb, (long long)nblocks); break; }
        ++seen[(size_t)cb];
        const int64_t c0 = cb * W;
        for (int tid = 0; tid < NT; ++tid) {
            for (int row = tid; row < R; row += NT) r.access("fwht_t x", (int64_t)row * ldx + c0, W, x_elems, block, tid, row);
            const int per_seg = (int)(R >> 3);
            for (int i = tid; i < W * per_seg; i += NT) r.access("fwht_t y", (c0 + i / per_seg) * ldy + (int64_t)(i % per_seg) * 8, 8, y_elems, block, tid, i);
        }
    }
    for (int64_t cb = 0; cb < nblocks && !r.bad; ++cb)
        if (seen[(size_t)cb] != 1) r.fail("fwht_t: column block %lld is transformed %d times", (long long)cb, (int)seen[(size_t)cb]);
    *n_checked = r.checked;
    return r.bad;
}

// ti8_quant_row -> quant_row_kernel<NLOAD, WG_ROW, GROUP16, HAD> (quant.hip)
int walk_quant_row(int64_t ldx, int64_t ldq, int64_t rows, int64_t cols, int group, int64_t x_elems, int64_t q_elems,
                   int64_t s_elems, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    const int nchunk = (int)(cols / 8);
    const QRowConfig cfg = qrow_config(nchunk, group == 128);
    const int64_t grid = cfg.wg_row ? rows : (rows + 3) / 4;
    const int T = cfg.wg_row ? 256 : 64;
    const int ngrp = (int)(cols >> 7);
    std::vector<uint8_t> seen((size_t)rows, 0);
    for (int64_t block = 0; block < grid && !r.bad; ++block)
        for (int tid = 0; tid < 256; ++tid) {
            const int t = cfg.wg_row ? tid : (tid & 63);
            const int64_t row = qrow_row(block, tid >> 6, cfg.wg_row);
            if (row >= rows) continue;
            if (t == 0) ++seen[(size_t)row];
            for (int i = 0; i < cfg.nload; ++i) {
                const int c = qrow_chunk(t, i, T);
                if (c >= nchunk) continue;
                r.access("quant_row x", row * ldx + c * 8, 8, x_elems, block, tid, i);
                r.access("quant_row q", row * ldq + c * 8, 8, q_elems, block, tid, i);
                if (group == 128 && (c & 15) == 0) r.access("quant_row s", row * ngrp + (c >> 4), 1, s_elems, block, tid, i);
            }
            if (group != 128 && t == 0) r.access("quant_row s", row, 1, s_elems, block, tid);
        }
    // every chunk of a row is taken by exactly one (thread, load): T * NLOAD covers the row
    if ((int64_t)T * cfg.nload < nchunk) r.fail("quant_row: %d threads x %d loads do not cover %d chunks", T, cfg.nload, nchunk);
    for (int64_t row = 0; row < rows && !r.bad; ++row)
        if (seen[(size_t)row] != 1) r.fail("quant_row: row %lld handled %d times", (long long)row, (int)seen[(size_t)row]);
    *n_checked = r.checked;
    return r.bad;
}

// ti8_quant_block -> quant_block_kernel<NSUB, WRITE_Q, WRITE_QT> (quant.hip)
int walk_quant_block(int64_t bsx, int64_t ldx, int has_q, int64_t bsq, int64_t ldq, int has_qt, int64_t bsqt, int64_t ldqt,
                     int64_t ssb, int64_t ssr, int64_t ssc, int64_t B, int64_t R, int64_t C, int group_c, int64_t x_elems,
                     int64_t q_elems, int64_t qt_elems, int64_t s_elems, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    const int nsub = group_c / 128;
    const int nrb = (int)(R / 128), ncb = (int)(C / group_c);
    const int64_t ntiles = B * nrb * ncb;
    for (int64_t block = 0; block < ntiles && !r.bad; ++block) {
        const TileId t = qblock_tile((int)block, nrb, ncb);
        const int64_t xo = qblock_origin(t.b, bsx, t.rb, ldx, t.cb, 128 * nsub);
        r.access("quant_block s", t.b * ssb + t.rb * ssr + t.cb * ssc, 1, s_elems, block);
        for (int tid = 0; tid < 256; ++tid) {
            for (int u = 0; u < nsub; ++u)
                for (int h = 0; h < 2; ++h)
                    for (int j = 0; j < 4; ++j) {
                        const int row = qblock_row(tid, h, j);
                        r.access("quant_block x", xo + (int64_t)row * ldx + u * 128 + qblock_col(tid), 8, x_elems, block, tid, h, j);
                        if (has_q)
                            r.access("quant_block q", qblock_origin(t.b, bsq, t.rb, ldq, t.cb, 128 * nsub) + u * 128 + qblock_col(tid) + (int64_t)row * ldq,
                                     8, q_elems, block, tid, h, j);
                    }
            if (has_qt) {
                const int64_t qo = qblock_origin(t.b, bsqt, t.cb, ldqt, t.rb, 128);
                for (int p = 0; p < 4; ++p) r.access("quant_block qT", qo + (int64_t)qblock_t_row(tid, p) * ldqt + qblock_t_col(tid), 16, qt_elems, block, tid, p);
            }
        }
    }
    *n_checked = r.checked;
    return r.bad;
}

struct ScaleArg {
    int mode;
    int64_t bs, rs, ks, elems;
};

// ti8_gemm_i8_nt / ti8_gemm_i8_nt_i32 -> gemm_i8_kernel<BM, BN, WM, WN, EPI> (gemm.hip); the
// tile shape and epilogue kind are chosen as the entry point chooses them (raw_i32 = 1: the
// int32-output entry point, always 256 x 256 tiles).  epi: 0 raw int32, 1 rows, 2 promote,
// 3 literal, 4 per-lane B factors, 5 chained promote.
int walk_gemm(int64_t bsa, int64_t lda, int64_t bsb, int64_t ldb, int64_t bsc, int64_t ldc, const ScaleArg* sa_in,
              const ScaleArg* sb_in, int64_t batch, int64_t M, int64_t N, int64_t K, int acc_i32_full, int strict, int large,
              int raw_i32, int num_cu, int64_t a_elems, int64_t b_elems, int64_t c_elems, int* picked, int64_t* n_checked,
              char* msg, int msglen) {
    Report r{msg, msglen};
    ScaleArg sa = sa_in ? *sa_in : ScaleArg{0, 0, 0, 0, 0}, sb = sb_in ? *sb_in : ScaleArg{0, 0, 0, 0, 0};
    GemmConfig cfg = raw_i32 ? GemmConfig{256, 256, 2, 4, 0}
                             : gemm_config(M, N, K, batch, acc_i32_full != 0, strict != 0, sa.mode, sb.mode, large != 0, num_cu);
    picked[0] = cfg.bm; picked[1] = cfg.bn; picked[2] = cfg.epi;
    const int BM = cfg.bm, BN = cfg.bn, WM = cfg.wm, WN = cfg.wn, EPI = cfg.epi;
    const int NW = WM * WN, TM = BM / WM / 32, TN = BN / WN / 32, A_INSTR = BM / 8 / NW, B_INSTR = BN / 8 / NW;
    const int A_BYTES = BM * 128, B_BYTES = BN * 128;
    const bool CHAIN = EPI == 5 || EPI == 6, LANEB = EPI == 4 || EPI == 6, FAST = EPI == 2 || EPI == 4 || CHAIN;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    const int nk = (int)(K >> 7), klast = (nk - 1) * 128;
    const int WCOLS = TN * 32, LPR = WCOLS / 8, RPI = 64 / LPR, NRR = 32 / RPI;
    const int GROUP = gemm_group_rows(BM);
    (void)CHAIN;
    std::vector<uint8_t> stored(c_elems <= (int64_t)1 << 30 ? (size_t)c_elems : 0, 0);
    std::vector<uint8_t> tile_seen((size_t)tiles_m * tiles_n, 0);
    // K tiles whose loads are checked: offsets grow with kt up to the clamp, so the first two and
    // the clamped ones (nk - 1, nk, nk + 1: the loop fetches up to two tiles ahead) cover all
    const int kts[5] = {0, 1, nk - 1, nk, nk + 1};
    for (int64_t by = 0; by < batch && !r.bad; ++by) {
        std::fill(tile_seen.begin(), tile_seen.end(), 0);
        for (int bx = 0; bx < tiles_m * tiles_n && !r.bad; ++bx) {
            const TileCoord tc = gemm_tile_of(bx, tiles_m, tiles_n, GROUP);
            if (tc.tile_m < 0 || tc.tile_m >= tiles_m || tc.tile_n < 0 || tc.tile_n >= tiles_n) {
                r.fail("gemm: workgroup %d maps to tile (%d, %d) outside %d x %d", bx, tc.tile_m, tc.tile_n, tiles_m, tiles_n);
                break;
            }
            ++tile_seen[(size_t)tc.tile_m * tiles_n + tc.tile_n];
            const int m0 = tc.tile_m * BM, n0 = tc.tile_n * BN;
            for (int wave = 0; wave < NW; ++wave) {
                const int wm = wave / WN, wn = wave % WN;
                const int rA0 = gemm_wave_first_row(m0, wave, A_INSTR, (int)M), rB0 = gemm_wave_first_row(n0, wave, B_INSTR, (int)N);
                const int tA0 = wave * A_INSTR, tB0 = wave * B_INSTR;
                for (int lane = 0; lane < 64; ++lane) {
                    // ---- global -> LDS loads (gemm.hip: voffA/voffB, baseA/baseB, issue_tile_loads)
                    for (int q = 0; q < 5; ++q) {
                        const int koff = gemm_k_offset(kts[q], klast);
                        for (int i = 0; i < A_INSTR; ++i) {
                            const uint32_t vo = gemm_lane_offset_bytes(lane, (tA0 + i) & 1, (int)lda);
                            r.access("gemm A", by * bsa + gemm_load_offset_bytes(rA0, lda, koff, i, vo), 16, a_elems, bx, wave, lane, kts[q]);
                            const int64_t lds = (int64_t)wave * A_INSTR * 1024 + i * 1024 + lane * 16;
                            r.access("gemm LDS A", lds, 16, A_BYTES, bx, wave, lane, i);
                        }
                        for (int i = 0; i < B_INSTR; ++i) {
                            const uint32_t vo = gemm_lane_offset_bytes(lane, (tB0 + i) & 1, (int)ldb);
                            r.access("gemm B", by * bsb + gemm_load_offset_bytes(rB0, ldb, koff, i, vo), 16, b_elems, bx, wave, lane, kts[q]);
                            const int64_t lds = (int64_t)wave * B_INSTR * 1024 + i * 1024 + lane * 16;
                            r.access("gemm LDS B", lds, 16, B_BYTES, bx, wave, lane, i);
                        }
                    }
                    const int fr_row = lane & 31, fr_half = lane >> 5;
                    // ---- per-K-tile factors of the fast promotion (gemm.hip: fraw_a / fraw_b, pfb)
                    if (FAST) {
                        const bool a_in = sa.mode != 0, b_in = sb.mode != 0;
                        const int sha = sa.mode == 3 ? 1 : 0, shb = sb.mode == 3 ? 1 : 0;
                        const int rowblk = gemm_factor_block(m0 + wm * TM * 32, (int)M), colblk = gemm_factor_block(n0 + wn * TN * 32, (int)N);
                        const int64_t ska = a_in ? sa.ks : 0, skb = (b_in && !LANEB) ? sb.ks : 0;
                        for (int c = 0; c < 4; ++c) {
                            const int kt = gemm_factor_kt(c, lane, nk);
                            r.access("gemm factor A", gemm_factor_index(by, sa.bs, rowblk, sa.rs, kt, sha, ska), 1, sa.elems, bx, wave, lane, c);
                            r.access("gemm factor B", gemm_factor_index(by, sb.bs, colblk, sb.rs, kt, shb, skb), 1, sb.elems, bx, wave, lane, c);
                        }
                        if (LANEB)
                            for (int j = 0; j < TN; ++j) {
                                const int64_t base = epi_col_scale_index(by, sb.bs, n0 + (wn * TN + j) * 32 + fr_row, (int)N, sb.rs);
                                for (int kt = 0; kt < nk; ++kt) r.access("gemm lane factor B", base + (int64_t)kt * sb.ks, 1, sb.elems, bx, wave, lane, kt);
                            }
                    }
                    // ---- literal promotion: one scale per element and K tile (gemm.hip: EPI_STRICT block)
                    if (EPI == 3) {
                        const int kk[2] = {0, nk - 1};
                        for (int q = 0; q < 2; ++q)
                            for (int i = 0; i < TM; ++i)
                                for (int j = 0; j < TN; ++j) {
                                    const int col = imin(n0 + (wn * TN + j) * 32 + fr_row, (int)N - 1);
                                    r.access("gemm strict B scale", scale_index(sb.mode, sb.bs, sb.rs, sb.ks, by, col, kk[q]), 1, sb.elems, bx, wave, lane, kk[q]);
                                    for (int e = 0; e < 16; ++e) {
                                        const int mrow = imin(m0 + (wm * TM + i) * 32 + 8 * (e >> 2) + 4 * fr_half + (e & 3), (int)M - 1);
                                        r.access("gemm strict A scale", scale_index(sa.mode, sa.bs, sa.rs, sa.ks, by, mrow, kk[q]), 1, sa.elems, bx, wave, lane, kk[q]);
                                    }
                                }
                    }
                    // ---- epilogue (gemm.hip: coln, cm, prow0 / rm_all, store_tile)
                    const bool col_part = EPI == 1 || (FAST && sb.mode == 0), row_part = EPI == 1 || (FAST && sa.mode == 0);
                    if (EPI == 1 || FAST) {   // column scales, fetched before the main loop by every wave
                        const int64_t cs = col_part ? sb.rs : 0;
                        const int ncol0 = n0 + wn * WCOLS + epi_scale_col_of_lane(lane);
                        for (int c = 0; c < 4; ++c) r.access("gemm column scale", epi_col_scale_index(by, sb.bs, ncol0 + c, (int)N, cs), 1, sb.elems, bx, wave, lane, c);
                    }
                    // a wave whose tile lies outside the output stops here
                    if (m0 + wm * TM * 32 >= M || n0 + wn * WCOLS >= N) continue;
                    const int rb_col = epi_col_of_lane(lane, WCOLS), rb_row = epi_row_of_lane(lane, WCOLS);
                    for (int c = 0; c < 8; ++c) {   // the lane that holds this lane's column scale c, and the column it fetched
                        const int src = epi_scale_lane(lane, c);
                        if (src < 0 || src >= 64 || epi_scale_col_of_lane(src) + (c & 3) != rb_col + c)
                            r.fail("gemm: lane %d takes column scale %d from lane %d, which holds column %d, not %d", lane, c, src,
                                   epi_scale_col_of_lane(src) + (c & 3), rb_col + c);
                    }
                    const int row0 = m0 + wm * TM * 32 + rb_row;
                    if (row_part) {
                        const int64_t base = epi_row_scale_base(by, sa.bs, row0, sa.rs);
                        for (int i = 0; i < TM; ++i)
                            for (int k = 0; k < NRR; ++k)
                                r.access("gemm row scale", base + (int64_t)(i * 32 + k * RPI) * sa.rs, 1, sa.elems, bx, wave, lane, i * NRR + k);
                    }
                    // slab: 32 rows of EPI_SLAB_LD words per wave, inside the operand buffers
                    for (int e = 0; e < 16; ++e)
                        for (int j = 0; j < TN; ++j) {
                            const int rr = 8 * (e >> 2) + 4 * fr_half + (e & 3);
                            r.access("gemm slab write", (int64_t)wave * 32 * EPI_SLAB_LD(WCOLS) + rr * EPI_SLAB_LD(WCOLS) + j * 32 + fr_row, 1,
                                     (2 * (A_BYTES + B_BYTES)) / 4, bx, wave, lane, e);
                        }
                    for (int k = 0; k < NRR; ++k)
                        r.access("gemm slab read", (int64_t)wave * 32 * EPI_SLAB_LD(WCOLS) + (rb_row + k * RPI) * EPI_SLAB_LD(WCOLS) + rb_col, 8,
                                 (2 * (A_BYTES + B_BYTES)) / 4, bx, wave, lane, k);
                    int64_t off = epi_out_offset(by, bsc, row0, ldc, n0 + wn * WCOLS + rb_col);
                    const int64_t c_step = (int64_t)RPI * ldc;
                    for (int i = 0; i < TM; ++i)
                        for (int k = 0; k < NRR; ++k, off += c_step) {
                            if (r.access("gemm C", off, 8, c_elems, bx, wave, lane, i * NRR + k) && !stored.empty())
                                for (int c = 0; c < 8; ++c) ++stored[(size_t)(off + c)];
                        }
                }
            }
        }
        for (size_t t = 0; t < tile_seen.size() && !r.bad; ++t)
            if (tile_seen[t] != 1) r.fail("gemm: tile %zu of batch %lld is computed %d times", t, (long long)by, (int)tile_seen[t]);
    }
    // every element of C [batch][M][N] stored exactly once, nothing else touched
    if (!stored.empty() && !r.bad) {
        int64_t expect = 0;
        for (int64_t b = 0; b < batch && !r.bad; ++b)
            for (int64_t m = 0; m < M && !r.bad; ++m)
                for (int64_t n = 0; n < N; ++n) {
                    const int64_t o = b * bsc + m * ldc + n;
                    if (stored[(size_t)o] != 1) {
                        r.fail("gemm: C[%lld][%lld][%lld] stored %d times", (long long)b, (long long)m, (long long)n, (int)stored[(size_t)o]);
                        break;
                    }
                    ++expect;
                }
        int64_t total = 0;
        for (size_t i = 0; i < stored.size(); ++i) total += stored[i];
        if (!r.bad && total != expect) r.fail("gemm: %lld stores, %lld elements of C", (long long)total, (long long)expect);
    }
    *n_checked = r.checked;
    return r.bad;
}

// Persistent chained kernel (gemm_chain.hip: gemm_i8_chain_kernel) on one GEMM with `batch` batches and `grid`
// workgroups: workgroup w walks tiles w, w + grid, ...; a tile's K tiles are fetched by its own iterations except
// K tiles 0 and 1, which the previous tile's last iterations (or, for a workgroup's first tile, its start) fetch, and
// the workgroup's last tile fetches its own K tiles 0 and 1 once more.  Checked: every tile of every batch is taken
// exactly once, every global -> LDS load, scale load, slab access and store lies inside its buffer, every element
// of C is stored exactly once.
int walk_gemm_chain(int64_t bsa, int64_t lda, int64_t bsb, int64_t ldb, int64_t bsc, int64_t ldc, const ScaleArg* sa_in,
                    const ScaleArg* sb_in, int64_t batch, int64_t M, int64_t N, int64_t K, int grid, int64_t a_elems,
                    int64_t b_elems, int64_t c_elems, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    const ScaleArg sa = *sa_in, sb = *sb_in;
    const int BM = 256, BN = 256, WN = 4, NW = 8, TM = 4, TN = 2, A_INSTR = 4, B_INSTR = 4, WCOLS = 64, RPI = 8;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN), per_batch = tiles_m * tiles_n;
    const int total = per_batch * (int)batch, nk = (int)(K >> 7), GROUP = gemm_group_rows(BM);
    const int64_t lds_words = (2 * (BM + BN) * 128 + NW * 16 * WCOLS * 4) / 4, slab0 = 2 * (BM + BN) * 128 / 4;
    if (nk < 2 || nk > 256 || (nk & 1)) { r.fail("gemm chain: K / 128 = %d is odd or outside [2, 256]", nk); *n_checked = 0; return 1; }
    std::vector<uint8_t> stored(c_elems <= (int64_t)1 << 30 ? (size_t)c_elems : 0, 0);
    std::vector<uint8_t> seen((size_t)total, 0);
    const bool a_in = sa.mode != 0, b_in = sb.mode != 0;
    for (int w = 0; w < grid && !r.bad; ++w)
        for (int T = w; T < total && !r.bad; T += grid) {
            ++seen[(size_t)T];
            const int64_t by = T / per_batch;
            const TileCoord tc = gemm_tile_of(T - (int)by * per_batch, tiles_m, tiles_n, GROUP);
            if (tc.tile_m < 0 || tc.tile_m >= tiles_m || tc.tile_n < 0 || tc.tile_n >= tiles_n) {
                r.fail("gemm chain: tile %d maps to (%d, %d) outside %d x %d", T, tc.tile_m, tc.tile_n, tiles_m, tiles_n);
                break;
            }
            const int m0 = tc.tile_m * BM, n0 = tc.tile_n * BN;
            for (int wave = 0; wave < NW; ++wave) {
                const int wm = wave / WN, wn = wave % WN;
                const int rA0 = gemm_wave_first_row(m0, wave, A_INSTR, (int)M), rB0 = gemm_wave_first_row(n0, wave, B_INSTR, (int)N);
                const int tA0 = wave * A_INSTR, tB0 = wave * B_INSTR;
                const int kts[4] = {0, 1, nk - 2, nk - 1};
                for (int lane = 0; lane < 64; ++lane) {
                    for (int q = 0; q < 4; ++q) {
                        const int koff = kts[q] * 128;
                        for (int i = 0; i < A_INSTR; ++i) {
                            const uint32_t vo = gemm_lane_offset_bytes(lane, (tA0 + i) & 1, (int)lda);
                            r.access("gemm chain A", by * bsa + gemm_load_offset_bytes(rA0, lda, koff, i, vo), 16, a_elems, T, wave, lane, kts[q]);
                        }
                        for (int i = 0; i < B_INSTR; ++i) {
                            const uint32_t vo = gemm_lane_offset_bytes(lane, (tB0 + i) & 1, (int)ldb);
                            r.access("gemm chain B", by * bsb + gemm_load_offset_bytes(rB0, ldb, koff, i, vo), 16, b_elems, T, wave, lane, kts[q]);
                        }
                    }
                    // per-K-tile factors: scalar base + (K tile >> shift) * stride per lane
                    const int64_t fa = gemm_factor_index(by, sa.bs, gemm_factor_block(m0 + wm * TM * 32, (int)M), sa.rs, 0, 0, 0);
                    const int64_t fb = gemm_factor_index(by, sb.bs, gemm_factor_block(n0 + wn * TN * 32, (int)N), sb.rs, 0, 0, 0);
                    for (int c = 0; c <= (nk - 1) >> 6; ++c) {   // the factor register is refilled every 64 K tiles
                        const uint32_t kt = (uint32_t)gemm_factor_kt(c, lane, nk);
                        r.access("gemm chain factor A", fa + (int64_t)((kt >> (sa.mode == 3 ? 1 : 0)) * (uint32_t)(a_in ? sa.ks : 0)), 1, sa.elems, T, wave, lane, c);
                        r.access("gemm chain factor B", fb + (int64_t)((kt >> (sb.mode == 3 ? 1 : 0)) * (uint32_t)(b_in ? sb.ks : 0)), 1, sb.elems, T, wave, lane, c);
                    }
                    // column scales: 4 per lane from the wave tile's first column (clamped for a tile outside N)
                    const uint32_t cs = b_in ? 0u : (uint32_t)sb.rs;
                    const int64_t colp = epi_col_scale_index(by, sb.bs, chain_col_scale_first(n0 + wn * WCOLS, (int)N), (int)N, cs);
                    for (int c = 0; c < 4; ++c)
                        r.access("gemm chain column scale", colp + (int64_t)(((uint32_t)epi_scale_col_of_lane(lane) + c) * cs), 1, sb.elems, T, wave, lane, c);
                    if (m0 + wm * TM * 32 >= M || n0 + wn * WCOLS >= N) continue;   // this wave stores nothing
                    const int rb_col = epi_col_of_lane(lane, WCOLS), rb_row = epi_row_of_lane(lane, WCOLS);
                    for (int c = 0; c < 8; ++c) {
                        const int src = epi_scale_lane(lane, c);
                        if (src < 0 || src >= 64 || epi_scale_col_of_lane(src) + (c & 3) != rb_col + c)
                            r.fail("gemm chain: lane %d takes column scale %d from lane %d", lane, c, src);
                    }
                    const int row0 = m0 + wm * TM * 32 + rb_row;
                    if (!a_in) {
                        const int64_t base = epi_row_scale_base(by, sa.bs, row0, sa.rs);
                        for (int q = 0; q < TM * 4; ++q) r.access("gemm chain row scale", base + (int64_t)(q * RPI) * sa.rs, 1, sa.elems, T, wave, lane, q);
                    }
                    const int fr_row = lane & 31, fr_half = lane >> 5;
                    for (int e = 0; e < 8; ++e)
                        for (int j = 0; j < TN; ++j)
                            r.access("gemm chain slab write", slab0 + wave * 16 * WCOLS + epi_chain_slab_word(epi_chain_slab_row(e, fr_half), j * 32 + fr_row), 1,
                                     lds_words, T, wave, lane, e);
                    for (int k = 0; k < 2; ++k)
                        for (int half = 0; half < 2; ++half)
                            r.access("gemm chain slab read", slab0 + wave * 16 * WCOLS + epi_chain_slab_word(rb_row + k * RPI, rb_col + 4 * half), 4, lds_words,
                                     T, wave, lane, k);
                    int64_t off = epi_out_offset(by, bsc, row0, ldc, n0 + wn * WCOLS + rb_col);
                    for (int q = 0; q < TM * 4; ++q, off += (int64_t)RPI * ldc)
                        if (r.access("gemm chain C", off, 8, c_elems, T, wave, lane, q) && !stored.empty())
                            for (int c = 0; c < 8; ++c) ++stored[(size_t)(off + c)];
                }
            }
        }
    for (int T = 0; T < total && !r.bad; ++T)
        if (seen[(size_t)T] != 1) r.fail("gemm chain: tile %d is computed %d times", T, (int)seen[(size_t)T]);
    if (!stored.empty() && !r.bad) {
        for (int64_t b = 0; b < batch && !r.bad; ++b)
            for (int64_t mm = 0; mm < M && !r.bad; ++mm)
                for (int64_t n = 0; n < N; ++n)
                    if (stored[(size_t)(b * bsc + mm * ldc + n)] != 1) {
                        r.fail("gemm chain: C[%lld][%lld][%lld] stored %d times", (long long)b, (long long)mm, (long long)n, (int)stored[(size_t)(b * bsc + mm * ldc + n)]);
                        break;
                    }
    }
    *n_checked = r.checked;
    return r.bad;
}

// Workgroup -> (GEMM, tile) map of a several-GEMM launch (gemm.hip: gemm_i8_multi_kernel, launch_multi):
// tiles[i] = workgroups of GEMM i.  Every workgroup of the grid must land in a GEMM i < count with
// a tile index in [0, tiles[i]), and every (GEMM, tile) must be taken exactly once.
int walk_gemm_multi_map(const int* tiles, int count, int64_t* n_checked, char* msg, int msglen) {
    Report r{msg, msglen};
    int first[4] = {0, 0, 0, 0};
    int total = 0;
    for (int i = 0; i < count; ++i) {
        first[i] = total;
        total += tiles[i];
    }
    for (int i = count; i < 4; ++i) first[i] = total;
    std::vector<std::vector<int>> seen(count);
    for (int i = 0; i < count; ++i) seen[i].assign(tiles[i], 0);
    for (int w = 0; w < total && !r.bad; ++w) {
        const int i = gemm_multi_pick(w, first[1], first[2], count);
        const int t = w - first[i];
        if (i < 0 || i >= count || t < 0 || t >= tiles[i]) {
            r.fail("gemm multi: workgroup %d maps to GEMM %d tile %d (of %d GEMMs, %d tiles)", w, i, t, count, i >= 0 && i < count ? tiles[i] : -1);
            break;
        }
        ++seen[i][t];
        ++r.checked;
    }
    for (int i = 0; i < count && !r.bad; ++i)
        for (int t = 0; t < tiles[i]; ++t)
            if (seen[i][t] != 1) {
                r.fail("gemm multi: tile %d of GEMM %d is computed %d times", t, i, seen[i][t]);
                break;
            }
    *n_checked = r.checked;
    return r.bad ? 1 : 0;
}

}  // extern "C"
