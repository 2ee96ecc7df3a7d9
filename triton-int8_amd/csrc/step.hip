// One training step of the INT8 linear layer -- Y = X W^T, dX = dY W, dW = dY^T X -- enqueued by ONE call:
// the quantiser launches and the GEMM launch(es) that the Python layer would otherwise issue one entry point at
// a time, on caller-provided outputs and a caller-provided workspace.  Nothing here computes: the entry points
// of quant.hip and gemm.hip are called in the order of a step with sub-buffers of the workspace, so every tensor
// (int8 operands, scales, bf16 outputs) has the bits the separate calls give.
#include "ti8_common.h"

namespace ti8 {

namespace {

// Sub-buffers of the workspace, each starting on a 256-byte boundary.
struct Carver {
    char* base;
    int64_t used = 0;
    template <class T>
    T* take(int64_t count) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += (count * (int64_t)sizeof(T) + 255) / 256 * 256;
        return p;
    }
};

// what one operand needs when it is quantised by rows and by columns (ti8_quant_row_col_t)
struct RowCol {
    int8_t* q;
    int8_t* qT;
    float* s_row;
    float* s_col;
    float* maxima;   // R + C words, zero on entry of the quantiser
    void carve(Carver& c, int64_t R, int64_t C, bool own_maxima) {
        q = c.take<int8_t>(R * C);
        qT = c.take<int8_t>(R * C);
        s_row = c.take<float>(R);
        s_col = c.take<float>(C);
        maxima = own_maxima ? c.take<float>(R + C) : nullptr;
    }
};

// what one operand needs when it is quantised by 128 x 128 blocks with a transposed copy (ti8_quant_block)
struct Blocks {
    int8_t* q;
    int8_t* qT;
    float* s;        // [R / 128][C / 128]
    void carve(Carver& c, int64_t R, int64_t C) {
        q = c.take<int8_t>(R * C);
        qT = c.take<int8_t>(R * C);
        s = c.take<float>((R / 128) * (C / 128));
    }
};

struct BlockChannelLayout {
    Blocks x, dy;
    RowCol w;
    int64_t carve(char* base, int64_t T, int64_t K, int64_t N) {
        Carver c{base};
        x.carve(c, T, K);
        dy.carve(c, T, N);
        w.carve(c, N, K, true);
        return c.used;
    }
};

struct DoubleChannelLayout {
    RowCol x, w, dy;
    float* maxima;     // the three operands' maxima in one piece, so that one fill clears them
    int64_t maxima_words;
    int64_t carve(char* base, int64_t T, int64_t K, int64_t N) {
        Carver c{base};
        x.carve(c, T, K, false);
        w.carve(c, N, K, false);
        dy.carve(c, T, N, false);
        maxima_words = (T + K) + (N + K) + (T + N);
        maxima = c.take<float>(maxima_words);
        x.maxima = maxima;
        w.maxima = maxima ? maxima + (T + K) : nullptr;
        dy.maxima = maxima ? maxima + (T + K) + (N + K) : nullptr;
        return c.used;
    }
};

ti8_gemm_problem gemm2d(const int8_t* A, int64_t lda, const float* sA, int modeA, int64_t sa_rs, int64_t sa_ks,
                        const int8_t* B, int64_t ldb, const float* sB, int modeB, int64_t sb_rs, int64_t sb_ks,
                        void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int acc_i32_full) {
    ti8_gemm_problem p;
    p.A = A; p.bsa = 0; p.lda = lda;
    p.B = B; p.bsb = 0; p.ldb = ldb;
    p.C = C; p.bsc = 0; p.ldc = ldc;
    p.sA = sA; p.modeA = modeA; p.sa_bs = 0; p.sa_rs = sa_rs; p.sa_ks = sa_ks;
    p.sB = sB; p.modeB = modeB; p.sb_bs = 0; p.sb_rs = sb_rs; p.sb_ks = sb_ks;
    p.batch = 1; p.M = M; p.N = N; p.K = K;
    p.acc_i32_full = acc_i32_full; p.combine = TI8_COMBINE_MUL_MUL;
    p.out_scale = 1.0f; p.post_scale = 0.0f;
    return p;
}

int check_step(const char* fn, const void* X, int64_t ldx, const void* W, int64_t ldw, const void* dY, int64_t lddy, const void* Y,
               int64_t ldy, const void* dX, int64_t lddx, const void* dW, int64_t lddw, int64_t T, int64_t tokens, int64_t K, int64_t N, int scheme) {
    if (scheme != TI8_SCHEME_BLOCK_CHANNEL && scheme != TI8_SCHEME_DOUBLE_CHANNEL)
        return fail(TI8_ERR_MODE, "%s: scheme must be TI8_SCHEME_BLOCK_CHANNEL or TI8_SCHEME_DOUBLE_CHANNEL, got %d", fn, scheme);
    if (!X || !W || !dY || !Y || !dX || !dW) return fail(TI8_ERR_NULL, "%s: X, W, dY, Y, dX and dW are required", fn);
    if (T <= 0 || K <= 0 || N <= 0 || T % 128 || K % 128 || N % 128 || T > 0x3fffffff || K > 0x3fffffff || N > 0x3fffffff)
        return fail(TI8_ERR_SHAPE, "%s: T, K and N must be positive multiples of 128 (zero-pad the tokens); got T=%lld K=%lld N=%lld", fn,
                    (long long)T, (long long)K, (long long)N);
    if (tokens < 1 || tokens > T) return fail(TI8_ERR_SHAPE, "%s: tokens must be in [1, T]; got tokens=%lld T=%lld", fn, (long long)tokens, (long long)T);
    if (ldx < K || ldw < K || lddy < N || ldy < N || lddx < K || lddw < K) return fail(TI8_ERR_SHAPE, "%s: leading dimension smaller than the row length", fn);
    // what the quantisers (inputs) and the GEMM epilogues (outputs) need, checked here so that nothing is launched before a rejection
    if (!aligned16(X) || !aligned16(W) || !aligned16(dY) || !aligned16(Y) || !aligned16(dX) || !aligned16(dW) || (ldx % 8) || (ldw % 8) ||
        (lddy % 8) || (ldy % 8) || (lddx % 8) || (lddw % 8))
        return fail(TI8_ERR_ALIGN, "%s: X, W, dY, Y, dX and dW must be 16-byte aligned with leading dimensions multiples of 8 elements", fn);
    return TI8_OK;
}

}  // namespace
}  // namespace ti8

using namespace ti8;

extern "C" int64_t ti8_linear_fwd_bwd_workspace(int64_t T, int64_t K, int64_t N, int scheme) {
    if (T <= 0 || K <= 0 || N <= 0 || T % 128 || K % 128 || N % 128) return -1;
    if (scheme == TI8_SCHEME_BLOCK_CHANNEL) return BlockChannelLayout().carve(nullptr, T, K, N);
    if (scheme == TI8_SCHEME_DOUBLE_CHANNEL) return DoubleChannelLayout().carve(nullptr, T, K, N);
    return -1;
}

// One GEMM of the step launched alone (what ti8_gemm_i8_nt selects for its shape: the few-rows kernel up to 256 rows).
// `live` rows of A are multiplied: with few tokens the padding rows of the 128-row-quantised operand are zeros whose
// products nobody reads.
static int one_gemm(const ti8_gemm_problem& p, int64_t live, int gemm_flags, ti8_stream_t stream) {
    return ti8_gemm_i8_nt(p.A, p.bsa, p.lda, p.B, p.bsb, p.ldb, p.C, p.bsc, p.ldc, p.sA, p.modeA, p.sa_bs, p.sa_rs, p.sa_ks,
                          p.sB, p.modeB, p.sb_bs, p.sb_rs, p.sb_ks, 1, live, p.N, p.K, p.acc_i32_full, p.combine, p.out_scale, p.post_scale,
                          gemm_flags, stream);
}

extern "C" int ti8_linear_fwd_bwd(const void* X, int64_t ldx, const void* W, int64_t ldw, const void* dY, int64_t lddy,
                                  void* Y, int64_t ldy, void* dX, int64_t lddx, void* dW, int64_t lddw,
                                  int64_t T, int64_t tokens, int64_t K, int64_t N, int scheme, int gemm_flags,
                                  void* workspace, int64_t workspace_bytes, ti8_stream_t stream) {
    const char* fn = "ti8_linear_fwd_bwd";
    if (int e = check_step(fn, X, ldx, W, ldw, dY, lddy, Y, ldy, dX, lddx, dW, lddw, T, tokens, K, N, scheme)) return e;
    const int64_t need = ti8_linear_fwd_bwd_workspace(T, K, N, scheme);
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) || workspace_bytes < need)
        return fail(TI8_ERR_SHAPE, "%s: the workspace must be 256-byte aligned and hold %lld bytes (ti8_linear_fwd_bwd_workspace); got %lld", fn,
                    (long long)need, (long long)(workspace ? workspace_bytes : 0));
    if (gemm_flags & ~(TI8_GEMM_TILED | TI8_GEMM_LARGE_TILES | TI8_GEMM_ONE_TILE)) return fail(TI8_ERR_MODE, "%s: only TI8_GEMM_TILED, TI8_GEMM_LARGE_TILES and TI8_GEMM_ONE_TILE apply here", fn);
    char* base = static_cast<char*>(workspace);
    const int q = TI8_Q_CLAMP;
    // rows of the token operands that Y and dX multiply: all of them, or with up to 256 (padded) tokens the real ones
    // rounded up to 32, which the few-rows kernel takes
    auto live_rows = [&](int64_t contraction) {
        if (T > 256 || (gemm_flags & (TI8_GEMM_TILED | TI8_GEMM_LARGE_TILES)) || contraction > 32768) return T;
        const int64_t r = (tokens + 31) / 32 * 32;
        return r < T ? r : T;
    };
    // the three GEMMs go into one launch where none of them has so few rows that it would take the few-rows kernel
    const bool one_launch = (T < N ? T : N) > 256;

    if (scheme == TI8_SCHEME_BLOCK_CHANNEL) {
        // triton/block_channel_fwd32.py:221-222 on (X, W) and on (dY, W^T), triton/block_channel_bwd33.py:153-154 on (dY^T, X^T):
        // X and dY per 128 x 128 block (one read each; the transposed copies are the dW GEMM's K-contiguous operands and
        // their scale grids the transposed grids), W per row and per column
        BlockChannelLayout L;
        L.carve(base, T, K, N);
        const ti8_qblock_operand ops[2] = {
            {X, 0, ldx, L.x.q, T * K, K, L.x.qT, T * K, T, L.x.s, 0, K / 128, 1, 1, T, K},
            {dY, 0, lddy, L.dy.q, T * N, N, L.dy.qT, T * N, T, L.dy.s, 0, N / 128, 1, 1, T, N}};
        // the same launch clears the words in which W's maxima are collected next
        if (int e = quant_block_multi_and_clear(ops, 2, q, TI8_INV_RCP_OF_SCALE, reinterpret_cast<unsigned int*>(L.w.maxima), N + K, stream)) return e;
        if (int e = ti8_quant_row_col_t(W, ldw, L.w.q, K, L.w.s_row, L.w.qT, N, L.w.s_col, L.w.maxima, N, K, q | TI8_Q_WS_IS_ZERO, TI8_INV_RCP_OF_SCALE, stream)) return e;
        const ti8_gemm_problem g[3] = {
            gemm2d(L.x.q, K, L.x.s, TI8_SCALE_BLOCK128, K / 128, 1, L.w.q, K, L.w.s_row, TI8_SCALE_ROW, 1, 0, Y, ldy, T, N, K, 0),
            gemm2d(L.dy.q, N, L.dy.s, TI8_SCALE_BLOCK128, N / 128, 1, L.w.qT, N, L.w.s_col, TI8_SCALE_ROW, 1, 0, dX, lddx, T, K, N, 0),
            gemm2d(L.dy.qT, T, L.dy.s, TI8_SCALE_BLOCK128, 1, N / 128, L.x.qT, T, L.x.s, TI8_SCALE_BLOCK128, 1, K / 128, dW, lddw, N, K, T, 0)};
        if (one_launch) return ti8_gemm_i8_nt_multi(g, 3, gemm_flags, stream);
        if (int e = one_gemm(g[0], live_rows(K), gemm_flags, stream)) return e;
        if (int e = one_gemm(g[1], live_rows(N), gemm_flags, stream)) return e;
        return one_gemm(g[2], N, gemm_flags, stream);
    }

    // double-channel: every operand per row and per column (triton/double-channle_fwd32.py:277-278 on (X, W) and (dY, W^T),
    // triton/double_channel_bwd33.py:193-194 on (dY^T, X^T)), int32 accumulation over the whole K
    DoubleChannelLayout L;
    L.carve(base, T, K, N);
    if (int e = fill_words(reinterpret_cast<unsigned int*>(L.maxima), L.maxima_words, 0u, static_cast<hipStream_t>(stream))) return e;
    const int qz = q | TI8_Q_WS_IS_ZERO;
    if (int e = ti8_quant_row_col_t(X, ldx, L.x.q, K, L.x.s_row, L.x.qT, T, L.x.s_col, L.x.maxima, T, K, qz, TI8_INV_AMAX_DIV_127, stream)) return e;
    if (int e = ti8_quant_row_col_t(W, ldw, L.w.q, K, L.w.s_row, L.w.qT, N, L.w.s_col, L.w.maxima, N, K, qz, TI8_INV_AMAX_DIV_127, stream)) return e;
    if (int e = ti8_quant_row_col_t(dY, lddy, L.dy.q, N, L.dy.s_row, L.dy.qT, T, L.dy.s_col, L.dy.maxima, T, N, qz, TI8_INV_AMAX_DIV_127, stream)) return e;
    const ti8_gemm_problem g[3] = {
        gemm2d(L.x.q, K, L.x.s_row, TI8_SCALE_ROW, 1, 0, L.w.q, K, L.w.s_row, TI8_SCALE_ROW, 1, 0, Y, ldy, T, N, K, 1),
        gemm2d(L.dy.q, N, L.dy.s_row, TI8_SCALE_ROW, 1, 0, L.w.qT, N, L.w.s_col, TI8_SCALE_ROW, 1, 0, dX, lddx, T, K, N, 1),
        gemm2d(L.dy.qT, T, L.dy.s_col, TI8_SCALE_ROW, 1, 0, L.x.qT, T, L.x.s_col, TI8_SCALE_ROW, 1, 0, dW, lddw, N, K, T, 1)};
    if (one_launch) return ti8_gemm_i8_nt_multi(g, 3, gemm_flags, stream);
    if (int e = one_gemm(g[0], live_rows(K), gemm_flags, stream)) return e;
    if (int e = one_gemm(g[1], live_rows(N), gemm_flags, stream)) return e;
    return one_gemm(g[2], N, gemm_flags, stream);
}
