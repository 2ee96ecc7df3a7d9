/* ti8.h -- C ABI of libti8.so: gfx950 (MI355X) kernels for the INT8 quantized linear
 * layer of jiaoch/Triton-INT8 (quantize -> int8 GEMM on i8 MFMA -> dequant, fwd + bwd).
 *
 * Conventions
 *   - Every pointer is a BORROWED DEVICE pointer (hipMalloc'd / torch CUDA storage);
 *     the library allocates nothing and keeps nothing after a call returns.
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = null
 *     stream) of the CURRENT device; calls return after enqueueing.
 *   - Strides and leading dimensions are in ELEMENTS of the tensor they describe.
 *   - Every function returns TI8_OK (0) or an error code and never throws; the
 *     message of the last failure on the calling thread is ti8_last_error().
 *     Arguments are validated on the host before anything is launched.
 *   - bf16 tensors are passed as void* / uint16_t bit patterns.
 *
 *   - Non-finite inputs of the quantisers, one rule for all of them: a NaN element is left out of
 *     its group's absmax (as v_max_f32 and the reference's tl.max leave it out; a group of nothing
 *     but NaN has absmax 0) and converts to -128; an infinite element is its group's absmax like any
 *     other number, so the group's multiplier is 0, its finite elements convert to 0, the infinity
 *     to -128 (inf * 0 = NaN) and the stored scale is infinite.  Nothing is rejected or reported.
 *
 * The reference has no FFI: its boundary is a set of Python functions, each a host
 * wrapper around one Triton kernel.  Each entry point below names the reference
 * wrapper + kernel it replaces (paths relative to the reference checkout).
 */
#ifndef TI8_H
#define TI8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ti8_stream_t;

enum ti8_status {
    TI8_OK = 0,
    TI8_ERR_NULL = 1,        /* a required pointer is NULL */
    TI8_ERR_SHAPE = 2,       /* a size is not positive or not a multiple of what the kernel needs */
    TI8_ERR_ALIGN = 3,       /* a pointer / leading dimension breaks the 16-byte access contract */
    TI8_ERR_MODE = 4,        /* unknown or unsupported flag / mode combination */
    TI8_ERR_HIP = 5          /* the HIP runtime reported an error at launch */
};

/* quantiser flags (bit set) */
enum ti8_qflags {
    TI8_Q_CLAMP = 1,        /* clamp floor(x*scale+0.5) to [-128,127] before the int8 cast.  The conversion
                               saturates with or without this flag: the unclamped reference kernels give
                               the same bytes on every finite input, |x*scale| <= 127 by construction */
    TI8_Q_EPS_ADD = 2,      /* amax + 1e-5 (fused kernels) instead of max(amax, 1e-4) */
    TI8_Q_SCALE_BF16 = 4,   /* round the stored scale through bf16 (TileLang copy) */
    TI8_Q_HAD128 = 8,       /* ti8_quant_row only: rotate every 128-column group by H_128 (fp32
                               butterflies, one bf16 rounding) before the absmax */
    TI8_Q_WS_PINGPONG = 16, /* ti8_quant_row_col_t only: two-part workspace that the calls keep clear for each */
    TI8_Q_WS_SECOND = 32,   /* other, and which part this call works in (see there) */
    TI8_Q_WS_IS_ZERO = 256, /* ti8_quant_row_col_t only: the caller guarantees that the R + C words of ws are all zero on
                               entry (it cleared them beside earlier work), so the call needs no clearing launch */
    TI8_Q_TORCH_ROUND = 64, /* ti8_quant_block (128 x 128 groups, q only) and ti8_quant_row (group = 0): the arithmetic of the
                               reference's pure-torch quantisers instead of its Triton kernels' -- scale =
                               reciprocal(max(amax, 1e-4)) * 127, q = clamp(round_half_even(x * scale), -127, 127), stored
                               scale = reciprocal(scale) (per_block_cast_to_int8 of tilelang/block_channel_bwd.py:96-104) */
    TI8_Q_TORCH_BF16 = 128  /* the same with every intermediate rounded to bf16, the product x * scale included: what torch
                               computes when the input is bf16 and nothing widens it (per_token_cast_to_int8 /
                               per_block_cast_to_int8 of tilelang/block_channel_fwd.py:215-230) */
};

/* which number is written to the scale tensor */
enum ti8_inv_mode {
    TI8_INV_RCP_OF_SCALE = 0,     /* 1.0f / (127.0f / amax)   block + per-token kernels */
    TI8_INV_AMAX_DIV_127 = 1,     /* amax / 127.0f            two-pass per-row quantiser */
    TI8_INV_AMAX_MUL_RCP127 = 2,  /* amax * (1.0f / 127.0f)   torch-GPU evaluation of the same */
    TI8_INV_MULTIPLIER = 3        /* 127.0f / amax            fused kernels keep the multiplier */
};

/* scale descriptor of a GEMM operand (rows = M for A, N for B; kb = K block of 128) */
enum ti8_scale_mode {
    TI8_SCALE_ROW = 0,       /* s[batch*bs + row*rs]                          */
    TI8_SCALE_BLOCK128 = 1,  /* s[batch*bs + (row/128)*rs + kb*ks]            */
    TI8_SCALE_ROW_K128 = 2,  /* s[batch*bs + row*rs + kb*ks]                  */
    TI8_SCALE_BLOCK_K256 = 3 /* s[batch*bs + (row/128)*rs + (kb/2)*ks]        */
};

/* how one K block's exact integer dot d enters the fp32 accumulator */
enum ti8_combine {
    TI8_COMBINE_MUL_MUL = 0,   /* acc += (f32(d) * sa) * sb      Triton block-channel kernels */
    TI8_COMBINE_MUL_PROD = 1,  /* acc += f32(d) * (sa * sb)      TileLang kernels            */
    TI8_COMBINE_DIV_PROD = 2   /* acc += f32(d) / (sa * sb)      fused kernels (s = multipliers) */
};

enum ti8_gemm_flags {
    TI8_GEMM_STRICT = 1,  /* evaluate the combine formula literally (separate roundings, true
                             division); without it the kernel may use fma / reciprocal, which
                             moves results by a few fp32 ulps before the bf16 rounding */
    TI8_GEMM_TILED = 2,   /* always take an LDS-tiled kernel (tile size still chosen by the shape) */
    TI8_GEMM_LARGE_TILES = 8, /* LDS-tiled kernel with the largest tiles (256 x 256) whatever the shape */
    TI8_GEMM_ONE_TILE = 16,   /* one workgroup per output tile also where the block-channel promotion would run on
                                 persistent workgroups (one per CU walking its tiles); same bits either way */
    TI8_GEMM_SKINNY = 4   /* take the few-rows kernel (no LDS staging, K split over waves) whenever
                             it supports the scale modes; by default it is used for M <= 256.  Both
                             kernels give bit-identical results with acc_i32_full; otherwise their
                             fp32 sums associate differently (few ulps before the bf16 rounding) */
};

/* Library version (major*10000 + minor*100 + patch). */
int ti8_version(void);
/* Message of the last error on this thread ("" if none). */
const char* ti8_last_error(void);
/* Name of the GPU architecture the kernels were compiled for ("gfx950"). */
const char* ti8_arch(void);

/* One-time set-up on the CURRENT device, for callers that want none of it inside their first (timed or
 * captured) call: raises the dynamic-LDS limit of every kernel that needs more than 64 KiB, looks up the
 * device's compute-unit count and the address of the library's fixed scratch array.  Optional -- every entry
 * point does its own part of this on first use -- and idempotent; call it once per device.  It plays the part
 * of the warm-up call in which the reference's Triton kernels are compiled and autotuned
 * (triton/block_channel_fwd32.py:12-21).  A device that refuses the persistent GEMM kernel's 160 KiB of LDS
 * is not an error: ti8_last_error() then says so and the one-workgroup-per-tile kernel serves its shapes. */
int ti8_init(void);

/* Which GEMM kernel the last ti8_gemm_i8_nt / _multi / _i32 / ti8_linear_fwd_bwd call of THIS thread launched
 * (the last one when a call launches several): kind | epilogue << 8 | (tile rows / 64) << 16 | (tile columns / 64) << 20.
 * The kernels of one family give bit-identical results whichever of them runs, so a caller (or a test) that
 * cares about WHICH one ran -- the persistent kernel is the fast one -- asks here. */
enum ti8_gemm_kernel {
    TI8_KERNEL_NONE = 0,
    TI8_KERNEL_ONE_TILE = 1,          /* one workgroup per output tile */
    TI8_KERNEL_ONE_TILE_MULTI = 2,    /* the same, several GEMMs in one launch */
    TI8_KERNEL_PERSISTENT_CHAIN = 3,  /* persistent workgroups, chained block-channel promotion (256 x 256 tiles) */
    TI8_KERNEL_FEW_ROWS = 4           /* M <= 256: 32 x 32 blocks, K split over the waves */
};
#define TI8_KERNEL_KIND(id) ((id) & 0xff)
int ti8_last_gemm_kernel(void);

/* ---------------------------------------------------------------------------------
 * Per-block absmax quantiser: replaces triton_per_block_quant + per_block_quant_kernel
 * (triton/block_channel_fwd32.py:160-212 clamped; triton/block_channel_bwd33.py:87-138
 * unclamped; tilelang/block_channel_fwd.py:152-203 with group_c = 256 and bf16 scales).
 *
 *   x   bf16 [B][R][C], rows contiguous, leading dim ldx, batch stride bsx
 *   q   int8 [B][R][C] (ldq, bsq)   same orientation as x            -- may be NULL
 *   qT  int8 [B][C][R] (ldqt, bsqt) the transposed copy of q          -- may be NULL
 *   s   fp32, scale of tile (b, rb, cb) at s[b*ssb + rb*ssr + cb*ssc]
 * Tiles are 128 x group_c (group_c = 128 or 256; qT needs 128).  A 128x128 block
 * quantisation commutes with transposition, so a transposed VIEW is quantised by
 * passing its underlying row-major memory and swapping (q, qT) and (ssr, ssc).
 * At least one of q / qT must be given.  R % 128 == 0, C % group_c == 0. */
int ti8_quant_block(const void* x, int64_t bsx, int64_t ldx,
                    int8_t* q, int64_t bsq, int64_t ldq,
                    int8_t* qT, int64_t bsqt, int64_t ldqt,
                    float* s, int64_t ssb, int64_t ssr, int64_t ssc,
                    int64_t B, int64_t R, int64_t C, int group_c,
                    int qflags, int inv_mode, ti8_stream_t stream);

/* The same for up to 4 operands in ONE launch (128 x 128 tiles, every operand with the same set of
 * outputs: q, qT or both): a training step quantises X and dY the same way (triton/block_channel_fwd32.py:221
 * for X, the same call on dY for dX = fwd_32(dY, W^T)), and one launch instead of two saves a kernel
 * boundary.  Each operand's fields mean what the arguments of ti8_quant_block mean; `operands` is a
 * HOST array.  Bit-identical to separate ti8_quant_block calls. */
typedef struct ti8_qblock_operand {
    const void* x; int64_t bsx, ldx;
    int8_t* q; int64_t bsq, ldq;
    int8_t* qT; int64_t bsqt, ldqt;
    float* s; int64_t ssb, ssr, ssc;
    int64_t B, R, C;
} ti8_qblock_operand;
int ti8_quant_block_multi(const ti8_qblock_operand* operands, int count,
                          int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Block quantiser with the block-diagonal 128-point Walsh-Hadamard rotation fused in: what
 * BASELINE config 4 calls the "fused Hadamard + quantize path".  The reference has no such
 * kernel (its Hadamard is the external full-length transform called before the quantiser,
 * triton/double-channle_fwd32.py:299-300); the arithmetic is x' = bf16(FWHT_128(f32(x))) per
 * group of 128 (butterfly strides 1,2,...,64) followed by per_block_quant_kernel
 * (triton/block_channel_fwd32.py:160-192) on x'.
 *   along_rows = 0: groups run along the columns of x, q int8 [B][R][C] (ldq, bsq)
 *   along_rows = 1: groups run along the rows of x,    q int8 [B][C][R] (TRANSPOSED output:
 *                   the K-contiguous operand of a GEMM that contracts over the rows)
 *   s: scale of tile (b, rb, cb) of x at s[b*ssb + rb*ssr + cb*ssc].   R, C multiples of 128. */
int ti8_quant_block_had128(const void* x, int64_t bsx, int64_t ldx,
                           int8_t* q, int64_t bsq, int64_t ldq,
                           float* s, int64_t ssb, int64_t ssr, int64_t ssc,
                           int64_t B, int64_t R, int64_t C, int along_rows,
                           int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Per-row absmax quantiser in ONE pass over x: replaces triton_per_token_quant +
 * per_token_quant_kernel (triton/block_channel_fwd32.py:101-157) and the two-pass
 * triton_per_row_quant_2d/3d + _pass1/_pass2 kernels with their torch glue
 * (triton/double-channle_fwd32.py:93-266, triton/double_channel_bwd33.py:90-176).
 *
 *   x bf16 [rows][cols] (ldx) -> q int8 [rows][cols] (ldq)
 *   group = 0:   one scale per row,                 s[rows]
 *   group = 128: one scale per (row, 128 columns),  s[rows][cols/128]   (B operand of
 *                the fused kernel, triton/fused_triton_fwd32.py:57-59)
 * cols % 128 == 0, cols <= 32768. */
int ti8_quant_row(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s,
                  int64_t rows, int64_t cols, int group,
                  int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Per-COLUMN absmax quantiser with transposed output = the per-row quantiser applied
 * to x^T without materialising x^T in bf16.  Serves the reference's calls on
 * transposed operands (fwd_32(dY, W^T): triton/block_channel_fwd32.py:221-222 with
 * b = W^T; bwd_33(dY^T, X^T) of the double-channel scheme).
 *
 *   x bf16 [R][C] (ldx) -> qT int8 [C][R] (ldqt), s[C]
 *   ws: workspace of C floats (column absmax), contents undefined afterwards.
 * R % 128 == 0, C % 128 == 0.
 * With TI8_Q_HAD128 every 128-row segment of every column is rotated by H_128 first (x^T rotated
 * along its contraction dim, the rule of ti8_quant_row's flag applied to x^T): the
 * hadamard = 128 mode of dX = dY W, whose second operand is W^T per row. */
int ti8_quant_col_t(const void* x, int64_t ldx, int8_t* qT, int64_t ldqt, float* s, float* ws,
                    int64_t R, int64_t C, int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Both of the above on one operand with one launch sequence: the per-row quantisation
 * (as ti8_quant_row, group = 0) AND the per-column quantisation with transposed output
 * (as ti8_quant_col_t), bit-identical to the two separate calls.  A training step needs
 * both for W (triton/block_channel_fwd32.py:221-222 called with b = W for Y and with
 * b = W^T for dX) and, in the double-channel scheme, for X and dY as well
 * (triton/double-channle_fwd32.py:277-278 on X, W and on the transposed operands of
 * triton/double_channel_bwd33.py:193-194); x is read twice instead of three times.
 *
 *   x bf16 [R][C] (ldx) -> q int8 [R][C] (ldq), s_row[R];  qT int8 [C][R] (ldqt), s_col[C]
 *   ws: workspace of R + C floats, contents undefined afterwards.
 *   With TI8_Q_WS_PINGPONG ws has two parts of R + C floats each and the call works in the first,
 *   or with TI8_Q_WS_SECOND in the second: that part must be ALL ZERO on entry, and the call
 *   zero-fills the other part.  Zero-fill the buffer once after allocating it and alternate
 *   TI8_Q_WS_SECOND from call to call (same R and C, calls in stream order, not overlapping):
 *   then no call needs the launch that clears the workspace.
 * R % 128 == 0, C % 128 == 0. */
int ti8_quant_row_col_t(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s_row,
                        int8_t* qT, int64_t ldqt, float* s_col, float* ws,
                        int64_t R, int64_t C, int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * ti8_quant_row_col_t for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without `ws`,
 * same bits.  It has no counterpart in the reference.  The row and column maxima are collected in
 * a fixed array of TI8_NOALLOC_MAX_ROWS_PLUS_COLS floats (256 KiB) that lives in the library's
 * device image: every GPU the library runs on holds its own copy until the process ends.  The call
 * allocates and frees nothing; its launches are kernels only (the array is cleared by a fill
 * kernel), so it may be captured.
 *   R + C <= TI8_NOALLOC_MAX_ROWS_PLUS_COLS, else TI8_ERR_SHAPE (use the entry point above).
 *   TI8_Q_WS_PINGPONG / TI8_Q_WS_SECOND are rejected (TI8_ERR_MODE).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * without ordering between them) race; calls on one stream, or ordered by events, are safe. */
#define TI8_NOALLOC_MAX_ROWS_PLUS_COLS 65536
int ti8_quant_row_col_t_noalloc(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s_row,
                                int8_t* qT, int64_t ldqt, float* s_col,
                                int64_t R, int64_t C, int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Un-normalised Walsh-Hadamard transform along the last dim (Sylvester order):
 * replaces fast_hadamard_transform.hadamard_transform at its call sites
 * (triton/double-channle_fwd32.py:273-274,299-300; triton/double_channel_bwd33.py:
 * 189-190,208-209).  bf16 in, fp32 butterflies (strides 1,2,4,...), times `scale`,
 * one rounding to bf16 out.  Transforms contiguous groups of n along each row:
 * n = cols is the reference's full-length rotation, n = 128 the block-diagonal one.
 * n a power of two, 128 <= n <= 32768, cols % n == 0.  x == y is allowed.
 * A row whose length is no power of two (n / 2 < cols < n, cols % 16 == 0, n the next power of two) is transformed as
 * the external library transforms it: zero-extended to n, multiplied by H_n, cut back to its first cols elements. */
int ti8_fwht(const void* x, int64_t ldx, void* y, int64_t ldy,
             int64_t rows, int64_t cols, int64_t n, float scale, ti8_stream_t stream);

/* The same transform of x^T along its rows, without materialising x^T: x bf16 [R][C] (ldx) ->
 * y bf16 [C][R] (ldy), y[c][:] = FWHT_R(x[:, c]) * scale, bit-identical to ti8_fwht on the
 * transposed copy.  Serves the transposed operands of the backward GEMMs (dX = fwd_32(dY, W^T),
 * dW = bwd_33(dY^T, X^T)) when the scheme rotates along the full contraction dim
 * (triton/double-channle_fwd32.py:299-300 applied to W^T, dY^T, X^T).
 * R a power of two, 128 <= R <= 32768; C % 8 == 0; not in place. */
int ti8_fwht_t(const void* x, int64_t ldx, void* y, int64_t ldy,
               int64_t R, int64_t C, float scale, ti8_stream_t stream);

/* The full-length rotation and the per-row quantiser behind it in one pass: replaces the pair
 *   a = hadamard_transform(a); a_q, a_s = triton_per_row_quant_2d/3d(a)
 * of triton/double-channle_fwd32.py:273-278 and triton/double_channel_bwd33.py:189-194 (there a bf16 tensor written
 * by one kernel and read back by two more).  Same arithmetic on the same bf16-rounded rotated values, so q and s are
 * bit-identical to ti8_fwht(scale = 1) followed by ti8_quant_row; the rotated row stays in the workgroup's LDS and
 * registers, i.e. 3 bytes of HBM traffic per element instead of 7.
 *   x bf16 [rows][cols] (ldx) -> q int8 [rows][cols] (ldq), s fp32 [rows]
 *   n = the transform length: cols itself (a power of two, 128 <= n <= 32768), or the next power of two above a
 *   row that is none (n / 2 < cols < n, zero-extended as in ti8_fwht); cols % 16 == 0.
 *   qflags: TI8_Q_CLAMP, TI8_Q_EPS_ADD; inv_mode as in ti8_quant_row (the reference's pipelines use
 *   TI8_INV_AMAX_DIV_127). */
int ti8_fwht_quant_row(const void* x, int64_t ldx, int8_t* q, int64_t ldq, float* s,
                       int64_t rows, int64_t cols, int64_t n, int qflags, int inv_mode, ti8_stream_t stream);

/* The same for a transposed operand: q, s = ti8_quant_row(ti8_fwht_t(x)), bit for bit, i.e. the rotation along the ROWS of
 * x [R][C] and the per-row quantiser of the rotated x^T -- what dX = fwd_32(dY, W^T) and dW = bwd_33(dY^T, X^T) need of
 * W, dY and X when the scheme rotates along the contraction dim (triton/double-channle_fwd32.py:299-304 applied to the
 * transposed operands).  Two launches: a tiled bf16 transposition into `scratch` (16-byte accesses both ways), then
 * ti8_fwht_quant_row on it: 7 bytes of HBM traffic per element against 4 (2-to-16-byte strided reads) + 3 for the pair.
 *   x bf16 [R][C] (ldx) -> q int8 [C][R] (ldq), s fp32 [C];  scratch: C * R bf16 elements, 16-byte aligned, contents
 *   undefined afterwards.  R a power of two in [128, 32768] or a multiple of 64 that is zero-extended (n / 2 < R < n);
 *   C % 64 == 0.  qflags, inv_mode as in ti8_fwht_quant_row. */
int ti8_fwht_t_quant_row(const void* x, int64_t ldx, void* scratch, int8_t* q, int64_t ldq, float* s,
                         int64_t R, int64_t C, int qflags, int inv_mode, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * INT8 NT GEMM with fused dequantising epilogue, C[b] = dequant(A[b] * B[b]^T):
 * replaces triton_gemm + int8_gemm_kernel of every scheme
 *   block-channel 3Dx2D  triton/block_channel_fwd32.py:12-96   (A BLOCK128, B ROW)
 *   block-channel 3Dx3D  triton/block_channel_bwd33.py:8-84    (A BLOCK128, B BLOCK128)
 *   double-channel       triton/double-channle_fwd32.py:11-90, double_channel_bwd33.py:11-87
 *   TileLang mains       tilelang/block_channel_fwd.py:46-86, block_channel_bwd.py:47-86
 * and the GEMM half of the fused kernels (triton/fused_triton_fwd32.py:42-65).
 *
 *   A int8 [batch][M][K] (lda, bsa), B int8 [batch][N][K] (ldb, bsb; bsb = 0 shares
 *   one B), C bf16 [batch][M][N] (ldc, bsc).  Both operands contiguous along K.
 *   acc_i32_full = 1: int32 accumulation over the whole K, both scales TI8_SCALE_ROW,
 *       C = bf16((f32(acc) * sA[m]) * sB[n]); if post_scale != 0 a second rounding
 *       C = bf16(f32(C) * post_scale) follows (the reference's `C * inv_K`).
 *   acc_i32_full = 0: per 128-deep K block, exact int32 dot d, then `combine`;
 *       C = bf16(acc * out_scale) (out_scale = 1 for none).
 * N, K multiples of 128.  M a multiple of 128, or any multiple of 32 up to 256 (decode
 * shapes: only the first M rows of a quantised, zero-padded operand are multiplied; block
 * scales are indexed by row / 128 as usual).  Those M are served by the few-rows kernel
 * only, i.e. not with TI8_GEMM_STRICT / TI8_GEMM_TILED, TI8_SCALE_ROW_K128 or K > 32768. */
int ti8_gemm_i8_nt(const int8_t* A, int64_t bsa, int64_t lda,
                   const int8_t* B, int64_t bsb, int64_t ldb,
                   void* C, int64_t bsc, int64_t ldc,
                   const float* sA, int modeA, int64_t sa_bs, int64_t sa_rs, int64_t sa_ks,
                   const float* sB, int modeB, int64_t sb_bs, int64_t sb_rs, int64_t sb_ks,
                   int64_t batch, int64_t M, int64_t N, int64_t K,
                   int acc_i32_full, int combine, float out_scale, float post_scale,
                   int gemm_flags, ti8_stream_t stream);

/* Up to 3 such GEMMs, each with batch = 1 and M % 128 == 0, in ONE launch: the three GEMMs of a
 * training step (Y = fwd_32(X, W), dX = fwd_32(dY, W^T), dW = bwd_33(dY^T, X^T); the reference
 * launches int8_gemm_kernel once for each, triton/block_channel_fwd32.py:83,
 * triton/block_channel_bwd33.py:72) when all their operands are at hand.  Every field means what the
 * argument of that name means in ti8_gemm_i8_nt; `problems` is a HOST array, read before the call
 * returns.  Each GEMM runs the kernel that ti8_gemm_i8_nt with TI8_GEMM_TILED selects for its shape
 * and scale modes, so results are bit-identical to such separate calls; one launch serves them when
 * they all select the same kernel (not TI8_GEMM_STRICT, not TI8_SCALE_ROW_K128), otherwise they are
 * launched one after the other.  TI8_GEMM_SKINNY is refused. */
typedef struct ti8_gemm_problem {
    const int8_t* A; int64_t bsa, lda;
    const int8_t* B; int64_t bsb, ldb;
    void* C; int64_t bsc, ldc;
    const float* sA; int modeA; int64_t sa_bs, sa_rs, sa_ks;
    const float* sB; int modeB; int64_t sb_bs, sb_rs, sb_ks;
    int64_t batch, M, N, K;
    int acc_i32_full, combine;
    float out_scale, post_scale;
} ti8_gemm_problem;
int ti8_gemm_i8_nt_multi(const ti8_gemm_problem* problems, int count, int gemm_flags, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * One whole training step of the layer in ONE call: Y = X W^T, dX = dY W, dW = dY^T X with every operand
 * quantised on the way, i.e. the launches of
 *   Y  = fwd_32(X, W)        int8_gemm_pipeline of triton/block_channel_fwd32.py:216-241  /  triton/double-channle_fwd32.py:269-285
 *   dX = fwd_32(dY, W^T)     the same pipeline on the transposed weight
 *   dW = bwd_33(dY^T, X^T)   int8_gemm_pipeline of triton/block_channel_bwd33.py:148-172  /  triton/double_channel_bwd33.py:186-201
 * enqueued back to back from C (the reference pays one Python-side wrapper per quantiser and per GEMM, each with
 * its own allocations).  Same kernels on the same operands as the separate entry points, so the same bits:
 *   TI8_SCHEME_BLOCK_CHANNEL   ti8_quant_block_multi(X, dY; q and qT) -> ti8_quant_row_col_t(W) ->
 *                              ti8_gemm_i8_nt_multi(Y, dX, dW)          (3 launches + W's absmax pass)
 *   TI8_SCHEME_DOUBLE_CHANNEL  ti8_quant_row_col_t on X, W, dY (TI8_INV_AMAX_DIV_127) ->
 *                              ti8_gemm_i8_nt_multi(Y, dX, dW; acc_i32_full = 1)
 *   X bf16 [T][K] (ldx), W bf16 [N][K] (ldw), dY bf16 [T][N] (lddy)  ->  Y bf16 [T][N], dX bf16 [T][K], dW bf16 [N][K]
 *   All six 16-byte aligned, leading dimensions multiples of 8 elements; every argument is checked before the first launch.
 *   T, K, N multiples of 128.  `tokens` (1 <= tokens <= T) = the rows of X and dY that hold data when the caller has
 *   zero-padded them to T rows (padded rows change no absmax and add nothing to dW; pass tokens = T otherwise).  With
 *   T <= 256 or N <= 256 the GEMMs are launched one by one, as ti8_gemm_i8_nt would launch them (few-rows kernel up to 256
 *   rows), and Y and dX are computed for the first ceil(tokens / 32) * 32 rows only.
 *   workspace: ti8_linear_fwd_bwd_workspace(T, K, N, scheme) bytes of device memory, 256-byte aligned, contents
 *   undefined before and after (it holds the int8 operands, their transposes, scales and maxima; the call clears
 *   what it needs cleared itself, so the same buffer serves any sequence of calls in stream order).
 *   gemm_flags: TI8_GEMM_TILED / TI8_GEMM_LARGE_TILES / TI8_GEMM_ONE_TILE or 0.
 * Nothing is allocated; the call only enqueues kernels, so it may be captured into a graph. */
enum ti8_scheme {
    TI8_SCHEME_BLOCK_CHANNEL = 0,
    TI8_SCHEME_DOUBLE_CHANNEL = 2
};
/* bytes of workspace the call below needs, or -1 for sizes / a scheme it does not take */
int64_t ti8_linear_fwd_bwd_workspace(int64_t T, int64_t K, int64_t N, int scheme);
int ti8_linear_fwd_bwd(const void* X, int64_t ldx, const void* W, int64_t ldw, const void* dY, int64_t lddy,
                       void* Y, int64_t ldy, void* dX, int64_t lddx, void* dW, int64_t lddw,
                       int64_t T, int64_t tokens, int64_t K, int64_t N, int scheme, int gemm_flags,
                       void* workspace, int64_t workspace_bytes, ti8_stream_t stream);

/* Raw int32 accumulators of the same GEMM over the whole K, C int32 [batch][M][N]:
 * the accumulator of int8_gemm_kernel in triton/double-channle_fwd32.py:44,56.
 * Exists so that tests can compare accumulators bit for bit. */
int ti8_gemm_i8_nt_i32(const int8_t* A, int64_t bsa, int64_t lda,
                       const int8_t* B, int64_t bsb, int64_t ldb,
                       int32_t* C, int64_t bsc, int64_t ldc,
                       int64_t batch, int64_t M, int64_t N, int64_t K, ti8_stream_t stream);

/* ---------------------------------------------------------------------------------
 * Measurement aid (no counterpart in the reference; used by bench.py --probe mfma): a loop of nothing
 * but v_mfma_i32_32x32x32_i8 on `workgroups` workgroups of 8 waves, `iters` x 16 MFMAs per wave,
 * operands all zero or pseudo-random, optionally with the block-channel promotion's vector work
 * (convert + fma per accumulator element per four MFMAs).  Operations = workgroups * 8 * iters * 16 *
 * 65536; time it with events around the call.
 *   sink   float [workgroups * 512]   scratch output that keeps the loop alive
 *   clocks int64 [2]                  [0] shader-clock cycles, [1] ticks of the constant 100 MHz
 *                                     counter, both across the loop of workgroup 0: [0] / [1] * 100 = MHz */
int ti8_probe_mfma(float* sink, int64_t sink_elems, int64_t* clocks, int workgroups, int iters,
                   int random_operands, int with_promotion, ti8_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TI8_H */
