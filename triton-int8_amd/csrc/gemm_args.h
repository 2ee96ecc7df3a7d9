// Argument block, scale descriptors and epilogue kinds shared by the INT8 GEMM kernels.
#pragma once
#include "ti8_common.h"
#include "index_math.h"

namespace ti8 {

struct ScaleDesc {
    const float* p;
    int mode;         // ti8_scale_mode
    int64_t bs, rs, ks;
};

struct GemmArgs {
    const int8_t* A;
    const int8_t* B;
    void* C;
    int64_t bsa, lda, bsb, ldb, bsc, ldc;
    ScaleDesc sa, sb;
    int M, N, K;
    int tiles_m, tiles_n;
    int combine;
    int strict;
    float out_scale, post_scale;
};

// EPI_PROMOTE: the per-K-tile factor is uniform over a wave's tile (block or per-row scales
// on both operands); EPI_PROMOTE_LANE: operand B carries one scale per (column, K tile).
// EPI_PROMOTE_CHAIN: EPI_PROMOTE without int32 accumulators that live across K tiles (see gemm.hip).
// EPI_PROMOTE_CHAIN_LANE: EPI_PROMOTE_CHAIN with operand B's factors per (column, K tile) as in EPI_PROMOTE_LANE.
enum { EPI_I32 = 0, EPI_ROWS = 1, EPI_PROMOTE = 2, EPI_STRICT = 3, EPI_PROMOTE_LANE = 4, EPI_PROMOTE_CHAIN = 5, EPI_PROMOTE_CHAIN_LANE = 6 };


// scale of operand row `row` at K block kb
__device__ __forceinline__ float scale_at(const ScaleDesc& d, int64_t batch, int row, int kb) {
    return d.p[idx::scale_index(d.mode, d.bs, d.rs, d.ks, batch, row, kb)];
}

#ifndef TI8_LOAD_AUX
#define TI8_LOAD_AUX 0   // cache policy bits of the operand loads (0: default; sc0, sc1 measured no different, nt slower)
#endif

// One wave's share of a K tile: NI global->LDS instructions of 64 x 16 bytes; instruction i
// fills the 1 KiB slab at lds + i*1024 (lane l lands at byte 16*l of the slab) from
// base + i*stride8 (wave-uniform: 8 rows further per instruction) + voff[(t0 + i) & 1] (per lane).
template <int NI>
__device__ __forceinline__ void issue_tile_loads(const int8_t* base, int64_t stride8, const uint32_t (&voff)[2], int t0,
                                                 int8_t* lds) {
#if defined(__HIP_DEVICE_COMPILE__)  // the builtin only exists in the device pass
    // the per-lane offsets are made opaque here so that their widening to 64 bits is not hoisted out
    // of the caller's loop: instruction selection then sees (uniform base) + zext(32-bit offset) and
    // uses the SGPR-base addressing form instead of a 64-bit vector add per instruction
    uint32_t vo[2] = {voff[0], voff[1]};
    asm volatile("" : "+v"(vo[0]), "+v"(vo[1]));
#pragma unroll
    for (int i = 0; i < NI; ++i)
        __builtin_amdgcn_global_load_lds(base + i * stride8 + vo[(t0 + i) & 1], lds + i * 1024, 16, 0, TI8_LOAD_AUX);   // = idx::gemm_load_offset_bytes
#else
    (void)base; (void)stride8; (void)voff; (void)t0; (void)lds;
#endif
}

// Several GEMMs in one launch: GEMM i owns the workgroups (one-tile kernels) or the tile numbers (persistent
// kernel) [first[i], first[i + 1]), first[0] = 0.
constexpr int GEMM_MULTI_MAX = 3;
struct GemmMulti {
    GemmArgs g[GEMM_MULTI_MAX];
    int first[GEMM_MULTI_MAX + 1];
    int count;
};

// Persistent-workgroup kernel for the chained block-channel promotion on 256 x 256 tiles (gemm_chain.hip).
// `m.g[i].tiles_m / tiles_n` and `m.first` must be filled for 256 x 256 tiles, batches included
// (first[i + 1] - first[i] = tiles_m * tiles_n * batch of GEMM i).  launch returns TI8_OK, an error, or
// CHAIN_UNAVAILABLE when the device refuses the 160 KiB of LDS (the caller then takes the one-tile kernel).
constexpr int CHAIN_UNAVAILABLE = -1;
bool chain_persistent_supported(const GemmMulti& m);
int launch_chain_persistent(const GemmMulti& m, int total_tiles, int num_cu, hipStream_t st);

// Kernel for few rows (gemm_skinny.hip): M a multiple of 128, operand A without per-(row, K tile)
// scales.  i32_full: int32 accumulation over the whole K with per-row scales (bit-exact path).
bool skinny_supported(const GemmArgs& a);
int launch_skinny(const GemmArgs& a, int64_t batch, bool i32_full, hipStream_t st);

}  // namespace ti8
