// Parameters shared by the two backward kernels of the fused selective scan.
#pragma once

#include "common.h"

namespace mpa {

struct BwdParams {
    const void* x;
    const void* delta;
    const void* Bm;
    const void* C;
    const void* z;
    const void* dy;
    const void* ypre;  // output before the gate saved by the forward (strides of dy); fast path with z
    const float* A;
    const float* D;
    const float* dbias;
    const float* h0;
    const float* ckpt;
    void* dx;
    void* ddelta;
    void* dz;
    float* partB;   // [CG] groups of [batch][L][N], part_gs floats apart
    float* partC;   // same layout
    int64_t part_gs;  // distance between the partials of two channel groups (see bwd_workspace)
    float* partA;   // [rows][ED][N]   rows = batch * nseg
    float* partD;   // [rows][ED]
    float* partDb;  // [rows][ED]  (ddelta_bias)
    // sequence cut into nseg segments of seg_tiles tiles, counted from the END of the forward
    // walk (the order in which the backward visits them); ag0 [rows][ED][N] = a*g flowing into
    // every segment from the one visited before it (NULL = zeros: not cut)
    const float* ag0;
    int nseg, seg_tiles;
    int expire_waits;  // test hook: treat every bounded wait as run out
    int reverse;       // the forward walk ran from the last physical step to the first
    int batch, L, ED, N, nchunks;
    // d_state above 64 runs as several passes over blocks of 64 states (general kernel only):
    // N = states of this pass, Nst = states of the whole call = row stride of every array indexed
    // by state (A, h0, checkpoints, partA/B/C; their pointers are advanced to the block's first
    // state by the host); a pass after the first adds its share to dx, ddelta, dz instead of
    // overwriting them and contributes nothing to dD; row0 = its first row in partD / partDb
    int Nst, accumulate, row0;
    int softplus;
    int delta_f32;  // delta and ddelta are float32 whatever the I/O type (MPA_DELTA_F32)
    int in_tmajor, dy_tmajor, out_tmajor;
    int64_t u_sb, u_sl, u_sd;
    int64_t z_sb, z_sl, z_sd;
    int64_t d_sb, d_sl, d_sd;
    int64_t y_sb, y_sl, y_sd;
    int64_t g_sb, g_sl, g_sd;
    int64_t bc_sb, bc_sl;
};

// Fast path (no gate): scan and service waves, see sscan_bwd_fast.hip.  Returns
// MPA_ERR_BAD_SHAPE when the shape is outside what it was instantiated for.
int launch_bwd_fast(const BwdParams& p, int ns, int nw, int io_dtype, hipStream_t stream);
bool bwd_fast_supported(int ns, int nw);

}  // namespace mpa
