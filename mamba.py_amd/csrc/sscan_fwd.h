// Parameters and launchers of the forward kernel of the fused selective scan, shared with the
// backward entry point (which runs the same kernel in a carry mode when it cuts the sequence).
#pragma once

#include "common.h"

namespace mpa {

struct FwdParams {
    const void* x;
    const void* delta;
    const void* z;
    const float* A;
    const float* D;
    const float* dbias;
    const float* h0;
    const float* bcpack;  // packed B/C, see pack_bc_kernel (only at 16 or more states per lane)
    const void* Bm;
    const void* C;
    int64_t bc_sb, bc_sl;
    void* y;
    void* ypre;  // output before the gate (only with z), strides of y
    float* ckpt;
    float* hlast;
    float* dsum;     // segmented mode, first pass: sums of delta per (row, step group, channel)
    int nseg;        // > 1: every batch row is cut into nseg segments of seg_tiles tiles, one
    int seg_tiles;   // workgroup row (blockIdx.y) per (batch row, segment)
    int batch, L, ED, N, nchunks;
    // A wide d_state runs as passes over blocks of states: N = states of this launch, and the
    // arrays indexed by state keep the row stride of the whole call, with their pointers advanced
    // to the block's first state by the host: a_st = states per row of A, h_st = of h0 / hlast,
    // ck_st = states per checkpoint.  A pass after the first gets D = NULL (no D*x term) and adds
    // what `yacc` holds (strides of y) to its output before the gate.
    int a_st, h_st, ck_st;
    const void* yacc;
    int group48;     // workgroups of 48 channels (six scan waves) instead of 64, see sscan_fwd.hip
    int softplus;
    int delta_f32;   // delta is float32 whatever the I/O type (MPA_DELTA_F32)
    int reverse;     // the walk runs from the last physical step to the first
    int in_tmajor;   // x / delta have unit stride along time
    int out_tmajor;  // y has unit stride along time
    int64_t u_sb, u_sl, u_sd;
    int64_t z_sb, z_sl, z_sd;
    int64_t d_sb, d_sl, d_sd;
    int64_t y_sb, y_sl, y_sd;
};

// What one launch of the kernel computes.
//   kScan    the selective scan: states, readout y, optional checkpoints and last state.
//   kCarry   states only (no readout, no reducer waves): the end state of every segment from a
//            zero state, and its sum of delta, for seg_carry_kernel.
//   kGCarry  the carry of the BACKWARD recurrence, g[t] = dy[t]*C[t] + a[t+1]*g[t+1], in the
//            form ag[t] = a[t]*(ag[t+1] + C[t]*dy[t]): the same kernel walking the other way
//            with dy (times silu(z) when gated) in place of delta*x, C in place of B and the
//            decay applied after the addition.
enum FwdMode { kScan = 0, kCarry = 1, kGCarry = 2 };

// A sequence cut into nseg segments of seg_tiles tiles (the last one may be shorter), and where
// the per-segment buffers sit in the workspace (offsets in floats): end states from zero
// [rows][dim][dstate], true initial states (same shape), sums of delta [rows][4][dim];
// rows = batch * nseg.  nseg = 1: not cut, no buffers.
struct SegPlan {
    int nseg, seg_tiles;
    size_t off_hend, off_h0, off_dsum, floats;
};
SegPlan seg_plan(const mpa_sscan_shape* s, int ns, int thin);
// Channels per workgroup of a launch that is not cut: 48 where the kernels have that form (two states
// per lane, d_state up to 16) and batch * ceil(dim / 48) workgroups still run in one round on the
// chip's 256 CUs, else 64.  The plan flags pin either.
int group_channels(const mpa_sscan_shape* s, int ns, int nseg);

// Launch sscan_fwd_kernel in `mode` (FwdMode) for the (ns, nw) decomposition; the carry modes
// exist for ns <= 8.
int launch_fwd_any(const FwdParams& p, int io_dtype, int ns, int nw, int mode, hipStream_t stream);
// segh0[row] = state at the start of every segment, from the end states and delta sums of the
// first pass; hlast (optional) = state after the last segment.
// (A has rows of a_st states, the caller's h0 / hlast rows of h_st states; the segment buffers are dense)
int launch_seg_carry(const float* A, const float* h0, const float* hend, const float* dsum, float* segh0,
                     float* hlast, int batch, int nseg, int ED, int N, int a_st, int h_st, hipStream_t st);

}  // namespace mpa
