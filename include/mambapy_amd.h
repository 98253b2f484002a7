/* C ABI of libmambapy_amd.so: hand-written gfx950 (MI355X) kernels for the selective-scan
 * hot path of alxndrTL/mamba.py.
 *
 * The reference has no FFI for this path: its operator boundary is a set of Python
 * symbols (cited per entry point below).  Each entry point here is what a ctypes binding
 * placed behind that symbol calls.  Conventions:
 *   - every pointer is a DEVICE pointer unless stated otherwise; the library allocates
 *     and frees nothing, outputs and workspaces are caller-allocated;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all work is
 *     enqueued on it and nothing synchronises the device;
 *   - sizes are in elements, strides are ELEMENT strides of the tensor they describe;
 *   - io_dtype selects the storage type of x, delta, B, C, z, y, dy and of their
 *     gradients (delta and its gradient may be float32 next to bfloat16 tensors, see
 *     MPA_DELTA_F32); A, D, delta_bias, the recurrent state and every accumulation are float32;
 *   - the return value is MPA_OK or one of the MPA_ERR_* codes; nothing is thrown.
 * All entry points are reentrant: nothing is read from the environment, every choice the
 * library makes is a function of the arguments (the workspace queries and the calls they size
 * therefore always agree).  They keep no global state, with two exceptions: a per-device flag
 * that remembers that a kernel's dynamic-LDS limit has been raised, and mpa_sscan_fwd_noalloc,
 * which owns a static device array per GPU and the address of it (see there).
 */
#ifndef MAMBAPY_AMD_H
#define MAMBAPY_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MPA_VERSION 20100 /* major*10000 + minor*100 + patch: 2.1.0 */

enum mpa_status {
    MPA_OK = 0,
    MPA_ERR_NULL_POINTER = 1,  /* a required pointer is NULL */
    MPA_ERR_BAD_SHAPE = 2,     /* non-positive size, d_state above the supported maximum, ... */
    MPA_ERR_BAD_DTYPE = 3,     /* io_dtype is not one of mpa_dtype */
    MPA_ERR_BAD_STRIDE = 4,    /* a stride the kernels cannot honour (see each entry point) */
    MPA_ERR_MISALIGNED = 5,    /* a pointer is not aligned to its element size */
    MPA_ERR_WORKSPACE = 6,     /* workspace_bytes is smaller than the *_workspace_bytes query */
    MPA_ERR_LAUNCH = 7         /* hipGetLastError() reported a launch failure */
};

enum mpa_dtype { MPA_F32 = 0, MPA_BF16 = 1 };

/* Number of time steps between two saved states (see mpa_sscan_fwd: h_ckpt). */
#define MPA_CKPT_STEPS 16
/* Largest supported d_state (N). */
#define MPA_MAX_DSTATE 256

/* Shape and layout of one selective-scan call.  Logical shapes (mambapy/mamba.py:275-282):
 *   x, delta, z, y, dy, dx, ddelta : (batch, seqlen, dim)      dim = ED = d_inner
 *   A : (dim, dstate) contiguous float32;  D, delta_bias : (dim) contiguous float32
 *   B, C, dB, dC : (batch, seqlen, dstate), innermost stride 1
 * u_* strides apply to x;  z_* to z;  d_* to delta;  y_* to y, dy, y_pregate;  g_* to dx, ddelta, dz;
 * bc_* to B and C;  dbc_* to dB and dC.
 * The reference calls this path both with fresh channel-contiguous tensors
 * (tests/compare_seq_pscan.py:24-29: strides (L*ED, ED, 1)) and, from MambaBlock.forward,
 * with time-contiguous views (mambapy/mamba.py:217-221, 247, 264: strides (ED*L, 1, L)) and
 * with B, C that are slices of one projection (mamba.py:245: row stride dt_rank+2N).
 * Both layouts are honoured without a copy. */
typedef struct mpa_sscan_shape {
    int64_t batch, seqlen, dim, dstate;
    int32_t io_dtype; /* enum mpa_dtype */
    int32_t flags;    /* bit set of MPA_SSCAN_* */
    int64_t u_sb, u_sl, u_sd;
    int64_t z_sb, z_sl, z_sd;
    int64_t d_sb, d_sl, d_sd;
    int64_t y_sb, y_sl, y_sd;
    int64_t g_sb, g_sl, g_sd;
    int64_t bc_sb, bc_sl;
    int64_t dbc_sb, dbc_sl;
    /* Launch plan.  0 = chosen by the library from the shape (the normal case); a caller that
     * tunes or tests may pin the decomposition.  The same values must be given to a call and
     * to the workspace query that sizes it. */
    int32_t plan_states_per_lane; /* states of d_state kept by one lane: a power of two */
    int32_t plan_segments;        /* pieces the sequence is cut into (1 = never cut) */
    int32_t plan_flags;           /* bit set of MPA_PLAN_* */
    int32_t delta_dtype;          /* 0: delta and ddelta have io_dtype; MPA_DELTA_F32: see below */
} mpa_sscan_shape;

/* mpa_sscan_shape.delta_dtype: delta (read) and ddelta (written) are float32 whatever io_dtype is
 * (d_* and g_* remain element strides).  This is the call the reference makes under
 * torch.autocast: softplus leaves delta in float32 while x, B, C are bfloat16
 * (mambapy/mamba.py:264-265 with :284-287).  Fast kernels only: mpa_sscan_bwd returns
 * MPA_ERR_BAD_DTYPE where it would need its general kernel. */
#define MPA_DELTA_F32 1

/* delta = softplus(delta + delta_bias) is applied inside the kernel (mamba.py:264-265);
 * without the flag `delta` is used as given and delta_bias must be NULL. */
#define MPA_SSCAN_DELTA_SOFTPLUS 1
/* The recurrence runs from the last step to the first: h[t] = a[t]*h[t+1] + ..., h0 is the
 * state before step seqlen-1 and h_last the state after step 0.  Equal to flipping x, delta,
 * z, B, C along time, scanning, and flipping y back, which is how the reference's
 * bidirectional block obtains its backward direction (mambapy/vim.py:228-261: xz.flip([1])
 * in, y_b.flip([1]) out) at the price of those copies. */
#define MPA_SSCAN_REVERSE 2

/* mpa_sscan_bwd: use the general backward kernel even where the fast one applies. */
#define MPA_PLAN_BWD_GENERAL 1
/* Test hook: the bounded waits inside the kernels behave as if they had run out (see
 * mpa_sscan_bwd); every kernel still runs to its end. */
#define MPA_PLAN_EXPIRE_WAITS 2
/* Channels of a batch row that one workgroup owns: 64 always / 48 wherever the kernels have that form
 * (neither bit: the library picks, see mpa_sscan_fwd). */
#define MPA_PLAN_GROUP_64 4
#define MPA_PLAN_GROUP_48 8

int mpa_version(void);
/* Host string naming the GPU architecture the kernels were compiled for ("gfx950"). */
const char* mpa_arch(void);
/* Host string: hash of the kernel sources this library was built from (16 hex digits, "unknown"
 * when the build did not say).  Measurements that are kept next to the sources (hardware-counter
 * summaries) quote it, so that a reader can tell whether they describe the kernels that run. */
const char* mpa_source_hash(void);
/* Host string describing a status code. */
const char* mpa_status_string(int status);

/* ---- fused selective scan, forward ------------------------------------------------------
 * Replaces MambaBlock.selective_scan(x, delta, A, B, C, D) (mambapy/mamba.py:274-295) and
 * its sequential twin selective_scan_seq (:297-327): discretisation exp(delta*A) /
 * delta*B*x, the scan that mambapy/pscan.py:151-186 performs on materialised
 * (B,L,ED,N) tensors, and the readout y = C.h + D*x, in one pass that never writes a
 * (B,L,ED,N) tensor.  Any seqlen >= 1 (no power-of-two padding, cf. pscan.py:165-174).
 *   z        optional: y is multiplied by silu(z) (mamba.py:229-231); NULL = no gate.
 *   h0       optional (batch, dim, dstate) float32 initial state; NULL = zeros (mamba.py:314).
 *   h_ckpt   optional float32 buffer of mpa_sscan_ckpt_elems() elements: the state after
 *            every MPA_CKPT_STEPS-th step, consumed by mpa_sscan_bwd; NULL when no
 *            gradient is needed.
 *   h_last   optional (batch, dim, dstate) float32: state after the last step, in the
 *            layout of the decode cache `h` (mamba.py:335, 341).
 *   y_pregate  optional, only with z: the output before the gate (C.h + D*x), io_dtype, strides
 *            of y.  mpa_sscan_bwd needs it on its fast path; NULL when no gradient is needed.
 *   workspace  scratch of mpa_sscan_fwd_workspace_bytes() bytes.
 * d_state above 64 runs in passes over blocks of 64 states, each adding its readout to y (in
 * y_pregate when that is given) in io_dtype.
 * When batch * dim/64 workgroups would cover a fraction of the chip, the sequence is cut into
 * segments that run side by side (end states of all segments from zero, a carry pass, then the
 * real pass from the true initial states); checkpoints, h_last and y are the same as without the
 * cut up to float32 rounding.
 * A launch that is not cut has batch * ceil(dim / 64) workgroups; where batch * ceil(dim / 48) still
 * fit the 256 CUs in one round (and d_state <= 16), workgroups of 48 channels are used instead: more
 * of the chip works, and every workgroup is faster (its scan waves have two SIMDs to themselves).
 */
int mpa_sscan_fwd(const mpa_sscan_shape* s, const void* x, const void* delta, const float* A,
                  const void* B, const void* C, const float* D, const void* z,
                  const float* delta_bias, const float* h0, void* y, void* y_pregate,
                  float* h_ckpt, float* h_last, void* workspace, size_t workspace_bytes,
                  void* stream);

/* Number of float32 elements of the h_ckpt buffer for this shape. */
int64_t mpa_sscan_ckpt_elems(const mpa_sscan_shape* s);

/* Bytes of the scratch `workspace` of mpa_sscan_fwd (256-byte aligned; holds B and C
 * repacked as float32 in the order the scan waves read them, or the per-segment states of a
 * cut sequence; contents are dead after the call).  with_ckpt = 1 for a call that passes
 * h_ckpt, 0 for one that does not (the two are cut differently). */
size_t mpa_sscan_fwd_workspace_bytes(const mpa_sscan_shape* s, int with_ckpt);

/* ---- fused selective scan, forward, for callers that cannot allocate ------------------------
 * No counterpart in the reference.  It is for callers that cannot provide a workspace because they
 * cannot call hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  Same arguments and results as mpa_sscan_fwd (bit for bit) without `workspace`: the
 * scratch is a static device array of MPA_NOALLOC_SCRATCH_BYTES that the library owns, one copy on
 * every GPU it runs on, held until the process ends.  The call allocates and frees nothing.
 * A shape whose mpa_sscan_fwd_workspace_bytes() exceeds MPA_NOALLOC_SCRATCH_BYTES is refused with
 * MPA_ERR_WORKSPACE before anything is launched (sequences cut into segments need
 * 2 * batch * segments * dim * min(dstate, 64) floats and a little more; a caller that pins 16 or
 * 32 states per lane needs the packed B/C of the whole sequence).  All calls on one GPU share that GPU's array: calls that overlap
 * on one GPU (different streams or threads) race; calls on one stream are ordered.
 * The first call on a device looks up the array's address and raises the kernels' dynamic-LDS limit
 * (host calls that do not belong into a stream capture): make one call per device and kernel variant
 * (same dtype, gate and states per lane) before capturing.
 */
#define MPA_NOALLOC_SCRATCH_BYTES (16u << 20)
int mpa_sscan_fwd_noalloc(const mpa_sscan_shape* s, const void* x, const void* delta, const float* A,
                          const void* B, const void* C, const float* D, const void* z,
                          const float* delta_bias, const float* h0, void* y, void* y_pregate,
                          float* h_ckpt, float* h_last, void* stream);

/* ---- fused selective scan, backward -----------------------------------------------------
 * Replaces what autograd records for mamba.py:284-293 plus PScan.backward
 * (mambapy/pscan.py:188-224): given dy it writes dx, ddelta (io_dtype), dB, dC (io_dtype),
 * dA (dim, dstate) and dD (dim) (float32, overwritten, not accumulated).
 * h_ckpt is the buffer mpa_sscan_fwd filled for the same inputs.  The gate z, delta_bias /
 * MPA_SSCAN_DELTA_SOFTPLUS and h0 must be the ones given to the forward call; dz (io_dtype,
 * u-strides of g_*) is required when z is given, ddelta is then the gradient w.r.t. the
 * raw (pre-softplus) delta, and ddelta_bias (dim) float32 is written when delta_bias is
 * given.  y_pregate (strides of dy) is what the forward call wrote for the same inputs; with z
 * and y_pregate == NULL the pre-gate output is recomputed by a slower, more general kernel.
 * `workspace` needs mpa_sscan_bwd_workspace_bytes() bytes, 256-byte aligned.
 * d_state up to MPA_MAX_DSTATE; above 16 the call runs in passes over blocks of 16 states (the
 * states are independent given x, delta, B, C), dx and ddelta being summed over the passes in
 * io_dtype.  Short batches of long sequences are cut into segments as in the forward call (the
 * carry runs from the end).
 * One kernel waits, with a bound, for a counter in shared memory; the wait cannot run out
 * unless the hardware scheduler misbehaves, and if it ever does the call does not return clean
 * numbers: dA of every channel whose sums may have been damaged is NaN.
 */
int mpa_sscan_bwd(const mpa_sscan_shape* s, const void* x, const void* delta, const float* A,
                  const void* B, const void* C, const float* D, const void* z,
                  const float* delta_bias, const float* h0, const void* dy,
                  const void* y_pregate, const float* h_ckpt, void* dx, void* ddelta, float* dA, void* dB, void* dC,
                  float* dD, void* dz, float* ddelta_bias, void* workspace,
                  size_t workspace_bytes, void* stream);

size_t mpa_sscan_bwd_workspace_bytes(const mpa_sscan_shape* s);

/* ---- causal depthwise convolution along time (+ bias, + SiLU) ------------------------------
 * Replaces, in MambaBlock.forward (mambapy/mamba.py:217-221),
 *     x.transpose(1,2) -> Conv1d(ED, ED, kernel, groups=ED, padding=kernel-1)(.)[:, :, :L]
 *       -> transpose(1,2) -> silu
 * on the (batch, seqlen, dim) tensor directly (any element strides: the caller passes the x half
 * of the in_proj output, mamba.py:213-214, without a copy), and its gradient.  weight is the
 * Conv1d weight (dim, 1, kernel) viewed as (dim, kernel) float32, bias (dim) float32 or NULL.
 * window_in  optional (batch, dim, kernel-1), io_dtype: the inputs before step 0 (the decode
 *            cache of mamba.py:344-346, 379), NULL = zeros (the reference's left padding).
 * window_out optional (batch, dim, kernel-1): the last kernel-1 inputs, i.e. the cache to
 *            continue from with MambaBlock.step.
 * y has the y_* strides, dy too; dx the g_* strides; dweight (dim, kernel), dbias (dim) float32,
 * overwritten.  No gradient flows into window_in.  window_out may equal window_in (the rolling
 * cache of a decode loop, updated in place: every (batch, channel) row is read and written by
 * one thread).
 */
#define MPA_CONV_SILU 1
typedef struct mpa_conv_shape {
    int64_t batch, seqlen, dim;
    int32_t kernel;   /* d_conv, 2..4 */
    int32_t io_dtype; /* enum mpa_dtype */
    int32_t flags;    /* bit set of MPA_CONV_* */
    int32_t reserved;
    int64_t x_sb, x_sl, x_sd;
    int64_t y_sb, y_sl, y_sd;
    int64_t g_sb, g_sl, g_sd;
} mpa_conv_shape;

int mpa_conv1d_fwd(const mpa_conv_shape* s, const void* x, const float* weight, const float* bias,
                   const void* window_in, void* y, void* window_out, void* stream);
int mpa_conv1d_bwd(const mpa_conv_shape* s, const void* x, const float* weight, const float* bias,
                   const void* window_in, const void* dy, void* dx, float* dweight, float* dbias,
                   void* workspace, size_t workspace_bytes, void* stream);
size_t mpa_conv1d_bwd_workspace_bytes(const mpa_conv_shape* s);

/* ---- RMSNorm --------------------------------------------------------------------------------
 * Replaces RMSNorm.forward (mambapy/mamba.py:427-433): y = x * rsqrt(mean(x^2, -1) + eps) * weight
 * on `rows` contiguous rows of `d` elements (io_dtype; d a multiple of 4 (float32) / 8 (bfloat16),
 * d <= 2048 / 4096), weight (d) float32 or NULL (the muP variant has none), and its gradient:
 * dx (io_dtype) and dweight (d) float32, overwritten.  rstd (rows) float32 is an optional output.
 * Pointers to x, y, dy, dx must be 16-byte aligned.
 *
 * The residual add of the layer stack (mambapy/mamba.py:106-112: mixer(norm(x)) + x, read by the
 * next layer's norm) can be folded in: with `residual` (rows x d, io_dtype) the forward writes
 * sum_out = x + residual (rounded to io_dtype, as the separate add would be) and normalises that
 * row; the backward then takes the sum as its `x` and `dsum`, the gradient that reaches the sum
 * from its other users, and returns dx = (gradient through the norm) + dsum, which is the gradient
 * of both x and residual.  residual, sum_out and dsum may be NULL (plain RMSNorm).
 */
int mpa_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* y, void* sum_out,
                    float* rstd, int64_t rows, int64_t d, float eps, int32_t io_dtype, void* stream);
int mpa_rmsnorm_bwd(const void* x, const float* weight, const void* dy, const void* dsum, void* dx,
                    float* dweight, int64_t rows, int64_t d, float eps, int32_t io_dtype,
                    void* workspace, size_t workspace_bytes, void* stream);
size_t mpa_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t d);

/* ---- generic first-order scan -----------------------------------------------------------
 * Replaces pscan = PScan.apply (mambapy/pscan.py:226; forward :151-186, backward :188-224)
 * for callers that hold materialised A, X of logical shape (batch, seqlen, dim, dstate):
 * H[t] = A[t]*H[t-1] + X[t], H[-1] = 0.  Strides are (sb, sl, sd, sn) element strides, one
 * set per tensor; any seqlen.  H is a new tensor: inputs are never modified
 * (pscan.py:167-174 clones).  Backward: gradX[t] = gradH[t] + A[t+1]*gradX[t+1],
 * gradA[t] = H[t-1]*gradX[t], gradA[0] = 0 (pscan.py:216-222).
 * The reference's scan has O(log L) depth at any batch size (pscan.py:36-92); here one lane owns
 * one (dim, dstate) recurrence, and when batch*dim*dstate offers too few lanes to keep the memory
 * system busy the sequence is cut into pieces that run side by side (aggregate pass, carry pass,
 * main pass).  `workspace` (mpa_pscan_workspace_bytes() bytes, 256-byte aligned) holds the
 * per-piece aggregates; contents are dead after the call.
 */
typedef struct mpa_pscan_shape {
    int64_t batch, seqlen, dim, dstate;
    int32_t io_dtype;
    int32_t reverse;          /* 1: scan from the last step to the first (pscan.py:94-149) */
    int64_t a_st[4];          /* A     (sb, sl, sd, sn) */
    int64_t x_st[4];          /* X or gradH */
    int64_t h_st[4];          /* H (output of fwd, input of bwd) */
    int64_t ga_st[4];         /* gradA */
    int64_t gx_st[4];         /* gradX */
    int32_t plan_chunks;      /* pieces the sequence is cut into; 0 = chosen from the shape, 1 = never cut */
    int32_t reserved;         /* 0 */
} mpa_pscan_shape;

size_t mpa_pscan_workspace_bytes(const mpa_pscan_shape* s);
int mpa_pscan_fwd(const mpa_pscan_shape* s, const void* A, const void* X, void* H, void* workspace,
                  size_t workspace_bytes, void* stream);
int mpa_pscan_bwd(const mpa_pscan_shape* s, const void* A, const void* H, const void* gradH,
                  void* gradA, void* gradX, void* workspace, size_t workspace_bytes, void* stream);

/* ---- decode step --------------------------------------------------------------------------
 * Replaces the state update and readout of MambaBlock.ssm_step (mambapy/mamba.py:400-412)
 * for one token: h' = exp(delta*A)*h + delta*B*x ; y = C.h' + D*x, optionally
 * delta = softplus(delta + delta_bias) (mamba.py:398) and y *= silu(z) (mamba.py:373-375).
 *   x, delta, y : (batch, dim) io_dtype contiguous;  z : (batch, dim) with row stride z_stride (it
 *   is a half of the in_proj output, mamba.py:356-357);  B, C : (batch, dstate) io_dtype,
 *   row stride bc_stride;  h_in, h_out : (batch, dim, dstate) float32 contiguous.
 * h_in == NULL means zeros (mamba.py:405-406).  h_out may equal h_in (in-place update);
 * with distinct buffers h_in is left untouched, which is the reference's behaviour
 * (ssm_step returns a new tensor).
 */
int mpa_ssm_step(const void* x, const void* delta, const float* A, const void* B, const void* C,
                 const float* D, const void* z, const float* delta_bias, const float* h_in,
                 float* h_out, void* y, int64_t batch, int64_t dim, int64_t dstate,
                 int64_t bc_stride, int64_t z_stride, int32_t io_dtype, int32_t delta_softplus,
                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MAMBAPY_AMD_H */
