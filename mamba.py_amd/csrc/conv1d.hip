// Causal depthwise convolution along time (+ bias, + SiLU) for gfx950, forward and backward.
//
// This is the step in front of the selective scan in MambaBlock.forward
// (mambapy/mamba.py:217-221: transpose, Conv1d(groups=ED, padding=K-1)[:, :, :L], transpose,
// silu) and, one token at a time, in MambaBlock.step (mamba.py:366-369).  It is a pure
// streaming kernel, bound by HBM: per (batch, step, channel) it reads one element and writes
// one (backward: reads two, writes one), with K multiply-adds in between.
//
//   * x is read in place with its own element strides: the caller passes the `x` half of the
//     in_proj output (a strided view, mamba.py:213) and gets a (B, L, ED) tensor back, so
//     neither of the two transposes of the reference exists here.
//   * One lane owns one channel and walks a span of kSpan steps with the last K-1 inputs in
//     registers; a wave step is one contiguous row of 64 channels.  The loads of a group of 16
//     steps are all issued before the first one is used, and the next group is requested
//     before the current one is computed, so 32 rows per wave are in flight.
//   * A span starts from the K-1 inputs before it (the caller's window for the first span,
//     zeros if there is none): spans are independent, which is where the parallelism along L
//     comes from.
//   * Backward recomputes the pre-activation (K multiply-adds) instead of saving it, forms
//     dpre = dy * silu'(pre), dx[t] = sum_k w[k] * dpre[t + K-1-k], and keeps per-lane sums of
//     dweight / dbias over its span; spans and batch rows are then summed by a second kernel
//     in a fixed order (no floating-point atomics).
#include <type_traits>

#include "common.h"

namespace mpa {

constexpr int kConvSpan = 64;   // steps per lane (doubled when the problem still fills the chip, see conv_span)
constexpr int kConvGroup = 16;  // steps loaded together
constexpr int kConvMaxK = 4;

struct ConvParams {
    const void* x;
    const float* w;      // (ED, K)
    const float* bias;   // (ED) or null
    const void* win;     // (B, ED, K-1) inputs before step 0, or null (zeros)
    void* y;
    void* wout;          // (B, ED, K-1) last K-1 inputs, or null
    const void* dy;
    void* dx;
    float* part;         // [B][nspan][K+1][ED]
    int batch, L, ED, K, nspan, span;
    int silu;
    int64_t x_sb, x_sl, x_sd;
    int64_t y_sb, y_sl, y_sd;
    int64_t g_sb, g_sl, g_sd;
};

// input element at step t of this lane's channel: the sequence, the caller's window before
// it, or zero
template <typename IO>
__device__ __forceinline__ float conv_input(const ConvParams& p, const IO* xrow, const IO* wrow, int t) {
    if (t >= 0) return t < p.L ? to_float(xrow[(int64_t)t * p.x_sl]) : 0.0f;
    return (wrow && t + p.K - 1 >= 0) ? to_float(wrow[t + p.K - 1]) : 0.0f;
}

template <typename IO, bool SILU>
__global__ void __launch_bounds__(256) conv1d_fwd_kernel(const ConvParams p) {
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= p.ED) return;
    const int b = blockIdx.z;
    const int t0 = blockIdx.y * p.span;
    const int K = p.K;
    const IO* xrow = static_cast<const IO*>(p.x) + b * p.x_sb + (int64_t)d * p.x_sd;
    const IO* wrow = p.win ? static_cast<const IO*>(p.win) + ((int64_t)b * p.ED + d) * (K - 1) : nullptr;
    IO* yrow = static_cast<IO*>(p.y) + b * p.y_sb + (int64_t)d * p.y_sd;
    // taps aligned to the newest input: wk[kConvMaxK-1] multiplies x[t]
    float wk[kConvMaxK];
#pragma unroll
    for (int k = 0; k < kConvMaxK; ++k) {
        const int src = k - (kConvMaxK - K);
        wk[k] = src >= 0 ? p.w[(int64_t)d * K + src] : 0.0f;
    }
    const float bv = p.bias ? p.bias[d] : 0.0f;
    float h1 = conv_input<IO>(p, xrow, wrow, t0 - 1);
    float h2 = conv_input<IO>(p, xrow, wrow, t0 - 2);
    float h3 = conv_input<IO>(p, xrow, wrow, t0 - 3);

    const int tend = min(t0 + p.span, p.L);
    IO cur[kConvGroup], nxt[kConvGroup];
    auto load_group = [&](int tg, IO (&dst)[kConvGroup]) {
        // steps beyond the sequence are clamped (valid memory); their results are not stored
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) dst[j] = xrow[(int64_t)min(tg + j, p.L - 1) * p.x_sl];
    };
    load_group(t0, cur);
    for (int tg = t0; tg < tend; tg += kConvGroup) {
        if (tg + kConvGroup < tend) load_group(tg + kConvGroup, nxt);
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) {
            const float xv = to_float(cur[j]);
            float acc = __builtin_fmaf(wk[3], xv, bv);
            acc = __builtin_fmaf(wk[2], h1, acc);
            acc = __builtin_fmaf(wk[1], h2, acc);
            acc = __builtin_fmaf(wk[0], h3, acc);
            h3 = h2;
            h2 = h1;
            h1 = xv;
            if (SILU) acc *= sigmoid_f(acc);
            if (tg + j < tend) yrow[(int64_t)(tg + j) * p.y_sl] = from_float<IO>(acc);
        }
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) cur[j] = nxt[j];
    }
    if (p.wout && tend == p.L) {
        // the last K-1 inputs of the sequence, oldest first (the decode cache of mamba.py:379)
        IO* wo = static_cast<IO*>(p.wout) + ((int64_t)b * p.ED + d) * (K - 1);
        for (int j = 0; j < K - 1; ++j) wo[j] = from_float<IO>(conv_input<IO>(p, xrow, wrow, p.L - (K - 1) + j));
    }
}

template <typename IO, bool SILU>
__global__ void __launch_bounds__(256) conv1d_bwd_kernel(const ConvParams p) {
    const int d = blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= p.ED) return;
    const int b = blockIdx.z;
    const int t0 = blockIdx.y * p.span;
    const int K = p.K;
    const IO* xrow = static_cast<const IO*>(p.x) + b * p.x_sb + (int64_t)d * p.x_sd;
    const IO* wrow = p.win ? static_cast<const IO*>(p.win) + ((int64_t)b * p.ED + d) * (K - 1) : nullptr;
    const IO* dyrow = static_cast<const IO*>(p.dy) + b * p.y_sb + (int64_t)d * p.y_sd;
    IO* dxrow = static_cast<IO*>(p.dx) + b * p.g_sb + (int64_t)d * p.g_sd;
    float wk[kConvMaxK];
#pragma unroll
    for (int k = 0; k < kConvMaxK; ++k) {
        const int src = k - (kConvMaxK - K);
        wk[k] = src >= 0 ? p.w[(int64_t)d * K + src] : 0.0f;
    }
    const float bv = p.bias ? p.bias[d] : 0.0f;
    float h1 = conv_input<IO>(p, xrow, wrow, t0 - 1);
    float h2 = conv_input<IO>(p, xrow, wrow, t0 - 2);
    float h3 = conv_input<IO>(p, xrow, wrow, t0 - 3);
    // dpre of the last three steps processed; dx[t] needs dpre[t .. t+3], so the walk runs
    // three steps past the span and dx lags three steps behind
    float g1 = 0.0f, g2 = 0.0f, g3 = 0.0f;
    float dw[kConvMaxK] = {0.0f, 0.0f, 0.0f, 0.0f}, db = 0.0f;

    const int tend = min(t0 + p.span, p.L);           // dweight / dbias / dx cover [t0, tend)
    const int twalk = min(tend + kConvMaxK - 1, p.L + kConvMaxK - 1);
    IO cx[kConvGroup], cy[kConvGroup], nx[kConvGroup], ny[kConvGroup];
    auto load_group = [&](int tg, IO (&dx_)[kConvGroup], IO (&dy_)[kConvGroup]) {
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) {
            const int tc = min(tg + j, p.L - 1);
            dx_[j] = xrow[(int64_t)tc * p.x_sl];
            dy_[j] = dyrow[(int64_t)tc * p.y_sl];
        }
    };
    // one group of kConvGroup steps; EDGE = the group touches the start or the end of the span or of
    // the sequence (the others need no predicate: every step is live, counted and stored)
    auto walk_group = [&](auto edge_c, int tg) {
        constexpr bool EDGE = decltype(edge_c)::value;
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) {
            const int t = tg + j;
            const bool live = !EDGE || t < p.L;  // steps past the sequence contribute dpre = 0
            const float xv = live ? to_float(cx[j]) : 0.0f;
            float pre = __builtin_fmaf(wk[3], xv, bv);
            pre = __builtin_fmaf(wk[2], h1, pre);
            pre = __builtin_fmaf(wk[1], h2, pre);
            pre = __builtin_fmaf(wk[0], h3, pre);
            float g = live ? to_float(cy[j]) : 0.0f;
            if (SILU) {
                const float s = sigmoid_f(pre);
                g *= s * __builtin_fmaf(pre, 1.0f - s, 1.0f);
            }
            if (!EDGE || t < tend) {
                dw[3] = __builtin_fmaf(g, xv, dw[3]);
                dw[2] = __builtin_fmaf(g, h1, dw[2]);
                dw[1] = __builtin_fmaf(g, h2, dw[1]);
                dw[0] = __builtin_fmaf(g, h3, dw[0]);
                db += g;
            }
            // dx[t-3] = w[K-1]*dpre[t-3] + w[K-2]*dpre[t-2] + w[K-3]*dpre[t-1] + w[K-4]*dpre[t]
            const float dxv = __builtin_fmaf(wk[3], g3, __builtin_fmaf(wk[2], g2, __builtin_fmaf(wk[1], g1, wk[0] * g)));
            const int tx = t - (kConvMaxK - 1);
            if (!EDGE || (tx >= t0 && tx < tend)) dxrow[(int64_t)tx * p.g_sl] = from_float<IO>(dxv);
            g3 = g2;
            g2 = g1;
            g1 = g;
            h3 = h2;
            h2 = h1;
            h1 = xv;
        }
    };
    load_group(t0, cx, cy);
    for (int tg = t0; tg < twalk; tg += kConvGroup) {
        if (tg + kConvGroup < twalk) load_group(tg + kConvGroup, nx, ny);
        if (tg > t0 && tg + kConvGroup <= tend)
            walk_group(std::false_type{}, tg);
        else
            walk_group(std::true_type{}, tg);
#pragma unroll
        for (int j = 0; j < kConvGroup; ++j) {
            cx[j] = nx[j];
            cy[j] = ny[j];
        }
    }
    float* part = p.part + (((int64_t)b * p.nspan + blockIdx.y) * (kConvMaxK + 1)) * p.ED + d;
#pragma unroll
    for (int k = 0; k < kConvMaxK; ++k) part[(int64_t)k * p.ED] = dw[k];
    part[(int64_t)kConvMaxK * p.ED] = db;
}

// dweight[d][k] / dbias[d] = sum over (batch, span) of the partial sums.  A block owns 64
// columns of the [(K+1) * ED] partial rows; its 16 row groups each sum every 16th partial in
// index order and the groups are combined in a fixed order through LDS (no atomics, so the
// result does not depend on scheduling).
constexpr int kFinCols = 64, kFinRows = 16;
__global__ void __launch_bounds__(kFinCols* kFinRows)
    conv1d_bwd_finish_kernel(const float* part, float* dweight, float* dbias, int ED, int K, int nparts) {
    __shared__ float acc[kFinRows][kFinCols];
    const int col = threadIdx.x % kFinCols, rg = threadIdx.x / kFinCols;
    const int i = blockIdx.x * kFinCols + col;  // (k5, d), d fastest
    const int width = (kConvMaxK + 1) * ED;
    float s = 0.0f;
    if (i < width)
        for (int q = rg; q < nparts; q += kFinRows) s += part[(int64_t)q * width + i];
    acc[rg][col] = s;
    __syncthreads();
    if (rg != 0 || i >= width) return;
    for (int r = 1; r < kFinRows; ++r) s += acc[r][col];
    const int k5 = i / ED, d = i % ED;
    if (k5 == kConvMaxK) {
        if (dbias) dbias[d] = s;
    } else {
        const int k = k5 - (kConvMaxK - K);  // tap index in the caller's (ED, K) layout
        if (k >= 0) dweight[(int64_t)d * K + k] = s;
    }
}

static int conv_validate(const mpa_conv_shape* s) {
    if (!s) return MPA_ERR_NULL_POINTER;
    if (s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->batch > 65535) return MPA_ERR_BAD_SHAPE;
    if (s->kernel < 2 || s->kernel > kConvMaxK) return MPA_ERR_BAD_SHAPE;
    if (s->seqlen > (int64_t)1 << 30 || s->dim > (int64_t)1 << 30) return MPA_ERR_BAD_SHAPE;
    if ((s->seqlen + kConvSpan - 1) / kConvSpan > 65535) return MPA_ERR_BAD_SHAPE;  // spans are the grid's y axis
    if (s->io_dtype != MPA_F32 && s->io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    const int64_t st[] = {s->x_sb, s->x_sl, s->x_sd, s->y_sb, s->y_sl, s->y_sd, s->g_sb, s->g_sl, s->g_sd};
    for (int64_t v : st)
        if (v < 0) return MPA_ERR_BAD_STRIDE;
    return MPA_OK;
}

// Steps per lane: longer spans mean fewer halo reads and fewer dweight partials, shorter spans
// more waves; 128 steps when that still leaves 16 waves per CU.
static int conv_span(const mpa_conv_shape* s) {
    const int64_t waves128 = s->batch * ((s->seqlen + 2 * kConvSpan - 1) / (2 * kConvSpan)) * ((s->dim + kWave - 1) / kWave);
    return waves128 >= 4096 ? 2 * kConvSpan : kConvSpan;
}

static ConvParams conv_params(const mpa_conv_shape* s) {
    ConvParams p{};
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.ED = (int)s->dim; p.K = s->kernel;
    p.span = conv_span(s);
    p.nspan = (p.L + p.span - 1) / p.span;
    p.silu = (s->flags & MPA_CONV_SILU) ? 1 : 0;
    p.x_sb = s->x_sb; p.x_sl = s->x_sl; p.x_sd = s->x_sd;
    p.y_sb = s->y_sb; p.y_sl = s->y_sl; p.y_sd = s->y_sd;
    p.g_sb = s->g_sb; p.g_sl = s->g_sl; p.g_sd = s->g_sd;
    return p;
}

}  // namespace mpa

using namespace mpa;

extern "C" int mpa_conv1d_fwd(const mpa_conv_shape* s, const void* x, const float* weight,
                              const float* bias, const void* window_in, void* y, void* window_out,
                              void* stream) {
    int rc = conv_validate(s);
    if (rc != MPA_OK) return rc;
    if (!x || !weight || !y) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(x, es) || !aligned_to(y, es) || !aligned_to(weight, 4) || (bias && !aligned_to(bias, 4)) ||
        (window_in && !aligned_to(window_in, es)) || (window_out && !aligned_to(window_out, es)))
        return MPA_ERR_MISALIGNED;
    ConvParams p = conv_params(s);
    p.x = x; p.w = weight; p.bias = bias; p.win = window_in; p.y = y; p.wout = window_out;
    dim3 grid((p.ED + 255) / 256, p.nspan, p.batch), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->io_dtype == MPA_F32) {
        if (p.silu) hipLaunchKernelGGL((conv1d_fwd_kernel<float, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((conv1d_fwd_kernel<float, false>), grid, block, 0, st, p);
    } else {
        if (p.silu) hipLaunchKernelGGL((conv1d_fwd_kernel<bf16_t, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((conv1d_fwd_kernel<bf16_t, false>), grid, block, 0, st, p);
    }
    return check_launch();
}

extern "C" size_t mpa_conv1d_bwd_workspace_bytes(const mpa_conv_shape* s) {
    if (conv_validate(s) != MPA_OK) return 0;
    const size_t span = (size_t)conv_span(s);
    const size_t nspan = ((size_t)s->seqlen + span - 1) / span;
    return ((size_t)s->batch * nspan * (kConvMaxK + 1) * s->dim * sizeof(float) + 255) / 256 * 256;
}

extern "C" int mpa_conv1d_bwd(const mpa_conv_shape* s, const void* x, const float* weight,
                              const float* bias, const void* window_in, const void* dy, void* dx,
                              float* dweight, float* dbias, void* workspace, size_t workspace_bytes,
                              void* stream) {
    int rc = conv_validate(s);
    if (rc != MPA_OK) return rc;
    if (!x || !weight || !dy || !dx || !dweight || !workspace) return MPA_ERR_NULL_POINTER;
    if (bias && !dbias) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(x, es) || !aligned_to(dy, es) || !aligned_to(dx, es) || !aligned_to(weight, 4) ||
        !aligned_to(dweight, 4) || (bias && !aligned_to(bias, 4)) || (dbias && !aligned_to(dbias, 4)) ||
        (window_in && !aligned_to(window_in, es)) || !aligned_to(workspace, 256))
        return MPA_ERR_MISALIGNED;
    if (workspace_bytes < mpa_conv1d_bwd_workspace_bytes(s)) return MPA_ERR_WORKSPACE;
    ConvParams p = conv_params(s);
    p.x = x; p.w = weight; p.bias = bias; p.win = window_in; p.dy = dy; p.dx = dx;
    p.part = static_cast<float*>(workspace);
    dim3 grid((p.ED + 255) / 256, p.nspan, p.batch), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->io_dtype == MPA_F32) {
        if (p.silu) hipLaunchKernelGGL((conv1d_bwd_kernel<float, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((conv1d_bwd_kernel<float, false>), grid, block, 0, st, p);
    } else {
        if (p.silu) hipLaunchKernelGGL((conv1d_bwd_kernel<bf16_t, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((conv1d_bwd_kernel<bf16_t, false>), grid, block, 0, st, p);
    }
    rc = check_launch();
    if (rc != MPA_OK) return rc;
    const int total = (kConvMaxK + 1) * p.ED;
    hipLaunchKernelGGL(conv1d_bwd_finish_kernel, dim3((total + kFinCols - 1) / kFinCols),
                       dim3(kFinCols * kFinRows), 0, st, p.part, dweight, dbias, p.ED, p.K, p.batch * p.nspan);
    return check_launch();
}
