// Generic first-order scan H[t] = A[t]*H[t-1] + X[t] over materialised (B, L, D, N) tensors,
// forward and backward, for gfx950.
//
// This path is bound by HBM traffic (12 bytes moved per fp32 element and step, one fma), so
// the kernel is organised around the memory system: one lane owns one (channel, state)
// recurrence, lanes follow the unit-stride axis of the tensors so that every step of a wave
// is one coalesced 256-byte line per operand, and the time loop is unrolled by kUnroll steps
// with all loads of a block issued before its arithmetic, which keeps
// kUnroll * 2 * 256 B per wave in flight.  When the tensors offer too few such lanes to keep
// the memory system busy (small batch * dim * dstate), the sequence is cut into pieces that run
// side by side: a first pass finds, per piece, the product of its A and its end value from
// zero, a carry pass chains them, and the main pass starts every piece from its true value
// (see pscan_plan).
#include "common.h"

namespace mpa {

constexpr int kUnroll = 8;

struct PscanParams {
    const void* A;
    const void* X;   // fwd: X; bwd: gradH
    const void* H;   // bwd only
    void* out0;      // fwd: H; bwd: gradX
    void* out1;      // bwd: gradA
    // sequence cut into nchunk pieces of chunk_len walk positions (nchunk = 1: not cut)
    float* agg;          // [batch][nchunk][2][D*N]: product of A over the piece, end value from zero
    const float* carry;  // [batch][nchunk][D*N]: value that flows into the piece (NULL: zero)
    int nchunk, chunk_len;
    int batch, L, D, N;
    int reverse;
    int64_t a_st[4], x_st[4], h_st[4], o0_st[4], o1_st[4];
};

// lane -> (d, n): the innermost unit-stride axis of A decides which index runs fastest
__device__ __forceinline__ void lane_to_dn(const PscanParams& p, int64_t e, int& d, int& n) {
    if (p.a_st[3] == 1 || p.a_st[2] != 1) {
        d = (int)(e / p.N);
        n = (int)(e % p.N);
    } else {
        n = (int)(e / p.D);
        d = (int)(e % p.D);
    }
}

// A launch row is one piece of one batch row: walk positions [w0, w1) of the order in which the
// kernel visits the steps (the scan direction for the forward kernels, against it for the
// backward ones).
struct Piece {
    int b, c, w0, w1;
};
__device__ __forceinline__ Piece piece_of(const PscanParams& p) {
    Piece q;
    q.b = blockIdx.y / p.nchunk;
    q.c = blockIdx.y - q.b * p.nchunk;
    q.w0 = q.c * p.chunk_len;
    q.w1 = min(p.L, q.w0 + p.chunk_len);
    return q;
}

template <typename IO>
__global__ void __launch_bounds__(256) pscan_fwd_kernel(const PscanParams p) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (int64_t)p.D * p.N) return;
    const Piece q = piece_of(p);
    int d, n;
    lane_to_dn(p, e, d, n);
    const int64_t step = p.reverse ? -1 : 1;
    const int64_t tfirst = p.reverse ? p.L - 1 - q.w0 : q.w0;
    int64_t ia = q.b * p.a_st[0] + tfirst * p.a_st[1] + d * p.a_st[2] + n * p.a_st[3];
    int64_t ix = q.b * p.x_st[0] + tfirst * p.x_st[1] + d * p.x_st[2] + n * p.x_st[3];
    int64_t io = q.b * p.o0_st[0] + tfirst * p.o0_st[1] + d * p.o0_st[2] + n * p.o0_st[3];
    const int64_t sa = step * p.a_st[1], sx = step * p.x_st[1], so = step * p.o0_st[1];
    float h = p.carry ? p.carry[((int64_t)q.b * p.nchunk + q.c) * p.D * p.N + e] : 0.0f;
    int w = q.w0;
    for (; w + kUnroll <= q.w1; w += kUnroll) {
        float av[kUnroll], xv[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            av[k] = load_as_float<IO>(p.A, ia + k * sa);
            xv[k] = load_as_float<IO>(p.X, ix + k * sx);
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            h = __builtin_fmaf(av[k], h, xv[k]);
            store_from_float<IO>(p.out0, io + k * so, h);
        }
        ia += kUnroll * sa;
        ix += kUnroll * sx;
        io += kUnroll * so;
    }
    for (; w < q.w1; ++w) {
        h = __builtin_fmaf(load_as_float<IO>(p.A, ia), h, load_as_float<IO>(p.X, ix));
        store_from_float<IO>(p.out0, io, h);
        ia += sa;
        ix += sx;
        io += so;
    }
}

// First pass of a cut sequence: per piece, the product of its A and its end value from a zero
// start.  Both recurrences are linear in the value they carry,
//     forward   h' = A*h + X            (walk in the scan direction)
//     backward  c' = A*(G + c)          (walk against it; c = A[t]*gradX[t] is what step t-1 adds)
// so the value that leaves a piece entered with v is (product of A) * v + (end value from zero).
template <typename IO, bool BWD>
__global__ void __launch_bounds__(256) pscan_agg_kernel(const PscanParams p) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t dn = (int64_t)p.D * p.N;
    if (e >= dn) return;
    const Piece q = piece_of(p);
    int d, n;
    lane_to_dn(p, e, d, n);
    const bool down = BWD ? !p.reverse : (p.reverse != 0);  // the walk runs towards lower t
    const int64_t step = down ? -1 : 1;
    const int64_t tfirst = down ? p.L - 1 - q.w0 : q.w0;
    int64_t ia = q.b * p.a_st[0] + tfirst * p.a_st[1] + d * p.a_st[2] + n * p.a_st[3];
    int64_t ix = q.b * p.x_st[0] + tfirst * p.x_st[1] + d * p.x_st[2] + n * p.x_st[3];
    const int64_t sa = step * p.a_st[1], sx = step * p.x_st[1];
    float v = 0.0f, prod = 1.0f;
    int w = q.w0;
    for (; w + kUnroll <= q.w1; w += kUnroll) {
        float av[kUnroll], xv[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            av[k] = load_as_float<IO>(p.A, ia + k * sa);
            xv[k] = load_as_float<IO>(p.X, ix + k * sx);
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            v = BWD ? av[k] * (xv[k] + v) : __builtin_fmaf(av[k], v, xv[k]);
            prod *= av[k];
        }
        ia += kUnroll * sa;
        ix += kUnroll * sx;
    }
    for (; w < q.w1; ++w) {
        const float a = load_as_float<IO>(p.A, ia), x = load_as_float<IO>(p.X, ix);
        v = BWD ? a * (x + v) : __builtin_fmaf(a, v, x);
        prod *= a;
        ia += sa;
        ix += sx;
    }
    float* out = p.agg + ((int64_t)q.b * p.nchunk + q.c) * 2 * dn + e;
    out[0] = prod;
    out[dn] = v;
}

// Between the passes: the value that flows into every piece, pieces taken in walk order.
__global__ void __launch_bounds__(256) pscan_carry_kernel(const float* __restrict__ agg, float* __restrict__ carry,
                                                          int nchunk, int64_t dn) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= dn) return;
    const int b = blockIdx.y;
    float v = 0.0f;
    // The chain over the pieces is serial, its operands are not: the aggregates of the next kAhead
    // pieces are requested while the chain runs over the kAhead before them (a launch has few
    // lanes here, so nothing else would hide the memory latency of every step).
    constexpr int kAhead = 16;
    float prod[2][kAhead], hend[2][kAhead];
    auto request = [&](int c0, float (&pr)[kAhead], float (&he)[kAhead]) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            const int64_t row = (int64_t)b * nchunk + min(c0 + k, nchunk - 1);
            pr[k] = agg[row * 2 * dn + e];
            he[k] = agg[(row * 2 + 1) * dn + e];
        }
    };
    auto chain = [&](int c0, const float (&pr)[kAhead], const float (&he)[kAhead]) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            if (c0 + k < nchunk) {
                carry[((int64_t)b * nchunk + c0 + k) * dn + e] = v;
                // (a zero value stays out of the product: it may have overflowed, and 0 * inf is
                // not what the step-by-step recurrence computes)
                v = v == 0.0f ? he[k] : __builtin_fmaf(pr[k], v, he[k]);
            }
        }
    };
    request(0, prod[0], hend[0]);
    for (int c0 = 0; c0 < nchunk; c0 += 2 * kAhead) {
        request(c0 + kAhead, prod[1], hend[1]);
        chain(c0, prod[0], hend[0]);
        request(c0 + 2 * kAhead, prod[0], hend[0]);
        chain(c0 + kAhead, prod[1], hend[1]);
    }
}

// gradX[t] = gradH[t] + A[t+1]*gradX[t+1];  gradA[t] = H[t-1]*gradX[t], gradA[0] = 0.
// With reverse = 1 (the scan ran from the end) the roles of t-1 / t+1 swap.
template <typename IO>
__global__ void __launch_bounds__(256) pscan_bwd_kernel(const PscanParams p) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (int64_t)p.D * p.N) return;
    const Piece q = piece_of(p);
    int d, n;
    lane_to_dn(p, e, d, n);
    // walk against the direction of the forward scan
    const int64_t step = p.reverse ? 1 : -1;
    const int64_t tfirst = p.reverse ? q.w0 : p.L - 1 - q.w0;
    int64_t ia = q.b * p.a_st[0] + tfirst * p.a_st[1] + d * p.a_st[2] + n * p.a_st[3];
    int64_t ig = q.b * p.x_st[0] + tfirst * p.x_st[1] + d * p.x_st[2] + n * p.x_st[3];
    int64_t ih = q.b * p.h_st[0] + tfirst * p.h_st[1] + d * p.h_st[2] + n * p.h_st[3];
    int64_t i0 = q.b * p.o0_st[0] + tfirst * p.o0_st[1] + d * p.o0_st[2] + n * p.o0_st[3];
    int64_t i1 = q.b * p.o1_st[0] + tfirst * p.o1_st[1] + d * p.o1_st[2] + n * p.o1_st[3];
    const int64_t sa = step * p.a_st[1], sg = step * p.x_st[1], sh = step * p.h_st[1];
    const int64_t s0 = step * p.o0_st[1], s1 = step * p.o1_st[1];
    // at walk position w: gx = grad + acarry * gx_prev, where acarry = A of the previously
    // visited step; gradA = H(next position in the walk) * gx, zero at the last position of the
    // sequence.  A piece that is not the first starts from the carried product acarry * gx_prev.
    float gx = 0.0f, acarry = 0.0f;
    if (p.carry) {
        gx = p.carry[((int64_t)q.b * p.nchunk + q.c) * p.D * p.N + e];
        acarry = 1.0f;
    }
    // full blocks read H one position ahead, which exists while w + kUnroll < L
    const int wfull = min(q.w1, p.L - 1);
    int w = q.w0;
    for (; w + kUnroll <= wfull; w += kUnroll) {
        float av[kUnroll], gv[kUnroll], hv[kUnroll];
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            av[k] = load_as_float<IO>(p.A, ia + k * sa);
            gv[k] = load_as_float<IO>(p.X, ig + k * sg);
            hv[k] = load_as_float<IO>(p.H, ih + (k + 1) * sh);
        }
#pragma unroll
        for (int k = 0; k < kUnroll; ++k) {
            gx = __builtin_fmaf(acarry, gx, gv[k]);
            acarry = av[k];
            store_from_float<IO>(p.out0, i0 + k * s0, gx);
            store_from_float<IO>(p.out1, i1 + k * s1, hv[k] * gx);
        }
        ia += kUnroll * sa;
        ig += kUnroll * sg;
        ih += kUnroll * sh;
        i0 += kUnroll * s0;
        i1 += kUnroll * s1;
    }
    for (; w < q.w1; ++w) {
        gx = __builtin_fmaf(acarry, gx, load_as_float<IO>(p.X, ig));
        acarry = load_as_float<IO>(p.A, ia);
        const float hprev = (w + 1 < p.L) ? load_as_float<IO>(p.H, ih + sh) : 0.0f;
        store_from_float<IO>(p.out0, i0, gx);
        store_from_float<IO>(p.out1, i1, hprev * gx);
        ia += sa;
        ig += sg;
        ih += sh;
        i0 += s0;
        i1 += s1;
    }
}

// How a launch is cut.  One lane owns one (channel, state) recurrence for the whole sequence, so
// a launch has batch*dim*dstate lanes; below about 64 K of them the memory system runs dry and
// the sequence is cut into pieces that run side by side: two extra reads of A and X (or gradH)
// for nchunk times the lanes.
struct PscanPlan {
    int nchunk, chunk_len;
    size_t off_carry, floats;  // agg at 0
};
static PscanPlan pscan_plan(const mpa_pscan_shape* s) {
    PscanPlan pl{1, (int)s->seqlen, 0, 0};
    const int64_t lanes = s->batch * s->dim * s->dstate;
    int64_t want = 1;
    if (s->plan_chunks > 0) {
        want = s->plan_chunks;
    } else if (lanes <= 65536 && s->seqlen >= 256) {
        want = (262144 + lanes - 1) / lanes;
        if (want > s->seqlen / 64) want = s->seqlen / 64;  // pieces of 64 steps or more
    }
    if (want > s->seqlen) want = s->seqlen;
    if (want < 2 || s->batch * want > 65535) return pl;
    int64_t len = (s->seqlen + want - 1) / want;
    len = (len + kUnroll - 1) / kUnroll * kUnroll;
    pl.chunk_len = (int)len;
    pl.nchunk = (int)((s->seqlen + len - 1) / len);
    if (pl.nchunk < 2) return PscanPlan{1, (int)s->seqlen, 0, 0};
    const size_t rows = (size_t)s->batch * pl.nchunk, dn = (size_t)s->dim * s->dstate;
    pl.off_carry = 2 * rows * dn;
    pl.floats = 3 * rows * dn;
    return pl;
}

static int fill_params(const mpa_pscan_shape* s, PscanParams& p) {
    if (!s) return MPA_ERR_NULL_POINTER;
    if (s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return MPA_ERR_BAD_SHAPE;
    if (s->batch > 65535 || s->seqlen > (int64_t)1 << 30 || s->dim * s->dstate > (int64_t)1 << 31)
        return MPA_ERR_BAD_SHAPE;
    if (s->plan_chunks < 0 || s->reserved != 0) return MPA_ERR_BAD_SHAPE;
    if (s->io_dtype != MPA_F32 && s->io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.D = (int)s->dim; p.N = (int)s->dstate;
    p.reverse = s->reverse ? 1 : 0;
    p.nchunk = 1;
    p.chunk_len = p.L;
    return MPA_OK;
}

// passes 1 and 2 of a cut sequence (aggregates, then the carried values); X is X or gradH
template <bool BWD>
static int launch_carry_passes(const mpa_pscan_shape* s, PscanParams& p, const PscanPlan& pl, float* ws,
                               hipStream_t st) {
    p.nchunk = pl.nchunk;
    p.chunk_len = pl.chunk_len;
    p.agg = ws;
    const int64_t dn = (int64_t)p.D * p.N;
    dim3 grid((unsigned)((dn + 255) / 256), (unsigned)(p.batch * pl.nchunk));
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL((pscan_agg_kernel<float, BWD>), grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL((pscan_agg_kernel<bf16_t, BWD>), grid, dim3(256), 0, st, p);
    int rc = check_launch();
    if (rc != MPA_OK) return rc;
    hipLaunchKernelGGL(pscan_carry_kernel, dim3((unsigned)((dn + 255) / 256), (unsigned)p.batch), dim3(256), 0, st,
                       ws, ws + pl.off_carry, pl.nchunk, dn);
    p.carry = ws + pl.off_carry;
    return check_launch();
}

}  // namespace mpa

using namespace mpa;

extern "C" size_t mpa_pscan_workspace_bytes(const mpa_pscan_shape* s) {
    PscanParams p{};
    if (fill_params(s, p) != MPA_OK) return 0;
    return (pscan_plan(s).floats * sizeof(float) + 255) / 256 * 256 + 256;
}

extern "C" int mpa_pscan_fwd(const mpa_pscan_shape* s, const void* A, const void* X, void* H,
                             void* workspace, size_t workspace_bytes, void* stream) {
    PscanParams p{};
    int rc = fill_params(s, p);
    if (rc != MPA_OK) return rc;
    if (!A || !X || !H || !workspace) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(A, es) || !aligned_to(X, es) || !aligned_to(H, es) || !aligned_to(workspace, 256))
        return MPA_ERR_MISALIGNED;
    if (workspace_bytes < mpa_pscan_workspace_bytes(s)) return MPA_ERR_WORKSPACE;
    p.A = A; p.X = X; p.out0 = H;
    for (int i = 0; i < 4; ++i) {
        p.a_st[i] = s->a_st[i]; p.x_st[i] = s->x_st[i]; p.o0_st[i] = s->h_st[i];
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const PscanPlan pl = pscan_plan(s);
    if (pl.nchunk > 1) {
        rc = launch_carry_passes<false>(s, p, pl, static_cast<float*>(workspace), st);
        if (rc != MPA_OK) return rc;
    }
    const int64_t dn = (int64_t)p.D * p.N;
    dim3 grid((unsigned)((dn + 255) / 256), (unsigned)(p.batch * p.nchunk));
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL(pscan_fwd_kernel<float>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(pscan_fwd_kernel<bf16_t>, grid, dim3(256), 0, st, p);
    return check_launch();
}

extern "C" int mpa_pscan_bwd(const mpa_pscan_shape* s, const void* A, const void* H,
                             const void* gradH, void* gradA, void* gradX, void* workspace,
                             size_t workspace_bytes, void* stream) {
    PscanParams p{};
    int rc = fill_params(s, p);
    if (rc != MPA_OK) return rc;
    if (!A || !H || !gradH || !gradA || !gradX || !workspace) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(A, es) || !aligned_to(H, es) || !aligned_to(gradH, es) ||
        !aligned_to(gradA, es) || !aligned_to(gradX, es) || !aligned_to(workspace, 256))
        return MPA_ERR_MISALIGNED;
    if (workspace_bytes < mpa_pscan_workspace_bytes(s)) return MPA_ERR_WORKSPACE;
    p.A = A; p.X = gradH; p.H = H; p.out0 = gradX; p.out1 = gradA;
    for (int i = 0; i < 4; ++i) {
        p.a_st[i] = s->a_st[i]; p.x_st[i] = s->x_st[i]; p.h_st[i] = s->h_st[i];
        p.o0_st[i] = s->gx_st[i]; p.o1_st[i] = s->ga_st[i];
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const PscanPlan pl = pscan_plan(s);
    if (pl.nchunk > 1) {
        rc = launch_carry_passes<true>(s, p, pl, static_cast<float*>(workspace), st);
        if (rc != MPA_OK) return rc;
    }
    const int64_t dn = (int64_t)p.D * p.N;
    dim3 grid((unsigned)((dn + 255) / 256), (unsigned)(p.batch * p.nchunk));
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL(pscan_bwd_kernel<float>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(pscan_bwd_kernel<bf16_t>, grid, dim3(256), 0, st, p);
    return check_launch();
}
