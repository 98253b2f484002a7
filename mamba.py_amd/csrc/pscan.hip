// Generic first-order scan H[t] = A[t]*H[t-1] + X[t] over materialised (B, L, D, N) tensors,
// forward and backward, for gfx950.
//
// This path is bound by HBM traffic (12 bytes moved per fp32 element and step, one fma), so
// the kernel is organised around the memory system: one lane owns one (channel, state)
// recurrence, lanes follow the unit-stride axis of the tensors so that every step of a wave
// is one coalesced 256-byte line per operand, and the time loop is unrolled by kUnroll steps
// with all loads of a block issued before its arithmetic, which keeps
// kUnroll * 2 * 256 B per wave in flight.
#include "common.h"

namespace mpa {

constexpr int kUnroll = 8;

struct PscanParams {
    const void* A;
    const void* X;   // fwd: X; bwd: gradH
    const void* H;   // bwd only
    void* out0;      // fwd: H; bwd: gradX
    void* out1;      // bwd: gradA
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

template <typename IO>
__global__ void __launch_bounds__(256) pscan_fwd_kernel(const PscanParams p) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (int64_t)p.D * p.N) return;
    const int b = blockIdx.y;
    int d, n;
    lane_to_dn(p, e, d, n);
    const int64_t step = p.reverse ? -1 : 1;
    const int64_t tfirst = p.reverse ? p.L - 1 : 0;
    int64_t ia = b * p.a_st[0] + tfirst * p.a_st[1] + d * p.a_st[2] + n * p.a_st[3];
    int64_t ix = b * p.x_st[0] + tfirst * p.x_st[1] + d * p.x_st[2] + n * p.x_st[3];
    int64_t io = b * p.o0_st[0] + tfirst * p.o0_st[1] + d * p.o0_st[2] + n * p.o0_st[3];
    const int64_t sa = step * p.a_st[1], sx = step * p.x_st[1], so = step * p.o0_st[1];
    float h = 0.0f;
    int t = 0;
    for (; t + kUnroll <= p.L; t += kUnroll) {
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
    for (; t < p.L; ++t) {
        h = __builtin_fmaf(load_as_float<IO>(p.A, ia), h, load_as_float<IO>(p.X, ix));
        store_from_float<IO>(p.out0, io, h);
        ia += sa;
        ix += sx;
        io += so;
    }
}

// gradX[t] = gradH[t] + A[t+1]*gradX[t+1];  gradA[t] = H[t-1]*gradX[t], gradA[0] = 0.
// With reverse = 1 (the scan ran from the end) the roles of t-1 / t+1 swap.
template <typename IO>
__global__ void __launch_bounds__(256) pscan_bwd_kernel(const PscanParams p) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (int64_t)p.D * p.N) return;
    const int b = blockIdx.y;
    int d, n;
    lane_to_dn(p, e, d, n);
    // walk against the direction of the forward scan
    const int64_t step = p.reverse ? 1 : -1;
    const int64_t tfirst = p.reverse ? 0 : p.L - 1;
    int64_t ia = b * p.a_st[0] + tfirst * p.a_st[1] + d * p.a_st[2] + n * p.a_st[3];
    int64_t ig = b * p.x_st[0] + tfirst * p.x_st[1] + d * p.x_st[2] + n * p.x_st[3];
    int64_t ih = b * p.h_st[0] + tfirst * p.h_st[1] + d * p.h_st[2] + n * p.h_st[3];
    int64_t i0 = b * p.o0_st[0] + tfirst * p.o0_st[1] + d * p.o0_st[2] + n * p.o0_st[3];
    int64_t i1 = b * p.o1_st[0] + tfirst * p.o1_st[1] + d * p.o1_st[2] + n * p.o1_st[3];
    const int64_t sa = step * p.a_st[1], sg = step * p.x_st[1], sh = step * p.h_st[1];
    const int64_t s0 = step * p.o0_st[1], s1 = step * p.o1_st[1];
    // at walk position k: gx = grad + acarry * gx_prev, where acarry = A of the previously
    // visited step; gradA = H(next position in the walk) * gx, zero at the last position
    float gx = 0.0f, acarry = 0.0f;
    int t = 0;
    for (; t + kUnroll < p.L; t += kUnroll) {
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
    for (; t < p.L; ++t) {
        gx = __builtin_fmaf(acarry, gx, load_as_float<IO>(p.X, ig));
        acarry = load_as_float<IO>(p.A, ia);
        const float hprev = (t + 1 < p.L) ? load_as_float<IO>(p.H, ih + sh) : 0.0f;
        store_from_float<IO>(p.out0, i0, gx);
        store_from_float<IO>(p.out1, i1, hprev * gx);
        ia += sa;
        ig += sg;
        ih += sh;
        i0 += s0;
        i1 += s1;
    }
}

static int fill_params(const mpa_pscan_shape* s, PscanParams& p) {
    if (!s) return MPA_ERR_NULL_POINTER;
    if (s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return MPA_ERR_BAD_SHAPE;
    if (s->batch > 65535 || s->seqlen > (int64_t)1 << 30 || s->dim * s->dstate > (int64_t)1 << 31)
        return MPA_ERR_BAD_SHAPE;
    if (s->io_dtype != MPA_F32 && s->io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.D = (int)s->dim; p.N = (int)s->dstate;
    p.reverse = s->reverse ? 1 : 0;
    return MPA_OK;
}

}  // namespace mpa

using namespace mpa;

extern "C" int mpa_pscan_fwd(const mpa_pscan_shape* s, const void* A, const void* X, void* H,
                             void* stream) {
    PscanParams p{};
    int rc = fill_params(s, p);
    if (rc != MPA_OK) return rc;
    if (!A || !X || !H) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(A, es) || !aligned_to(X, es) || !aligned_to(H, es)) return MPA_ERR_MISALIGNED;
    p.A = A; p.X = X; p.out0 = H;
    for (int i = 0; i < 4; ++i) {
        p.a_st[i] = s->a_st[i]; p.x_st[i] = s->x_st[i]; p.o0_st[i] = s->h_st[i];
    }
    const int64_t dn = (int64_t)p.D * p.N;
    dim3 grid((unsigned)((dn + 255) / 256), p.batch);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL(pscan_fwd_kernel<float>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(pscan_fwd_kernel<bf16_t>, grid, dim3(256), 0, st, p);
    return check_launch();
}

extern "C" int mpa_pscan_bwd(const mpa_pscan_shape* s, const void* A, const void* H,
                             const void* gradH, void* gradA, void* gradX, void* stream) {
    PscanParams p{};
    int rc = fill_params(s, p);
    if (rc != MPA_OK) return rc;
    if (!A || !H || !gradH || !gradA || !gradX) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(A, es) || !aligned_to(H, es) || !aligned_to(gradH, es) ||
        !aligned_to(gradA, es) || !aligned_to(gradX, es))
        return MPA_ERR_MISALIGNED;
    p.A = A; p.X = gradH; p.H = H; p.out0 = gradX; p.out1 = gradA;
    for (int i = 0; i < 4; ++i) {
        p.a_st[i] = s->a_st[i]; p.x_st[i] = s->x_st[i]; p.h_st[i] = s->h_st[i];
        p.o0_st[i] = s->gx_st[i]; p.o1_st[i] = s->ga_st[i];
    }
    const int64_t dn = (int64_t)p.D * p.N;
    dim3 grid((unsigned)((dn + 255) / 256), p.batch);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL(pscan_bwd_kernel<float>, grid, dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(pscan_bwd_kernel<bf16_t>, grid, dim3(256), 0, st, p);
    return check_launch();
}
