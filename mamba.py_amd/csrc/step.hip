// Single-token decode step for gfx950: h' = exp(delta*A)*h + delta*B*x ; y = C.h' + D*x.
//
// The step moves the whole recurrent state once (read + write, float32) and does a handful
// of flops per element, so it is bound by HBM traffic and, at decode batch sizes, by launch
// latency.  One lane owns one (batch, channel) row: it streams the row's d_state values of h
// and A as 16-byte vectors (a wave touches 64 consecutive rows = one contiguous 4 KB block
// of h), keeps the readout sum in a register and writes h' back in place or to a second
// buffer.  softplus(delta + bias) and the output gate y*silu(z) are folded in so that the
// caller needs no extra elementwise launches around the step.
#include "common.h"

namespace mpa {

struct StepParams {
    const void* x;
    const void* delta;
    const void* Bm;
    const void* C;
    const void* z;
    const float* A;
    const float* D;
    const float* dbias;
    const float* hin;
    float* hout;
    void* y;
    int batch, ED, N;
    int64_t bc_stride;
    int64_t z_stride;  // row stride of z (elements)
    int softplus;
};

template <typename IO, int VEC>
__global__ void __launch_bounds__(256) ssm_step_kernel(const StepParams p) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // b*ED + d
    if (row >= (int64_t)p.batch * p.ED) return;
    const int b = (int)(row / p.ED);
    const int d = (int)(row % p.ED);
    const float xv = load_as_float<IO>(p.x, row);
    float dv = load_as_float<IO>(p.delta, row);
    if (p.softplus) dv = softplus_f(dv + (p.dbias ? p.dbias[d] : 0.0f));
    const float dl2 = dv * kLog2e;
    const float u = dv * xv;
    const float* Arow = p.A + (int64_t)d * p.N;
    const float* hin = p.hin ? p.hin + row * p.N : nullptr;
    float* hout = p.hout + row * p.N;
    const int64_t bc = (int64_t)b * p.bc_stride;
    float acc = 0.0f;
    if (VEC == 4) {
        for (int n = 0; n < p.N; n += 4) {
            const float4 a4 = *reinterpret_cast<const float4*>(Arow + n);
            float4 h4 = hin ? *reinterpret_cast<const float4*>(hin + n) : make_float4(0, 0, 0, 0);
            const float av[4] = {a4.x, a4.y, a4.z, a4.w};
            float hv[4] = {h4.x, h4.y, h4.z, h4.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float bv = load_as_float<IO>(p.Bm, bc + n + k);
                const float cv = load_as_float<IO>(p.C, bc + n + k);
                hv[k] = __builtin_fmaf(u, bv, fast_exp2(dl2 * av[k]) * hv[k]);
                acc = __builtin_fmaf(cv, hv[k], acc);
            }
            *reinterpret_cast<float4*>(hout + n) = make_float4(hv[0], hv[1], hv[2], hv[3]);
        }
    } else {
        for (int n = 0; n < p.N; ++n) {
            const float bv = load_as_float<IO>(p.Bm, bc + n);
            const float cv = load_as_float<IO>(p.C, bc + n);
            const float hv =
                __builtin_fmaf(u, bv, fast_exp2(dl2 * Arow[n]) * (hin ? hin[n] : 0.0f));
            hout[n] = hv;
            acc = __builtin_fmaf(cv, hv, acc);
        }
    }
    float yv = __builtin_fmaf(p.D[d], xv, acc);
    if (p.z) {
        const float zv = load_as_float<IO>(p.z, b * p.z_stride + d);
        yv *= zv * sigmoid_f(zv);
    }
    store_from_float<IO>(p.y, row, yv);
}

// Variant for d_state = 4*Q with Q a power of two: Q lanes share one row, four states each.
// A wave then reads and writes h as one contiguous, fully used block per instruction (the
// one-lane-per-row kernel touches every cache line of a 4 KB block with each of its loads),
// all of a lane's loads are issued before the first use, and four times as many waves are in
// flight, which is what a kernel this short needs.  The readout is summed over the Q lanes of
// a row with lane exchanges.
template <typename IO, int Q>
__global__ void __launch_bounds__(256) ssm_step_quad_kernel(const StepParams p) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t row = gid / Q;  // b*ED + d
    const int part = (int)(gid % Q);
    if (row >= (int64_t)p.batch * p.ED) return;  // Q divides 64: a row's lanes leave together
    const int b = (int)(row / p.ED);
    const int d = (int)(row % p.ED);
    const int n0 = 4 * part;
    const float4 h4 = p.hin ? *reinterpret_cast<const float4*>(p.hin + row * p.N + n0) : make_float4(0, 0, 0, 0);
    const float4 a4 = *reinterpret_cast<const float4*>(p.A + (int64_t)d * p.N + n0);
    const int64_t bc = (int64_t)b * p.bc_stride + n0;
    float bv[4], cv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        bv[k] = load_as_float<IO>(p.Bm, bc + k);
        cv[k] = load_as_float<IO>(p.C, bc + k);
    }
    const float xv = load_as_float<IO>(p.x, row);
    float dv = load_as_float<IO>(p.delta, row);
    const float zv = p.z ? load_as_float<IO>(p.z, b * p.z_stride + d) : 0.0f;
    const float Dv = p.D[d];
    if (p.softplus) dv = softplus_f(dv + (p.dbias ? p.dbias[d] : 0.0f));
    const float dl2 = dv * kLog2e;
    const float u = dv * xv;
    const float av[4] = {a4.x, a4.y, a4.z, a4.w};
    float hv[4] = {h4.x, h4.y, h4.z, h4.w};
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        hv[k] = __builtin_fmaf(u, bv[k], fast_exp2(dl2 * av[k]) * hv[k]);
        acc = __builtin_fmaf(cv[k], hv[k], acc);
    }
    *reinterpret_cast<float4*>(p.hout + row * p.N + n0) = make_float4(hv[0], hv[1], hv[2], hv[3]);
#pragma unroll
    for (int m = 1; m < Q; m *= 2) acc += __shfl_xor(acc, m);
    if (part == 0) {
        float yv = __builtin_fmaf(Dv, xv, acc);
        if (p.z) yv *= zv * sigmoid_f(zv);
        store_from_float<IO>(p.y, row, yv);
    }
}

template <typename IO>
static bool launch_step_quad(const StepParams& p, int q, hipStream_t st) {
    const int64_t threads = (int64_t)p.batch * p.ED * q;
    dim3 grid((unsigned)((threads + 255) / 256));
#define MPA_Q(Q_) \
    if (q == Q_) { hipLaunchKernelGGL((ssm_step_quad_kernel<IO, Q_>), grid, dim3(256), 0, st, p); return true; }
    MPA_Q(1) MPA_Q(2) MPA_Q(4) MPA_Q(8) MPA_Q(16)
#undef MPA_Q
    return false;
}

}  // namespace mpa

using namespace mpa;

extern "C" int mpa_ssm_step(const void* x, const void* delta, const float* A, const void* B,
                            const void* C, const float* D, const void* z, const float* delta_bias,
                            const float* h_in, float* h_out, void* y, int64_t batch, int64_t dim,
                            int64_t dstate, int64_t bc_stride, int64_t z_stride, int32_t io_dtype,
                            int32_t delta_softplus, void* stream) {
    if (!x || !delta || !A || !B || !C || !D || !h_out || !y) return MPA_ERR_NULL_POINTER;
    if (batch <= 0 || dim <= 0 || dstate <= 0 || batch * dim > (int64_t)1 << 40)
        return MPA_ERR_BAD_SHAPE;
    if (io_dtype != MPA_F32 && io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    if (bc_stride < dstate || (z && z_stride < dim)) return MPA_ERR_BAD_STRIDE;
    if (!delta_softplus && delta_bias) return MPA_ERR_BAD_SHAPE;
    const size_t es = dtype_size(io_dtype);
    if (!aligned_to(x, es) || !aligned_to(delta, es) || !aligned_to(B, es) || !aligned_to(C, es) ||
        !aligned_to(y, es) || (z && !aligned_to(z, es)))
        return MPA_ERR_MISALIGNED;
    const bool vec4 = dstate % 4 == 0 && aligned_to(A, 16) && aligned_to(h_out, 16) &&
                      (!h_in || aligned_to(h_in, 16));
    if (!aligned_to(A, 4) || !aligned_to(h_out, 4) || (h_in && !aligned_to(h_in, 4)))
        return MPA_ERR_MISALIGNED;
    StepParams p{};
    p.x = x; p.delta = delta; p.Bm = B; p.C = C; p.z = z; p.A = A; p.D = D; p.dbias = delta_bias;
    p.hin = h_in; p.hout = h_out; p.y = y;
    p.batch = (int)batch; p.ED = (int)dim; p.N = (int)dstate; p.bc_stride = bc_stride;
    p.z_stride = z_stride;
    p.softplus = delta_softplus ? 1 : 0;
    const int64_t rows = batch * dim;
    dim3 grid((unsigned)((rows + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    // d_state = 4*Q, Q a power of two up to 16: the lanes-per-row kernel
    const int q = (int)(dstate / 4);
    if (vec4 && q >= 1 && q <= 16 && (q & (q - 1)) == 0 && rows * q < ((int64_t)1 << 31) * 256) {
        const bool ok = io_dtype == MPA_F32 ? launch_step_quad<float>(p, q, st) : launch_step_quad<bf16_t>(p, q, st);
        if (ok) return check_launch();
    }
    if (io_dtype == MPA_F32) {
        if (vec4) hipLaunchKernelGGL((ssm_step_kernel<float, 4>), grid, dim3(256), 0, st, p);
        else hipLaunchKernelGGL((ssm_step_kernel<float, 1>), grid, dim3(256), 0, st, p);
    } else {
        if (vec4) hipLaunchKernelGGL((ssm_step_kernel<bf16_t, 4>), grid, dim3(256), 0, st, p);
        else hipLaunchKernelGGL((ssm_step_kernel<bf16_t, 1>), grid, dim3(256), 0, st, p);
    }
    return check_launch();
}

extern "C" int mpa_version(void) { return MPA_VERSION; }
extern "C" const char* mpa_arch(void) { return "gfx950"; }
#ifndef MPA_SOURCE_SHA
#define MPA_SOURCE_SHA "unknown"
#endif
extern "C" const char* mpa_source_hash(void) { return MPA_SOURCE_SHA; }
extern "C" const char* mpa_status_string(int status) {
    switch (status) {
        case MPA_OK: return "ok";
        case MPA_ERR_NULL_POINTER: return "a required pointer is NULL";
        case MPA_ERR_BAD_SHAPE: return "unsupported or inconsistent shape / flags";
        case MPA_ERR_BAD_DTYPE: return "unsupported io_dtype";
        case MPA_ERR_BAD_STRIDE: return "unsupported stride";
        case MPA_ERR_MISALIGNED: return "misaligned pointer";
        case MPA_ERR_WORKSPACE: return "workspace too small";
        case MPA_ERR_LAUNCH: return "kernel launch failed";
        default: return "unknown status";
    }
}
