// RMSNorm for gfx950, forward and backward: y = x * rsqrt(mean(x^2) + eps) * weight
// (mambapy/mamba.py:416-433; no weight under muP).
//
// The reference evaluates this as five elementwise / reduction kernels per call (pow, mean,
// add + rsqrt, two multiplies), each a full pass over the activations.  Here one wave owns one
// row: it reads the row with 16-byte loads, sums the squares across its lanes with lane
// exchanges, and writes the scaled row; the second read of the row comes from cache.  The
// kernels are bound by HBM: forward x in, y out; backward x, dy in, dx out, plus per-block
// partial sums of dweight that a second kernel adds up in a fixed order.
//
// The residual add that precedes every norm of the layer stack (mambapy/mamba.py:106-112:
// output = mixer(norm(x)) + x, then the next layer's norm reads it) can ride along: the forward
// takes a second input, writes the sum (rounded to the I/O type, as the separate add would) and
// normalises it; the backward adds the gradient that reaches the sum from its other users.
#include "common.h"

namespace mpa {

constexpr int kNormRowsPerWave = 16;  // backward: rows walked by one wave (dweight partials per wave)

template <typename IO>
struct RowVec;
template <>
struct RowVec<float> {
    static constexpr int kN = 4;
    typedef float4 T;
    static __device__ __forceinline__ void unpack(const T& v, float (&f)[4]) { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
    static __device__ __forceinline__ T pack(const float (&f)[4]) { return make_float4(f[0], f[1], f[2], f[3]); }
};
template <>
struct RowVec<bf16_t> {
    static constexpr int kN = 8;
    typedef uint4 T;
    static __device__ __forceinline__ void unpack(const T& v, float (&f)[8]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ T pack(const float (&f)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = from_float<bf16_t>(f[2 * i]).bits, hi = from_float<bf16_t>(f[2 * i + 1]).bits;
            w[i] = lo | (hi << 16);
        }
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    return v;
}

// rows x d, contiguous rows; d a multiple of the vector width.  rstd (rows) is optional.
// With `res`: the row that is normalised is round(x + res), also written to `sum_out`.
template <typename IO>
__global__ void __launch_bounds__(256) rmsnorm_fwd_kernel(const IO* __restrict__ x, const IO* __restrict__ res,
                                                          const float* __restrict__ w, IO* __restrict__ y,
                                                          IO* __restrict__ sum_out, float* __restrict__ rstd_out,
                                                          int64_t rows, int d, float eps) {
    typedef RowVec<IO> V;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
    if (row >= rows) return;
    const int nvec = d / V::kN;
    const typename V::T* xr = reinterpret_cast<const typename V::T*>(x + row * d);
    typename V::T* yr = reinterpret_cast<typename V::T*>(y + row * d);
    const typename V::T* rr = reinterpret_cast<const typename V::T*>(res + row * d);
    typename V::T* sr = reinterpret_cast<typename V::T*>(sum_out + row * d);
    auto load_row = [&](int i, float (&f)[V::kN]) {
        V::unpack(xr[i], f);
        if (res) {
            float g[V::kN];
            V::unpack(rr[i], g);
#pragma unroll
            for (int j = 0; j < V::kN; ++j) f[j] = to_float(from_float<IO>(f[j] + g[j]));
        }
    };
    float ss = 0.0f;
    for (int i = lane; i < nvec; i += kWave) {
        float f[V::kN];
        load_row(i, f);
        if (res) sr[i] = V::pack(f);
#pragma unroll
        for (int j = 0; j < V::kN; ++j) ss = __builtin_fmaf(f[j], f[j], ss);
    }
    const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)d + eps);
    if (rstd_out && lane == 0) rstd_out[row] = rstd;
    for (int i = lane; i < nvec; i += kWave) {
        float f[V::kN], o[V::kN];
        load_row(i, f);
#pragma unroll
        for (int j = 0; j < V::kN; ++j) o[j] = f[j] * rstd * (w ? w[i * V::kN + j] : 1.0f);
        yr[i] = V::pack(o);
    }
}

// dx = rstd * (w*dy) - x * rstd^3 * mean(w*dy*x);  dweight[c] = sum_rows dy*x*rstd.
// A wave walks kNormRowsPerWave rows and writes its dweight sums as one row of `part`.
// `dres` (optional) is added to dx: the gradient that reaches the normalised row from its
// other users (the residual stream).
template <typename IO, int MAXV>
__global__ void __launch_bounds__(256) rmsnorm_bwd_kernel(const IO* __restrict__ x, const float* __restrict__ w,
                                                          const IO* __restrict__ dy, const IO* __restrict__ dres,
                                                          IO* __restrict__ dx, float* __restrict__ part,
                                                          int64_t rows, int d, float eps) {
    typedef RowVec<IO> V;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
    const int nvec = d / V::kN;
    float dwacc[MAXV][V::kN];
#pragma unroll
    for (int v = 0; v < MAXV; ++v)
#pragma unroll
        for (int j = 0; j < V::kN; ++j) dwacc[v][j] = 0.0f;
    for (int r = 0; r < kNormRowsPerWave; ++r) {
        const int64_t row = wave * kNormRowsPerWave + r;
        if (row >= rows) break;
        const typename V::T* xr = reinterpret_cast<const typename V::T*>(x + row * d);
        const typename V::T* gr = reinterpret_cast<const typename V::T*>(dy + row * d);
        typename V::T* dr = reinterpret_cast<typename V::T*>(dx + row * d);
        const typename V::T* qr = reinterpret_cast<const typename V::T*>(dres + row * d);
        float ss = 0.0f, sg = 0.0f;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                float f[V::kN], g[V::kN];
                V::unpack(xr[i], f);
                V::unpack(gr[i], g);
#pragma unroll
                for (int j = 0; j < V::kN; ++j) {
                    ss = __builtin_fmaf(f[j], f[j], ss);
                    sg = __builtin_fmaf(g[j] * (w ? w[i * V::kN + j] : 1.0f), f[j], sg);
                }
            }
        }
        const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)d + eps);
        const float c = wave_sum(sg) / (float)d * rstd * rstd * rstd;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                float f[V::kN], g[V::kN], o[V::kN];
                V::unpack(xr[i], f);
                V::unpack(gr[i], g);
#pragma unroll
                for (int j = 0; j < V::kN; ++j) {
                    o[j] = __builtin_fmaf(g[j] * (w ? w[i * V::kN + j] : 1.0f), rstd, -f[j] * c);
                    dwacc[v][j] = __builtin_fmaf(g[j] * rstd, f[j], dwacc[v][j]);
                }
                if (dres) {
                    float q[V::kN];
                    V::unpack(qr[i], q);
#pragma unroll
                    for (int j = 0; j < V::kN; ++j) o[j] += q[j];
                }
                dr[i] = V::pack(o);
            }
        }
    }
    if (part) {
        float* pr = part + wave * d;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec)
#pragma unroll
                for (int j = 0; j < V::kN; ++j) pr[i * V::kN + j] = dwacc[v][j];
        }
    }
}

// dweight[c] = sum over the per-wave partial rows, fixed order (32 columns x 32 row groups per block)
constexpr int kNormFinCols = 32, kNormFinRows = 32;
__global__ void __launch_bounds__(1024) rmsnorm_bwd_finish_kernel(const float* part, float* dweight, int d,
                                                                  int64_t nparts) {
    __shared__ float acc[kNormFinRows][kNormFinCols + 1];
    const int col = threadIdx.x % kNormFinCols, rg = threadIdx.x / kNormFinCols;
    const int c = blockIdx.x * kNormFinCols + col;
    float s = 0.0f;
    if (c < d)
        for (int64_t q = rg; q < nparts; q += kNormFinRows) s += part[q * d + c];
    acc[rg][col] = s;
    __syncthreads();
    if (rg != 0 || c >= d) return;
    for (int r = 1; r < kNormFinRows; ++r) s += acc[r][col];
    dweight[c] = s;
}

static int norm_validate(int64_t rows, int64_t d, int io_dtype) {
    if (rows <= 0 || d <= 0 || rows > (int64_t)1 << 40) return MPA_ERR_BAD_SHAPE;
    if (io_dtype != MPA_F32 && io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    const int vec = io_dtype == MPA_BF16 ? 8 : 4;
    if (d % vec != 0 || d / vec > 8 * kWave) return MPA_ERR_BAD_SHAPE;  // d <= 4096 (bf16) / 2048 (f32)
    return MPA_OK;
}

static int64_t norm_waves(int64_t rows) { return (rows + kNormRowsPerWave - 1) / kNormRowsPerWave; }

}  // namespace mpa

using namespace mpa;

extern "C" int mpa_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* y, void* sum_out,
                               float* rstd, int64_t rows, int64_t d, float eps, int32_t io_dtype, void* stream) {
    int rc = norm_validate(rows, d, io_dtype);
    if (rc != MPA_OK) return rc;
    if (!x || !y || (residual && !sum_out)) return MPA_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || (weight && !aligned_to(weight, 4)) ||
        (residual && (!aligned_to(residual, 16) || !aligned_to(sum_out, 16))))
        return MPA_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (io_dtype == MPA_F32)
        hipLaunchKernelGGL(rmsnorm_fwd_kernel<float>, grid, block, 0, st, static_cast<const float*>(x),
                           static_cast<const float*>(residual), weight, static_cast<float*>(y),
                           static_cast<float*>(sum_out), rstd, rows, (int)d, eps);
    else
        hipLaunchKernelGGL(rmsnorm_fwd_kernel<bf16_t>, grid, block, 0, st, static_cast<const bf16_t*>(x),
                           static_cast<const bf16_t*>(residual), weight, static_cast<bf16_t*>(y),
                           static_cast<bf16_t*>(sum_out), rstd, rows, (int)d, eps);
    return check_launch();
}

extern "C" size_t mpa_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t d) {
    if (rows <= 0 || d <= 0) return 0;
    const int64_t waves = (norm_waves(rows) + 3) / 4 * 4;
    return ((size_t)waves * d * sizeof(float) + 255) / 256 * 256;
}

extern "C" int mpa_rmsnorm_bwd(const void* x, const float* weight, const void* dy, const void* dsum, void* dx,
                               float* dweight, int64_t rows, int64_t d, float eps, int32_t io_dtype,
                               void* workspace, size_t workspace_bytes, void* stream) {
    int rc = norm_validate(rows, d, io_dtype);
    if (rc != MPA_OK) return rc;
    if (!x || !dy || !dx) return MPA_ERR_NULL_POINTER;
    if (weight && (!dweight || !workspace)) return MPA_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(dy, 16) || !aligned_to(dx, 16) || (weight && !aligned_to(weight, 4)) ||
        (dsum && !aligned_to(dsum, 16)) ||
        (workspace && !aligned_to(workspace, 256)))
        return MPA_ERR_MISALIGNED;
    if (weight && workspace_bytes < mpa_rmsnorm_bwd_workspace_bytes(rows, d)) return MPA_ERR_WORKSPACE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t waves = norm_waves(rows);
    dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    float* part = weight ? static_cast<float*>(workspace) : nullptr;
    const int vec = io_dtype == MPA_BF16 ? 8 : 4;
    const int nv = (int)((d / vec + kWave - 1) / kWave);  // vectors per lane: 1..8
#define MPA_NORM_CASE(IO_, MV_)                                                                               \
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<IO_, MV_>), grid, block, 0, st, static_cast<const IO_*>(x), weight, \
                       static_cast<const IO_*>(dy), static_cast<const IO_*>(dsum), static_cast<IO_*>(dx), part, \
                       rows, (int)d, eps)
    if (io_dtype == MPA_F32) {
        if (nv <= 1) MPA_NORM_CASE(float, 1);
        else if (nv <= 2) MPA_NORM_CASE(float, 2);
        else if (nv <= 4) MPA_NORM_CASE(float, 4);
        else MPA_NORM_CASE(float, 8);
    } else {
        if (nv <= 1) MPA_NORM_CASE(bf16_t, 1);
        else if (nv <= 2) MPA_NORM_CASE(bf16_t, 2);
        else if (nv <= 4) MPA_NORM_CASE(bf16_t, 4);
        else MPA_NORM_CASE(bf16_t, 8);
    }
#undef MPA_NORM_CASE
    rc = check_launch();
    if (rc != MPA_OK || !weight) return rc;
    // rows of the partial buffer beyond the last wave of a partially filled block were written
    // by waves that own no row (all zeros), so every one of the grid's waves counts
    hipLaunchKernelGGL(rmsnorm_bwd_finish_kernel, dim3((unsigned)((d + kNormFinCols - 1) / kNormFinCols)), dim3(1024), 0, st, part, dweight,
                       (int)d, (int64_t)grid.x * 4);
    return check_launch();
}
