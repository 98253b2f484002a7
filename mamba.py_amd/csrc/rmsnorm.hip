// RMSNorm for gfx950, forward and backward: y = x * rsqrt(mean(x^2) + eps) * weight
// (mambapy/mamba.py:416-433; no weight under muP).
//
// The reference evaluates this as five elementwise / reduction kernels per call (pow, mean,
// add + rsqrt, two multiplies), each a full pass over the activations.  Here one wave owns a
// row: it reads the row once with 16-byte loads into registers, sums across its lanes with six
// DPP additions (no LDS round trips), and writes the result from the same registers.  The
// kernels are bound by HBM, so they are organised to keep bytes in flight: the forward holds four
// rows per wave at a time (two: 37 us, four: 34 us at 32768 x 768 bfloat16), the backward requests the next row before it works on the current
// one.  Backward: dweight is summed per wave in registers, per block through LDS, and over the
// blocks by a second kernel in a fixed order (no float atomics).
//
// The residual add that precedes every norm of the layer stack (mambapy/mamba.py:106-112:
// output = mixer(norm(x)) + x, then the next layer's norm reads it) can ride along: the forward
// takes a second input, writes the sum (rounded to the I/O type, as the separate add would) and
// normalises it; the backward adds the gradient that reaches the sum from its other users.
#include "common.h"

namespace mpa {

constexpr int kNormBwdWaves = 8;  // waves per block of the backward kernel (one dweight partial per block)

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

// v + (v moved by the DPP control CTRL); rows outside ROW_MASK add zero
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false);
    return v + __builtin_bit_cast(float, moved);
}
// Sum over the 64 lanes, returned wave-uniform.  Four exchanges inside every row of 16 lanes
// (after each, the partners hold the same partial sum, so the mirrors act as lane ^ 4 and
// lane ^ 8), then lane 15 of row 0 / 2 into rows 1 / 3 and lane 31 into rows 2 and 3: lane 63
// holds the total.
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1, 0xf>(v);   // quad_perm:[1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);   // quad_perm:[2,3,0,1]
    v = dpp_add<0x141, 0xf>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xf>(v);  // row_mirror
    v = dpp_add<0x142, 0xa>(v);  // row_bcast:15
    v = dpp_add<0x143, 0xc>(v);  // row_bcast:31
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// rows x d, contiguous rows; d a multiple of the vector width, at most MAXV vectors per lane.
// A wave takes R consecutive rows and holds all of them in registers.  With `res` the row that
// is normalised is round(x + res), also written to `sum_out`.  rstd (rows) is optional.
template <typename IO, int MAXV, int R>
__global__ void __launch_bounds__(256) rmsnorm_fwd_kernel(const IO* __restrict__ x, const IO* __restrict__ res,
                                                          const float* __restrict__ w, IO* __restrict__ y,
                                                          IO* __restrict__ sum_out, float* __restrict__ rstd_out,
                                                          int64_t rows, int d, float eps) {
    typedef RowVec<IO> V;
    typedef typename V::T VT;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row0 = ((int64_t)blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave)) * R;
    if (row0 >= rows) return;
    const int nvec = d / V::kN;
    VT xv[R][MAXV], rv[R][MAXV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t row = row0 + r < rows ? row0 + r : rows - 1;  // a clamped copy is not stored
        const VT* xr = reinterpret_cast<const VT*>(x + row * d);
        const VT* rr = reinterpret_cast<const VT*>(res + row * d);
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                xv[r][v] = xr[i];
                if (res) rv[r][v] = rr[i];
            }
        }
    }
    float wv[MAXV][V::kN];
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int i = lane + v * kWave;
#pragma unroll
        for (int j = 0; j < V::kN; ++j) wv[v][j] = (w && i < nvec) ? w[i * V::kN + j] : 1.0f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (row0 + r >= rows) break;
        const int64_t row = row0 + r;
        VT* yr = reinterpret_cast<VT*>(y + row * d);
        VT* sr = reinterpret_cast<VT*>(sum_out + row * d);
        float f[MAXV][V::kN];
        float ss = 0.0f;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                V::unpack(xv[r][v], f[v]);
                if (res) {
                    float g[V::kN];
                    V::unpack(rv[r][v], g);
#pragma unroll
                    for (int j = 0; j < V::kN; ++j) f[v][j] = to_float(from_float<IO>(f[v][j] + g[j]));
                    sr[i] = V::pack(f[v]);
                }
#pragma unroll
                for (int j = 0; j < V::kN; ++j) ss = __builtin_fmaf(f[v][j], f[v][j], ss);
            }
        }
        const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)d + eps);
        if (rstd_out && lane == 0) rstd_out[row] = rstd;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                float o[V::kN];
#pragma unroll
                for (int j = 0; j < V::kN; ++j) o[j] = f[v][j] * rstd * wv[v][j];
                yr[i] = V::pack(o);
            }
        }
    }
}

// dx = rstd * (w*dy) - x * rstd^3 * mean(w*dy*x) [+ dres];  dweight[c] = sum_rows dy*x*rstd.
// A wave walks `rpw` consecutive rows, requesting row r+1 before it works on row r; its dweight
// sums stay in registers, the kNormBwdWaves waves of a block add theirs through LDS and the
// block writes one row of `part`.  `dres` (optional) is the gradient that reaches the
// normalised row from its other users (the residual stream).  Rows of more than two vectors per
// lane (LEAN) would not fit the register file that way: they are walked without the prefetch
// and read the weight from cache instead of registers.
template <typename IO, int MAXV>
__global__ void __launch_bounds__(kNormBwdWaves* kWave) rmsnorm_bwd_kernel(
    const IO* __restrict__ x, const float* __restrict__ w, const IO* __restrict__ dy, const IO* __restrict__ dres,
    IO* __restrict__ dx, float* __restrict__ part, int64_t rows, int d, float eps, int rpw) {
    typedef RowVec<IO> V;
    typedef typename V::T VT;
    extern __shared__ float sacc[];  // [kNormBwdWaves][d]
    const int lane = threadIdx.x & (kWave - 1);
    const int wib = wave_id();
    const int64_t row_begin = ((int64_t)blockIdx.x * kNormBwdWaves + wib) * rpw;
    const int64_t row_end = row_begin + rpw < rows ? row_begin + rpw : rows;
    const int nvec = d / V::kN;
    constexpr bool LEAN = MAXV > 2;
    float wv[LEAN ? 1 : MAXV][V::kN], dwacc[MAXV][V::kN];
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int i = lane + v * kWave;
#pragma unroll
        for (int j = 0; j < V::kN; ++j) {
            if (!LEAN) wv[v][j] = (w && i < nvec) ? w[i * V::kN + j] : 1.0f;
            dwacc[v][j] = 0.0f;
        }
    }
    auto weights = [&](int v, int i, float (&wj)[V::kN]) {
#pragma unroll
        for (int j = 0; j < V::kN; ++j) wj[j] = LEAN ? (w ? w[i * V::kN + j] : 1.0f) : wv[LEAN ? 0 : v][j];
    };
    struct Raw {
        VT x[MAXV], g[MAXV], q[MAXV];
    };
    auto load_row = [&](int64_t row, Raw& raw) {
        const VT* xr = reinterpret_cast<const VT*>(x + row * d);
        const VT* gr = reinterpret_cast<const VT*>(dy + row * d);
        const VT* qr = reinterpret_cast<const VT*>(dres + row * d);
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                raw.x[v] = xr[i];
                raw.g[v] = gr[i];
                if (dres) raw.q[v] = qr[i];
            }
        }
    };
    Raw cur, nxt;
    if (row_begin < row_end) load_row(row_begin, cur);
    for (int64_t row = row_begin; row < row_end; ++row) {
        if (!LEAN && row + 1 < row_end) load_row(row + 1, nxt);
        VT* dr = reinterpret_cast<VT*>(dx + row * d);
        float ss = 0.0f, sg = 0.0f;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                float f[V::kN], g[V::kN], wj[V::kN];
                V::unpack(cur.x[v], f);
                V::unpack(cur.g[v], g);
                weights(v, i, wj);
#pragma unroll
                for (int j = 0; j < V::kN; ++j) {
                    ss = __builtin_fmaf(f[j], f[j], ss);
                    sg = __builtin_fmaf(g[j] * wj[j], f[j], sg);
                }
            }
        }
        const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)d + eps);
        const float c = wave_sum(sg) / (float)d * rstd * rstd * rstd;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int i = lane + v * kWave;
            if (i < nvec) {
                float f[V::kN], g[V::kN], wj[V::kN], o[V::kN];
                V::unpack(cur.x[v], f);
                V::unpack(cur.g[v], g);
                weights(v, i, wj);
#pragma unroll
                for (int j = 0; j < V::kN; ++j) {
                    o[j] = __builtin_fmaf(g[j] * wj[j], rstd, -f[j] * c);
                    dwacc[v][j] = __builtin_fmaf(g[j] * rstd, f[j], dwacc[v][j]);
                }
                if (dres) {
                    float q[V::kN];
                    V::unpack(cur.q[v], q);
#pragma unroll
                    for (int j = 0; j < V::kN; ++j) o[j] += q[j];
                }
                dr[i] = V::pack(o);
            }
        }
        if (LEAN) {
            if (row + 1 < row_end) load_row(row + 1, cur);
        } else {
            cur = nxt;
        }
    }
    if (!part) return;  // uniform over the grid
    float* mine = sacc + wib * d;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int i = lane + v * kWave;
        if (i < nvec)
#pragma unroll
            for (int j = 0; j < V::kN; ++j) mine[i * V::kN + j] = dwacc[v][j];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < d; c += kNormBwdWaves * kWave) {
        float s = sacc[c];
#pragma unroll
        for (int k = 1; k < kNormBwdWaves; ++k) s += sacc[k * d + c];
        part[(int64_t)blockIdx.x * d + c] = s;
    }
}

// dweight[c] = sum over the per-block partial rows, fixed order (32 columns x 32 row groups per block)
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
    if (rows <= 0 || d <= 0 || rows > (int64_t)1 << 31) return MPA_ERR_BAD_SHAPE;  // one wave per one or two rows
    if (io_dtype != MPA_F32 && io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    const int vec = io_dtype == MPA_BF16 ? 8 : 4;
    if (d % vec != 0 || d / vec > 8 * kWave) return MPA_ERR_BAD_SHAPE;  // d <= 4096 (bf16) / 2048 (f32)
    return MPA_OK;
}

// vectors per lane, rounded up to a power of two: 1, 2, 4, 8
static int norm_maxv(int64_t d, int io_dtype) {
    const int vec = io_dtype == MPA_BF16 ? 8 : 4;
    const int nv = (int)((d / vec + kWave - 1) / kWave);
    return nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : 8;
}

// Backward launch: rows per wave chosen for about 4096 waves (16 per CU) when the problem has
// that many rows, at most 16 rows per wave; one dweight partial per block.
struct NormBwdPlan {
    int rpw;
    int64_t blocks;
};
static NormBwdPlan norm_bwd_plan(int64_t rows) {
    int64_t rpw = rows / 4096;
    rpw = rpw < 1 ? 1 : rpw > 16 ? 16 : rpw;
    const int64_t waves = (rows + rpw - 1) / rpw;
    return NormBwdPlan{(int)rpw, (waves + kNormBwdWaves - 1) / kNormBwdWaves};
}

template <typename IO, int MAXV>
static int launch_norm_fwd(const void* x, const void* res, const float* w, void* y, void* sum_out, float* rstd,
                           int64_t rows, int d, float eps, hipStream_t st) {
    constexpr int R = MAXV <= 2 ? 4 : 1;
    const int64_t waves = (rows + R - 1) / R;
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<IO, MAXV, R>), dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, st,
                       static_cast<const IO*>(x), static_cast<const IO*>(res), w, static_cast<IO*>(y),
                       static_cast<IO*>(sum_out), rstd, rows, d, eps);
    return check_launch();
}

template <typename IO, int MAXV>
static int launch_norm_bwd(const void* x, const float* w, const void* dy, const void* dsum, void* dx, float* part,
                           int64_t rows, int d, float eps, hipStream_t st) {
    const NormBwdPlan plan = norm_bwd_plan(rows);
    const size_t lds = part ? (size_t)kNormBwdWaves * d * sizeof(float) : 0;
    // the widest rows of this instantiation need more than the 64 KB a kernel gets by default
    static LdsLimitOnce lds_limit;
    const int attr_rc = lds_limit.ensure(rmsnorm_bwd_kernel<IO, MAXV>,
                                                 (size_t)kNormBwdWaves * MAXV * kWave * RowVec<IO>::kN * sizeof(float));
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<IO, MAXV>), dim3((unsigned)plan.blocks), dim3(kNormBwdWaves * kWave), lds,
                       st, static_cast<const IO*>(x), w, static_cast<const IO*>(dy), static_cast<const IO*>(dsum),
                       static_cast<IO*>(dx), part, rows, d, eps, plan.rpw);
    return check_launch();
}

}  // namespace mpa

using namespace mpa;

#define MPA_NORM_DISPATCH(FN, ...)                                                     \
    (io_dtype == MPA_F32                                                               \
         ? (maxv == 1   ? FN<float, 1>(__VA_ARGS__)                                    \
            : maxv == 2 ? FN<float, 2>(__VA_ARGS__)                                    \
            : maxv == 4 ? FN<float, 4>(__VA_ARGS__)                                    \
                        : FN<float, 8>(__VA_ARGS__))                                   \
         : (maxv == 1   ? FN<bf16_t, 1>(__VA_ARGS__)                                   \
            : maxv == 2 ? FN<bf16_t, 2>(__VA_ARGS__)                                   \
            : maxv == 4 ? FN<bf16_t, 4>(__VA_ARGS__)                                   \
                        : FN<bf16_t, 8>(__VA_ARGS__)))

extern "C" int mpa_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* y, void* sum_out,
                               float* rstd, int64_t rows, int64_t d, float eps, int32_t io_dtype, void* stream) {
    int rc = norm_validate(rows, d, io_dtype);
    if (rc != MPA_OK) return rc;
    if (!x || !y || (residual && !sum_out)) return MPA_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || (weight && !aligned_to(weight, 4)) ||
        (residual && (!aligned_to(residual, 16) || !aligned_to(sum_out, 16))))
        return MPA_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int maxv = norm_maxv(d, io_dtype);
    return MPA_NORM_DISPATCH(launch_norm_fwd, x, residual, weight, y, sum_out, rstd, rows, (int)d, eps, st);
}

extern "C" size_t mpa_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t d) {
    if (rows <= 0 || d <= 0) return 0;
    return ((size_t)norm_bwd_plan(rows).blocks * d * sizeof(float) + 255) / 256 * 256;
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
    float* part = weight ? static_cast<float*>(workspace) : nullptr;
    const int maxv = norm_maxv(d, io_dtype);
    rc = MPA_NORM_DISPATCH(launch_norm_bwd, x, weight, dy, dsum, dx, part, rows, (int)d, eps, st);
    if (rc != MPA_OK || !weight) return rc;
    hipLaunchKernelGGL(rmsnorm_bwd_finish_kernel, dim3((unsigned)((d + kNormFinCols - 1) / kNormFinCols)),
                       dim3(1024), 0, st, part, dweight, (int)d, norm_bwd_plan(rows).blocks);
    return check_launch();
}
