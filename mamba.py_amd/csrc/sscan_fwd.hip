// Fused selective-scan forward for gfx950: discretise -> scan -> readout in one pass.
//
// Work decomposition.  The recurrence h[t] = a[t]*h[t-1] + bx[t] is serial in t and
// independent per (batch, channel, state).  A workgroup owns 64 channels of one batch row;
// its NW waves split the d_state axis: wave w keeps NS states (n = w*NS .. w*NS+NS-1) of the
// 64 channels in registers, one channel per lane, and walks the sequence in time order.
// Per state and step the VALU work is one multiply for the exponent, one v_exp_f32, one
// multiply a*h, one fma for +u*B and one fma for the readout; nothing else scales with N.
//
// Per tile of kTile steps:
//   A. the whole workgroup converts the (kTile x 64) slices of delta and x to float32 in LDS
//      (delta, u = delta*x, x), and the (kTile x N) slices of B and C; the global loads of
//      the NEXT tile are issued before the arithmetic of this one (register prefetch);
//   B. every wave runs its NS recurrences and writes a partial readout sum_n C*h to LDS;
//   C. the workgroup sums the NW partials, adds D*x, applies the optional gate and stores y.
// Both channel-contiguous and time-contiguous (B,ED,L memory) operands are read and written
// coalesced: the thread -> (step, channel) map of phases A and C follows the unit stride.
#include "common.h"

namespace mpa {

struct FwdParams {
    const void* x;
    const void* delta;
    const void* Bm;
    const void* C;
    const void* z;
    const float* A;
    const float* D;
    const float* dbias;
    const float* h0;
    void* y;
    float* ckpt;
    float* hlast;
    int batch, L, ED, N, nchunks;
    int softplus;
    int in_tmajor;   // x / delta have unit stride along time
    int out_tmajor;  // y has unit stride along time
    int64_t u_sb, u_sl, u_sd;
    int64_t d_sb, d_sl, d_sd;
    int64_t y_sb, y_sl, y_sd;
    int64_t bc_sb, bc_sl;
};

constexpr int kPitch = kWave + 1;  // LDS row pitch (floats): conflict-free for both maps

template <typename IO, int NS, int NW>
__global__ void __launch_bounds__(NW* kWave) sscan_fwd_kernel(const FwdParams p) {
    constexpr int NT = NW * kWave;
    constexpr int NP = NS * NW;                    // padded state count
    constexpr int EPT = (kTile * kWave + NT - 1) / NT;  // (step, channel) elements per thread
    constexpr int BPT = (kTile * NP + NT - 1) / NT;     // B/C elements per thread

    extern __shared__ float smem[];
    typedef float Tile[kTile][kPitch];
    typedef float TileN[kTile][NP];
    Tile* sDelta = reinterpret_cast<Tile*>(smem);                 // [2]
    Tile* sU = sDelta + 2;                                        // [2]
    Tile* sX = sU + 2;                                            // [2]
    Tile* sY = sX + 2;                                            // [NW]
    TileN* sB = reinterpret_cast<TileN*>(sY + NW);                // [2]
    TileN* sC = sB + 2;                                           // [2]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = wave_id();
    const int b = blockIdx.y;
    const int d0 = blockIdx.x * kWave;
    const int d = d0 + lane;
    const bool dvalid = d < p.ED;

    float A2[NS], h[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = w * NS + i;
        const bool ok = dvalid && n < p.N;
        A2[i] = ok ? p.A[(int64_t)d * p.N + n] * kLog2e : 0.0f;
        h[i] = (ok && p.h0) ? p.h0[((int64_t)b * p.ED + d) * p.N + n] : 0.0f;
    }

    // register staging of the next tile
    float rX[EPT], rDl[EPT], rB[BPT], rC[BPT];

    auto elem_map = [&](int idx, bool tmajor, int& tt, int& cc) {
        if (tmajor) {
            tt = idx % kTile;
            cc = idx / kTile;
        } else {
            tt = idx / kWave;
            cc = idx % kWave;
        }
    };

    auto prefetch = [&](int t0) {
        const int tl = min(kTile, p.L - t0);
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
            const int idx = tid + k * NT;
            int tt, cc;
            elem_map(idx, p.in_tmajor, tt, cc);
            float xv = 0.0f, dv = 0.0f;
            if (idx < kTile * kWave && tt < tl && d0 + cc < p.ED) {
                const int64_t t = t0 + tt;
                xv = load_as_float<IO>(p.x, b * p.u_sb + t * p.u_sl + (int64_t)(d0 + cc) * p.u_sd);
                dv = load_as_float<IO>(p.delta, b * p.d_sb + t * p.d_sl + (int64_t)(d0 + cc) * p.d_sd);
            }
            rX[k] = xv;
            rDl[k] = dv;
        }
#pragma unroll
        for (int k = 0; k < BPT; ++k) {
            const int idx = tid + k * NT;
            const int tt = idx / NP, n = idx % NP;
            float bv = 0.0f, cv = 0.0f;
            if (idx < kTile * NP && tt < tl && n < p.N) {
                const int64_t off = b * p.bc_sb + (int64_t)(t0 + tt) * p.bc_sl + n;
                bv = load_as_float<IO>(p.Bm, off);
                cv = load_as_float<IO>(p.C, off);
            }
            rB[k] = bv;
            rC[k] = cv;
        }
    };

    // the softplus is applied here, not in prefetch(), so that the loads stay in flight
    // during the arithmetic of the previous tile; padded elements keep delta = 0
    auto stage = [&](int buf, int t0) {
        const int tl = min(kTile, p.L - t0);
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
            const int idx = tid + k * NT;
            int tt, cc;
            elem_map(idx, p.in_tmajor, tt, cc);
            if (idx < kTile * kWave) {
                if (p.softplus && tt < tl && d0 + cc < p.ED)
                    rDl[k] = softplus_f(rDl[k] + (p.dbias ? p.dbias[d0 + cc] : 0.0f));
                sDelta[buf][tt][cc] = rDl[k];
                sU[buf][tt][cc] = rDl[k] * rX[k];
                sX[buf][tt][cc] = rX[k];
            }
        }
#pragma unroll
        for (int k = 0; k < BPT; ++k) {
            const int idx = tid + k * NT;
            if (idx < kTile * NP) {
                sB[buf][idx / NP][idx % NP] = rB[k];
                sC[buf][idx / NP][idx % NP] = rC[k];
            }
        }
    };

    prefetch(0);
    int buf = 0;
    for (int t0 = 0, c = 0; t0 < p.L; t0 += kTile, ++c, buf ^= 1) {
        const int tl = min(kTile, p.L - t0);
        stage(buf, t0);
        __syncthreads();
        if (t0 + kTile < p.L) prefetch(t0 + kTile);

        // phase B: steps beyond the sequence end were staged as delta = 0, u = 0, which
        // leaves h unchanged (a = 2^0 = 1), so the loop needs no tail handling
#pragma unroll
        for (int tt = 0; tt < kTile; ++tt) {
            const float dv = sDelta[buf][tt][lane];
            const float uv = sU[buf][tt][lane];
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const float a = fast_exp2(dv * A2[i]);
                const float bv = sB[buf][tt][w * NS + i];
                const float cv = sC[buf][tt][w * NS + i];
                h[i] = __builtin_fmaf(uv, bv, a * h[i]);
                acc = __builtin_fmaf(cv, h[i], acc);
            }
            sY[w][tt][lane] = acc;
        }
        if (p.ckpt && dvalid) {
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const int n = w * NS + i;
                if (n < p.N)
                    p.ckpt[(((int64_t)b * p.nchunks + c) * p.N + n) * p.ED + d] = h[i];
            }
        }
        __syncthreads();

        // phase C
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
            const int idx = tid + k * NT;
            int tt, cc;
            elem_map(idx, p.out_tmajor, tt, cc);
            if (idx < kTile * kWave && tt < tl && d0 + cc < p.ED) {
                float s = 0.0f;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww) s += sY[ww][tt][cc];
                s = __builtin_fmaf(p.D[d0 + cc], sX[buf][tt][cc], s);
                const int64_t t = t0 + tt;
                if (p.z) {
                    const float zv =
                        load_as_float<IO>(p.z, b * p.u_sb + t * p.u_sl + (int64_t)(d0 + cc) * p.u_sd);
                    s *= zv * sigmoid_f(zv);
                }
                store_from_float<IO>(p.y, b * p.y_sb + t * p.y_sl + (int64_t)(d0 + cc) * p.y_sd, s);
            }
        }
        // the next stage() writes the other input buffer; sY is rewritten only after the
        // barrier that follows it, so no third barrier is needed here
    }

    if (p.hlast && dvalid) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = w * NS + i;
            if (n < p.N) p.hlast[((int64_t)b * p.ED + d) * p.N + n] = h[i];
        }
    }
}

template <typename IO, int NS, int NW>
static int launch_fwd(const FwdParams& p, hipStream_t stream) {
    dim3 grid((p.ED + kWave - 1) / kWave, p.batch);
    dim3 block(NW * kWave);
    constexpr size_t lds = sizeof(float) * ((6 + NW) * kTile * kPitch + 4 * kTile * NS * NW);
    static const int attr_rc = allow_dynamic_lds(sscan_fwd_kernel<IO, NS, NW>, lds);
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((sscan_fwd_kernel<IO, NS, NW>), grid, block, lds, stream, p);
    return check_launch();
}

template <typename IO>
static int dispatch_fwd(const FwdParams& p, int ns, int nw, hipStream_t stream) {
#define MPA_CASE(NS_, NW_) \
    if (ns == NS_ && nw == NW_) return launch_fwd<IO, NS_, NW_>(p, stream);
    MPA_CASE(1, 16) MPA_CASE(2, 8) MPA_CASE(4, 4) MPA_CASE(8, 2) MPA_CASE(16, 1)
    MPA_CASE(2, 16) MPA_CASE(4, 8) MPA_CASE(8, 4) MPA_CASE(16, 2)
    MPA_CASE(4, 16) MPA_CASE(8, 8) MPA_CASE(16, 4)
    MPA_CASE(8, 16) MPA_CASE(16, 8)
    MPA_CASE(16, 16)
#undef MPA_CASE
    return MPA_ERR_BAD_SHAPE;
}

}  // namespace mpa

using namespace mpa;

extern "C" int64_t mpa_sscan_ckpt_elems(const mpa_sscan_shape* s) {
    if (!s || s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return 0;
    const int64_t nchunks = (s->seqlen + kTile - 1) / kTile;
    return s->batch * nchunks * s->dstate * s->dim;
}

namespace mpa {
int validate_shape(const mpa_sscan_shape* s) {
    if (!s) return MPA_ERR_NULL_POINTER;
    if (s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return MPA_ERR_BAD_SHAPE;
    if (s->dstate > MPA_MAX_DSTATE || s->batch > 65535) return MPA_ERR_BAD_SHAPE;
    if (s->seqlen > (int64_t)1 << 30 || s->dim > (int64_t)1 << 30) return MPA_ERR_BAD_SHAPE;
    if (s->io_dtype != MPA_F32 && s->io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    return MPA_OK;
}

int padded_states(int64_t n) {
    int np = 16;
    while (np < n) np *= 2;
    return np;
}

int pick_states_per_lane(int64_t batch, int64_t dim, int64_t dstate, int ns_max, const char* env) {
    const int np = padded_states(dstate);
    const int ns_min = np / 16;  // at most 16 waves per workgroup
    if (env) {
        const char* v = getenv(env);
        if (v) {
            const int ns = atoi(v);
            if (ns >= ns_min && ns <= ns_max && ns <= np && (ns & (ns - 1)) == 0) return ns;
        }
    }
    // waves in flight = batch * ceil(dim/64) * np/ns; ask for two per SIMD (2048) if the
    // problem has them, otherwise expose all the parallelism there is
    const int64_t groups = batch * ((dim + kWave - 1) / kWave);
    int ns = ns_max < np ? ns_max : np;
    while (ns > ns_min && groups * (np / ns) < 2048) ns /= 2;
    return ns < ns_min ? ns_min : ns;
}
}  // namespace mpa

extern "C" int mpa_sscan_fwd(const mpa_sscan_shape* s, const void* x, const void* delta,
                             const float* A, const void* B, const void* C, const float* D,
                             const void* z, const float* delta_bias, const float* h0, void* y,
                             float* h_ckpt, float* h_last, void* stream) {
    int rc = validate_shape(s);
    if (rc != MPA_OK) return rc;
    if (!x || !delta || !A || !B || !C || !D || !y) return MPA_ERR_NULL_POINTER;
    const bool softplus = (s->flags & MPA_SSCAN_DELTA_SOFTPLUS) != 0;
    if (!softplus && delta_bias) return MPA_ERR_BAD_SHAPE;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(x, es) || !aligned_to(delta, es) || !aligned_to(B, es) || !aligned_to(C, es) ||
        !aligned_to(y, es) || (z && !aligned_to(z, es)) || !aligned_to(A, 4) || !aligned_to(D, 4))
        return MPA_ERR_MISALIGNED;

    FwdParams p{};
    p.x = x; p.delta = delta; p.Bm = B; p.C = C; p.z = z; p.A = A; p.D = D;
    p.dbias = delta_bias; p.h0 = h0; p.y = y; p.ckpt = h_ckpt; p.hlast = h_last;
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.ED = (int)s->dim; p.N = (int)s->dstate;
    p.nchunks = (p.L + kTile - 1) / kTile;
    p.softplus = softplus ? 1 : 0;
    p.u_sb = s->u_sb; p.u_sl = s->u_sl; p.u_sd = s->u_sd;
    p.d_sb = s->d_sb; p.d_sl = s->d_sl; p.d_sd = s->d_sd;
    p.y_sb = s->y_sb; p.y_sl = s->y_sl; p.y_sd = s->y_sd;
    p.bc_sb = s->bc_sb; p.bc_sl = s->bc_sl;
    p.in_tmajor = (s->u_sd != 1 && s->u_sl == 1) ? 1 : 0;
    p.out_tmajor = (s->y_sd != 1 && s->y_sl == 1) ? 1 : 0;

    const int np = padded_states(s->dstate);
    const int ns = pick_states_per_lane(s->batch, s->dim, s->dstate, 16, "MPA_FWD_NS");
    const int nw = np / ns;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (s->io_dtype == MPA_F32) return dispatch_fwd<float>(p, ns, nw, st);
    return dispatch_fwd<bf16_t>(p, ns, nw, st);
}
