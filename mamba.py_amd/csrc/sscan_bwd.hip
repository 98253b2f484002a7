// Fused selective-scan backward for gfx950.
//
// Same decomposition as the forward pass: a workgroup owns 64 channels of one batch row and
// its NW waves split d_state, NS states per lane.  The sequence is walked from the last
// chunk of kTile steps to the first.  For each chunk a wave
//   1. reloads the state at the chunk start from the checkpoints the forward pass wrote and
//      recomputes the kTile steps, keeping a[t] and a[t]*h[t-1] of every step in registers
//      (the recurrence is never inverted: dividing by a[t] amplifies rounding error);
//   2. sweeps the chunk backwards with the reverse recurrence
//          g[t] = dy[t]*C[t] + a[t+1]*g[t+1]
//      and forms, per state and step,
//          d(delta*A) = g*a*h[t-1]      -> dA += .*delta,  ddelta += .*A
//          sum_n g*B                    -> dx = delta*., ddelta += x*.
//          g*u (u = delta*x)            -> dB (summed over channels)
//          dy*h[t]                      -> dC (summed over channels)
// Reductions: over d_state across the NW waves through LDS (phase C, like the forward
// readout); over the 64 channels of a wave by a wave-private LDS transposition every four
// steps; over channel groups, batch and time by deterministic partial buffers that a small
// second kernel sums (no floating-point atomics: results are bitwise reproducible).
#include "sscan_bwd.h"
#include "sscan_fwd.h"

namespace mpa {

constexpr int kPitchB = kWave + 1;
constexpr int kRedPitch = kWave + 4;  // keeps 16-byte row alignment, conflict-free b128 reads

__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// LDS budget (160 KB per CU).  PS = steps per cross-wave reduction (phase C): a 16-wave
// workgroup reduces twice per chunk so that its partial buffers stay at 8 steps.  kRows = rows
// of one wave's channel-reduction buffer (two per state and step); RS = steps between two
// channel reductions.
template <int NS, int NW>
struct BwdLds {
    static constexpr int NP = NS * NW;
    static constexpr int PS = NW == 16 ? kTile / 2 : kTile;
    static constexpr int kRows = 128 / NW;
    static constexpr int RS = kRows / (2 * NS);
    static_assert(RS >= 1 && RS <= 4, "unsupported (NS, NW)");
    static constexpr size_t floats(bool has_z) {
        return (size_t)5 * kTile * kPitchB + (size_t)(has_z ? 3 : 2) * NW * PS * kPitchB +
               2 * kTile * NP + (size_t)NW * kRows * kRedPitch;
    }
};

template <typename IO, int NS, int NW, bool HAS_Z>
__global__ void __launch_bounds__(NW* kWave) sscan_bwd_kernel(const BwdParams p) {
    constexpr int NT = NW * kWave;
    constexpr int NP = NS * NW;
    constexpr int EPT = (kTile * kWave + NT - 1) / NT;
    constexpr int BPT = (kTile * NP + NT - 1) / NT;
    constexpr int PS = BwdLds<NS, NW>::PS;
    constexpr int NSEG = kTile / PS;
    constexpr int EPS = (PS * kWave + NT - 1) / NT;  // phase-C elements per thread
    constexpr int kRows = BwdLds<NS, NW>::kRows;
    constexpr int RS = BwdLds<NS, NW>::RS;
    constexpr int LPR = kWave / kRows;  // lanes that share one reduction row
    static_assert(kRows <= kWave && LPR >= 1, "reduction rows must fit one wave");

    extern __shared__ float smem[];
    typedef float Tile[kTile][kPitchB];
    typedef float Part[PS][kPitchB];
    typedef float TileN[kTile][NP];
    typedef float RedBuf[kRows][kRedPitch];
    Tile* sDelta = reinterpret_cast<Tile*>(smem);  // [1]
    Tile* sU = sDelta + 1;
    Tile* sX = sU + 1;
    Tile* sDy = sX + 1;
    Tile* sZg = sDy + 1;       // ungated dy when HAS_Z (else unused)
    TileN* sB = reinterpret_cast<TileN*>(sZg + 1);
    TileN* sC = sB + 1;
    RedBuf* sR = reinterpret_cast<RedBuf*>(sC + 1);  // [NW]
    Part* sP1 = reinterpret_cast<Part*>(sR + NW);     // [NW] sum_n g*B
    Part* sP2 = sP1 + NW;      // [NW] sum_n g*a*h[t-1]*A*log2(e)
    Part* sP3 = sP2 + NW;      // [NW] sum_n C*h, HAS_Z only

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = wave_id();
    const int b = blockIdx.y;
    const int cg = blockIdx.x;
    const int d0 = cg * kWave;
    const int d = d0 + lane;
    const bool dvalid = d < p.ED;

    float A2[NS], ag[NS], dAacc[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = w * NS + i;
        A2[i] = (dvalid && n < p.N) ? p.A[(int64_t)d * p.Nst + n] * kLog2e : 0.0f;
        ag[i] = 0.0f;
        dAacc[i] = 0.0f;
    }
    float dDacc[NSEG * EPS], dDbacc[NSEG * EPS];
#pragma unroll
    for (int k = 0; k < NSEG * EPS; ++k) dDacc[k] = dDbacc[k] = 0.0f;

    float rX[EPT], rDl[EPT], rDy[EPT], rZ[EPT], rB[BPT], rC[BPT], rH[NS];

    auto elem_map = [&](int idx, bool tmajor, int& tt, int& cc) {
        if (tmajor) {
            tt = idx % kTile;
            cc = idx / kTile;
        } else {
            tt = idx / kWave;
            cc = idx % kWave;
        }
    };

    // c counts the tiles in the order of the forward walk (the index of their checkpoints) and tt
    // the steps inside a tile likewise; with a reverse walk both are mirrored in memory
    const bool rev = p.reverse != 0;
    auto first_step = [&](int c) { return (rev ? p.nchunks - 1 - c : c) * kTile; };
    auto phys_step = [&](int tt) { return rev ? kTile - 1 - tt : tt; };

    auto prefetch = [&](int c) {
        const int t0 = first_step(c);
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
            const int idx = tid + k * NT;
            int tt, cc;
            elem_map(idx, p.in_tmajor, tt, cc);
            float xv = 0.0f, dv = 0.0f, dyv = 0.0f, zv = 0.0f;
            if (idx < kTile * kWave && t0 + phys_step(tt) < p.L && d0 + cc < p.ED) {
                const int64_t t = t0 + phys_step(tt);
                const int64_t ch = d0 + cc;
                xv = load_as_float<IO>(p.x, b * p.u_sb + t * p.u_sl + ch * p.u_sd);
                dv = load_as_float<IO>(p.delta, b * p.d_sb + t * p.d_sl + ch * p.d_sd);
                dyv = load_as_float<IO>(p.dy, b * p.y_sb + t * p.y_sl + ch * p.y_sd);
                if (HAS_Z) zv = load_as_float<IO>(p.z, b * p.z_sb + t * p.z_sl + ch * p.z_sd);
            }
            rX[k] = xv;
            rDl[k] = dv;
            rDy[k] = dyv;
            rZ[k] = zv;
        }
#pragma unroll
        for (int k = 0; k < BPT; ++k) {
            const int idx = tid + k * NT;
            const int tt = idx / NP, n = idx % NP;
            float bv = 0.0f, cv = 0.0f;
            if (idx < kTile * NP && t0 + phys_step(tt) < p.L && n < p.N) {
                const int64_t off = b * p.bc_sb + (int64_t)(t0 + phys_step(tt)) * p.bc_sl + n;
                bv = load_as_float<IO>(p.Bm, off);
                cv = load_as_float<IO>(p.C, off);
            }
            rB[k] = bv;
            rC[k] = cv;
        }
        // state at the start of chunk c = checkpoint written after chunk c-1
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = w * NS + i;
            float hv = 0.0f;
            if (dvalid && n < p.N) {
                if (c > 0)
                    hv = p.ckpt[(((int64_t)b * p.nchunks + (c - 1)) * p.Nst + n) * p.ED + d];
                else if (p.h0)
                    hv = p.h0[((int64_t)b * p.ED + d) * p.Nst + n];
            }
            rH[i] = hv;
        }
    };

    // sDelta holds the delta the recurrence uses (after softplus); the raw value that the
    // softplus derivative needs is recomputed from it: sigmoid(raw) = 1 - exp(-softplus(raw))
    auto stage = [&](int t0) {
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
            const int idx = tid + k * NT;
            int tt, cc;
            elem_map(idx, p.in_tmajor, tt, cc);
            if (idx < kTile * kWave) {
                float dv = rDl[k];
                const bool live = (t0 + phys_step(tt) < p.L && d0 + cc < p.ED);
                if (p.softplus && live) dv = softplus_f(dv + (p.dbias ? p.dbias[d0 + cc] : 0.0f));
                float dyv = rDy[k];
                if (HAS_Z) {
                    const float zv = rZ[k];
                    const float sg = sigmoid_f(zv);
                    // keep the raw dy for dz; the recurrence sees dy * silu(z)
                    sZg[0][tt][cc] = dyv;
                    dyv = dyv * zv * sg;
                }
                sDelta[0][tt][cc] = dv;
                sU[0][tt][cc] = dv * rX[k];
                sX[0][tt][cc] = rX[k];
                sDy[0][tt][cc] = dyv;
            }
        }
#pragma unroll
        for (int k = 0; k < BPT; ++k) {
            const int idx = tid + k * NT;
            if (idx < kTile * NP) {
                sB[0][idx / NP][idx % NP] = rB[k];
                sC[0][idx / NP][idx % NP] = rC[k];
            }
        }
    };

    const int last = p.nchunks - 1;
    prefetch(last);
    for (int c = last; c >= 0; --c) {
        const int t0 = first_step(c);
        float h[NS];
        // a tail chunk was prefetched with zero padding (delta = 0: a = 1, u = 0; dy = 0),
        // which makes the padded steps exact no-ops in both sweeps
        stage(t0);
#pragma unroll
        for (int i = 0; i < NS; ++i) h[i] = rH[i];
        __syncthreads();
        if (c > 0) prefetch(c - 1);

        // ---- 1. recompute the chunk forward, keeping a and a*h[t-1] ----
        float aS[kTile][NS], tS[kTile][NS];
#pragma unroll
        for (int tt = 0; tt < kTile; ++tt) {
            const float dv = sDelta[0][tt][lane];
            const float uv = sU[0][tt][lane];
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const float a = fast_exp2(dv * A2[i]);
                const float th = a * h[i];
                aS[tt][i] = a;
                tS[tt][i] = th;
                h[i] = __builtin_fmaf(uv, sB[0][tt][w * NS + i], th);
            }
        }

        // ---- 2. reverse sweep, in NSEG segments of PS steps, each followed by phase C ----
#pragma unroll
        for (int seg = NSEG - 1; seg >= 0; --seg) {
#pragma unroll
            for (int ts = PS - 1; ts >= 0; --ts) {
                const int tt = seg * PS + ts;
                const float dv = sDelta[0][tt][lane];
                const float uv = sU[0][tt][lane];
                const float dyv = sDy[0][tt][lane];
                float gB = 0.0f, dd = 0.0f, yp = 0.0f;
                const int slot = tt % RS;
#pragma unroll
                for (int i = 0; i < NS; ++i) {
                    const float bv = sB[0][tt][w * NS + i];
                    const float cv = sC[0][tt][w * NS + i];
                    const float g = __builtin_fmaf(dyv, cv, ag[i]);
                    const float hh = __builtin_fmaf(uv, bv, tS[tt][i]);
                    const float gha = g * tS[tt][i];
                    dAacc[i] = __builtin_fmaf(gha, dv, dAacc[i]);
                    dd = __builtin_fmaf(gha, A2[i], dd);
                    gB = __builtin_fmaf(g, bv, gB);
                    ag[i] = aS[tt][i] * g;
                    if (HAS_Z) yp = __builtin_fmaf(cv, hh, yp);
                    sR[w][slot * 2 * NS + i][lane] = g * uv;
                    sR[w][slot * 2 * NS + NS + i][lane] = dyv * hh;
                }
                sP1[w][ts][lane] = gB;
                sP2[w][ts][lane] = dd;
                if (HAS_Z) sP3[w][ts][lane] = yp;

                if (slot == 0) {
                    // channel reduction of the last RS steps: row r = (step, dB|dC, state);
                    // LPR lanes share a row, each sums kWave/LPR consecutive channels
                    wave_lds_sync();
                    const int row = lane / LPR, part = lane % LPR;
                    const float4* src =
                        reinterpret_cast<const float4*>(&sR[w][row][part * (kWave / LPR)]);
                    float s = 0.0f;
#pragma unroll
                    for (int j = 0; j < kWave / LPR / 4; ++j) {
                        const float4 v = src[j];
                        s += (v.x + v.y) + (v.z + v.w);
                    }
#pragma unroll
                    for (int m = 1; m < LPR; m *= 2) s += __shfl_xor(s, m, kWave);
                    const int rs = row / (2 * NS), o = row % (2 * NS);
                    const int t = t0 + phys_step(tt + rs);
                    const int n = w * NS + (o % NS);
                    if (part == 0 && t < p.L && n < p.N) {
                        float* dst = (o < NS) ? p.partB : p.partC;
                        dst[cg * p.part_gs + ((int64_t)b * p.L + t) * p.Nst + n] = s;
                    }
                    wave_lds_sync();
                }
            }
            __syncthreads();

            // ---- phase C: sum over the waves, finish dx / ddelta (/ dz), accumulate dD ----
#pragma unroll
            for (int k = 0; k < EPS; ++k) {
                const int idx = tid + k * NT;
                int ts, cc;
                if (p.out_tmajor) {
                    ts = idx % PS;
                    cc = idx / PS;
                } else {
                    ts = idx / kWave;
                    cc = idx % kWave;
                }
                const int tt = seg * PS + ts;
                if (idx < PS * kWave && t0 + phys_step(tt) < p.L && d0 + cc < p.ED) {
                    float gB = 0.0f, dd = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < NW; ++ww) {
                        gB += sP1[ww][ts][cc];
                        dd += sP2[ww][ts][cc];
                    }
                    const float xv = sX[0][tt][cc];
                    const float dv = sDelta[0][tt][cc];
                    const float dyg = sDy[0][tt][cc];  // dy, already gated when HAS_Z
                    const float Dv = p.D[d0 + cc];
                    const int64_t t = t0 + phys_step(tt);
                    const int64_t ch = d0 + cc;
                    // (a later pass over another block of states adds dv * gB only: D*dy and dD
                    // belong to the first)
                    float dxv = __builtin_fmaf(dv, gB, p.accumulate ? 0.0f : Dv * dyg);
                    float ddv = __builtin_fmaf(xv, gB, dd * kLn2);
                    if (!p.accumulate) dDacc[seg * EPS + k] = __builtin_fmaf(dyg, xv, dDacc[seg * EPS + k]);
                    if (p.softplus) {
                        // d softplus(r)/dr = sigmoid(r) = 1 - exp(-softplus(r))
                        ddv *= (1.0f - __expf(-dv));
                        dDbacc[seg * EPS + k] += ddv;
                    }
                    const int64_t go = b * p.g_sb + t * p.g_sl + ch * p.g_sd;
                    if (p.accumulate) {
                        dxv += load_as_float<IO>(p.dx, go);
                        ddv += load_as_float<IO>(p.ddelta, go);
                    }
                    store_from_float<IO>(p.dx, go, dxv);
                    store_from_float<IO>(p.ddelta, go, ddv);
                    if (HAS_Z) {
                        float yp = 0.0f;
#pragma unroll
                        for (int ww = 0; ww < NW; ++ww) yp += sP3[ww][ts][cc];
                        if (!p.accumulate) yp = __builtin_fmaf(Dv, xv, yp);  // pre-gate output
                        const float zv =
                            load_as_float<IO>(p.z, b * p.z_sb + t * p.z_sl + ch * p.z_sd);
                        const float sg = sigmoid_f(zv);
                        const float dyraw = sZg[0][tt][cc];
                        // d(z*sigmoid(z))/dz = sg * (1 + z*(1-sg))
                        float dzv = dyraw * yp * sg * (1.0f + zv * (1.0f - sg));
                        if (p.accumulate) dzv += load_as_float<IO>(p.dz, go);
                        store_from_float<IO>(p.dz, go, dzv);
                    }
                }
            }
            __syncthreads();
        }
    }

    // ---- epilogue: per-batch partials of dA, dD (and ddelta_bias) ----
    if (dvalid) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = w * NS + i;
            if (n < p.N) p.partA[((int64_t)b * p.ED + d) * p.Nst + n] = dAacc[i];
        }
    }
    // dD: every thread holds sums for its fixed (step slot, channel) elements; reduce over
    // the step slots through LDS (sDelta .. sDy are free now: use them as one [kTile] tile)
    for (int pass = 0; pass < (p.softplus ? 2 : 1); ++pass) {
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {
#pragma unroll
            for (int k = 0; k < EPS; ++k) {
                const int idx = tid + k * NT;
                int ts, cc;
                if (p.out_tmajor) {
                    ts = idx % PS;
                    cc = idx / PS;
                } else {
                    ts = idx / kWave;
                    cc = idx % kWave;
                }
                if (idx < PS * kWave)
                    sDelta[0][seg * PS + ts][cc] =
                        pass == 0 ? dDacc[seg * EPS + k] : dDbacc[seg * EPS + k];
            }
        }
        __syncthreads();
        if (tid < kWave && d0 + tid < p.ED) {
            float s = 0.0f;
#pragma unroll
            for (int tt = 0; tt < kTile; ++tt) s += sDelta[0][tt][tid];
            float* dst = pass == 0 ? p.partD : p.partDb;
            dst[(int64_t)(p.row0 + b) * p.ED + d0 + tid] = s;
        }
        __syncthreads();
    }
}

// Sums the partial buffers: dB/dC over channel groups, dA over its rows_a rows (batch rows, or
// their segments), dD/ddelta_bias over their rows_d rows (the same, or batch rows times the state
// blocks of a wide d_state).  V = 4: d_state is a multiple of 4, a thread sums
// four consecutive states with 16-byte loads.
template <typename IO, int V>
__global__ void __launch_bounds__(256) sscan_bwd_finish_kernel(
    const float* partB, const float* partC, const float* partA, const float* partD,
    const float* partDb, void* dB, void* dC, float* dA, float* dD, float* dDb, int CG, int64_t gs,
    int batch, int rows_a, int rows_d, int L, int ED, int N, int64_t dbc_sb, int64_t dbc_sl) {
    const int64_t bln = (int64_t)batch * L * N;
    const int64_t edn = (int64_t)ED * N;
    const int64_t nbc = bln / V;  // threads of the dB/dC part
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t i = t - nbc + bln;  // index into the dA / dD parts, as if V were 1
    if (t < nbc) {
        float sb[V], sc[V];
#pragma unroll
        for (int v = 0; v < V; ++v) sb[v] = sc[v] = 0.0f;
        // eight groups per round: all sixteen loads are issued before the first sum (the kernel is
        // bound by memory latency, not by instructions); the order of the additions is fixed
        constexpr int kRound = 8;
        for (int g0 = 0; g0 < CG; g0 += kRound) {
            if constexpr (V == 4) {
                float4 b4[kRound], c4[kRound];
#pragma unroll
                for (int r = 0; r < kRound; ++r) {
                    const int g = g0 + r < CG ? g0 + r : CG - 1;  // clamped copies are not added
                    b4[r] = *reinterpret_cast<const float4*>(partB + g * gs + 4 * t);
                    c4[r] = *reinterpret_cast<const float4*>(partC + g * gs + 4 * t);
                }
#pragma unroll
                for (int r = 0; r < kRound; ++r) {
                    if (g0 + r < CG) {
                        sb[0] += b4[r].x; sb[1] += b4[r].y; sb[2] += b4[r].z; sb[3] += b4[r].w;
                        sc[0] += c4[r].x; sc[1] += c4[r].y; sc[2] += c4[r].z; sc[3] += c4[r].w;
                    }
                }
            } else {
                float b1[kRound], c1[kRound];
#pragma unroll
                for (int r = 0; r < kRound; ++r) {
                    const int g = g0 + r < CG ? g0 + r : CG - 1;
                    b1[r] = partB[g * gs + t];
                    c1[r] = partC[g * gs + t];
                }
#pragma unroll
                for (int r = 0; r < kRound; ++r) {
                    if (g0 + r < CG) {
                        sb[0] += b1[r];
                        sc[0] += c1[r];
                    }
                }
            }
        }
        const int64_t e = V * t;
        const int n = (int)(e % N);
        const int64_t bt = e / N;
        const int64_t off = (bt / L) * dbc_sb + (bt % L) * dbc_sl + n;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            store_from_float<IO>(dB, off + v, sb[v]);
            store_from_float<IO>(dC, off + v, sc[v]);
        }
    } else if (i < bln + edn) {
        const int64_t j = i - bln;
        float s = 0.0f;
        for (int bb = 0; bb < rows_a; ++bb) s += partA[bb * edn + j];
        dA[j] = s;
    } else if (i < bln + edn + ED) {
        const int64_t j = i - bln - edn;
        float s = 0.0f, sdb = 0.0f;
        for (int bb = 0; bb < rows_d; ++bb) {
            s += partD[(int64_t)bb * ED + j];
            if (dDb) sdb += partDb[(int64_t)bb * ED + j];
        }
        dD[j] = s;
        if (dDb) dDb[j] = sdb;
    }
}

// states per lane of the backward kernels (at most 4) and, for that choice, how a thin launch
// is cut: half of the CUs or fewer covered (the first pass of a cut costs a quarter of the second)
static constexpr int kBwdThin = 2;
static int bwd_states_per_lane(const mpa_sscan_shape* s) {
    const int ns = pick_states_per_lane(s->batch, s->dim, s->dstate, 4, s->plan_states_per_lane);
    return ns < 0 ? 4 : ns;
}
// The fast kernel holds 16 states.  A wider d_state runs on it as passes over blocks of 16 states
// (the states are independent given x, delta, B, C; dx, ddelta add up over the passes), each pass cut
// into segments like a 16-state call.  `blk` = the shape of one such pass.
constexpr int kFastStates = 16;
static mpa_sscan_shape fast_block_shape(const mpa_sscan_shape* s) {
    mpa_sscan_shape blk = *s;
    if (blk.dstate > kFastStates) blk.dstate = kFastStates;
    return blk;
}
// The cut exists on the fast kernel only.
static SegPlan bwd_seg_plan(const mpa_sscan_shape* s) {
    const mpa_sscan_shape blk = fast_block_shape(s);
    const int ns = bwd_states_per_lane(&blk);
    if (!bwd_fast_supported(ns, padded_states(blk.dstate) / ns) || (s->plan_flags & MPA_PLAN_BWD_GENERAL))
        return SegPlan{1, 0, 0, 0, 0, 0};
    return seg_plan(&blk, ns, kBwdThin);
}

constexpr int kStateBlock = 64;  // states one launch of the general kernel holds (4 per lane, 16 waves)

struct BwdWorkspace {
    size_t offB, offC, offA, offD, offDb, offSeg, total, group_stride;
    SegPlan seg;
};

static BwdWorkspace bwd_workspace(const mpa_sscan_shape* s) {
    BwdWorkspace w;
    w.seg = bwd_seg_plan(s);
    // rows of the per-row partials of dD / ddelta_bias: batch rows, times the segments of a cut
    // sequence, times the passes over state blocks of a wide d_state (16 states on the fast kernel,
    // 64 on the general one, which is never cut: the larger count covers both); dA has one row per
    // batch row and segment, every pass writes its own states of it
    const size_t nseg = w.seg.nseg > 1 ? (size_t)w.seg.nseg : 1;
    const size_t nblk = (size_t)(s->dstate + kFastStates - 1) / kFastStates;
    const size_t rows = (size_t)s->batch * nseg * nblk;
    const size_t cg = (size_t)(s->dim + kWave - 1) / kWave;
    const size_t bln = (size_t)s->batch * s->seqlen * s->dstate;
    const size_t ren = (size_t)s->batch * nseg * s->dim * s->dstate;
    const size_t re = rows * s->dim;
    auto up = [](size_t v) { return (v + 63) / 64 * 64; };  // 256-byte granules of floats
    // The partial sums of the channel groups for one (batch, step, state) are written at the same
    // time by different workgroups and read together by the finish kernel.  batch*L*N floats is
    // often a power of two (1 MiB at the headline shape), which would put all of them on the same
    // memory channel: an odd number of 256-byte lines between groups spreads them.
    w.group_stride = up(bln) + 17 * 64;
    w.offB = 0;
    w.offC = w.offB + cg * w.group_stride;
    w.offA = w.offC + cg * w.group_stride;
    w.offD = w.offA + up(ren);
    w.offDb = w.offD + up(re);
    w.offSeg = w.offDb + up(re);
    w.total = (w.offSeg + up(w.seg.floats)) * sizeof(float);
    return w;
}

template <typename IO, int NS, int NW, bool HAS_Z>
static int launch_bwd(const BwdParams& p, hipStream_t stream) {
    dim3 grid((p.ED + kWave - 1) / kWave, p.batch);
    dim3 block(NW * kWave);
    constexpr size_t lds = sizeof(float) * BwdLds<NS, NW>::floats(HAS_Z);
    static LdsLimitOnce lds_limit;
    const int attr_rc = lds_limit.ensure(sscan_bwd_kernel<IO, NS, NW, HAS_Z>, lds);
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((sscan_bwd_kernel<IO, NS, NW, HAS_Z>), grid, block, lds, stream, p);
    return check_launch();
}

template <typename IO, bool HAS_Z>
static int dispatch_bwd(const BwdParams& p, int ns, int nw, hipStream_t stream) {
#define MPA_CASE(NS_, NW_) \
    if (ns == NS_ && nw == NW_) return launch_bwd<IO, NS_, NW_, HAS_Z>(p, stream);
    MPA_CASE(1, 16) MPA_CASE(2, 8) MPA_CASE(4, 4)
    MPA_CASE(2, 16) MPA_CASE(4, 8)
    MPA_CASE(4, 16)
#undef MPA_CASE
    return MPA_ERR_BAD_SHAPE;
}

}  // namespace mpa

using namespace mpa;

extern "C" size_t mpa_sscan_bwd_workspace_bytes(const mpa_sscan_shape* s) {
    if (validate_shape(s) != MPA_OK) return 0;
    return bwd_workspace(s).total;
}

extern "C" int mpa_sscan_bwd(const mpa_sscan_shape* s, const void* x, const void* delta,
                             const float* A, const void* B, const void* C, const float* D,
                             const void* z, const float* delta_bias, const float* h0,
                             const void* dy, const void* y_pregate, const float* h_ckpt, void* dx,
                             void* ddelta,
                             float* dA, void* dB, void* dC, float* dD, void* dz,
                             float* ddelta_bias, void* workspace, size_t workspace_bytes,
                             void* stream) {
    int rc = validate_shape(s);
    if (rc != MPA_OK) return rc;
    if (!x || !delta || !A || !B || !C || !D || !dy || !h_ckpt || !dx || !ddelta || !dA || !dB ||
        !dC || !dD || !workspace)
        return MPA_ERR_NULL_POINTER;
    if (z && !dz) return MPA_ERR_NULL_POINTER;
    const bool softplus = (s->flags & MPA_SSCAN_DELTA_SOFTPLUS) != 0;
    if (!softplus && (delta_bias || ddelta_bias)) return MPA_ERR_BAD_SHAPE;
    if (delta_bias && !ddelta_bias) return MPA_ERR_NULL_POINTER;
    const size_t es = dtype_size(s->io_dtype);
    const size_t esd = s->delta_dtype == MPA_DELTA_F32 ? 4 : es;
    if (!aligned_to(x, es) || !aligned_to(delta, esd) || !aligned_to(B, es) || !aligned_to(C, es) ||
        !aligned_to(dy, es) || !aligned_to(dx, es) || !aligned_to(ddelta, esd) ||
        !aligned_to(dB, es) || !aligned_to(dC, es) || (z && !aligned_to(z, es)) ||
        (dz && !aligned_to(dz, es)) || (y_pregate && !aligned_to(y_pregate, es)) ||
        !aligned_to(workspace, 256))
        return MPA_ERR_MISALIGNED;
    const BwdWorkspace ws = bwd_workspace(s);
    if (workspace_bytes < ws.total) return MPA_ERR_WORKSPACE;

    float* wsf = static_cast<float*>(workspace);
    BwdParams p{};
    p.x = x; p.delta = delta; p.Bm = B; p.C = C; p.z = z; p.dy = dy; p.A = A; p.D = D;
    p.ypre = z ? y_pregate : nullptr;
    p.dbias = delta_bias; p.h0 = h0; p.ckpt = h_ckpt; p.dx = dx; p.ddelta = ddelta; p.dz = dz;
    p.partB = wsf + ws.offB; p.partC = wsf + ws.offC; p.partA = wsf + ws.offA;
    p.part_gs = (int64_t)ws.group_stride;
    p.partD = wsf + ws.offD; p.partDb = wsf + ws.offDb;
    p.expire_waits = (s->plan_flags & MPA_PLAN_EXPIRE_WAITS) ? 1 : 0;
    p.reverse = (s->flags & MPA_SSCAN_REVERSE) ? 1 : 0;
    p.nseg = 1;
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.ED = (int)s->dim; p.N = (int)s->dstate;
    p.nchunks = (p.L + kTile - 1) / kTile;
    p.Nst = p.N;
    p.softplus = softplus ? 1 : 0;
    p.delta_f32 = s->delta_dtype == MPA_DELTA_F32 ? 1 : 0;
    p.u_sb = s->u_sb; p.u_sl = s->u_sl; p.u_sd = s->u_sd;
    p.z_sb = s->z_sb; p.z_sl = s->z_sl; p.z_sd = s->z_sd;
    p.d_sb = s->d_sb; p.d_sl = s->d_sl; p.d_sd = s->d_sd;
    p.y_sb = s->y_sb; p.y_sl = s->y_sl; p.y_sd = s->y_sd;
    p.g_sb = s->g_sb; p.g_sl = s->g_sl; p.g_sd = s->g_sd;
    p.bc_sb = s->bc_sb; p.bc_sl = s->bc_sl;
    p.in_tmajor = (s->u_sd != 1 && s->u_sl == 1) ? 1 : 0;
    p.out_tmajor = (s->g_sd != 1 && s->g_sl == 1) ? 1 : 0;

    hipStream_t st = static_cast<hipStream_t>(stream);
    // the fast kernel (16 states per launch, in passes over blocks of 16 for a wider d_state) unless
    // the gate comes without the saved pre-gate output or the caller asks for the general kernel
    const mpa_sscan_shape blk_shape = fast_block_shape(s);
    const int fns = bwd_states_per_lane(&blk_shape);
    const int fnw = padded_states(blk_shape.dstate) / fns;
    const bool fast = (!z || p.ypre) && bwd_fast_supported(fns, fnw) && !(s->plan_flags & MPA_PLAN_BWD_GENERAL);
    const int np = padded_states(s->dstate);
    const int ns = bwd_states_per_lane(s);
    const int nw = np / ns;
    int rows = p.batch, rows_a = p.batch;
    // (float32 delta next to bfloat16 tensors exists on the fast kernels only)
    if (!fast && p.delta_f32 && s->io_dtype != MPA_F32) return MPA_ERR_BAD_DTYPE;
    if (fast) {
        const int nseg = ws.seg.nseg > 1 ? ws.seg.nseg : 1;
        const int nblk = (p.N + kFastStates - 1) / kFastStates;
        const size_t es_ = dtype_size(s->io_dtype);
        for (int sb = 0; sb < nblk && rc == MPA_OK; ++sb) {
            const int n0 = sb * kFastStates;
            BwdParams q = p;
            q.N = p.N - n0 < kFastStates ? p.N - n0 : kFastStates;
            q.A = A + n0;
            q.Bm = static_cast<const char*>(B) + n0 * es_;
            q.C = static_cast<const char*>(C) + n0 * es_;
            q.h0 = h0 ? h0 + n0 : nullptr;
            q.ckpt = h_ckpt + (int64_t)n0 * p.ED;
            q.partA = p.partA + n0; q.partB = p.partB + n0; q.partC = p.partC + n0;
            q.accumulate = sb > 0 ? 1 : 0;
            q.row0 = sb * p.batch * nseg;
            if (nseg > 1) {
                // Sequence cut into segments that run side by side.  The reverse recurrence
                // ag[t] = a[t] * (ag[t+1] + C[t]*dy[t]) is linear in its state like the forward one,
                // so the forward kernel in its carry mode, walking against the forward direction,
                // finds every segment's end value from zero and its sum of delta; seg_carry_kernel
                // chains them into the value that flows into each segment.
                float* seg = wsf + ws.offSeg;
                FwdParams g{};
                g.x = dy; g.delta = delta; g.z = z; g.A = q.A; g.D = D; g.dbias = delta_bias;
                g.Bm = q.C; g.C = q.C; g.bc_sb = s->bc_sb; g.bc_sl = s->bc_sl;
                g.hlast = seg + ws.seg.off_hend; g.dsum = seg + ws.seg.off_dsum;
                g.nseg = nseg; g.seg_tiles = ws.seg.seg_tiles;
                g.batch = p.batch; g.L = p.L; g.ED = p.ED; g.N = q.N; g.nchunks = p.nchunks;
                g.a_st = p.N; g.h_st = q.N; g.ck_st = q.N;
                g.softplus = p.softplus; g.delta_f32 = p.delta_f32; g.reverse = p.reverse ? 0 : 1;
                g.u_sb = s->y_sb; g.u_sl = s->y_sl; g.u_sd = s->y_sd;
                g.z_sb = s->z_sb; g.z_sl = s->z_sl; g.z_sd = s->z_sd;
                g.d_sb = s->d_sb; g.d_sl = s->d_sl; g.d_sd = s->d_sd;
                g.in_tmajor = (s->d_sd != 1 && s->d_sl == 1) ? 1 : 0;
                rc = launch_fwd_any(g, s->io_dtype, fns, fnw, kGCarry, st);
                if (rc != MPA_OK) return rc;
                rc = launch_seg_carry(q.A, nullptr, seg + ws.seg.off_hend, seg + ws.seg.off_dsum, seg + ws.seg.off_h0,
                                      nullptr, p.batch, nseg, p.ED, q.N, p.N, q.N, st);
                if (rc != MPA_OK) return rc;
                q.nseg = nseg; q.seg_tiles = ws.seg.seg_tiles; q.ag0 = seg + ws.seg.off_h0;
            }
            rc = launch_bwd_fast(q, fns, fnw, s->io_dtype, st);
        }
        rows_a = p.batch * nseg;
        rows = rows_a * nblk;
    } else {
        auto general = [&](const BwdParams& q, int qns, int qnw) {
            if (s->io_dtype == MPA_F32)
                return z ? dispatch_bwd<float, true>(q, qns, qnw, st) : dispatch_bwd<float, false>(q, qns, qnw, st);
            return z ? dispatch_bwd<bf16_t, true>(q, qns, qnw, st) : dispatch_bwd<bf16_t, false>(q, qns, qnw, st);
        };
        if (p.N <= kStateBlock) {
            rc = general(p, ns, nw);
        } else {
            // d_state above 64: one launch per block of 64 states, in order on the stream.  Each
            // pass owns its states' dA, dB, dC; dx, ddelta and dz are sums over all states, so
            // the passes after the first add to what is there; dD comes from the first.
            const int nblk = (p.N + kStateBlock - 1) / kStateBlock;
            const size_t es_ = dtype_size(s->io_dtype);
            for (int sb = 0; sb < nblk && rc == MPA_OK; ++sb) {
                const int n0 = sb * kStateBlock;
                BwdParams q = p;
                q.N = p.N - n0 < kStateBlock ? p.N - n0 : kStateBlock;
                q.A = A + n0;
                q.Bm = static_cast<const char*>(B) + n0 * es_;
                q.C = static_cast<const char*>(C) + n0 * es_;
                q.h0 = h0 ? h0 + n0 : nullptr;
                q.ckpt = h_ckpt + (int64_t)n0 * p.ED;
                q.partA = p.partA + n0; q.partB = p.partB + n0; q.partC = p.partC + n0;
                q.accumulate = sb > 0 ? 1 : 0;
                q.row0 = sb * p.batch;
                rc = general(q, 4, kStateBlock / 4);
            }
            rows = p.batch * nblk;
        }
    }
    if (rc != MPA_OK) return rc;

    const int cg = (p.ED + kWave - 1) / kWave;
    // the partial buffers start on 256-byte granules, so rows of four states are 16-byte aligned
    const int vec = p.N % 4 == 0 ? 4 : 1;
    const int64_t total = (int64_t)p.batch * p.L * p.N / vec + (int64_t)p.ED * p.N + p.ED;
    dim3 fgrid((unsigned)((total + 255) / 256));
#define MPA_FINISH(IO_, V_)                                                                                    \
    hipLaunchKernelGGL((sscan_bwd_finish_kernel<IO_, V_>), fgrid, dim3(256), 0, st, p.partB, p.partC, p.partA, \
                       p.partD, softplus && ddelta_bias ? p.partDb : nullptr, dB, dC, dA, dD, ddelta_bias, cg,  \
                       p.part_gs, p.batch, rows_a, rows, p.L, p.ED, p.N, s->dbc_sb, s->dbc_sl)
    if (s->io_dtype == MPA_F32) {
        if (vec == 4) MPA_FINISH(float, 4);
        else MPA_FINISH(float, 1);
    } else {
        if (vec == 4) MPA_FINISH(bf16_t, 4);
        else MPA_FINISH(bf16_t, 1);
    }
#undef MPA_FINISH
    return check_launch();
}
