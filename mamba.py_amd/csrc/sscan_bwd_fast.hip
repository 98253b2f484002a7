// Fused selective-scan backward for gfx950, fast path (no output gate).
//
// Same roles as the forward kernel.  A workgroup owns 64 channels of one batch row and walks
// the sequence from the last tile of kTile steps to the first.
//   * NW scan waves split d_state (NS states per lane, one channel per lane).  Per tile a
//     scan wave reloads the state at the tile start from the forward checkpoints, recomputes
//     the kTile steps keeping a[t] and a[t]*h[t-1] in registers (the recurrence is never
//     inverted: dividing by a[t] amplifies rounding error), then sweeps the tile backwards:
//         g[t] = dy[t]*C[t] + a[t+1]*g[t+1]
//         d(delta*A) = g*a*h[t-1]   -> dA += .*delta ;  ddelta += .*A
//         sum_n g*B                 -> dx = delta*. ;   ddelta += x*.
//         g*u (u = delta*x), dy*h   -> dB, dC, summed over the 64 channels of the wave by a
//                                      wave by an in-register reduce-scatter (rs_stage).
//     B and C come through scalar loads from the float32 pack the pre-pass wrote.
//   * two loader waves fetch x, delta, dy two tiles ahead, convert, apply softplus and
//     publish delta, u, dy and x as float32 LDS tiles; they also accumulate dD.
//   * two reducer waves, one tile behind, sum the partial sum_n over the scan waves, finish
//     dx and ddelta (softplus chain rule included), store them, and forward the per-tile
//     dB/dC sums to the per-channel-group partial buffers.
// Tiles in LDS are [64 channels][16 steps] float32 at a pitch of 20 floats.
// Reductions over channel groups, batch and time go through deterministic partial buffers
// summed by sscan_bwd_finish_kernel (no floating-point atomics: results are bitwise
// reproducible).
#include "sscan_bwd.h"

namespace mpa {

constexpr int kPitchT = kTile + 4;         // row pitch (floats) of a [channel][step] LDS tile: rows stay
                                          // 16-byte aligned and 16-byte accesses are conflict-free
constexpr int kTileF = kWave * kPitchT;   // floats per LDS tile


// float index of the 16-byte column q (4 steps) of channel ch inside a tile
__device__ __forceinline__ int tile_off(int ch, int q) { return ch * kPitchT + 4 * q; }

__device__ __forceinline__ float4 tile_ld(const float* tile, int ch, int q) {
    return *reinterpret_cast<const float4*>(tile + tile_off(ch, q));
}
__device__ __forceinline__ void tile_st(float* tile, int ch, int q, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(tile + tile_off(ch, q)) = make_float4(a, b, c, d);
}

// ---- in-register reduce-scatter over the 64 lanes of a wave ------------------------------
// 64 values per lane are summed over all lanes in six halving stages; after stage s only
// half of the registers remain, and a lane keeps the value whose index bit s equals the
// matching lane bit, so that at the end lane l holds the complete sum of value number l and
// each value cost (32+16+8+4+2+1)/64 adds plus the data movement, all on the VALU (no LDS
// round trip sits in the dependency chain of the reverse sweep).
//   stage 1: v_permlane32_swap  (lane bit 5)     stage 4: DPP row_half_mirror (lane bit 2)
//   stage 2: v_permlane16_swap  (lane bit 4)     stage 5: DPP quad_perm 3210  (lane bit 1)
//   stage 3: DPP row_mirror     (lane bit 3)     stage 6: DPP quad_perm 1032  (lane bit 0)
// `lo` is the value with index bit 0 (kept by lanes whose bit is clear), `hi` the other one.
__device__ __forceinline__ float rs_swap32(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float rs_swap16(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int CTRL>
__device__ __forceinline__ float rs_dpp(float lo, float hi, bool lane_bit) {
    const float keep = lane_bit ? hi : lo;
    const float send = lane_bit ? lo : hi;
    const float got = __uint_as_float(
        __builtin_amdgcn_update_dpp(0u, __float_as_uint(send), CTRL, 0xf, 0xf, false));
    return keep + got;
}
// stage number (1..6) -> combine
template <int STAGE>
__device__ __forceinline__ float rs_stage(float lo, float hi, int lane) {
    if constexpr (STAGE == 1) return rs_swap32(lo, hi);
    else if constexpr (STAGE == 2) return rs_swap16(lo, hi);
    else if constexpr (STAGE == 3) return rs_dpp<0x140>(lo, hi, (lane & 8) != 0);
    else if constexpr (STAGE == 4) return rs_dpp<0x141>(lo, hi, (lane & 4) != 0);
    else if constexpr (STAGE == 5) return rs_dpp<0x1B>(lo, hi, (lane & 2) != 0);
    else return rs_dpp<0xB1>(lo, hi, (lane & 1) != 0);
}

template <int NS, int NW>
struct BwdFastLds {
    static constexpr int NP = NS * NW;
    static constexpr size_t kInputs = 3 * 4 + 2;     // delta, x, dy: four buffers each; u: two
    static constexpr size_t floats = (kInputs + 2 * NW) * kTileF + 2 * kTile * 2 * NP + 2 * 4 * kWave + 4;
};

template <typename IO, int NS, int NW>
__global__ void __launch_bounds__((NW + 4) * kWave)
    sscan_bwd_fast_kernel(const BwdParams p, const float* __restrict__ bcpack) {
    constexpr int NP = NS * NW;
    constexpr int NQ = kTile / 4;
    // channel reduction of dB/dC: 64 values (2 * NS per step, kBatch steps) per reduce-scatter
    constexpr int kStepBits = NS == 2 ? 2 : 3;  // stages spent inside one step: log2(2*NS)
    constexpr int kBatch = 64 / (2 * NS);       // steps per batch
    static_assert(NS == 2 || NS == 4, "reduce-scatter layout written for 2 or 4 states per lane");
    constexpr int kSS = BcPack<NS>::kSS;        // steps per B/C sub-tile
    constexpr int NSUB = kTile / kSS;
    constexpr int kSub = 2 * kSS * NS;          // floats per sub-tile: B then C

    extern __shared__ float4 smem4[];
    float* const smem = reinterpret_cast<float*>(smem4);
    float* const sDl = smem;                      // [4] delta (after softplus)
    float* const sX = sDl + 4 * kTileF;           // [4] x
    float* const sDy = sX + 4 * kTileF;           // [4] dy
    float* const sU = sDy + 4 * kTileF;           // [2] u = delta*x
    float* const sP1 = sU + 2 * kTileF;           // [NW] sum_n g*B
    float* const sP2 = sP1 + NW * kTileF;         // [NW] sum_n g*a*h[t-1]*A*log2(e)
    float* const sRed = sP2 + NW * kTileF;        // [2][kTile][2][NP] dB | dC tile sums
    float* const sDD = sRed + 2 * kTile * 2 * NP;      // [2][4][kWave] dD, ddelta_bias partials
    // one word per reducer wave: index of the last tile whose partial sums it has consumed
    int* const sConsumed = reinterpret_cast<int*>(sDD + 2 * 4 * kWave);

    const int lane = threadIdx.x & (kWave - 1);
    const int w = wave_id();
    const int b = blockIdx.y;
    const int cg = blockIdx.x;
    const int d0 = cg * kWave;
    const int ntiles = p.nchunks;
    const int cmax = min(kWave, p.ED - d0) - 1;  // last valid channel of the group

    // tile index k counts from the END of the sequence: tile k covers chunk c = ntiles-1-k
    auto chunk_of = [&](int k) { return ntiles - 1 - k; };

    if (w >= NW + 2) {
        // ================================ reducers ================================
        const int sw = w - NW - 2;
        int co[2], qo[2];
        bool co_ok[2];
        uint32_t cgo[2];
        float Dr[2];
        float dDb[2] = {0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int item = sw * kWave + lane + r * 2 * kWave;
            co[r] = p.out_tmajor ? item / NQ : item % kWave;
            qo[r] = p.out_tmajor ? item % NQ : item / kWave;
            co_ok[r] = co[r] <= cmax;
            cgo[r] = (uint32_t)min(co[r], cmax) * (uint32_t)p.g_sd;
            Dr[r] = p.D[d0 + min(co[r], cmax)];
        }
        IO* const dxg = static_cast<IO*>(p.dx) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        IO* const ddg = static_cast<IO*>(p.ddelta) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        const int rtid = sw * kWave + lane;  // 0..127: dB/dC forwarding

        auto reduce_store = [&](int k) {
            const int c = chunk_of(k);
            IO* dxk = dxg + (int64_t)c * kTile * p.g_sl;
            IO* ddk = ddg + (int64_t)c * kTile * p.g_sl;
            float4 gBs[2], dds[2];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int ch = co[r], q = qo[r];
                float4 gB = make_float4(0.f, 0.f, 0.f, 0.f), dd = gB;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww) {
                    const float4 a = tile_ld(sP1 + ww * kTileF, ch, q);
                    const float4 e = tile_ld(sP2 + ww * kTileF, ch, q);
                    gB.x += a.x; gB.y += a.y; gB.z += a.z; gB.w += a.w;
                    dd.x += e.x; dd.y += e.y; dd.z += e.z; dd.w += e.w;
                }
                gBs[r] = gB;
                dds[r] = dd;
            }
            // the partial sums of tile k are in registers: the scan waves may overwrite them
            // (the release orders this store after the LDS reads above)
            if (lane == 0)
                __hip_atomic_store(sConsumed + sw, k, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int ch = co[r], q = qo[r];
                const float4 gB = gBs[r], dd = dds[r];
                const float4 dl = tile_ld(sDl + (k & 3) * kTileF, ch, q);
                const float4 xv = tile_ld(sX + (k & 3) * kTileF, ch, q);
                const float4 ddy = tile_ld(sDy + (k & 3) * kTileF, ch, q);
                const float gBv[4] = {gB.x, gB.y, gB.z, gB.w}, ddv[4] = {dd.x, dd.y, dd.z, dd.w};
                const float dlv[4] = {dl.x, dl.y, dl.z, dl.w}, xvv[4] = {xv.x, xv.y, xv.z, xv.w};
                const float dyv[4] = {ddy.x, ddy.y, ddy.z, ddy.w};
                const int t0 = c * kTile + 4 * q;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float dxv = __builtin_fmaf(dlv[j], gBv[j], Dr[r] * dyv[j]);
                    float dv = __builtin_fmaf(xvv[j], gBv[j], ddv[j] * kLn2);
                    if (p.softplus) {
                        // d softplus(r)/dr = sigmoid(r) = 1 - exp(-softplus(r))
                        dv *= (1.0f - __expf(-dlv[j]));
                        if (co_ok[r] && t0 + j < p.L) dDb[r] += dv;
                    }
                    if (co_ok[r] && t0 + j < p.L) {
                        const uint32_t o = (uint32_t)(4 * q + j) * (uint32_t)p.g_sl + cgo[r];
                        dxk[o] = from_float<IO>(dxv);
                        ddk[o] = from_float<IO>(dv);
                    }
                }
            }
            // forward this tile's dB / dC sums over the 64 channels to the partial buffers
            const float* red = sRed + (k & 1) * (kTile * 2 * NP);
            for (int e = rtid; e < kTile * 2 * NP; e += 2 * kWave) {
                const int tt = e / (2 * NP), which = (e / NP) & 1, n = e % NP;
                const int t = c * kTile + tt;
                if (t < p.L && n < p.N) {
                    float* dst = which ? p.partC : p.partB;
                    dst[(((int64_t)cg * p.batch + b) * p.L + t) * p.N + n] = red[e];
                }
            }
        };

        if (lane == 0) sConsumed[sw] = -1;
        __syncthreads();
        __syncthreads();
        for (int k = 0; k < ntiles; ++k) {
            if (k >= 1) reduce_store(k - 1);
            __syncthreads();  // end of interval k
        }
        reduce_store(ntiles - 1);
        if (p.softplus) {
#pragma unroll
            for (int r = 0; r < 2; ++r) sDD[(4 + qo[r]) * kWave + co[r]] = dDb[r];
        }
        __syncthreads();  // final
        return;
    }

    if (w >= NW) {
        // ================================ loaders ================================
        const int sw = w - NW;
        int ci[2], qi[2];
        bool ci_ok[2];
        uint32_t cx[2], cd[2], cy[2];
        float bias[2], dDacc[2] = {0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int item = sw * kWave + lane + r * 2 * kWave;
            ci[r] = p.in_tmajor ? item / NQ : item % kWave;
            qi[r] = p.in_tmajor ? item % NQ : item / kWave;
            ci_ok[r] = ci[r] <= cmax;
            const int cic = min(ci[r], cmax);
            cx[r] = (uint32_t)cic * (uint32_t)p.u_sd;
            cd[r] = (uint32_t)cic * (uint32_t)p.d_sd;
            cy[r] = (uint32_t)cic * (uint32_t)p.y_sd;
            bias[r] = p.dbias ? p.dbias[d0 + cic] : 0.0f;
        }
        const IO* const xg = static_cast<const IO*>(p.x) + (b * p.u_sb + (int64_t)d0 * p.u_sd);
        const IO* const dg = static_cast<const IO*>(p.delta) + (b * p.d_sb + (int64_t)d0 * p.d_sd);
        const IO* const yg = static_cast<const IO*>(p.dy) + (b * p.y_sb + (int64_t)d0 * p.y_sd);

        IO rx[2][4], rd[2][4], ry[2][4];
        auto load_tile = [&](int k) {
            // steps beyond the sequence end are clamped to the last one: loads stay in bounds
            // and free of branches
            const int c = chunk_of(k);
            const int tmax = min(kTile, p.L - c * kTile) - 1;
            const IO* xk = xg + (int64_t)c * kTile * p.u_sl;
            const IO* dk = dg + (int64_t)c * kTile * p.d_sl;
            const IO* yk = yg + (int64_t)c * kTile * p.y_sl;
#pragma unroll
            for (int r = 0; r < 2; ++r) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t tc = (uint32_t)min(4 * qi[r] + j, tmax);
                    rx[r][j] = xk[tc * (uint32_t)p.u_sl + cx[r]];
                    rd[r][j] = dk[tc * (uint32_t)p.d_sl + cd[r]];
                    ry[r][j] = yk[tc * (uint32_t)p.y_sl + cy[r]];
                }
            }
        };
        auto stage_tile = [&](int k) {
            const int c = chunk_of(k);
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int t0 = c * kTile + 4 * qi[r];
                float dl[4], uu[4], xx[4], yy[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // padding (beyond the sequence or the channel count): delta = 0, u = 0,
                    // dy = 0 make the step an exact no-op in both sweeps
                    const bool ok = ci_ok[r] && t0 + j < p.L;
                    const float xv = ok ? to_float(rx[r][j]) : 0.0f;
                    const float yv = ok ? to_float(ry[r][j]) : 0.0f;
                    float dv = to_float(rd[r][j]);
                    if (p.softplus) dv = softplus_f(dv + bias[r]);
                    dv = ok ? dv : 0.0f;
                    dl[j] = dv;
                    uu[j] = dv * xv;
                    xx[j] = xv;
                    yy[j] = yv;
                    dDacc[r] = __builtin_fmaf(yv, xv, dDacc[r]);
                }
                const int ch = ci[r], q = qi[r], s4 = (k & 3) * kTileF;
                tile_st(sDl + s4, ch, q, dl[0], dl[1], dl[2], dl[3]);
                tile_st(sU + (k & 1) * kTileF, ch, q, uu[0], uu[1], uu[2], uu[3]);
                tile_st(sDy + s4, ch, q, yy[0], yy[1], yy[2], yy[3]);
                tile_st(sX + s4, ch, q, xx[0], xx[1], xx[2], xx[3]);
            }
        };

        load_tile(0);
        stage_tile(0);
        if (ntiles > 1) {
            load_tile(1);
            stage_tile(1);
        }
        if (ntiles > 2) load_tile(2);
        __syncthreads();  // tiles 0 and 1 are published
        __syncthreads();
        for (int k = 0; k < ntiles; ++k) {
            if (k + 2 < ntiles) stage_tile(k + 2);
            if (k + 3 < ntiles) load_tile(k + 3);
            __syncthreads();  // end of interval k
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) sDD[qi[r] * kWave + ci[r]] = dDacc[r];
        __syncthreads();  // final
        // dD (and ddelta_bias): sum the four step groups of every channel
        if (sw == 0 && lane <= cmax) {
            float s = 0.0f, sb = 0.0f;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                s += sDD[q * kWave + lane];
                sb += sDD[(4 + q) * kWave + lane];
            }
            p.partD[(int64_t)b * p.ED + d0 + lane] = s;
            if (p.softplus) p.partDb[(int64_t)b * p.ED + d0 + lane] = sb;
        }
        return;
    }

    // ================================= scan waves =================================
    const int d = d0 + lane;
    const bool dvalid = d < p.ED;
    float A2[NS], ag[NS], dAacc[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = w * NS + i;
        const int64_t dn = (int64_t)min(d, p.ED - 1) * p.N + min(n, p.N - 1);
        const float av = p.A[dn];
        A2[i] = (dvalid && n < p.N) ? av * kLog2e : 0.0f;
        ag[i] = 0.0f;
        dAacc[i] = 0.0f;
    }
    // state at the start of chunk c: checkpoint written after chunk c-1, or h0 / zero
    const int64_t ck_lane = (int64_t)min(d, p.ED - 1);
    auto load_state = [&](int k, float (&hs)[NS]) {
        const int c = chunk_of(min(k, ntiles - 1));
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = min(w * NS + i, p.N - 1);
            // branch-free: chunk 0 reads slot 0 (or h0) and the value is masked below
            const float* src = p.ckpt + (((int64_t)b * ntiles + max(c - 1, 0)) * p.N + n) * p.ED + ck_lane;
            const float* src0 = p.h0 ? p.h0 + ((int64_t)b * p.ED + ck_lane) * p.N + n : src;
            const float v = *(c > 0 ? src : src0);
            hs[i] = (c > 0 || p.h0) ? v : 0.0f;
        }
    };
    const float* bc = bcpack + ((int64_t)b * ntiles * NW + w) * (NSUB * kSub);
    const int64_t bc_tile = (int64_t)NW * NSUB * kSub;

    auto read_fwd_inputs = [&](int k, float (&dl)[kTile], float (&uu)[kTile]) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float4 v = tile_ld(sDl + (k & 3) * kTileF, lane, q);
            const float4 u4 = tile_ld(sU + (k & 1) * kTileF, lane, q);
            dl[4 * q] = v.x; dl[4 * q + 1] = v.y; dl[4 * q + 2] = v.z; dl[4 * q + 3] = v.w;
            uu[4 * q] = u4.x; uu[4 * q + 1] = u4.y; uu[4 * q + 2] = u4.z; uu[4 * q + 3] = u4.w;
        }
    };

    // B/C sub-tiles are consumed in the order F0..F(NSUB-1) (recompute, B only) then
    // R(NSUB-1)..R0 (reverse sweep, B and C); fetch number s of a tile lands in bcb[s & 1]
    float bcb[2][kSub];
    float hnext[NS];

    auto tile_pass = [&](int k, const float (&dl)[kTile], const float (&uu)[kTile],
                         float (&dl_next)[kTile], float (&uu_next)[kTile]) {
        const int c = chunk_of(k);
        const float* bck = bc + (int64_t)c * bc_tile;
        const float* bck_next = bc + (int64_t)max(c - 1, 0) * bc_tile;
        float h[NS];
#pragma unroll
        for (int i = 0; i < NS; ++i) h[i] = hnext[i];

        // ---- 1. recompute the tile forward, keeping a and a*h[t-1] ----
        float aS[kTile][NS], tS[kTile][NS], dyq[2][4];
#pragma unroll
        for (int tt = 0; tt < kTile; ++tt) {
            const int sub = tt / kSS, ts = tt % kSS;
            const float(&cur)[kSub] = bcb[sub & 1];
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const float a = fast_exp2(dl[tt] * A2[i]);
                const float th = a * h[i];
                aS[tt][i] = a;
                tS[tt][i] = th;
                h[i] = __builtin_fmaf(uu[tt], cur[ts * NS + i], th);
            }
            if (ts == 0) {
                // next fetch right after the first use of the current one (the wait before a
                // first use drains every scalar load and LDS read in flight)
                __builtin_amdgcn_sched_barrier(0);
                if (sub + 1 < NSUB)
                    scalar_load<kSub>(bck + (sub + 1) * kSub, bcb[(sub + 1) & 1]);
                else
                    scalar_load<kSub>(bck + (NSUB - 1) * kSub, bcb[NSUB & 1]);
                if (sub == 0) load_state(k + 1, hnext);
                if (sub == NSUB - 1) {
                    // dy of the last four steps, needed when the reverse sweep starts
                    const float4 v = tile_ld(sDy + (k & 3) * kTileF, lane, NQ - 1);
                    dyq[(NQ - 1) & 1][0] = v.x; dyq[(NQ - 1) & 1][1] = v.y;
                    dyq[(NQ - 1) & 1][2] = v.z; dyq[(NQ - 1) & 1][3] = v.w;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- 2. reverse sweep ----
        float gBv[kTile], ddv[kTile];
        float pend[4];
#pragma unroll
        for (int tt = kTile - 1; tt >= 0; --tt) {
            const int sub = tt / kSS, ts = tt % kSS;
            const int fetch = NSUB + (NSUB - 1 - sub);  // fetch number of this sub-tile
            const float(&cur)[kSub] = bcb[fetch & 1];
            if ((tt & 3) == 3 && tt >= 4) {
                // dy of the next (earlier) four steps, one group ahead of use
                const int qn = (tt >> 2) - 1;
                const float4 v = tile_ld(sDy + (k & 3) * kTileF, lane, qn);
                dyq[qn & 1][0] = v.x; dyq[qn & 1][1] = v.y; dyq[qn & 1][2] = v.z; dyq[qn & 1][3] = v.w;
            }
            const float dyv = dyq[(tt >> 2) & 1][tt & 3];
            float gB = 0.0f, dd = 0.0f;
            float pB[NS], pC[NS];
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const float bv = cur[ts * NS + i];
                const float cv = cur[kSS * NS + ts * NS + i];
                const float g = __builtin_fmaf(dyv, cv, ag[i]);
                const float hh = __builtin_fmaf(uu[tt], bv, tS[tt][i]);
                const float gha = g * tS[tt][i];
                dAacc[i] = __builtin_fmaf(gha, dl[tt], dAacc[i]);
                dd = __builtin_fmaf(gha, A2[i], dd);
                gB = __builtin_fmaf(g, bv, gB);
                ag[i] = aS[tt][i] * g;
                pB[i] = g * uu[tt];
                pC[i] = dyv * hh;
            }
            gBv[tt] = gB;
            ddv[tt] = dd;

            if (ts == kSS - 1) {
                // first use of this sub-tile is done: fetch the next one in reverse order, or
                // the first forward sub-tile of the next tile
                __builtin_amdgcn_sched_barrier(0);
                if (sub > 0)
                    scalar_load<kSub>(bck + (sub - 1) * kSub, bcb[(fetch + 1) & 1]);
                else
                    scalar_load<kSub>(bck_next, bcb[0]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (tt == 2) {
                // the registers of the consumed steps are free: fetch delta/u of the next tile
                __builtin_amdgcn_sched_barrier(0);
                read_fwd_inputs(k + 1, dl_next, uu_next);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- channel reduction of this step's dB / dC products (see rs_stage) ----
            // value index bits, from stage 1 up: dB|dC, the state index, then the step index
            // inside the batch; steps arrive in descending order, so a step with a set index
            // bit waits in `pend` for its partner with the bit clear
            {
                float r;
                if constexpr (NS == 2) {
                    r = rs_stage<2>(rs_stage<1>(pB[0], pC[0], lane), rs_stage<1>(pB[1], pC[1], lane), lane);
                } else {
                    const float a0 = rs_stage<1>(pB[0], pC[0], lane), a1 = rs_stage<1>(pB[1], pC[1], lane);
                    const float a2 = rs_stage<1>(pB[2], pC[2], lane), a3 = rs_stage<1>(pB[3], pC[3], lane);
                    r = rs_stage<3>(rs_stage<2>(a0, a2, lane), rs_stage<2>(a1, a3, lane), lane);
                }
                const int sb = tt % kBatch;  // step inside the batch
                if (sb & 1) {
                    pend[0] = r;
                } else {
                    r = rs_stage<kStepBits + 1>(r, pend[0], lane);
                    if (sb & 2) {
                        pend[1] = r;
                    } else {
                        r = rs_stage<kStepBits + 2>(r, pend[1], lane);
                        if (sb & 4) {
                            pend[2] = r;
                        } else {
                            r = rs_stage<kStepBits + 3>(r, pend[2], lane);
                            if constexpr (kBatch == 16) {
                                if (sb & 8) {
                                    pend[3] = r;
                                } else {
                                    r = rs_stage<6>(r, pend[3], lane);
                                }
                            }
                            if (sb == 0) {
                                // lane l holds value number l: decode (step, dB|dC, state)
                                const int which = lane >> 5;
                                const int st = NS == 2 ? (lane >> 4) & 1 : (((lane >> 4) & 1) << 1) | ((lane >> 3) & 1);
                                const int stp = NS == 2 ? (lane & 1) << 3 | (lane & 2) << 1 | (lane & 4) >> 1 | (lane & 8) >> 3
                                                        : (lane & 1) << 2 | (lane & 2) | (lane & 4) >> 2;
                                sRed[(k & 1) * (kTile * 2 * NP) + ((tt + stp) * 2 + which) * NP + w * NS + st] = r;
                            }
                        }
                    }
                }
            }
        }
        // The partial sums go to single-buffered LDS tiles.  The reducers read tile k-1 at the
        // start of this interval and publish that in sConsumed; by the end of the sweep that
        // has long happened, so this wait normally falls through (bounded: a wave never
        // spins forever).
        if (k >= 1) {
            int spins = 0;
            while ((__hip_atomic_load(sConsumed, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < k - 1 ||
                    __hip_atomic_load(sConsumed + 1, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < k - 1) &&
                   ++spins < (1 << 20))
                __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            tile_st(sP1 + w * kTileF, lane, q, gBv[4 * q], gBv[4 * q + 1], gBv[4 * q + 2], gBv[4 * q + 3]);
            tile_st(sP2 + w * kTileF, lane, q, ddv[4 * q], ddv[4 * q + 1], ddv[4 * q + 2], ddv[4 * q + 3]);
        }
        __syncthreads();  // end of interval k: partial sums and dB/dC sums of tile k are visible
    };

    float dlA[kTile], uuA[kTile], dlB[kTile], uuB[kTile];
    scalar_load<kSub>(bc + (int64_t)chunk_of(0) * bc_tile, bcb[0]);
    load_state(0, hnext);
    __syncthreads();
    read_fwd_inputs(0, dlA, uuA);
    __syncthreads();
    for (int k = 0; k < ntiles; k += 2) {
        tile_pass(k, dlA, uuA, dlB, uuB);
        if (k + 1 >= ntiles) break;
        tile_pass(k + 1, dlB, uuB, dlA, uuA);
    }
    // per-batch partial of dA
    if (dvalid) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = w * NS + i;
            if (n < p.N) p.partA[((int64_t)b * p.ED + d) * p.N + n] = dAacc[i];
        }
    }
    __syncthreads();  // final
}

template <typename IO, int NS, int NW>
static int launch_fast(const BwdParams& p, const float* bcpack, hipStream_t stream) {
    dim3 grid((p.ED + kWave - 1) / kWave, p.batch);
    dim3 block((NW + 4) * kWave);
    constexpr size_t lds = sizeof(float) * BwdFastLds<NS, NW>::floats;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static const int attr_rc = allow_dynamic_lds(sscan_bwd_fast_kernel<IO, NS, NW>, lds);
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((sscan_bwd_fast_kernel<IO, NS, NW>), grid, block, lds, stream, p, bcpack);
    return check_launch();
}

bool bwd_fast_supported(int ns, int nw) { return (ns == 2 && nw == 8) || (ns == 4 && nw == 4); }

int launch_bwd_fast(const BwdParams& p, const float* bcpack, int ns, int nw, int io_dtype,
                    hipStream_t stream) {
#define MPA_CASE(NS_, NW_)                                                           \
    if (ns == NS_ && nw == NW_)                                                      \
        return io_dtype == MPA_F32 ? launch_fast<float, NS_, NW_>(p, bcpack, stream) \
                                   : launch_fast<bf16_t, NS_, NW_>(p, bcpack, stream);
    MPA_CASE(2, 8) MPA_CASE(4, 4)
#undef MPA_CASE
    return MPA_ERR_BAD_SHAPE;
}

}  // namespace mpa
