// Fused selective-scan backward for gfx950, fast path.
//
// A workgroup owns 64 channels of one batch row and walks the sequence from the last tile of
// kTile steps to the first.
//   * NW scan waves split d_state (NS states per lane, one channel per lane).  Per tile a
//     scan wave reloads the state at the tile start from the forward checkpoints, recomputes
//     the kTile steps keeping a[t] and h[t] in registers (the recurrence is never
//     inverted: dividing by a[t] amplifies rounding error), then sweeps the tile backwards:
//         g[t] = dy[t]*C[t] + a[t+1]*g[t+1]
//         d(delta*A) = g*a*h[t-1]   -> dA += .*delta ;  ddelta += .*A
//         sum_n g*B                 -> dx = delta*. ;   ddelta += x*.
//         g*u (u = delta*x), dy*h   -> dB, dC: summed over the lanes of a row as far as plain DPP
//                                      additions go (rs_stage), the rest by the service waves.
//     B and C of a tile sit in one register per state whose lane t of every row of 16 lanes
//     holds step t; the FMAs pick their step with a DPP row broadcast (fmac_bcast), so B and C
//     cost neither scalar registers nor extra instructions.
//   * four service waves, one item of (channel, 4 steps) per thread and tile, do everything
//     else: they request x, delta, dy, B, C five tiles ahead (three tiles in flight), convert,
//     apply softplus and publish delta, u, dy, x, B, C as float32 LDS tiles two tiles ahead
//     (accumulating dD on the way); one tile behind the scan they sum the partial sum_n over
//     the scan waves, finish dx and ddelta (softplus chain rule included), store them, and
//     forward the per-tile dB/dC sums to the per-channel-group partial buffers.  Their
//     per-tile code is short and has one uniform branch for the ragged edge: a lone wave
//     issues an instruction only every ~6 clocks and pays tens of clocks per branch, and every
//     instruction it issues takes a VALU slot away from the scan waves of its SIMD.
// Tiles in LDS are float32 planes of [64 channels][4 steps] (see tile_off).
// Reductions over channel groups, batch and time go through deterministic partial buffers
// summed by sscan_bwd_finish_kernel (no floating-point atomics: results are bitwise
// reproducible).
#include <type_traits>

#include "sscan_bwd.h"

namespace mpa {

// A tile of (64 channels x kTile steps) in LDS is kTile/4 planes; plane q holds steps 4q..4q+3 of every
// channel, the channel index fastest (16 bytes per channel).  A wave that reads or writes one plane with
// one channel per lane touches 1 KB of consecutive addresses: no bank conflicts and no padding inside the
// plane (a [channel][step] tile needs a pitch of 20 floats for that).  Planes are 8 floats further apart
// than their 256 floats, so that threads that walk the planes of a few channels (the step-major item map
// of the service waves) do not all start in the same bank.
constexpr int kPlane = kWave * 4 + 8;
constexpr int kTileF = (kTile / 4) * kPlane;  // floats per LDS tile

// float index of the 16-byte column q (4 steps) of channel ch inside a tile
__device__ __forceinline__ int tile_off(int ch, int q) { return q * kPlane + ch * 4; }

__device__ __forceinline__ float4 tile_ld(const float* tile, int ch, int q) {
    return *reinterpret_cast<const float4*>(tile + tile_off(ch, q));
}
__device__ __forceinline__ void tile_st(float* tile, int ch, int q, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(tile + tile_off(ch, q)) = make_float4(a, b, c, d);
}

// ---- reduce-scatter over the lanes of a row (first part of the dB / dC channel sums) ---------
// A sum over the lanes of a wave can be taken in halving stages: a stage combines two registers
// into one, a lane keeping the value whose index bit equals the stage's lane bit and receiving
// its partner lane's share of it, so each value costs less than one addition per stage and no
// LDS round trip sits in the dependency chain of the reverse sweep.  The scan waves run only the
// stages that stay inside a row of 16 lanes and are plain DPP additions (two at two states per
// lane, three at four); the 16 / 2^stages partial sums per value and row that are left go to LDS
// as they are and the service waves add them one tile later (the stages across rows are lane
// swaps at twice the cost of a DPP addition each, and the scattered stores that followed them
// cost more than the 30 additions per service thread that replaced them).
//   stage 1: DPP row_mirror      (lane bit 3)     stage 3: DPP quad_perm 3210  (lane bit 1)
//   stage 2: DPP row_half_mirror (lane bit 2)
// (every stage's partner lane agrees with the lane in the bits of the stages before it)
// `lo` is the value with index bit 0 (kept by lanes whose bit is clear), `hi` the other one.
template <int CTRL>
__device__ __forceinline__ float rs_dpp(float lo, float hi, bool lane_bit) {
    const float keep = lane_bit ? hi : lo;
    const float send = lane_bit ? lo : hi;
    const float got = __uint_as_float(
        __builtin_amdgcn_update_dpp(0u, __float_as_uint(send), CTRL, 0xf, 0xf, false));
    return keep + got;
}
// Stages 1 and 2 without selects: the lanes whose bit is clear form whole banks (groups of four
// lanes) of a row, so two additions that each write only their banks do the work: lanes with the
// bit clear get lo + lo[partner], the others hi + hi[partner].  (The compiler does not see into
// inline assembly: the two wait states a DPP read needs after a VALU write of the same register
// are written out.)
__device__ __forceinline__ float rs_mirror8(float lo, float hi) {
    float r;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %1, %1 row_mirror row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %2, %2 row_mirror row_mask:0xf bank_mask:0xc"
        : "=&v"(r)
        : "v"(lo), "v"(hi));
    return r;
}
__device__ __forceinline__ float rs_mirror4(float lo, float hi) {
    float r;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %1, %1 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %0, %2, %2 row_half_mirror row_mask:0xf bank_mask:0xa"
        : "=&v"(r)
        : "v"(lo), "v"(hi));
    return r;
}
// stage number (1..3) -> combine
template <int STAGE>
__device__ __forceinline__ float rs_stage(float lo, float hi, int lane) {
    static_assert(STAGE >= 1 && STAGE <= 3, "the scan waves run the stages inside a row only");
    if constexpr (STAGE == 1) return rs_mirror8(lo, hi);
    else if constexpr (STAGE == 2) return rs_mirror4(lo, hi);
    else return rs_dpp<0x1B>(lo, hi, (lane & 2) != 0);
}

constexpr int kSvc = 4;  // service waves per workgroup

// compile-time loop: f(std::integral_constant<int, I>) for I = 0 .. N-1
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// dB/dC products of one scan wave and tile, summed over groups of 2*NS lanes by the wave's in-register
// stages: [kTile steps][64 lanes]; four floats between the waves' blocks, so that service threads that
// read the same row of different waves start in different banks
constexpr int kRpW = kTile * kWave + 4;

template <int NS, int NW>
struct BwdFastLds {
    static constexpr int NP = NS * NW;
    static constexpr size_t kInputs = 3 * 4 + 2;     // delta, x, dy: four buffers each; u: two
    // + partial sums per scan wave, dB|dC lane-group sums [NW][kRpW], B|C tiles
    // [2][2][NP][kTile], consumption flags
    static constexpr size_t floats =
        (kInputs + 2 * NW) * kTileF + NW * kRpW + 2 * 2 * NP * kTile + 4;
};

// HAS_Z: the forward multiplied its output by silu(z).  The service waves then read z and the
// saved pre-gate output next to dy, publish dy*silu(z) as the dy tile (everything downstream is
// unchanged) and store dz = dy * y_pre * d silu(z)/dz.
// ACC: a pass after the first over the states of a wide d_state: it adds to the dx and ddelta
// that are there and leaves D*dy, dD and dz to the first pass.
template <typename IO, int NS, int NW, bool HAS_Z, bool ACC>
__global__ void __launch_bounds__((NW + kSvc) * kWave) sscan_bwd_fast_kernel(const BwdParams p) {
    constexpr int NP = NS * NW;
    constexpr int NQ = kTile / 4;
    static_assert(kSvc == NQ, "one service thread per (channel, 4 steps) item of a tile");
    // channel reduction of dB/dC: the 2 * NS products of a step are summed over groups of 2 * NS lanes in
    // registers (reduce-scatter stages inside a row of 16 lanes); kLanesPer lanes of every row then hold
    // partial sums of one (dB|dC, state) value, and the service waves add those up
    static_assert(NS == 2 || NS == 4, "reduce-scatter layout written for 2 or 4 states per lane");
    constexpr int kLanesPer = 16 / (2 * NS);
    constexpr int kRedF = kTile * 2 * NP;       // dB|dC values of one tile
    constexpr int kBcF = 2 * NP * kTile;        // floats of one B|C tile

    extern __shared__ float4 smem4[];
    float* const smem = reinterpret_cast<float*>(smem4);
    float* const sDl = smem;                      // [4] delta (after softplus)
    float* const sX = sDl + 4 * kTileF;           // [4] x
    float* const sDy = sX + 4 * kTileF;           // [4] dy
    float* const sU = sDy + 4 * kTileF;           // [2] u = delta*x
    float* const sP1 = sU + 2 * kTileF;           // [NW] sum_n g*B
    float* const sP2 = sP1 + NW * kTileF;         // [NW] sum_n g*a*h[t-1]*A*log2(e)
    float* const sRP = sP2 + NW * kTileF;         // [NW][kTile][64] dB | dC lane-group sums
    float* const sBC = sRP + NW * kRpW;           // [2][B|C][NP][kTile]
    // counts (service wave, tile) pairs whose partial sums have been consumed: kSvc * (k + 1)
    // once every service wave is done with tile k
    int* const sConsumed = reinterpret_cast<int*>(sBC + 2 * kBcF);

    const int lane = threadIdx.x & (kWave - 1);
    const int w = wave_id();
    // Row of the launch: a batch row, or one segment of it.  Tiles of the row are counted from
    // the end of the forward walk: tile k of the row is backward-walk tile k0 + k.
    const int bs = blockIdx.y;
    int b = bs, k0 = 0, ntiles = p.nchunks;
    if (p.nseg > 1) {
        b = bs / p.nseg;
        k0 = (bs - b * p.nseg) * p.seg_tiles;
        ntiles = min(p.seg_tiles, p.nchunks - k0);
    }
    const int cg = blockIdx.x;
    const int d0 = cg * kWave;
    const int cmax = min(kWave, p.ED - d0) - 1;  // last valid channel of the group
    const bool rev = p.reverse != 0;
    const int last_chunk = p.nchunks - 1;
    const bool ragged_seq = p.nchunks * kTile > p.L;
    // dD / ddelta_bias partials [2][4][kWave]: written once at the very end, into the delta
    // buffer that no tile uses any more
    float* const sDD = sDl + (ntiles & 3) * kTileF;

    // tile k of the row is walk tile c of the forward pass (the index of its checkpoint), which
    // covers physical chunk c, or last_chunk - c when the forward walk ran in reverse; inside a
    // tile walk step s is physical step s or kTile-1-s
    auto chunk_of = [&](int k) { return last_chunk - (k0 + k); };
    auto phys_of = [&](int c) { return rev ? last_chunk - c : c; };

    if (w >= NW) {
        // ================================ service waves ================================
        const int sw = w - NW;
        const int item = sw * kWave + lane;  // 0 .. 255
        // with softplus or the gate the service waves carry long chains of transcendental
        // functions and would reach the tile barrier last: they then go first when ready
#ifndef MPA_PRIO_SVC
#define MPA_PRIO_SVC 1
#endif
        if (HAS_Z || p.softplus) __builtin_amdgcn_s_setprio(2);
        else __builtin_amdgcn_s_setprio(MPA_PRIO_SVC);
        constexpr uint32_t kES = sizeof(IO);
        const bool group_full = cmax == kWave - 1;
        // With a gate the service waves carry two more input streams, set the kernel's register count
        // and spill scalar registers into vector lanes; three of the forms below (marked kLean: a few
        // instructions less, a few more live values) measured slower there (gated backward +1.5 % with
        // the first two, +2 % with the third) and a gated kernel keeps the plainer ones.
        constexpr bool kLean = !HAS_Z;

        // ---- input side: item -> (channel, step group), offsets that never change ----
        const int ci = p.in_tmajor ? item / NQ : item % kWave;
        const int qi = p.in_tmajor ? item % NQ : item / kWave;  // walk step group of the item
        // its physical step group (recomputed where it is used: not kept alive across the tiles)
        auto qp_now = [&]() { return rev ? NQ - 1 - qi : qi; };
        const int qp = qp_now();
        auto jw = [&](int j) { return (uint32_t)(rev ? 3 - j : j); };  // walk step j of an item -> physical
        const bool ci_ok = ci <= cmax;
        const int cic = min(ci, cmax);
        const float bias = p.dbias ? p.dbias[d0 + cic] : 0.0f;
        IO* const dzg = static_cast<IO*>(p.dz) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        // byte offset of the item's lowest physical step (one vector register per tensor); walk
        // step j of the item is jw(j) row strides further, which goes into the scalar offset
        const uint32_t offx = ((uint32_t)(4 * qp) * (uint32_t)p.u_sl + (uint32_t)cic * (uint32_t)p.u_sd) * kES;
        // (delta and ddelta may be float32 next to bfloat16 tensors: element size and conversion shift of their own)
        const bool d_wide = sizeof(IO) == 4 || p.delta_f32;
        const uint32_t kESd = d_wide ? 4u : 2u;
        const uint32_t dshift = __builtin_amdgcn_readfirstlane(d_wide ? 0u : 16u);
        const uint32_t offd = ((uint32_t)(4 * qp) * (uint32_t)p.d_sl + (uint32_t)cic * (uint32_t)p.d_sd) * kESd;
        const uint32_t offy = ((uint32_t)(4 * qp) * (uint32_t)p.y_sl + (uint32_t)cic * (uint32_t)p.y_sd) * kES;
        const uint32_t offzi = ((uint32_t)(4 * qp) * (uint32_t)p.z_sl + (uint32_t)cic * (uint32_t)p.z_sd) * kES;
        const uint32_t offz = ((uint32_t)(4 * qp) * (uint32_t)p.g_sl + (uint32_t)cic * (uint32_t)p.g_sd) * kES;  // dz
        // Scalar byte offsets of an item's four walk steps: jw(j) row strides.  Only the row stride of
        // each tensor is kept (one scalar register); the four products are formed by the scalar unit
        // where they are used.  Computed once and kept, the twenty offsets did not fit the scalar
        // register file next to the tensor addresses: they were parked in lanes of a vector register
        // and every access paid a lane read on the vector unit and its wait states.
        // (readfirstlane: told to the compiler as wave-uniform; an offset it takes for per-lane costs
        // a loop over its values per access)
        const uint32_t rowx = __builtin_amdgcn_readfirstlane((uint32_t)p.u_sl * kES);
        const uint32_t rowd = __builtin_amdgcn_readfirstlane((uint32_t)p.d_sl * kESd);
        const uint32_t rowy = __builtin_amdgcn_readfirstlane((uint32_t)p.y_sl * kES);
        const uint32_t rowz = __builtin_amdgcn_readfirstlane((uint32_t)p.z_sl * kES);
        const uint32_t rowg = __builtin_amdgcn_readfirstlane((uint32_t)p.g_sl * kES);
        // the four offsets of a tensor, from a copy of the stride that the compiler cannot trace back
        // (it would otherwise hoist the products out of the tile loop and keep all of them again)
        struct Steps { uint32_t at[4]; };
        auto steps_of = [&](uint32_t row) {
            asm volatile("" : "+s"(row));
            Steps r;
#pragma unroll
            for (int j = 0; j < 4; ++j) r.at[j] = jw(j) * row;
            return r;
        };
        // origin of physical chunk pc in a tensor whose rows are `row` bytes (`stride` elements of the
        // pointer's type) apart.  Without a gate: a 32 x 32 -> 64 bit product of the scalar unit on the
        // stride register that steps_of uses (with the 64-bit element strides of the arguments, each
        // tensor keeps two more scalar registers alive and every tile pays a 64 x 64 bit product:
        // backward at B=8, L=2048, 1536 channels, float32: 0.302 -> 0.297 ms).  The gated kernels
        // measured 2 % slower with it (their register allocation again) and keep the 64-bit form.
        auto at_chunk = [&](auto* base, int pc, uint32_t row, int64_t stride) {
            typedef decltype(base) P;
            if constexpr (kLean) {
                const uint64_t off = (uint64_t)(uint32_t)(pc * kTile) * (uint64_t)row;
                return reinterpret_cast<P>(reinterpret_cast<uintptr_t>(base) + off);
            } else {
                return base + (int64_t)pc * kTile * stride;
            }
        };
        const uint32_t rowbc = __builtin_amdgcn_readfirstlane((uint32_t)p.bc_sl * kES);
        const uint32_t rowfw = __builtin_amdgcn_readfirstlane((uint32_t)p.Nst * 4u);
        // tensor origins of this (batch row, channel group)
        const IO* const xb = static_cast<const IO*>(p.x) + (b * p.u_sb + (int64_t)d0 * p.u_sd);
        const char* const db = static_cast<const char*>(p.delta) + (b * p.d_sb + (int64_t)d0 * p.d_sd) * (int64_t)kESd;
        const IO* const yb = static_cast<const IO*>(p.dy) + (b * p.y_sb + (int64_t)d0 * p.y_sd);
        const IO* const zb = static_cast<const IO*>(p.z) + (b * p.z_sb + (int64_t)d0 * p.z_sd);
        const IO* const ypb = static_cast<const IO*>(p.ypre) + (b * p.y_sb + (int64_t)d0 * p.y_sd);
        const IO* const Bb = static_cast<const IO*>(p.Bm) + b * p.bc_sb;
        const IO* const Cb = static_cast<const IO*>(p.C) + b * p.bc_sb;
        // Loads of the ragged chunk run past the sequence end.  That is harmless (the values are
        // masked at staging) as long as the address is inside the tensor: the ragged chunk is
        // read through windows that end with the tensor's last element, whatever the strides
        // (out-of-window loads return zero).
        // B/C of a tile: kTile * NP elements each, kBcPer per service thread, step fastest
        constexpr int kBcPer = NP * kTile / (kSvc * kWave);
        static_assert(NP * kTile % (kSvc * kWave) == 0, "whole elements per thread");
        int bct[kBcPer], bcn[kBcPer];
        uint32_t offbc[kBcPer];
#pragma unroll
        for (int r = 0; r < kBcPer; ++r) {
            const int e = item + r * (kSvc * kWave);
            bct[r] = e % kTile;  // walk step
            bcn[r] = e / kTile;
            offbc[r] = ((uint32_t)(rev ? kTile - 1 - bct[r] : bct[r]) * (uint32_t)p.bc_sl +
                        (uint32_t)min(bcn[r], p.N - 1)) * kES;
        }

        // ---- output side: item -> (channel, step group) ----
        const int co = p.out_tmajor ? item / NQ : item % kWave;
        const int qo = p.out_tmajor ? item % NQ : item / kWave;
        const int qpo = rev ? NQ - 1 - qo : qo;
        const bool co_ok = co <= cmax;
        // (a pass after the first over the states of a wide d_state adds to dx, ddelta; D*dy, dD and dz
        // belong to the first one)
        const float Dr = ACC ? 0.0f : p.D[d0 + min(co, cmax)];
        const uint32_t offg = ((uint32_t)(4 * qpo) * (uint32_t)p.g_sl + (uint32_t)min(co, cmax) * (uint32_t)p.g_sd) * kES;
        IO* const dxg = static_cast<IO*>(p.dx) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        IO* const ddg = static_cast<IO*>(p.ddelta) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        // ddelta as float32 next to bfloat16 tensors: same element offsets, twice the bytes
        const bool dd_wide = sizeof(IO) == 2 && p.delta_f32;
        float* const ddgf = static_cast<float*>(p.ddelta) + (b * p.g_sb + (int64_t)d0 * p.g_sd);
        // dB/dC forwarding: kFw consecutive states of one (step, dB|dC) per thread
        constexpr int kFw = kRedF / (kSvc * kWave);
        static_assert(kRedF % (kSvc * kWave) == 0 && NP % kFw == 0 && (kFw == 2 || kFw == 4), "forwarding layout");
        // (even service waves forward dB, odd ones dC, so that the destination is wave-uniform)
        const int fw_which = sw & 1;
        const int fw_i = ((sw >> 1) * kWave + lane) * kFw;  // index inside the [kTile][NP] half
        const int fw_tt = fw_i / NP, fw_n = fw_i % NP;        // walk step, state
        const int fw_tp = rev ? kTile - 1 - fw_tt : fw_tt;    // physical step inside the chunk
        // its values in a scan wave's block of lane-group sums: row fw_tt, lanes (of every row of 16)
        // fw_which * 8 + (state inside the wave) * kLanesPer onwards, kFw * kLanesPer of them
        static_assert(kFw == 2 && NS % kFw == 0, "a thread forwards two states of one scan wave");
        const int fw_rp = (fw_n / NS) * kRpW + fw_tt * kWave + fw_which * 8 + (fw_n % NS) * kLanesPer;
        float* const fw_base = (fw_which ? p.partC : p.partB) + cg * p.part_gs + (int64_t)b * p.L * p.Nst;
        const uint32_t fw_off = ((uint32_t)fw_tp * (uint32_t)p.Nst + (uint32_t)fw_n) * 4u;
        const bool fw_vec = p.N == NP && p.Nst % 4 == 0;  // rows of the partial buffers are then aligned for vector stores

        float dDacc = 0.0f, dDb = 0.0f;

        // Raw values of three tiles in flight (see the forward kernel: HBM latency under load
        // is longer than one tile interval)
        struct Raw { IO x[4], y[4], z[HAS_Z ? 4 : 1], yp[HAS_Z ? 4 : 1], b[kBcPer], c[kBcPer]; uint32_t d[4]; };
        auto load_tile = [&](int kk, Raw& raw) {
            // tiles beyond the last one are clamped to it; steps beyond the sequence end are read
            // as whatever follows inside the tensor (or zero past its end) and masked at staging
            const int k = min(kk, ntiles - 1);
            const int pc = phys_of(chunk_of(k));
            const IO* xk = at_chunk(xb, pc, rowx, p.u_sl);
            const char* dk = at_chunk(db, pc, rowd, p.d_sl * (int64_t)kESd);
            const IO* yk = at_chunk(yb, pc, rowy, p.y_sl);
            const IO* zk = at_chunk(zb, pc, rowz, p.z_sl);
            const IO* ypk = at_chunk(ypb, pc, rowy, p.y_sl);
            const IO* Bk = at_chunk(Bb, pc, rowbc, p.bc_sl);
            const IO* Ck = at_chunk(Cb, pc, rowbc, p.bc_sl);
            uint32_t wx = 0xffffffffu, wd = wx, wy = wx, wz = wx, wbc = wx;
            if (ragged_seq && pc == last_chunk) {
                // elements from this chunk's origin to one past the tensor's last element
                const int64_t tb = (int64_t)pc * kTile;
                auto left = [&](int64_t sb_, int64_t sl_, int64_t sd_, int64_t width, int es = (int)sizeof(IO)) {
                    const int64_t end = (p.batch - 1) * sb_ + (p.L - 1) * sl_ + (width - 1) * sd_ + 1;
                    return window_bytes(end, b * sb_ + tb * sl_ + (int64_t)d0 * sd_, es);
                };
                wx = left(p.u_sb, p.u_sl, p.u_sd, p.ED);
                wd = left(p.d_sb, p.d_sl, p.d_sd, p.ED, kESd);
                wy = left(p.y_sb, p.y_sl, p.y_sd, p.ED);
                wz = left(p.z_sb, p.z_sl, p.z_sd, p.ED);
                wbc = window_bytes((p.batch - 1) * p.bc_sb + (p.L - 1) * p.bc_sl + p.N, b * p.bc_sb + tb * p.bc_sl, kES);
            }
            const Steps sx = steps_of(rowx), sy = steps_of(rowy), sd = steps_of(rowd);
            const Steps sz = steps_of(rowz);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                raw.x[j] = ld_off(xk, offx, sx.at[j], wx);
                raw.y[j] = ld_off(yk, offy, sy.at[j], wy);
                if constexpr (HAS_Z) {
                    raw.z[j] = ld_off(zk, offzi, sz.at[j], wz);
                    raw.yp[j] = ld_off(ypk, offy, sy.at[j], wy);
                }
            }
            if (d_wide) {
#pragma unroll
                for (int j = 0; j < 4; ++j) raw.d[j] = ld_bits32(dk, offd, sd.at[j], wd);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) raw.d[j] = ld_bits16(dk, offd, sd.at[j], wd);
            }
#pragma unroll
            for (int r = 0; r < kBcPer; ++r) {
                raw.b[r] = ld_off(Bk, offbc[r], 0, wbc);
                raw.c[r] = ld_off(Ck, offbc[r], 0, wbc);
            }
        };
        auto stage_tile = [&](int k, const Raw& raw) {
            const int pc = phys_of(chunk_of(k));
            float xv[4], dv[4], yv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                xv[j] = to_float(raw.x[j]);
                dv[j] = bits_to_float(raw.d[j], dshift);
                yv[j] = to_float(raw.y[j]);
            }
            if (p.softplus) {
#pragma unroll
                for (int j = 0; j < 4; ++j) dv[j] = softplus_f(dv[j] + bias);
            }
            float dzv[4];
            if constexpr (HAS_Z) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float zv = to_float(raw.z[j]);
                    const float sg = sigmoid_f(zv);
                    // d/dz (z*sigmoid(z)) = sigmoid(z) * (1 + z*(1 - sigmoid(z)))
                    dzv[j] = yv[j] * to_float(raw.yp[j]) * sg * __builtin_fmaf(zv, 1.0f - sg, 1.0f);
                    yv[j] *= zv * sg;
                }
            }
            const bool ragged = !group_full || (ragged_seq && pc == last_chunk);
            if constexpr (HAS_Z && !ACC) {
                IO* dzk = at_chunk(dzg, pc, rowg, p.g_sl);
                const Steps sg = steps_of(rowg);
                if (!ragged) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) st_off(dzk, offz, from_float<IO>(dzv[j]), sg.at[j]);
                } else {
                    const int t0 = pc * kTile + 4 * qp_now();
                    for (int j = 0; j < 4; ++j)
                        if (ci_ok && t0 + (int)jw(j) < p.L) st_off(dzk, offz, from_float<IO>(dzv[j]), sg.at[j]);
                }
            }
            if (ragged) {
                // padding (beyond the sequence or the channel count): delta = 0, u = 0, dy = 0
                // make the step an exact no-op in both sweeps
                const int t0 = pc * kTile + 4 * qp_now();
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool ok = ci_ok && t0 + (int)jw(j) < p.L;
                    xv[j] = ok ? xv[j] : 0.0f;
                    dv[j] = ok ? dv[j] : 0.0f;
                    yv[j] = ok ? yv[j] : 0.0f;
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) dDacc = __builtin_fmaf(yv[j], xv[j], dDacc);  // (dropped at the end by a later pass)
            const int s4 = (k & 3) * kTileF;
            tile_st(sDl + s4, ci, qi, dv[0], dv[1], dv[2], dv[3]);
            tile_st(sU + (k & 1) * kTileF, ci, qi, dv[0] * xv[0], dv[1] * xv[1], dv[2] * xv[2], dv[3] * xv[3]);
            tile_st(sDy + s4, ci, qi, yv[0], yv[1], yv[2], yv[3]);
            tile_st(sX + s4, ci, qi, xv[0], xv[1], xv[2], xv[3]);
#pragma unroll
            for (int r = 0; r < kBcPer; ++r) {
                // states beyond d_state: B = C = 0 (padded steps need no care: u = dy = 0)
                const bool ok = bcn[r] < p.N;
                float* dst = sBC + (k & 1) * kBcF + bcn[r] * kTile + bct[r];
                dst[0] = ok ? to_float(raw.b[r]) : 0.0f;
                dst[NP * kTile] = ok ? to_float(raw.c[r]) : 0.0f;
            }
        };
        // A pass after the first over the states of a wide d_state adds its share to the dx and
        // ddelta that are there.  They are requested one interval before the tile is reduced, ahead
        // of that interval's input loads: a wave's loads return in order, so a load that is
        // waited for right after its issue would make the wave wait for every tile in flight.
        struct Acc { IO dx[4]; uint32_t dd[4]; };
        Acc acc;
        auto load_acc = [&](int kk) {
            if constexpr (!ACC) return;
            const int pc = phys_of(chunk_of(min(kk, ntiles - 1)));
            const IO* dxk = at_chunk(dxg, pc, rowg, p.g_sl);
            const IO* ddk = at_chunk(ddg, pc, rowg, p.g_sl);
            uint32_t wg = 0xffffffffu, wgd = 0xffffffffu;
            if (ragged_seq && pc == last_chunk) {
                const int64_t end = (p.batch - 1) * p.g_sb + (p.L - 1) * p.g_sl + (p.ED - 1) * p.g_sd + 1;
                wg = window_bytes(end, b * p.g_sb + (int64_t)pc * kTile * p.g_sl + (int64_t)d0 * p.g_sd, kES);
                wgd = window_bytes(end, b * p.g_sb + (int64_t)pc * kTile * p.g_sl + (int64_t)d0 * p.g_sd, kESd);
            }
            const Steps sg = steps_of(rowg);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc.dx[j] = ld_off(dxk, offg, sg.at[j], wg);
            if (dd_wide) {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc.dd[j] = ld_bits32(at_chunk(ddgf, pc, rowg * 2u, p.g_sl), offg * 2u, sg.at[j] * 2u, wgd);
            } else if (sizeof(IO) == 4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc.dd[j] = ld_bits32(ddk, offg, sg.at[j], wgd);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc.dd[j] = ld_bits16(ddk, offg, sg.at[j], wgd);
            }
        };
        auto reduce_tile = [&](int k) {
            const int pc = phys_of(chunk_of(k));
            // this thread's share of the tile's dB / dC sums over the 64 channels: the four rows of
            // lanes, then the lanes of a state's group, always in this order
            float fw[kFw];
            {
                const float* rp = sRP + fw_rp;
                float4 s0 = *reinterpret_cast<const float4*>(rp), s1 = make_float4(0.f, 0.f, 0.f, 0.f);
                if constexpr (kLanesPer == 4) s1 = *reinterpret_cast<const float4*>(rp + 4);
#pragma unroll
                for (int r = 1; r < 4; ++r) {
                    const float4 v = *reinterpret_cast<const float4*>(rp + 16 * r);
                    s0.x += v.x; s0.y += v.y; s0.z += v.z; s0.w += v.w;
                    if constexpr (kLanesPer == 4) {
                        const float4 u = *reinterpret_cast<const float4*>(rp + 16 * r + 4);
                        s1.x += u.x; s1.y += u.y; s1.z += u.z; s1.w += u.w;
                    }
                }
                if constexpr (kLanesPer == 4) {
                    fw[0] = (s0.x + s0.y) + (s0.z + s0.w);
                    fw[1] = (s1.x + s1.y) + (s1.z + s1.w);
                } else {
                    fw[0] = s0.x + s0.y;
                    fw[1] = s0.z + s0.w;
                }
            }
            // (summed before the loads below are issued: together the two groups of loads hold more
            // registers than the wave has)
            asm volatile("" : "+v"(fw[0]), "+v"(fw[1]));
            __builtin_amdgcn_sched_barrier(0);
            float4 gB = make_float4(0.f, 0.f, 0.f, 0.f), dd = gB;
            if constexpr (kLean) {
                gB = tile_ld(sP1, co, qo);
                dd = tile_ld(sP2, co, qo);
            }
#pragma unroll
            for (int ww = kLean ? 1 : 0; ww < NW; ++ww) {
                const float4 a = tile_ld(sP1 + ww * kTileF, co, qo);
                const float4 e = tile_ld(sP2 + ww * kTileF, co, qo);
                gB.x += a.x; gB.y += a.y; gB.z += a.z; gB.w += a.w;
                dd.x += e.x; dd.y += e.y; dd.z += e.z; dd.w += e.w;
            }
            // the partial sums of tile k are in registers: the scan waves may overwrite them
            // (the release orders this store after the LDS reads above)
            if (lane == 0)
                __hip_atomic_fetch_add(sConsumed, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            const float4 dl4 = tile_ld(sDl + (k & 3) * kTileF, co, qo);
            const float4 x4 = tile_ld(sX + (k & 3) * kTileF, co, qo);
            const float4 dy4 = tile_ld(sDy + (k & 3) * kTileF, co, qo);
            const float gBv[4] = {gB.x, gB.y, gB.z, gB.w}, ddv[4] = {dd.x, dd.y, dd.z, dd.w};
            const float dlv[4] = {dl4.x, dl4.y, dl4.z, dl4.w}, xvv[4] = {x4.x, x4.y, x4.z, x4.w};
            const float dyv[4] = {dy4.x, dy4.y, dy4.z, dy4.w};
            float dxv[4], dv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                dxv[j] = __builtin_fmaf(dlv[j], gBv[j], Dr * dyv[j]);
                dv[j] = __builtin_fmaf(xvv[j], gBv[j], ddv[j] * kLn2);
            }
            if (p.softplus) {
                // d softplus(r)/dr = sigmoid(r) = 1 - exp(-softplus(r)); padded elements have
                // delta = 0 and all-zero partial sums, so they add nothing to ddelta_bias
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    dv[j] *= 1.0f - fast_exp2(-dlv[j] * kLog2e);
                    dDb += dv[j];
                }
            }
            if constexpr (ACC) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    dxv[j] += to_float(acc.dx[j]);
                    dv[j] += bits_to_float(acc.dd[j], dshift);
                }
            }
            IO* dxk = at_chunk(dxg, pc, rowg, p.g_sl);
            IO* ddk = at_chunk(ddg, pc, rowg, p.g_sl);
            float* ddkf = at_chunk(ddgf, pc, rowg * 2u, p.g_sl);  // (float32 next to bfloat16 tensors: rows twice as wide)
            const Steps sg = steps_of(rowg);
            auto st_dd = [&](int j, float v) {
                if (dd_wide) st_off(ddkf, offg * 2u, v, sg.at[j] * 2u);
                else st_off(ddk, offg, from_float<IO>(v), sg.at[j]);
            };
            float* fwk = at_chunk(fw_base, pc, rowfw, p.Nst);
            if (group_full && !(ragged_seq && pc == last_chunk) && fw_vec) {
                if constexpr (kLean) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) st_off(dxk, offg, from_float<IO>(dxv[j]), sg.at[j]);
                    // (one branch per tile on the width of ddelta, not one per element)
                    if (dd_wide) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) st_off(ddkf, offg * 2u, dv[j], sg.at[j] * 2u);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j) st_off(ddk, offg, from_float<IO>(dv[j]), sg.at[j]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        st_off(dxk, offg, from_float<IO>(dxv[j]), sg.at[j]);
                        st_dd(j, dv[j]);
                    }
                }
                if constexpr (kFw == 2)
                    st_off(reinterpret_cast<float2*>(fwk), fw_off, make_float2(fw[0], fw[1]));
                else
                    st_off(reinterpret_cast<float4*>(fwk), fw_off, make_float4(fw[0], fw[1], fw[2], fw[3]));
            } else {
                const int t0 = pc * kTile + 4 * (rev ? NQ - 1 - qo : qo);
                for (int j = 0; j < 4; ++j)
                    if (co_ok && t0 + (int)jw(j) < p.L) {
                        st_off(dxk, offg, from_float<IO>(dxv[j]), sg.at[j]);
                        st_dd(j, dv[j]);
                    }
                for (int i = 0; i < kFw; ++i)
                    if (pc * kTile + (rev ? kTile - 1 - fw_tt : fw_tt) < p.L && fw_n + i < p.N)
                        st_off(fwk, fw_off + 4u * i, fw[i]);
            }
        };

        // tile j travels in register set j % 3; staging runs two tiles ahead of the scan, the
        // reduction one tile behind
        Raw ra, rb, rc;
        if (sw == 0 && lane == 0) sConsumed[0] = 0;
        load_tile(0, ra);
        load_tile(1, rb);
        load_tile(2, rc);
        stage_tile(0, ra);
        load_tile(3, ra);
        if (ntiles > 1) stage_tile(1, rb);
        load_tile(4, rb);
        __syncthreads();  // tiles 0 and 1 are published
        __syncthreads();
        // The steady-state loop has one exit, at its top: with exits between the intervals the
        // compiler's wait-count bookkeeping sees an edge from the end of every interval back to
        // the first one, takes the loads issued last for the ones a tile is staged from, and
        // makes every interval wait for all loads and stores in flight.
        int k = 0;
        for (; k + 3 <= ntiles; k += 3) {
            if (k >= 1) reduce_tile(k - 1);
            load_acc(k);
            stage_tile(k + 2, rc);
            load_tile(k + 5, rc);
            __syncthreads();  // end of interval k
            reduce_tile(k);
            load_acc(k + 1);
            if (k + 3 < ntiles) stage_tile(k + 3, ra);
            load_tile(k + 6, ra);
            __syncthreads();  // end of interval k + 1
            reduce_tile(k + 1);
            load_acc(k + 2);
            if (k + 4 < ntiles) stage_tile(k + 4, rb);
            load_tile(k + 7, rb);
            __syncthreads();  // end of interval k + 2
        }
        // the last one or two intervals: every tile is staged already
        if (k < ntiles) {
            if (k >= 1) reduce_tile(k - 1);
            load_acc(k);
            __syncthreads();  // end of interval k
            if (k + 1 < ntiles) {
                reduce_tile(k);
                load_acc(k + 1);
                __syncthreads();  // end of interval k + 1
            }
        }
        reduce_tile(ntiles - 1);
        sDD[qi * kWave + ci] = ACC ? 0.0f : dDacc;
        sDD[(4 + qo) * kWave + co] = dDb;
        __syncthreads();  // final
        // dD (and ddelta_bias): sum the four step groups of every channel
        if (sw == 0 && lane <= cmax) {
            float s = 0.0f, sb = 0.0f;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                s += sDD[q * kWave + lane];
                sb += sDD[(4 + q) * kWave + lane];
            }
            p.partD[(int64_t)(p.row0 + bs) * p.ED + d0 + lane] = s;
            if (p.softplus) p.partDb[(int64_t)(p.row0 + bs) * p.ED + d0 + lane] = sb;
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
        // (A, h0, the checkpoints and the dA partials are rows of Nst states, the states of the whole
        // call; this launch works on N of them, starting where the host put the pointers)
        const int64_t dn = (int64_t)min(d, p.ED - 1) * p.N + min(n, p.N - 1);
        const float av = p.A[(int64_t)min(d, p.ED - 1) * p.Nst + min(n, p.N - 1)];
        const bool ok = dvalid && n < p.N;
        A2[i] = ok ? av * kLog2e : 0.0f;
        // a*g flowing in from the steps after this row's last one (zero at the sequence end)
        const float ag_in = p.ag0 ? p.ag0[(int64_t)bs * p.ED * p.N + dn] : 0.0f;
        ag[i] = ok ? ag_in : 0.0f;
        dAacc[i] = 0.0f;
    }
    // state at the start of chunk c: checkpoint written after chunk c-1, or h0 / zero.  A checkpoint is
    // fetched with one buffer instruction per state: wave-uniform slot address and state row (scalar
    // registers) + the lane's channel offset, the one per-lane value, kept for the whole kernel (built
    // from the lane index at every tile, the address cost each scan wave a dozen half-rate instructions
    // per tile).
    const uint32_t ck_voff = (uint32_t)min(d, p.ED - 1) * 4u;
    auto load_state = [&](int k, float (&hs)[NS]) {
        const int c = chunk_of(min(k, ntiles - 1));
        if (c > 0) {
            const float* ck_base = p.ckpt + ((int64_t)b * p.nchunks + (c - 1)) * p.Nst * p.ED;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const uint32_t n = (uint32_t)min(w * NS + i, p.N - 1);
                hs[i] = ld_off(ck_base, ck_voff, __builtin_amdgcn_readfirstlane(n * (uint32_t)p.ED * 4u));
            }
        } else {
            // the row starts here: its initial state, or zero
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const int n = min(w * NS + i, p.N - 1);
                hs[i] = p.h0 ? p.h0[((int64_t)b * p.ED + min(d, p.ED - 1)) * p.Nst + n] : 0.0f;
            }
        }
    };

    // registers of one tile: delta and u of the lane's channel, and one register per state for
    // B and for C whose lane t of every row holds step t
    struct TileIn {
        float dl[kTile], uu[kTile], vb[NS], vc[NS];
    };
    auto read_fwd_inputs = [&](int k, TileIn& r) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float4 v = tile_ld(sDl + (k & 3) * kTileF, lane, q);
            const float4 u4 = tile_ld(sU + (k & 1) * kTileF, lane, q);
            r.dl[4 * q] = v.x; r.dl[4 * q + 1] = v.y; r.dl[4 * q + 2] = v.z; r.dl[4 * q + 3] = v.w;
            r.uu[4 * q] = u4.x; r.uu[4 * q + 1] = u4.y; r.uu[4 * q + 2] = u4.z; r.uu[4 * q + 3] = u4.w;
        }
        const float* bck = sBC + (k & 1) * kBcF + (w * NS) * kTile + (lane & (kTile - 1));
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            r.vb[i] = bck[i * kTile];
            r.vc[i] = bck[NP * kTile + i * kTile];
        }
    };

    float hnext[NS];
    float poison = 0.0f;

    auto tile_pass = [&](int k, const TileIn& in, TileIn& next) {
        float hin[NS];  // state at the tile start
#pragma unroll
        for (int i = 0; i < NS; ++i) hin[i] = hnext[i];
        // The two scan waves of a SIMD share its VALU.  The hardware prefers the older wave, which
        // would then run the tile at the speed of a lone wave and wait at the barrier while the
        // younger one does most of its work alone (a lone wave issues one instruction per five
        // clocks, half of what the SIMD takes).  A wave's priority therefore falls as it advances
        // through the tile: the wave that is behind goes first, both finish together.
        __builtin_amdgcn_s_setprio(3);

        // ---- 1. recompute the tile forward, keeping a[t] and h[t] ----
        float aS[kTile][NS], hS[kTile][NS], dyq[2][4];
        int consumed = 0;
        static_for<0, kTile>([&](auto TT) {
            constexpr int tt = decltype(TT)::value;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const float a = fast_exp2(in.dl[tt] * A2[i]);
                float hprev;
                if constexpr (tt == 0) hprev = hin[i];
                else hprev = hS[tt > 0 ? tt - 1 : 0][i];
                aS[tt][i] = a;
                hS[tt][i] = fmac_bcast<tt>(a * hprev, in.vb[i], in.uu[tt]);
            }
            if (tt == 0) {
                // checkpoint of the next tile: a global load with a whole tile to arrive
                __builtin_amdgcn_sched_barrier(0);
                load_state(k + 1, hnext);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (tt == kTile - 4) {
                // first look at the consumption counter (see the wait below), early enough to hide the
                // LDS latency
                consumed = __hip_atomic_load(sConsumed, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
                // dy of the last four steps, needed when the reverse sweep starts
                const float4 v = tile_ld(sDy + (k & 3) * kTileF, lane, NQ - 1);
                dyq[(NQ - 1) & 1][0] = v.x; dyq[(NQ - 1) & 1][1] = v.y;
                dyq[(NQ - 1) & 1][2] = v.z; dyq[(NQ - 1) & 1][3] = v.w;
            }
        });

        // ---- 2. reverse sweep ----
        // The sweep writes this wave's single-buffered LDS blocks: the dB/dC lane-group sums step by
        // step, the partial sums over the states at its end.  The service waves read those of tile
        // k-1 at the start of this interval and publish that in sConsumed; by the end of the
        // recomputation that has normally happened, so this wait falls through.  It is bounded (a
        // wave never spins forever); if the bound is ever reached the blocks may be overwritten while
        // they are still being read, so the wave poisons its sums of dA: the call then returns NaN
        // in dA for these channels (and in one element of dx and ddelta per channel, see the end of the
        // kernel) instead of silently wrong gradients.
        auto wait_consumed = [&]() {
            if (k >= 1) {
                int spins = 0;
                while (consumed < kSvc * k && ++spins < (1 << 20)) {
                    __builtin_amdgcn_s_sleep(1);
                    consumed = __hip_atomic_load(sConsumed, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
                // (added to the sums at the very end of the kernel)
                if (consumed < kSvc * k || p.expire_waits) poison = __builtin_nanf("");
            }
        };
        // With a gate the service waves need longer for the previous tile, and the wait moves eight
        // steps into the sweep: the lane-group sums of those steps are held in registers, and they and
        // the two groups' partial sums are stored behind the wait (gated backward at B=4, L=4096, 4096
        // channels, bfloat16: 0.752 ms waiting at the start, 0.744 with four steps held, 0.715 with eight,
        // 0.750 with twelve;
        // without a gate the signal has come by the end of the recomputation and holding values costs
        // 1.5 %).
        constexpr bool kHoldSteps = HAS_Z;
        constexpr int kHold = 8;  // steps held (a multiple of four)
        if constexpr (!kHoldSteps) wait_consumed();
        __builtin_amdgcn_s_setprio(2);
        float rhold[kHold];
        float gBv[kTile], ddv[kTile];
        const int ln = lane;
        float* const rp_lane = sRP + w * kRpW + ln;
        float* const p_lane = sP1 + w * kTileF + tile_off(ln, 0);  // (sP2 is NW tiles further: a constant offset)
        static_for<0, kTile>([&](auto RT) {
            constexpr int tt = kTile - 1 - decltype(RT)::value;
            if constexpr ((tt & 3) == 3 && tt >= 4) {
                // dy of the next (earlier) four steps, one group ahead of use
                constexpr int qn = (tt >> 2) - (tt >= 4 ? 1 : 0);
                const float4 v = tile_ld(sDy + (k & 3) * kTileF, lane, qn);
                dyq[qn & 1][0] = v.x; dyq[qn & 1][1] = v.y; dyq[qn & 1][2] = v.z; dyq[qn & 1][3] = v.w;
            }
            if (tt == 10) __builtin_amdgcn_s_setprio(1);
            if (tt == 4) __builtin_amdgcn_s_setprio(0);
            const float dyv = dyq[(tt >> 2) & 1][tt & 3];
            float gB, dd = 0.0f;
            float pB[NS], pC[NS];
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                // g[t] = dy*C + a[t+1]*g[t+1];  a[t]*g[t] serves the next (earlier) step and,
                // times h[t-1], is d(delta*A)
                const float g = fmac_bcast<tt>(ag[i], in.vc[i], dyv);
                float hprev;
                if constexpr (tt == 0) hprev = hin[i];
                else hprev = hS[tt > 0 ? tt - 1 : 0][i];
                ag[i] = aS[tt][i] * g;
                const float gha = ag[i] * hprev;
                dAacc[i] = __builtin_fmaf(gha, in.dl[tt], dAacc[i]);
                dd = __builtin_fmaf(gha, A2[i], dd);
                gB = i == 0 ? mul_bcast<tt>(in.vb[i], g) : fmac_bcast<tt>(gB, in.vb[i], g);
                pB[i] = g * in.uu[tt];
                pC[i] = dyv * hS[tt][i];
            }
            gBv[tt] = gB;
            ddv[tt] = dd;
            // the partial sums of a group of four steps leave as soon as they are complete: written
            // together at the end of the tile, the stores of all scan waves (16 KB per wave) would
            // meet in the LDS queue in front of the barrier
            auto store_p_group = [&]() {
                constexpr int q = tt >> 2;
                *reinterpret_cast<float4*>(p_lane + q * kPlane) =
                    make_float4(gBv[4 * q], gBv[4 * q + 1], gBv[4 * q + 2], gBv[4 * q + 3]);
                *reinterpret_cast<float4*>(p_lane + NW * kTileF + q * kPlane) =
                    make_float4(ddv[4 * q], ddv[4 * q + 1], ddv[4 * q + 2], ddv[4 * q + 3]);
            };
            // (the first group of a gated kernel's sweep goes behind the wait, below)
            if constexpr ((tt & 3) == 0 && !(kHoldSteps && tt >= kTile - kHold)) store_p_group();

            if (tt == 2) {
                // fetch delta, u, B, C of the next tile (published two intervals ahead)
                __builtin_amdgcn_sched_barrier(0);
                read_fwd_inputs(k + 1, next);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- channel reduction of this step's dB / dC products, first part (see rs_stage) ----
            // value index bits, from stage 1 up: dB|dC, then the state index.  The lanes of a row then
            // hold 16 / (2 * NS) partial sums of each of the step's 2 * NS values; they go to this
            // wave's block of sRP as they are, and the service waves add them up one tile later.
            {
                float r;
                if constexpr (NS == 2) {
                    r = rs_stage<2>(rs_stage<1>(pB[0], pC[0], lane), rs_stage<1>(pB[1], pC[1], lane), lane);
                } else {
                    const float a0 = rs_stage<1>(pB[0], pC[0], lane), a1 = rs_stage<1>(pB[1], pC[1], lane);
                    const float a2 = rs_stage<1>(pB[2], pC[2], lane), a3 = rs_stage<1>(pB[3], pC[3], lane);
                    r = rs_stage<3>(rs_stage<2>(a0, a2, lane), rs_stage<2>(a1, a3, lane), lane);
                }
                if constexpr (kHoldSteps && tt >= kTile - kHold) {
                    rhold[tt - (kTile - kHold)] = r;
                    if constexpr (tt == kTile - kHold) {
                        __builtin_amdgcn_sched_barrier(0);
                        wait_consumed();
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int j = kHold - 1; j >= 0; --j) rp_lane[(kTile - kHold + j) * kWave] = rhold[j];
#pragma unroll
                        for (int q = NQ - 1; q >= NQ - kHold / 4; --q) {
                            *reinterpret_cast<float4*>(p_lane + q * kPlane) =
                                make_float4(gBv[4 * q], gBv[4 * q + 1], gBv[4 * q + 2], gBv[4 * q + 3]);
                            *reinterpret_cast<float4*>(p_lane + NW * kTileF + q * kPlane) =
                                make_float4(ddv[4 * q], ddv[4 * q + 1], ddv[4 * q + 2], ddv[4 * q + 3]);
                        }
                    }
                } else {
                    rp_lane[tt * kWave] = r;
                }
            }
        });
        __syncthreads();  // end of interval k: partial sums and dB/dC sums of tile k are visible
    };

    TileIn ta, tb;
    load_state(0, hnext);
    __syncthreads();
    read_fwd_inputs(0, ta);
    __syncthreads();
    for (int k = 0; k < ntiles; k += 2) {
        tile_pass(k, ta, tb);
        if (k + 1 >= ntiles) break;
        tile_pass(k + 1, tb, ta);
    }
    // per-batch partial of dA
    if (dvalid) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = w * NS + i;
            if (n < p.N) p.partA[((int64_t)bs * p.ED + d) * p.Nst + n] = dAacc[i] + poison;
        }
    }
    __syncthreads();  // final
    // A caller that drops dA (a frozen A) must still see an expired wait: the wave also overwrites one
    // element of dx and of ddelta per channel with NaN, in the tile the row ends with (the barrier
    // above orders these stores after the service waves' stores of that tile).
    if (poison != poison && dvalid) {
        const int64_t at = b * p.g_sb + (int64_t)phys_of(chunk_of(ntiles - 1)) * kTile * p.g_sl + (int64_t)d * p.g_sd;
        static_cast<IO*>(p.dx)[at] = from_float<IO>(poison);
        if (sizeof(IO) == 2 && p.delta_f32) static_cast<float*>(p.ddelta)[at] = poison;
        else static_cast<IO*>(p.ddelta)[at] = from_float<IO>(poison);
    }
}

template <typename IO, int NS, int NW, bool HAS_Z, bool ACC>
static int launch_fast(const BwdParams& p, hipStream_t stream) {
    dim3 grid((p.ED + kWave - 1) / kWave, p.batch * (p.nseg > 1 ? p.nseg : 1));
    dim3 block((NW + kSvc) * kWave);
    constexpr size_t lds = sizeof(float) * BwdFastLds<NS, NW>::floats;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static LdsLimitOnce lds_limit;
    const int attr_rc = lds_limit.ensure(sscan_bwd_fast_kernel<IO, NS, NW, HAS_Z, ACC>, lds);
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((sscan_bwd_fast_kernel<IO, NS, NW, HAS_Z, ACC>), grid, block, lds, stream, p);
    return check_launch();
}

bool bwd_fast_supported(int ns, int nw) { return (ns == 2 && nw == 8) || (ns == 4 && nw == 4); }

int launch_bwd_fast(const BwdParams& p, int ns, int nw, int io_dtype, hipStream_t stream) {
#define MPA_CASE2(NS_, NW_, Z_, ACC_)                                                    \
    return io_dtype == MPA_F32 ? launch_fast<float, NS_, NW_, Z_, ACC_>(p, stream)        \
                               : launch_fast<bf16_t, NS_, NW_, Z_, ACC_>(p, stream)
#define MPA_CASE(NS_, NW_)                                          \
    if (ns == NS_ && nw == NW_) {                                   \
        if (p.z && p.accumulate) MPA_CASE2(NS_, NW_, true, true);   \
        if (p.z) MPA_CASE2(NS_, NW_, true, false);                  \
        if (p.accumulate) MPA_CASE2(NS_, NW_, false, true);         \
        MPA_CASE2(NS_, NW_, false, false);                          \
    }
    MPA_CASE(2, 8) MPA_CASE(4, 4)
#undef MPA_CASE
#undef MPA_CASE2
    return MPA_ERR_BAD_SHAPE;
}

}  // namespace mpa
