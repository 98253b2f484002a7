// Fused selective-scan forward for gfx950: discretise -> scan -> readout in one pass.
//
// Work decomposition.  The recurrence h[t] = a[t]*h[t-1] + bx[t] is serial in t and
// independent per (batch, channel, state); with N = 16 there is nothing to contract, so the
// kernel is bound by fp32 VALU issue (one v_exp_f32 and four multiply/fma per state and
// step), not by HBM.  Everything is organised to keep the VALU fed:
//
//  * A workgroup owns 64 channels of one batch row.  NW "scan" waves split the d_state axis:
//    wave w keeps NS states (n = w*NS ..) of the 64 channels in registers, one channel per
//    lane, and walks the sequence in tiles of kTile steps.
//  * Eight "service" waves do everything that is per (step, channel) rather than per state.
//    Four loader waves request x, delta (z), B, C five tiles ahead, convert them, apply
//    softplus, form u = delta*x and D*x, and publish float32 tiles in LDS two tiles ahead of
//    the scan; four reducer waves, one tile behind, sum the NW partial readouts, apply the
//    gate and store y.  Scan and service waves meet at ONE workgroup barrier per tile, so HBM
//    latency, conversions and the cross-wave reduction overlap with the recurrence
//    arithmetic instead of preceding it.
//  * B and C are wave-uniform (they do not depend on the channel).  Up to 8 states per lane
//    they are staged in LDS and each scan wave loads, per state, one register whose lane t of
//    every 16-lane row holds step t; the FMAs read their step through a DPP row broadcast
//    (fmac_bcast), so B and C cost no extra instructions and no scalar registers.  Above that
//    a small pre-pass packs them as float32 in the order each scan wave consumes them and the
//    scan waves fetch them with scalar loads into SGPRs.
//  * The only parallel axes are batch * dim/64 workgroups and the states inside them.  When a
//    launch would cover a fraction of the chip, the sequence is cut into segments that run side
//    by side: a first pass (kernel mode kCarry: no readout) finds every segment's end state
//    from zero and its sum of delta, seg_carry_kernel chains them, a second pass is the normal
//    kernel from the true initial states (see seg_plan).  The backward uses the same first pass
//    for its own carry (mode kGCarry, see sscan_bwd.hip).
//  * Time is addressed through one mapping, walk position -> physical step, so that the scan
//    can run from the last step to the first (MPA_SSCAN_REVERSE) without flipped copies: the
//    service waves stage every tile in walk order and the scan waves never see the direction.
//  * Both channel-contiguous and time-contiguous ((B,ED,L) memory) operands are read and
//    written coalesced: a service thread owns 4 consecutive steps of one channel, and the
//    thread -> (channel, step group) map follows the unit-stride axis.
#include "sscan_fwd.h"

namespace mpa {


// ---------------------------------------------------------------------------------------------
// B/C pre-pass.  Output layout, float32:
//     [batch][tile][wave][sub-tile][B | C][kSS steps][NS states]
// i.e. the values one scan wave needs for one sub-tile of kSS steps are contiguous (the scan
// waves fetch them one sub-tile ahead of use); tiles and steps are in walk order.  Steps beyond
// the sequence end and states beyond d_state are written as zeros.
// ---------------------------------------------------------------------------------------------
template <typename IO>
__global__ void __launch_bounds__(256) pack_bc_kernel(const void* Bm, const void* C, float* out,
                                                      int L, int N, int NS, int NW, int kSS,
                                                      int nchunks, int reverse, int64_t bc_sb, int64_t bc_sl) {
    const int NP = NS * NW;
    const int64_t per_b = (int64_t)nchunks * 2 * kTile * NP;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= per_b) return;
    const int b = blockIdx.y;
    // decompose the OUTPUT index
    int r = (int)(i % (2 * kTile * NP));
    const int c = (int)(i / (2 * kTile * NP));
    const int w = r / (2 * kTile * NS);
    r %= 2 * kTile * NS;
    const int sub = r / (2 * kSS * NS);
    r %= 2 * kSS * NS;
    const int which = r / (kSS * NS);
    r %= kSS * NS;
    const int tt = sub * kSS + r / NS, s = r % NS;
    // (c, tt) count tiles and steps in walk order; a reverse walk starts at the physical end
    const int t = reverse ? (nchunks - 1 - c) * kTile + (kTile - 1 - tt) : c * kTile + tt;
    const int n = w * NS + s;
    float v = 0.0f;
    if (t < L && n < N)
        v = load_as_float<IO>(which ? C : Bm, b * bc_sb + (int64_t)t * bc_sl + n);
    out[b * per_b + i] = v;
}

// Packed B/C of the forward kernel: sub-tiles of 16 floats (32 at 16 states per lane, 64 at
// 32), and as many of them resident in scalar registers as 64 registers hold.  A scalar load
// that hits L2 takes 200+ clocks (500+ on a miss) while a scan step takes ~25, so a sub-tile is
// requested three sub-tiles before its first use.
template <int NS>
struct FwdPack {
    static constexpr int kSS = NS >= 8 ? 1 : 8 / NS;       // steps per sub-tile
    static constexpr int kSub = 2 * kSS * NS;              // floats per sub-tile
    static constexpr int kRing = kSub <= 16 ? 4 : 2;       // resident sub-tiles
};

constexpr int kCP = kTile + 4;  // pitch (floats) of a [channel][step] LDS tile: rows stay
                                // 16-byte aligned and 16-byte accesses of 16 lanes hit 64
                                // distinct banks
constexpr int kLoaders = 4;     // loader waves per workgroup (one item of (channel, 4 steps) per thread)
constexpr int kReducers = 4;    // reducer waves per workgroup (one item per thread)
constexpr int kService = kLoaders + kReducers;

// Up to 8 states per lane B and C reach the scan waves through LDS and a register per state
// whose 16 lanes of a row hold the 16 steps of a tile (see fmac_bcast); above that the register
// and LDS cost is too high and they come packed through the scalar cache (FwdPack).
template <int NS>
constexpr bool kBcastBC = NS <= 8;

// A workgroup owns CH channels of a batch row: 64 (one channel per lane of a scan wave, the wave's
// lanes all on the same NS states), or 48.  With 48, a row of 16 lanes is the unit: 3 rows of channels
// times 8 groups of two states are 24 units, four per scan wave, six scan waves; the rows of a wave
// then work on different state groups (B and C reach an FMA through a broadcast inside the row, so
// every row can have its own).  Batch * dim/48 workgroups fill the chip for shapes where batch *
// dim/64 leaves CUs idle (8 x 1536: 256 instead of 192), and the six scan waves occupy two SIMDs
// alone: the service waves are given wave numbers that land on the other two.
template <int NS, int NW, int CH>
constexpr int kStateGroups = CH == 64 ? NW : 16 / NS;  // groups of NS states = partial readouts per channel

template <int NS, int NW, int CH = 64>
struct FwdLds {
    static constexpr int NG = kStateGroups<NS, NW, CH>;
    // delta, u double-buffered (written two tiles ahead of use, read one tile ahead); D*x and
    // the gate in four buffers (written two tiles ahead, read one tile behind); readout
    // partials double-buffered per state group; B/C tiles [2][B|C][state][step] double-buffered
    static constexpr size_t tiles = (size_t)(2 * 2 + 2 * 4 + 2 * NG) * kWave * kCP;
    static constexpr size_t floats = tiles + (kBcastBC<NS> ? 2 * 2 * NS * NG * kTile : 0);
};


// One scan step / one group of four steps on the broadcast path: B and C of step TT come out of
// lane TT of the registers vb[i] / vc[i] inside the FMA (fmac_bcast).
// The decay factors a = 2^(delta * A2) of a group of four steps.  They do not depend on the state, so a
// scan wave computes them one group ahead of the recurrence: the multiply and the exponential (the
// longest latencies of a step) then sit off the chain h -> a*h -> +B*u -> next h, and a wave has
// independent work to issue while that chain waits for its own results.
// (With 8 states per lane a wave has eight independent chains and no registers to spare: the factors
// of a step are then computed when the step needs them.)
template <int NS>
constexpr bool kDecayAhead = NS <= 4;
template <int NS>
struct Decay4 {
    float a[kDecayAhead<NS> ? 4 : 1][NS];
    const float* dl;  // without look-ahead: the group's four values of delta, and A2
    const float* A2;
};
template <int Q, int NS>
__device__ __forceinline__ void decay_group(const float (&dl)[kTile], const float (&A2)[NS], Decay4<NS>& out) {
    if constexpr (kDecayAhead<NS>) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < NS; ++i) out.a[j][i] = fast_exp2(dl[4 * Q + j] * A2[i]);
    } else {
        out.dl = dl + 4 * Q;
        out.A2 = A2;
    }
}
// decay factors of step j of the group
template <int NS>
__device__ __forceinline__ void decay_step(const Decay4<NS>& dk, int j, float (&a)[NS]) {
#pragma unroll
    for (int i = 0; i < NS; ++i) a[i] = kDecayAhead<NS> ? dk.a[kDecayAhead<NS> ? j : 0][i] : fast_exp2(dk.dl[j] * dk.A2[i]);
}
template <int TT, int NS, int MODE>
__device__ __forceinline__ float scan_step_bcast(const float (&a)[NS], float uuv, float (&h)[NS],
                                                 const float (&vb)[NS], const float (&vc)[NS]) {
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        if constexpr (MODE == kGCarry) {
            h[i] = a[i] * fmac_bcast<TT>(h[i], vb[i], uuv);
        } else {
            h[i] = fmac_bcast<TT>(a[i] * h[i], vb[i], uuv);
        }
        if constexpr (MODE == kScan) sum = i == 0 ? mul_bcast<TT>(vc[i], h[i]) : fmac_bcast<TT>(sum, vc[i], h[i]);
    }
    return sum;
}
template <int Q, int NS, int MODE>
__device__ __forceinline__ float4 scan_group_bcast(const Decay4<NS>& dk, const float (&uu)[kTile], float (&h)[NS],
                                                   const float (&vb)[NS], const float (&vc)[NS]) {
    float4 y;
    float a[NS];
    decay_step<NS>(dk, 0, a);
    y.x = scan_step_bcast<4 * Q + 0, NS, MODE>(a, uu[4 * Q + 0], h, vb, vc);
    decay_step<NS>(dk, 1, a);
    y.y = scan_step_bcast<4 * Q + 1, NS, MODE>(a, uu[4 * Q + 1], h, vb, vc);
    decay_step<NS>(dk, 2, a);
    y.z = scan_step_bcast<4 * Q + 2, NS, MODE>(a, uu[4 * Q + 2], h, vb, vc);
    decay_step<NS>(dk, 3, a);
    y.w = scan_step_bcast<4 * Q + 3, NS, MODE>(a, uu[4 * Q + 3], h, vb, vc);
    return y;
}

// waves of a workgroup: the carry modes store no output and run without reducer waves; a 48-channel
// workgroup has sixteen wave numbers of which four do nothing (see service_role)
template <int NW, int MODE, int CH = 64>
constexpr int kFwdWaves = CH == 48 ? 16 : NW + (MODE == kScan ? kService : kLoaders);

// Role of wave w >= NW: 0..3 loaders, 4..7 reducers, -1 none.  Waves w and w + 4 of a workgroup share
// a SIMD.  In a 48-channel workgroup the six scan waves are waves 0..5 (two each on SIMDs 0 and 1, one
// each on SIMDs 2 and 3); its three loaders and three reducers (192 items of (channel, 4 steps)) take
// the wave numbers of SIMDs 2 and 3, and the numbers in between end at once.
template <int NW, int CH>
__device__ __forceinline__ int service_role(int w) {
    if constexpr (CH == 64) return w - NW;
    switch (w) {
        case 6: return 0;
        case 7: return 1;
        case 10: return 2;
        case 11: return 4;
        case 14: return 5;
        case 15: return 6;
        default: return -1;
    }
}

template <typename IO, int NS, int NW, bool HAS_Z, int MODE, int CH = 64>
__global__ void __launch_bounds__((kFwdWaves<NW, MODE, CH>) * kWave) sscan_fwd_kernel(const FwdParams p) {
    constexpr int NQ = kTile / 4;  // step groups (of 4) per tile
    static_assert(kLoaders == NQ && kReducers == NQ, "a tile has 64 * NQ items of (channel, 4 steps)");
    static_assert(CH == 64 || (CH == 48 && NS == 2 && NW == 6 && MODE == kScan), "48-channel groups: six scan waves of two states per lane");
    constexpr int NG = kStateGroups<NS, NW, CH>;
    constexpr int kSvcThreads = (CH == 64 ? 4 : 3) * kWave;  // loader (and reducer) threads: one per item

    extern __shared__ float4 smem4[];
    typedef float CTile[kWave][kCP];  // [channel][step]
    CTile* sDl = reinterpret_cast<CTile*>(smem4);  // [2]
    CTile* sU = sDl + 2;                           // [2]
    CTile* sDx = sU + 2;                           // [4] D*x
    CTile* sG = sDx + 4;                           // [4] gate silu(z) (only with z)
    CTile* sY = sG + 4;                            // [2][NG]
    float* const sBC = reinterpret_cast<float*>(sY + 2 * NG);  // [2][B|C][NP states][kTile steps]
    constexpr int NP = NS * NG;
    constexpr bool kBcast = kBcastBC<NS>;
    static_assert(MODE == kScan || kBcast, "the carry modes exist on the broadcast path only");

    const int lane = threadIdx.x & (kWave - 1);
    const int w = wave_id();
    // Row of the launch: a batch row, or one segment of it (segmented mode).  h0 / h_last / dsum
    // are indexed by the launch row, the caller's tensors by (batch row, physical step).
    // Tiles are counted in WALK order: walk tile kk is the kk-th tile the recurrence visits.
    const int bs = blockIdx.y;
    int b = bs, tile0 = 0, ntiles = p.nchunks;
    if (p.nseg > 1) {
        b = bs / p.nseg;
        tile0 = (bs - b * p.nseg) * p.seg_tiles;
        ntiles = min(p.seg_tiles, p.nchunks - tile0);
    }
    // walk tile -> physical chunk of kTile steps; inside a tile walk step s is physical step
    // s (forward) or kTile-1-s (reverse).  The ragged chunk is always the physical last one, so a
    // reverse walk starts with its padded steps: delta = 0 and u = 0 there leave the state alone.
    const bool rev = p.reverse != 0;
    const int last_chunk = p.nchunks - 1;
    auto phys_chunk = [&](int k) { return rev ? last_chunk - (tile0 + k) : tile0 + k; };
    const bool ragged_seq = p.nchunks * kTile > p.L;
    const int d0 = blockIdx.x * CH;
    constexpr bool has_z = HAS_Z;

    if (w >= NW) {
        // =============================== service waves ===============================
        // Four loader waves and four reducer waves, one item of (channel, 4 steps) per thread.
        // The roles are split across waves because loads and stores share one in-order
        // counter per wave: a wave that stores y would wait for those stores to drain every
        // time it waits for its next input tile.  A lone wave issues an instruction only every
        // 6-10 clocks and pays tens of clocks for every branch, so the per-tile code of these
        // waves is kept short (offsets precomputed, one uniform branch for the ragged edge)
        // and spread over four waves per role.
        const int sw = service_role<NW, CH>(w);      // 0..3: loaders   4..7: reducers
        if (CH != 64 && sw < 0) return;
        // With softplus or the gate the service waves carry long dependent chains of
        // transcendental functions and must still publish their tile before the interval ends:
        // they then go first whenever they are ready (gated forward at the headline shape: 0.258 ms at
        // priority 3, 0.277 at 2, 0.282 at 1; without gate and softplus priority 1 is best)
        if (has_z || p.softplus) __builtin_amdgcn_s_setprio(3);
        else __builtin_amdgcn_s_setprio(1);
        const int cmax = min(CH, p.ED - d0) - 1;     // last valid channel of the group
        const int item = (sw & 3) * kWave + lane;    // 0 .. 4 * CH - 1
        constexpr uint32_t kES = sizeof(IO);
        if (sw < kLoaders) {
            // ------------------------------- loaders -------------------------------
            const int ci = p.in_tmajor ? item / NQ : item % CH;
            const int qi = p.in_tmajor ? item % NQ : item / CH;     // walk step group of the item
            const int qp = rev ? NQ - 1 - qi : qi;                  // its physical step group
            const bool ci_ok = ci <= cmax;
            const int cic = min(ci, cmax);
            const float Dv = p.D ? p.D[d0 + cic] : 0.0f;  // (NULL: a pass after the first over a wide d_state)
            const float bias = p.dbias ? p.dbias[d0 + cic] : 0.0f;
            // wave-uniform chunk origins (scalar registers) + per-thread 32-bit element
            // offsets that do not change from tile to tile: one load per element and no
            // address arithmetic in the loop
            const IO* const xg = static_cast<const IO*>(p.x) + (b * p.u_sb + (int64_t)d0 * p.u_sd);
            const char* const dg = static_cast<const char*>(p.delta) + (b * p.d_sb + (int64_t)d0 * p.d_sd) * (int64_t)(sizeof(IO) == 4 || p.delta_f32 ? 4 : 2);
            const IO* const zg = static_cast<const IO*>(p.z) + (b * p.z_sb + (int64_t)d0 * p.z_sd);
            // byte offset of the item's lowest physical step (one vector register per tensor, see
            // ld_off); walk step j of the item is jw(j) row strides further, which goes into the
            // scalar offset of the access
            const uint32_t offx = ((uint32_t)(4 * qp) * (uint32_t)p.u_sl + (uint32_t)cic * (uint32_t)p.u_sd) * kES;
            // (delta may be float32 next to bfloat16 tensors: element size and conversion shift of its own)
            const bool d_wide = sizeof(IO) == 4 || p.delta_f32;
            const uint32_t kESd = d_wide ? 4u : 2u;
            const uint32_t dshift = __builtin_amdgcn_readfirstlane(d_wide ? 0u : 16u);
            const uint32_t offd = ((uint32_t)(4 * qp) * (uint32_t)p.d_sl + (uint32_t)cic * (uint32_t)p.d_sd) * kESd;
            const uint32_t offz = ((uint32_t)(4 * qp) * (uint32_t)p.z_sl + (uint32_t)cic * (uint32_t)p.z_sd) * kES;
            auto jw = [&](int j) { return (uint32_t)(rev ? 3 - j : j); };
            // scalar byte offsets of the item's four walk steps, computed once (scalar registers)
            uint32_t sxj[4], sdj[4], szj[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // (readfirstlane: told to the compiler as wave-uniform, so that they stay in scalar
                // registers; an offset it takes for per-lane costs a loop over its values per access)
                sxj[j] = __builtin_amdgcn_readfirstlane(jw(j) * (uint32_t)p.u_sl * kES);
                sdj[j] = __builtin_amdgcn_readfirstlane(jw(j) * (uint32_t)p.d_sl * kESd);
                szj[j] = __builtin_amdgcn_readfirstlane(jw(j) * (uint32_t)p.z_sl * kES);
            }
            // Loads of the ragged chunk run past the sequence end.  That is harmless (the values
            // are masked at staging) as long as the address is inside the tensor: the ragged
            // chunk is read through windows that end with the tensor's last element, whatever
            // the strides (out-of-window loads return zero).
            const bool group_full = cmax == CH - 1;
            // B/C of a tile: kTile * NP elements each, kBcPer per loader thread (the last of them only
            // for some threads when the division leaves a rest), step fastest
            constexpr int kBcPer = kBcast ? (NP * kTile + kSvcThreads - 1) / kSvcThreads : 0;
            const IO* const Bg = static_cast<const IO*>(p.Bm) + b * p.bc_sb;
            const IO* const Cg = static_cast<const IO*>(p.C) + b * p.bc_sb;
            int bct[kBcPer > 0 ? kBcPer : 1], bcn[kBcPer > 0 ? kBcPer : 1];
            uint32_t offbc[kBcPer > 0 ? kBcPer : 1];
#pragma unroll
            for (int r = 0; r < kBcPer; ++r) {
                const int e = min(item + r * kSvcThreads, NP * kTile - 1);
                bct[r] = e % kTile;  // walk step
                bcn[r] = item + r * kSvcThreads < NP * kTile ? e / kTile : 2 * NP;  // (beyond the tile: never staged)
                offbc[r] = ((uint32_t)(rev ? kTile - 1 - bct[r] : bct[r]) * (uint32_t)p.bc_sl +
                            (uint32_t)min(bcn[r], p.N - 1)) * kES;
            }

            // Raw values of three tiles in flight: HBM latency under load is longer than one
            // tile interval, so a tile is requested five intervals before the scan waves use
            // it and staged (converted, published in LDS) three intervals after the request.
            // The scan waves fetch packed B/C through the scalar cache.  All workgroups of a
            // batch row walk the sequence in step, so without help every one of those scalar
            // loads would wait for the same trip to memory; each loader thread therefore
            // touches 16 bytes of the pack five tiles ahead, which brings the lines into L2.
            constexpr int kPackVec = 2 * kTile * NS * NW / 4;  // float4 per tile of the pack
            const float4* const warm =
                kBcast ? nullptr
                       : reinterpret_cast<const float4*>(p.bcpack) + (int64_t)b * ntiles * kPackVec + min(item, kPackVec - 1);
            float dsum = 0.0f;  // delta summed over the thread's steps of the row
            struct Raw { IO x[4], z[4], b[kBcPer > 0 ? kBcPer : 1], c[kBcPer > 0 ? kBcPer : 1]; uint32_t d[4]; float4 warm; };
            auto load_tile = [&](int kk, Raw& raw) {
                // tiles beyond the last one are clamped to it; the loads are unconditional (a
                // branch around them would force a wait on their data)
                const int k = min(kk, ntiles - 1);
                const int pc = phys_chunk(k);
                const IO* xk = xg + (int64_t)pc * kTile * p.u_sl;
                const char* dk = dg + ((int64_t)pc * kTile * p.d_sl) * kESd;
                const IO* zk = zg + (int64_t)pc * kTile * p.z_sl;
                const IO* Bk = Bg + (int64_t)pc * kTile * p.bc_sl;
                const IO* Ck = Cg + (int64_t)pc * kTile * p.bc_sl;
                uint32_t wx = 0xffffffffu, wd = wx, wz = wx, wbc = wx;
                if (ragged_seq && pc == last_chunk) {
                    // elements from this chunk's origin to one past the tensor's last element
                    const int64_t tb = (int64_t)pc * kTile;
                    auto left = [&](int64_t sb_, int64_t sl_, int64_t sd_, int64_t width, int es = (int)sizeof(IO)) {
                        const int64_t end = (p.batch - 1) * sb_ + (p.L - 1) * sl_ + (width - 1) * sd_ + 1;
                        return window_bytes(end, b * sb_ + tb * sl_ + (int64_t)d0 * sd_, es);
                    };
                    wx = left(p.u_sb, p.u_sl, p.u_sd, p.ED);
                    wd = left(p.d_sb, p.d_sl, p.d_sd, p.ED, kESd);
                    wz = left(p.z_sb, p.z_sl, p.z_sd, p.ED);
                    wbc = window_bytes((p.batch - 1) * p.bc_sb + (p.L - 1) * p.bc_sl + p.N, b * p.bc_sb + tb * p.bc_sl, kES);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    raw.x[j] = ld_off(xk, offx, sxj[j], wx);
                    if (has_z) raw.z[j] = ld_off(zk, offz, szj[j], wz);
                }
                if (d_wide) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) raw.d[j] = ld_bits32(dk, offd, sdj[j], wd);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) raw.d[j] = ld_bits16(dk, offd, sdj[j], wd);
                }
#pragma unroll
                for (int r = 0; r < kBcPer; ++r) {
                    raw.b[r] = ld_off(Bk, offbc[r], 0, wbc);
                    if constexpr (MODE == kScan) raw.c[r] = ld_off(Ck, offbc[r], 0, wbc);
                }
                if (!kBcast) raw.warm = warm[(int64_t)k * kPackVec];
            };
            auto stage_tile = [&](int k, const Raw& raw) {
                if (!kBcast) asm volatile("" ::"v"(raw.warm.x), "v"(raw.warm.w));  // keeps the touch alive
#pragma unroll
                for (int r = 0; r < kBcPer; ++r) {
                    // states beyond d_state: B = C = 0 (padded steps need no care: u = 0 there
                    // and their y is never stored)
                    const bool ok = bcn[r] < p.N;
                    if (NP * kTile % kSvcThreads != 0 && bcn[r] >= NP) continue;
                    float* dst = sBC + (k & 1) * (2 * NP * kTile) + bcn[r] * kTile + bct[r];
                    dst[0] = ok ? to_float(raw.b[r]) : 0.0f;
                    if constexpr (MODE == kScan) dst[NP * kTile] = ok ? to_float(raw.c[r]) : 0.0f;
                }
                float xv[4], dv[4], gg[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    xv[j] = to_float(raw.x[j]);
                    dv[j] = bits_to_float(raw.d[j], dshift);
                }
                if (p.softplus) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) dv[j] = softplus_f(dv[j] + bias);
                }
                const int pc = phys_chunk(k);
                if (!group_full || (ragged_seq && pc == last_chunk)) {
                    // ragged edge: delta = 0, u = 0 keeps the state of padded steps/channels
                    const int t0 = pc * kTile + 4 * qp;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const bool ok = ci_ok && t0 + (int)jw(j) < p.L;
                        xv[j] = ok ? xv[j] : 0.0f;
                        dv[j] = ok ? dv[j] : 0.0f;
                    }
                }
                if constexpr (MODE != kScan) dsum += (dv[0] + dv[1]) + (dv[2] + dv[3]);  // only the carry needs it
                const int q4 = 4 * qi;
                *reinterpret_cast<float4*>(&sDl[k & 1][ci][q4]) = make_float4(dv[0], dv[1], dv[2], dv[3]);
                if (has_z) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float zv = to_float(raw.z[j]);
                        gg[j] = zv * sigmoid_f(zv);
                    }
                }
                if constexpr (MODE == kGCarry) {
                    // `x` is the upstream gradient dy here; the recurrence sees dy * silu(z)
                    if (has_z) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) xv[j] *= gg[j];
                    }
                    *reinterpret_cast<float4*>(&sU[k & 1][ci][q4]) = make_float4(xv[0], xv[1], xv[2], xv[3]);
                } else {
                    *reinterpret_cast<float4*>(&sU[k & 1][ci][q4]) =
                        make_float4(dv[0] * xv[0], dv[1] * xv[1], dv[2] * xv[2], dv[3] * xv[3]);
                }
                if constexpr (MODE == kScan) {
                    *reinterpret_cast<float4*>(&sDx[k & 3][ci][q4]) =
                        make_float4(Dv * xv[0], Dv * xv[1], Dv * xv[2], Dv * xv[3]);
                    if (has_z) *reinterpret_cast<float4*>(&sG[k & 3][ci][q4]) = make_float4(gg[0], gg[1], gg[2], gg[3]);
                }
            };
            // tile j travels in register set j % 3; staging runs two tiles ahead of the scan
            Raw ra, rb, rc;
            load_tile(0, ra);
            load_tile(1, rb);
            load_tile(2, rc);
            stage_tile(0, ra);
            load_tile(3, ra);
            if (ntiles > 1) stage_tile(1, rb);
            load_tile(4, rb);
            __syncthreads();  // tiles 0 and 1 are published
            __syncthreads();  // the scan waves hold tile 0 in registers: its buffer is free
            // The steady-state loop has one exit, at its top: with exits between the intervals
            // the compiler's wait-count bookkeeping sees an edge from the end of every interval
            // back to the first one and makes the wave wait for the loads it has just issued.
            int k = 0;
            for (; k + 3 <= ntiles; k += 3) {
                stage_tile(k + 2, rc);
                load_tile(k + 5, rc);
                __syncthreads();
                if (k + 3 < ntiles) stage_tile(k + 3, ra);
                load_tile(k + 6, ra);
                __syncthreads();
                if (k + 4 < ntiles) stage_tile(k + 4, rb);
                load_tile(k + 7, rb);
                __syncthreads();
            }
            // the last one or two intervals: every tile is staged already
            if (k < ntiles) {
                __syncthreads();
                if (k + 1 < ntiles) __syncthreads();
            }
            if (p.dsum && ci_ok) p.dsum[((int64_t)bs * NQ + qi) * p.ED + d0 + ci] = dsum;
        } else if constexpr (MODE == kScan) {
            // ------------------------------- reducers -------------------------------
            const int co = p.out_tmajor ? item / NQ : item % CH;
            const int qo = p.out_tmajor ? item % NQ : item / CH;     // walk step group
            const int qpo = rev ? NQ - 1 - qo : qo;                  // physical step group
            const bool co_ok = co <= cmax;
            const int q4 = 4 * qo;
            const uint32_t offy = ((uint32_t)(4 * qpo) * (uint32_t)p.y_sl + (uint32_t)min(co, cmax) * (uint32_t)p.y_sd) * kES;
            auto jw = [&](int j) { return (uint32_t)(rev ? 3 - j : j); };
            uint32_t syj[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) syj[j] = __builtin_amdgcn_readfirstlane(jw(j) * (uint32_t)p.y_sl * kES);
            IO* const yg = static_cast<IO*>(p.y) + (b * p.y_sb + (int64_t)d0 * p.y_sd);
            IO* const ypg = static_cast<IO*>(p.ypre) + (b * p.y_sb + (int64_t)d0 * p.y_sd);
            // What is already in the output (a pass after the first over a wide d_state adds to
            // it): requested one interval before the tile is reduced, so that the wait for it
            // is not a wait for a load just issued.
            const IO* const yag = static_cast<const IO*>(p.yacc) + (b * p.y_sb + (int64_t)d0 * p.y_sd);
            IO yav[4];
            auto load_yacc = [&](int kk) {
                if (!p.yacc) return;
                const int pc = phys_chunk(min(kk, ntiles - 1));
                uint32_t wy = 0xffffffffu;
                if (ragged_seq && pc == last_chunk) {
                    const int64_t end = (p.batch - 1) * p.y_sb + (p.L - 1) * p.y_sl + (p.ED - 1) * p.y_sd + 1;
                    wy = window_bytes(end, b * p.y_sb + (int64_t)pc * kTile * p.y_sl + (int64_t)d0 * p.y_sd, kES);
                }
                const IO* yak = yag + (int64_t)pc * kTile * p.y_sl;
#pragma unroll
                for (int j = 0; j < 4; ++j) yav[j] = ld_off(yak, offy, syj[j], wy);
            };
            auto reduce_store = [&](int k) {
                const int pc = phys_chunk(k);
                IO* yk = yg + (int64_t)pc * kTile * p.y_sl;
                IO* ypk = ypg + (int64_t)pc * kTile * p.y_sl;
                float4 s = *reinterpret_cast<const float4*>(&sDx[k & 3][co][q4]);
#pragma unroll
                for (int ww = 0; ww < NG; ++ww) {
                    const float4 v = *reinterpret_cast<const float4*>(&sY[(k & 1) * NG + ww][co][q4]);
                    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
                }
                if (p.yacc) {
                    s.x += to_float(yav[0]); s.y += to_float(yav[1]); s.z += to_float(yav[2]); s.w += to_float(yav[3]);
                }
                const int t0 = pc * kTile + 4 * qpo;  // lowest physical step of the item
                const bool whole = !(ragged_seq && pc == last_chunk) || t0 + 3 < p.L;
                if (has_z) {
                    if (p.ypre) {
                        const float pv[4] = {s.x, s.y, s.z, s.w};
                        for (int j = 0; j < 4; ++j)
                            if (co_ok && t0 + (int)jw(j) < p.L) st_off(ypk, offy, from_float<IO>(pv[j]), syj[j]);
                    }
                    const float4 g = *reinterpret_cast<const float4*>(&sG[k & 3][co][q4]);
                    s.x *= g.x; s.y *= g.y; s.z *= g.z; s.w *= g.w;
                }
                const float sv[4] = {s.x, s.y, s.z, s.w};
                if (co_ok && whole) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) st_off(yk, offy, from_float<IO>(sv[j]), syj[j]);
                } else if (co_ok) {
                    for (int j = 0; j < 4; ++j)
                        if (t0 + (int)jw(j) < p.L) st_off(yk, offy, from_float<IO>(sv[j]), syj[j]);
                }
            };
            // the reducers run one tile behind the scan waves
            __syncthreads();
            __syncthreads();
            for (int k = 0; k < ntiles; ++k) {
                if (k >= 1) reduce_store(k - 1);
                load_yacc(k);
                __syncthreads();
            }
            reduce_store(ntiles - 1);
        }
        return;
    }

    // ================================= scan waves =================================
    // lane -> (channel inside the group, group of NS states): see FwdLds
    int ch = lane, sg = w;
    if constexpr (CH == 48) {
        const int unit = 4 * w + (lane >> 4);
        sg = unit / 3;
        ch = (unit - 3 * sg) * 16 + (lane & 15);
    }
    const int d = d0 + ch;
    const bool dvalid = d < p.ED;
    float A2[NS], h[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = sg * NS + i;
        const bool ok = dvalid && n < p.N;
        const int dc = min(d, p.ED - 1), nc = min(n, p.N - 1);
        const float av = p.A[(int64_t)dc * p.a_st + nc];
        const float hv = p.h0 ? p.h0[((int64_t)bs * p.ED + dc) * p.h_st + nc] : 0.0f;
        A2[i] = ok ? av * kLog2e : 0.0f;
        h[i] = ok ? hv : 0.0f;
    }
    // registers of one tile: delta and u of the lane's channel and, on the broadcast path, one
    // register per state for B and for C whose lane t of every row holds step t
    struct TileRegs {
        float dl[kTile], uu[kTile];
        float vb[kBcast ? NS : 1], vc[kBcast ? NS : 1];
    };
    // (in two parts, so that a wave can spread its LDS reads over the tile: delta first, then u, B, C)
    auto read_tile_delta = [&](int k, TileRegs& r) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float4 v = *reinterpret_cast<const float4*>(&sDl[k & 1][ch][4 * q]);
            r.dl[4 * q] = v.x; r.dl[4 * q + 1] = v.y; r.dl[4 * q + 2] = v.z; r.dl[4 * q + 3] = v.w;
        }
    };
    auto read_tile_rest = [&](int k, TileRegs& r) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float4 u4 = *reinterpret_cast<const float4*>(&sU[k & 1][ch][4 * q]);
            r.uu[4 * q] = u4.x; r.uu[4 * q + 1] = u4.y; r.uu[4 * q + 2] = u4.z; r.uu[4 * q + 3] = u4.w;
        }
        if constexpr (kBcast) {
            const float* bck = sBC + (k & 1) * (2 * NP * kTile) + (sg * NS) * kTile + (lane & (kTile - 1));
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                r.vb[i] = bck[i * kTile];
                if constexpr (MODE == kScan) r.vc[i] = bck[NP * kTile + i * kTile];
            }
        }
    };
    auto read_tile = [&](int k, TileRegs& r) {
        read_tile_delta(k, r);
        read_tile_rest(k, r);
    };
    // state after walk tile tile0 + k of the batch row (the state after the very last tile is
    // h_last, not a checkpoint)
    auto store_ckpt = [&](int k) {
        if (MODE == kScan && p.ckpt && dvalid && tile0 + k < last_chunk) {
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const int n = sg * NS + i;
                if (n < p.N) p.ckpt[(((int64_t)b * p.nchunks + tile0 + k) * p.ck_st + n) * p.ED + d] = h[i];
            }
        }
    };

    // Software pipeline of one scan wave.  In interval k (between two barriers) it computes
    // tile k from registers that were filled during interval k-1 and fetches the inputs of
    // tile k+1 from LDS (published by the loader waves two intervals ahead), so no load
    // latency sits between two dependent steps.  Padded steps were staged as delta = 0, u = 0
    // (a = 2^0 = 1: h unchanged) and padded states have A2 = 0, B = C = 0, so there is no tail
    // handling.
    TileRegs ra, rb;
    if constexpr (kBcast) {
        Decay4<NS> d0q;  // decay factors of the first four steps of the tile that comes next
        auto tile_compute = [&](int k, const TileRegs& cur, TileRegs& next) {
            CTile& yt = sY[(k & 1) * NG + sg];
            // The scan waves of a SIMD share its VALU and the hardware prefers the older one, which
            // would run ahead and then wait at the barrier while the younger one works alone (a
            // lone wave cannot keep the SIMD busy).  A wave's priority falls as it advances
            // through the tile, so the wave that is behind goes first.
            __builtin_amdgcn_s_setprio(3);
            Decay4<NS> d1, d2, d3;
            decay_group<1, NS>(cur.dl, A2, d1);
            const float4 y0 = scan_group_bcast<0, NS, MODE>(d0q, cur.uu, h, cur.vb, cur.vc);
            if constexpr (MODE == kScan) *reinterpret_cast<float4*>(&yt[ch][0]) = y0;
            __builtin_amdgcn_sched_barrier(0);
            read_tile_delta(k + 1, next);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(2);
            decay_group<2, NS>(cur.dl, A2, d2);
            const float4 y1 = scan_group_bcast<1, NS, MODE>(d1, cur.uu, h, cur.vb, cur.vc);
            // (every group's readout leaves as soon as it is complete: written together at the end of the
            // tile, the stores of all scan waves would meet in the LDS queue in front of the barrier)
            if constexpr (MODE == kScan) *reinterpret_cast<float4*>(&yt[ch][4]) = y1;
            __builtin_amdgcn_sched_barrier(0);
            read_tile_rest(k + 1, next);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
            decay_group<3, NS>(cur.dl, A2, d3);
            const float4 y2 = scan_group_bcast<2, NS, MODE>(d2, cur.uu, h, cur.vb, cur.vc);
            if constexpr (MODE == kScan) *reinterpret_cast<float4*>(&yt[ch][8]) = y2;
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(0);
            // (the first group of the next tile, whose delta has arrived in `next` by now)
            decay_group<0, NS>(next.dl, A2, d0q);
            const float4 y3 = scan_group_bcast<3, NS, MODE>(d3, cur.uu, h, cur.vb, cur.vc);
            if constexpr (MODE == kScan) *reinterpret_cast<float4*>(&yt[ch][12]) = y3;
            store_ckpt(k);
        };
        __syncthreads();
        read_tile(0, ra);
        __syncthreads();
        decay_group<0, NS>(ra.dl, A2, d0q);
        for (int k = 0; k < ntiles; k += 2) {
            tile_compute(k, ra, rb);
            __syncthreads();
            if (k + 1 >= ntiles) break;
            tile_compute(k + 1, rb, ra);
            __syncthreads();
        }
    } else {
        // packed B/C of this (batch, wave): sub-tile j of tile k at + (k*NW*NSUB + j) * kSub,
        // fetched through the scalar cache a few sub-tiles ahead of use
        constexpr int kSS = FwdPack<NS>::kSS;        // steps per sub-tile
        constexpr int NSUB = kTile / kSS;            // sub-tiles per tile
        constexpr int kSub = 2 * kSS * NS;           // floats per sub-tile: B then C
        constexpr int kRing = FwdPack<NS>::kRing;    // sub-tiles resident in scalar registers
        static_assert(NSUB % kRing == 0, "a sub-tile always lands in the same ring slot");
        const float* bc = p.bcpack + ((int64_t)b * ntiles * NW + w) * (NSUB * kSub);  // whole rows only
        const int64_t bc_tile = (int64_t)NW * NSUB * kSub;
        float bcb[kRing][kSub];  // wave-uniform: live in SGPRs; sub-tile j of a tile uses slot j % kRing
        auto tile_compute = [&](int k, const TileRegs& cur_t, TileRegs& next) {
            const float* bck = bc + (int64_t)k * bc_tile;
            float acc[4];
#pragma unroll
            for (int tt = 0; tt < kTile; ++tt) {
                const int sub = tt / kSS, ts = tt % kSS;
                const float(&cur)[kSub] = bcb[sub % kRing];
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < NS; ++i) {
                    const float a = fast_exp2(cur_t.dl[tt] * A2[i]);
                    h[i] = __builtin_fmaf(cur_t.uu[tt], cur[ts * NS + i], a * h[i]);
                    sum = __builtin_fmaf(cur[kSS * NS + ts * NS + i], h[i], sum);
                }
                acc[tt & 3] = sum;
                if ((tt & 3) == 3)
                    *reinterpret_cast<float4*>(&sY[(k & 1) * NW + w][lane][tt - 3]) =
                        make_float4(acc[0], acc[1], acc[2], acc[3]);
                if (ts == 0) {
                    // Prefetches are issued right AFTER the first step of a sub-tile has
                    // consumed its B/C: scalar loads return out of order and share their
                    // counter with LDS, so the wait that precedes the first use of a sub-tile
                    // drains everything in flight.  (After the last tile the prefetches
                    // re-read valid memory and are ignored: no branch, so that the compiler
                    // cannot sink the arithmetic below them.)
                    __builtin_amdgcn_sched_barrier(0);
                    constexpr int kAhead = kRing - 1;  // the slot of the sub-tile just finished is free
                    if (sub + kAhead < NSUB)
                        scalar_load<kSub>(bck + (sub + kAhead) * kSub, bcb[(sub + kAhead) % kRing]);
                    else
                        scalar_load<kSub>(bc + (int64_t)min(k + 1, ntiles - 1) * bc_tile + (sub + kAhead - NSUB) * kSub,
                                          bcb[(sub + kAhead) % kRing]);
                    if (sub == 0) read_tile(k + 1, next);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            store_ckpt(k);
        };
#pragma unroll
        for (int j = 0; j < kRing - 1; ++j) scalar_load<kSub>(bc + j * kSub, bcb[j]);
        __syncthreads();
        read_tile(0, ra);
        __syncthreads();
        for (int k = 0; k < ntiles; k += 2) {
            tile_compute(k, ra, rb);
            __syncthreads();
            if (k + 1 >= ntiles) break;
            tile_compute(k + 1, rb, ra);
            __syncthreads();
        }
    }

    if (p.hlast && dvalid) {
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int n = sg * NS + i;
            if (n < p.N) p.hlast[((int64_t)bs * p.ED + d) * p.h_st + n] = h[i];
        }
    }
}

// Segmented mode, between the passes: the state at the start of every segment.  The first pass
// ran every segment from a zero state: hend = its end state, dsum = its sums of delta; with
// P = exp(A * sum of delta) (the product of the segment's decay factors) the true end state of a
// segment that starts from h is P*h + hend.  One thread per (batch row, channel, state) walks the
// segments in order.
__global__ void __launch_bounds__(256) seg_carry_kernel(const float* __restrict__ A, const float* __restrict__ h0,
                                                        const float* __restrict__ hend, const float* __restrict__ dsum,
                                                        float* __restrict__ segh0, float* __restrict__ hlast,
                                                        int batch, int nseg, int ED, int N, int a_st, int h_st) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t per_b = (int64_t)ED * N;
    if (i >= batch * per_b) return;
    const int b = (int)(i / per_b);
    const int64_t dn = i - b * per_b;
    const int d = (int)(dn / N), n = (int)(dn - (int64_t)d * N);
    const float a2 = A[(int64_t)d * a_st + n] * kLog2e;
    const int64_t ih = ((int64_t)b * ED + d) * h_st + n;  // in the caller's h0 / hlast
    float h = h0 ? h0[ih] : 0.0f;
    for (int sg = 0; sg < nseg; ++sg) {
        const int64_t row = (int64_t)b * nseg + sg;
        segh0[row * per_b + dn] = h;
        const float* ds = dsum + row * (kTile / 4) * ED + d;
        const float sd = (ds[0] + ds[ED]) + (ds[2 * (int64_t)ED] + ds[3 * (int64_t)ED]);
        // (a zero state stays out of the product: with A > 0 the factor can overflow, and 0 * inf
        // is not what the step-by-step recurrence computes)
        const float e = hend[row * per_b + dn];
        h = h == 0.0f ? e : __builtin_fmaf(fast_exp2(a2 * sd), h, e);
    }
    if (hlast) hlast[ih] = h;
}

// Segments per batch row.  The scan is serial in time, so a launch has only batch * dim/64
// workgroups; when those cover a fraction of the chip's 256 CUs the sequence is cut into
// segments that run side by side: up to twice the arithmetic, nseg times the parallelism.
// `thin` is the coverage below which the cut pays: a third of the CUs for the forward (its first
// pass costs 0.8 of the second), half of them for the backward (its first pass costs a quarter).
SegPlan seg_plan(const mpa_sscan_shape* s, int ns, int thin) {
    SegPlan sp{1, 0, 0, 0, 0, 0};
    if (ns > 8) return sp;
    const int64_t ntiles = (s->seqlen + kTile - 1) / kTile;
    const int64_t groups = s->batch * ((s->dim + kWave - 1) / kWave);
    int64_t want = 1;
    if (s->plan_segments > 0) {
        want = s->plan_segments;
    } else if (groups * thin <= 256 && ntiles >= 32) {
        want = 256 / groups;
        if (want > ntiles / 8) want = ntiles / 8;  // segments of 128 steps or more
        if (want > 64) want = 64;
    }
    if (want > ntiles) want = ntiles;
    if (want < 2 || s->batch * want > 65535) return sp;
    sp.seg_tiles = (int)((ntiles + want - 1) / want);
    sp.nseg = (int)((ntiles + sp.seg_tiles - 1) / sp.seg_tiles);
    if (sp.nseg < 2) return SegPlan{1, 0, 0, 0, 0, 0};
    const size_t rows = (size_t)s->batch * sp.nseg, per = (size_t)s->dim * s->dstate;
    sp.off_hend = 0;
    sp.off_h0 = rows * per;
    sp.off_dsum = 2 * rows * per;
    sp.floats = sp.off_dsum + rows * (kTile / 4) * (size_t)s->dim;
    return sp;
}

int group_channels(const mpa_sscan_shape* s, int ns, int nseg) {
    if (ns != 2 || s->dstate > 16 || nseg > 1 || (s->plan_flags & MPA_PLAN_GROUP_64)) return 64;
    if (s->plan_flags & MPA_PLAN_GROUP_48) return 48;
    return s->batch * ((s->dim + 47) / 48) <= 256 ? 48 : 64;
}

template <typename IO, int NS, int NW, bool HAS_Z, int MODE, int CH = 64>
static int launch_fwd(const FwdParams& p, hipStream_t stream) {
    dim3 grid((p.ED + CH - 1) / CH, p.batch * (p.nseg > 1 ? p.nseg : 1));
    dim3 block(kFwdWaves<NW, MODE, CH> * kWave);
    constexpr size_t lds = sizeof(float) * FwdLds<NS, NW, CH>::floats;
    static LdsLimitOnce lds_limit;
    const int attr_rc = lds_limit.ensure(sscan_fwd_kernel<IO, NS, NW, HAS_Z, MODE, CH>, lds);
    if (attr_rc != MPA_OK) return attr_rc;
    hipLaunchKernelGGL((sscan_fwd_kernel<IO, NS, NW, HAS_Z, MODE, CH>), grid, block, lds, stream, p);
    return check_launch();
}

template <typename IO>
static int dispatch_fwd(const FwdParams& p, int ns, int nw, int mode, hipStream_t stream) {
    if (p.group48) {  // (chosen by the host only where this instance exists: see fwd_group_channels)
        if (ns != 2 || mode != kScan) return MPA_ERR_BAD_SHAPE;
        return p.z ? launch_fwd<IO, 2, 6, true, kScan, 48>(p, stream) : launch_fwd<IO, 2, 6, false, kScan, 48>(p, stream);
    }
#define MPA_CASE(NS_, NW_)                                                        \
    if (ns == NS_ && nw == NW_ && mode == kScan)                                  \
        return p.z ? launch_fwd<IO, NS_, NW_, true, kScan>(p, stream)             \
                   : launch_fwd<IO, NS_, NW_, false, kScan>(p, stream);
    MPA_CASE(2, 8) MPA_CASE(4, 4) MPA_CASE(8, 2) MPA_CASE(16, 1)
    MPA_CASE(4, 8) MPA_CASE(8, 4) MPA_CASE(16, 2) MPA_CASE(32, 1)
    MPA_CASE(8, 8) MPA_CASE(16, 4) MPA_CASE(32, 2)
    MPA_CASE(16, 8) MPA_CASE(32, 4)
    MPA_CASE(32, 8)
#undef MPA_CASE
    // carry passes: the gate only matters to the backward's carry (dy * silu(z))
#define MPA_CASE(NS_, NW_)                                                        \
    if (ns == NS_ && nw == NW_ && mode == kCarry)                                 \
        return launch_fwd<IO, NS_, NW_, false, kCarry>(p, stream);                \
    if (ns == NS_ && nw == NW_ && mode == kGCarry)                                \
        return p.z ? launch_fwd<IO, NS_, NW_, true, kGCarry>(p, stream)           \
                   : launch_fwd<IO, NS_, NW_, false, kGCarry>(p, stream);
    MPA_CASE(2, 8) MPA_CASE(4, 4) MPA_CASE(8, 2)
    MPA_CASE(4, 8) MPA_CASE(8, 4)
    MPA_CASE(8, 8)
#undef MPA_CASE
    return MPA_ERR_BAD_SHAPE;
}

int launch_fwd_any(const FwdParams& p, int io_dtype, int ns, int nw, int mode, hipStream_t stream) {
    return io_dtype == MPA_F32 ? dispatch_fwd<float>(p, ns, nw, mode, stream)
                               : dispatch_fwd<bf16_t>(p, ns, nw, mode, stream);
}

int launch_seg_carry(const float* A, const float* h0, const float* hend, const float* dsum, float* segh0,
                     float* hlast, int batch, int nseg, int ED, int N, int a_st, int h_st, hipStream_t st) {
    const int64_t total = (int64_t)batch * ED * N;
    hipLaunchKernelGGL(seg_carry_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, A, h0, hend, dsum,
                       segh0, hlast, batch, nseg, ED, N, a_st, h_st);
    return check_launch();
}

int validate_shape(const mpa_sscan_shape* s) {
    if (!s) return MPA_ERR_NULL_POINTER;
    if (s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return MPA_ERR_BAD_SHAPE;
    if (s->dstate > MPA_MAX_DSTATE || s->batch > 65535) return MPA_ERR_BAD_SHAPE;
    if (s->seqlen > (int64_t)1 << 30 || s->dim > (int64_t)1 << 30) return MPA_ERR_BAD_SHAPE;
    if (s->io_dtype != MPA_F32 && s->io_dtype != MPA_BF16) return MPA_ERR_BAD_DTYPE;
    if (s->plan_states_per_lane < 0 || s->plan_segments < 0) return MPA_ERR_BAD_SHAPE;
    if (s->delta_dtype != 0 && s->delta_dtype != MPA_DELTA_F32) return MPA_ERR_BAD_DTYPE;
    const int64_t st[] = {s->z_sb, s->z_sl, s->z_sd, s->u_sb, s->u_sl, s->u_sd, s->d_sb, s->d_sl, s->d_sd, s->y_sb, s->y_sl,
                          s->y_sd, s->g_sb, s->g_sl, s->g_sd, s->bc_sb, s->bc_sl, s->dbc_sb, s->dbc_sl};
    for (int64_t v : st)
        if (v < 0) return MPA_ERR_BAD_STRIDE;
    // one (kTile steps x 64 channels) tile is addressed with 32-bit byte offsets; so are a
    // tile of B / C and one checkpoint (d_state x dim floats)
    const int64_t tile[][2] = {{s->z_sl, s->z_sd}, {s->u_sl, s->u_sd}, {s->d_sl, s->d_sd}, {s->y_sl, s->y_sd},
                               {s->g_sl, s->g_sd}};
    for (const auto& v : tile)
        if (v[0] * kTile + v[1] * kWave >= ((int64_t)1 << 30)) return MPA_ERR_BAD_STRIDE;
    if (s->bc_sl * kTile + s->dstate >= ((int64_t)1 << 30) || s->dbc_sl * kTile + s->dstate >= ((int64_t)1 << 30))
        return MPA_ERR_BAD_STRIDE;
    if (s->dstate * s->dim >= ((int64_t)1 << 30)) return MPA_ERR_BAD_SHAPE;
    return MPA_OK;
}

int padded_states(int64_t n) {
    int np = 16;
    while (np < n) np *= 2;
    return np;
}

// States per lane (NS) for a launch.  The only parallel axes are batch*dim/64 workgroups and
// d_state/NS scan waves inside each; a workgroup holds at most 8 scan waves.  Fewer states per
// lane mean more waves (better latency hiding) but more LDS traffic per state; ask for about
// two scan waves per SIMD over the chip's 1024 SIMDs when the problem offers them.  `pinned`
// (the caller's plan_states_per_lane) wins when it is a value the kernels exist for.
int pick_states_per_lane(int64_t batch, int64_t dim, int64_t dstate, int ns_cap, int pinned) {
    const int np = padded_states(dstate);
    const int ns_min = np / 8 > 2 ? np / 8 : 2;
    const int ns_max = ns_cap < np ? ns_cap : np;
    if (ns_max < ns_min) return -1;
    if (pinned >= ns_min && pinned <= ns_max && (pinned & (pinned - 1)) == 0) return pinned;
    const int64_t groups = batch * ((dim + kWave - 1) / kWave);
    int ns = ns_max;
    while (ns > ns_min && groups * (np / ns) < 2048) ns /= 2;
    return ns;
}

size_t bcpack_floats(const mpa_sscan_shape* s) {
    const size_t nchunks = (size_t)(s->seqlen + kTile - 1) / kTile;
    return (size_t)s->batch * nchunks * 2 * kTile * padded_states(s->dstate);
}

int launch_pack_bc(const mpa_sscan_shape* s, const void* B, const void* C, float* out, int ns,
                   int kss, hipStream_t st) {
    const int np = padded_states(s->dstate);
    const int nchunks = (int)((s->seqlen + kTile - 1) / kTile);
    const int64_t per_b = (int64_t)nchunks * 2 * kTile * np;
    const int reverse = (s->flags & MPA_SSCAN_REVERSE) ? 1 : 0;
    dim3 grid((unsigned)((per_b + 255) / 256), (unsigned)s->batch);
    if (s->io_dtype == MPA_F32)
        hipLaunchKernelGGL(pack_bc_kernel<float>, grid, dim3(256), 0, st, B, C, out, (int)s->seqlen,
                           (int)s->dstate, ns, np / ns, kss, nchunks, reverse, s->bc_sb, s->bc_sl);
    else
        hipLaunchKernelGGL(pack_bc_kernel<bf16_t>, grid, dim3(256), 0, st, B, C, out, (int)s->seqlen,
                           (int)s->dstate, ns, np / ns, kss, nchunks, reverse, s->bc_sb, s->bc_sl);
    return check_launch();
}

}  // namespace mpa

using namespace mpa;

extern "C" int64_t mpa_sscan_ckpt_elems(const mpa_sscan_shape* s) {
    if (!s || s->batch <= 0 || s->seqlen <= 0 || s->dim <= 0 || s->dstate <= 0) return 0;
    const int64_t nchunks = (s->seqlen + kTile - 1) / kTile;
    return s->batch * nchunks * s->dstate * s->dim;
}

// forward cut: a third of the CUs or fewer covered (see seg_plan)
static constexpr int kFwdThin = 3;

// d_state above 64: the states are independent given x, delta, B, C, so the call runs as passes
// over blocks of 64 states on the broadcast path (8 states per lane, 8 scan waves; cut into segments
// like any other launch), each pass adding its readout to the output.  A caller that pins more than
// 8 states per lane gets the single launch with packed B/C instead.
static constexpr int kFwdStateBlock = 64;
static bool fwd_in_state_blocks(const mpa_sscan_shape* s) {
    return s->dstate > kFwdStateBlock && s->plan_states_per_lane <= 8;
}

extern "C" size_t mpa_sscan_fwd_workspace_bytes(const mpa_sscan_shape* s, int with_ckpt) {
    (void)with_ckpt;  // both kinds of call are cut by the same rule
    if (validate_shape(s) != MPA_OK) return 0;
    // the packed B/C exist only on the scalar-load path (more than 8 states per lane)
    if (fwd_in_state_blocks(s)) {
        // passes over blocks of kFwdStateBlock states: the first block needs the most
        mpa_sscan_shape sb = *s;
        sb.dstate = kFwdStateBlock;
        const int nsb = pick_states_per_lane(sb.batch, sb.dim, sb.dstate, 8, sb.plan_states_per_lane);
        return (seg_plan(&sb, nsb, kFwdThin).floats * sizeof(float) + 255) / 256 * 256 + 256;
    }
    const int ns = pick_states_per_lane(s->batch, s->dim, s->dstate, 32, s->plan_states_per_lane);
    if (ns <= 8) return (seg_plan(s, ns, kFwdThin).floats * sizeof(float) + 255) / 256 * 256 + 256;
    return (bcpack_floats(s) * sizeof(float) + 255) / 256 * 256;
}

static int sscan_fwd_impl(const mpa_sscan_shape* s, const void* x, const void* delta,
                          const float* A, const void* B, const void* C, const float* D,
                          const void* z, const float* delta_bias, const float* h0, void* y,
                          void* y_pregate, float* h_ckpt, float* h_last, void* workspace,
                          size_t workspace_bytes, void* stream) {
    int rc = validate_shape(s);
    if (rc != MPA_OK) return rc;
    if (!x || !delta || !A || !B || !C || !D || !y || !workspace) return MPA_ERR_NULL_POINTER;
    const bool softplus = (s->flags & MPA_SSCAN_DELTA_SOFTPLUS) != 0;
    if (!softplus && delta_bias) return MPA_ERR_BAD_SHAPE;
    const size_t es = dtype_size(s->io_dtype);
    if (!aligned_to(x, es) || !aligned_to(delta, s->delta_dtype == MPA_DELTA_F32 ? 4 : es) || !aligned_to(B, es) || !aligned_to(C, es) ||
        !aligned_to(y, es) || (z && !aligned_to(z, es)) || (y_pregate && !aligned_to(y_pregate, es)) || !aligned_to(A, 4) || !aligned_to(D, 4) ||
        !aligned_to(workspace, 256))
        return MPA_ERR_MISALIGNED;
    if (workspace_bytes < mpa_sscan_fwd_workspace_bytes(s, h_ckpt != nullptr)) return MPA_ERR_WORKSPACE;

    hipStream_t st = static_cast<hipStream_t>(stream);
    float* wsf = static_cast<float*>(workspace);

    FwdParams p{};
    p.x = x; p.delta = delta; p.z = z; p.A = A; p.D = D;
    p.dbias = delta_bias; p.h0 = h0; p.bcpack = static_cast<const float*>(workspace);
    p.Bm = B; p.C = C; p.bc_sb = s->bc_sb; p.bc_sl = s->bc_sl;
    p.y = y; p.ypre = z ? y_pregate : nullptr; p.ckpt = h_ckpt; p.hlast = h_last;
    p.batch = (int)s->batch; p.L = (int)s->seqlen; p.ED = (int)s->dim; p.N = (int)s->dstate;
    p.a_st = p.h_st = p.ck_st = p.N;
    p.nchunks = (p.L + kTile - 1) / kTile;
    p.softplus = softplus ? 1 : 0;
    p.delta_f32 = s->delta_dtype == MPA_DELTA_F32 ? 1 : 0;
    p.reverse = (s->flags & MPA_SSCAN_REVERSE) ? 1 : 0;
    p.u_sb = s->u_sb; p.u_sl = s->u_sl; p.u_sd = s->u_sd;
    p.z_sb = s->z_sb; p.z_sl = s->z_sl; p.z_sd = s->z_sd;
    p.d_sb = s->d_sb; p.d_sl = s->d_sl; p.d_sd = s->d_sd;
    p.y_sb = s->y_sb; p.y_sl = s->y_sl; p.y_sd = s->y_sd;
    p.in_tmajor = (s->u_sd != 1 && s->u_sl == 1) ? 1 : 0;
    p.out_tmajor = (s->y_sd != 1 && s->y_sl == 1) ? 1 : 0;

    // the launches for the states q describes (q.N of them, pointers at the first one): one
    // launch, or a sequence cut into segments (end states of every segment from zero, carry,
    // then the real pass)
    auto run_states = [&](const FwdParams& q, int ns, int nw, const SegPlan& sp) -> int {
        if (sp.nseg <= 1) {
            FwdParams q1 = q;
            q1.group48 = q.N == s->dstate && group_channels(s, ns, 1) == 48 ? 1 : 0;
            return launch_fwd_any(q1, s->io_dtype, ns, nw, kScan, st);
        }
        FwdParams p1 = q;
        p1.nseg = sp.nseg; p1.seg_tiles = sp.seg_tiles;
        p1.z = nullptr; p1.y = nullptr; p1.ypre = nullptr; p1.yacc = nullptr; p1.h0 = nullptr; p1.ckpt = nullptr;
        p1.hlast = wsf + sp.off_hend; p1.dsum = wsf + sp.off_dsum; p1.h_st = q.N;
        int r = launch_fwd_any(p1, s->io_dtype, ns, nw, kCarry, st);
        if (r != MPA_OK) return r;
        r = launch_seg_carry(q.A, q.h0, wsf + sp.off_hend, wsf + sp.off_dsum, wsf + sp.off_h0, q.hlast, q.batch,
                             sp.nseg, q.ED, q.N, q.a_st, q.h_st, st);
        if (r != MPA_OK) return r;
        FwdParams p2 = q;
        p2.nseg = sp.nseg; p2.seg_tiles = sp.seg_tiles;
        p2.h0 = wsf + sp.off_h0; p2.hlast = nullptr; p2.h_st = q.N;
        return launch_fwd_any(p2, s->io_dtype, ns, nw, kScan, st);
    };

    if (fwd_in_state_blocks(s)) {
        // The passes before the last write the sum of their readouts where the last one finds it:
        // in y_pregate when there is a gate and the caller wants that output, else in y.  The last
        // pass adds its own, writes the pre-gate output and applies the gate.
        void* const ysum = (z && y_pregate) ? y_pregate : y;
        const int nblk = (p.N + kFwdStateBlock - 1) / kFwdStateBlock;
        for (int blk = 0; blk < nblk; ++blk) {
            const int n0 = blk * kFwdStateBlock;
            mpa_sscan_shape sb = *s;
            sb.dstate = p.N - n0 < kFwdStateBlock ? p.N - n0 : kFwdStateBlock;
            const int ns = pick_states_per_lane(sb.batch, sb.dim, sb.dstate, 8, sb.plan_states_per_lane);
            if (ns < 0) return MPA_ERR_BAD_SHAPE;
            const int nw = padded_states(sb.dstate) / ns;
            const bool last = blk == nblk - 1;
            FwdParams q = p;
            q.N = (int)sb.dstate;
            q.A = A + n0;
            q.Bm = static_cast<const char*>(B) + n0 * es;
            q.C = static_cast<const char*>(C) + n0 * es;
            q.h0 = h0 ? h0 + n0 : nullptr;
            q.hlast = h_last ? h_last + n0 : nullptr;
            q.ckpt = h_ckpt ? h_ckpt + (int64_t)n0 * p.ED : nullptr;
            q.D = blk == 0 ? D : nullptr;
            q.yacc = blk > 0 ? ysum : nullptr;
            if (!last) { q.z = nullptr; q.y = ysum; q.ypre = nullptr; }
            rc = run_states(q, ns, nw, seg_plan(&sb, ns, kFwdThin));
            if (rc != MPA_OK) return rc;
        }
        return MPA_OK;
    }

    const int np = padded_states(s->dstate);
    const int ns = pick_states_per_lane(s->batch, s->dim, s->dstate, 32, s->plan_states_per_lane);
    if (ns < 0) return MPA_ERR_BAD_SHAPE;
    const int nw = np / ns;
    if (ns > 8) {  // !kBcastBC<NS>: B/C go through the scalar cache, repacked per scan wave
        rc = launch_pack_bc(s, B, C, wsf, ns, 1 /* FwdPack<NS>::kSS */, st);
        if (rc != MPA_OK) return rc;
    }
    return run_states(p, ns, nw, seg_plan(s, ns, kFwdThin));
}

extern "C" int mpa_sscan_fwd(const mpa_sscan_shape* s, const void* x, const void* delta,
                             const float* A, const void* B, const void* C, const float* D,
                             const void* z, const float* delta_bias, const float* h0, void* y,
                             void* y_pregate, float* h_ckpt, float* h_last, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return sscan_fwd_impl(s, x, delta, A, B, C, D, z, delta_bias, h0, y, y_pregate, h_ckpt, h_last, workspace,
                          workspace_bytes, stream);
}

// ---- the entry point that allocates nothing -------------------------------------------------
// Scratch of mpa_sscan_fwd_noalloc: device memory that belongs to the library's code object, one
// copy per GPU the library is loaded on, held until the process ends.  In host code the name
// below is only a handle for hipGetSymbolAddress; the device address it yields (different on
// every GPU) is what goes to the kernels.
static __device__ __align__(256) unsigned char scratch[MPA_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device, resolved once per device
int scratch_address(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MPA_ERR_LAUNCH;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MPA_ERR_LAUNCH;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return MPA_OK;
}
}  // namespace

extern "C" int mpa_sscan_fwd_noalloc(const mpa_sscan_shape* s, const void* x, const void* delta,
                                     const float* A, const void* B, const void* C, const float* D,
                                     const void* z, const float* delta_bias, const float* h0, void* y,
                                     void* y_pregate, float* h_ckpt, float* h_last, void* stream) {
    const int rc = validate_shape(s);
    if (rc != MPA_OK) return rc;
    // the scratch the call needs is a function of the shape alone: too large a call is refused
    // before anything touches the device
    if (mpa_sscan_fwd_workspace_bytes(s, h_ckpt != nullptr) > MPA_NOALLOC_SCRATCH_BYTES) return MPA_ERR_WORKSPACE;
    void* ptr = nullptr;
    const int arc = scratch_address(&ptr);
    if (arc != MPA_OK) return arc;
    // Nothing in the scratch has to start at zero: every word the kernels read (segment end
    // states, sums of delta, packed B/C) is written earlier in the same call.
    return sscan_fwd_impl(s, x, delta, A, B, C, D, z, delta_bias, h0, y, y_pregate, h_ckpt, h_last, ptr,
                          MPA_NOALLOC_SCRATCH_BYTES, stream);
}
