// Instruction issue-rate probe for gfx950 (a measuring tool, not part of the library): how many
// clocks a SIMD spends per wave64 VALU instruction, by instruction kind and by the number of waves
// resident on the SIMD.  The scan kernels are bound by this rate; the figures this program prints
// are the cost model their design notes use.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops issue_probe.hip -o issue_probe
//   ./issue_probe            (python bench.py --workload issue-probe runs it)
//
// Every stream is inline assembly, so the compiler neither packs nor reorders it.  A launch puts W
// waves on each of the 1024 SIMDs (blocks of 4*W waves on 256 CUs); clocks per instruction and SIMD =
// kernel time * shader clock / (instructions per wave * W).
#include <hip/hip_runtime.h>

#include <cstdio>

#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);  \
            return 1;                                                              \
        }                                                                          \
    } while (0)

enum Stream {
    kFmaIndependent, kFmaDependent, kExp, kExpDependent, kDppBroadcast, kLaneSwap32, kForwardMix, kForwardMixPlain,
    kBackwardMix, kBackwardMixPlain, kFmaSgpr, kForwardMixSgpr,
    kG0, kG1, kG2, kG3, kG4, kG5, kG6, kG7, kG8, kG9, kG10, kG11, kG12, kG13, kG14, kG15, kG16, kG17, kG18, kG19, kMixBatched, kMixAlt, kMixAlt2
};
#define GEN8(T) T("0") T("1") T("2") T("3") T("4") T("5") T("6") T("7")
#define G0(i) "v_fmac_f32 %" i ", 1.0, %9\n"
#define G1(i) "v_mul_f32 %" i ", 0x3fb8aa3b, %" i "\n"
#define G2(i) "v_lshlrev_b32 %" i ", 16, %" i "\n"
#define G3(i) "v_and_b32 %" i ", 0xffff0000, %" i "\n"
#define G4(i) "v_cndmask_b32 %" i ", %" i ", %9, vcc\n"
#define G5(i) "v_add_u32 %" i ", %" i ", %9\n"
#define G6(i) "v_add_f32 %" i ", %" i ", %9\n"
#define G7(i) "v_mov_b32 %" i ", %9\n"
#define G8(i) "v_cmp_lt_f32 vcc, %" i ", %9\n"
#define G10(i) "v_cndmask_b32_e64 %" i ", %" i ", %9, s[20:21]\n"
#define G11(i) "v_cmp_lt_f32 vcc, %" i ", %9\n v_cndmask_b32 %" i ", %" i ", %9, vcc\n"
#define G12(i) "v_readlane_b32 s22, %" i ", 3\n"
#define G13(i) "v_max_f32 %" i ", %" i ", %9\n"
#define G14(i) "v_cvt_pk_bf16_f32 %" i ", %" i ", %9\n"
#define G15(i) "v_writelane_b32 %" i ", s22, 5\n"
#define G16(i) "v_add_f32_dpp %" i ", %" i ", %9 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n"
#define G17(i) "v_add_f32_dpp %" i ", %" i ", %9 row_mirror row_mask:0xf bank_mask:0xf\n"
#define G18(i) "v_mov_b32_dpp %" i ", %9 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n"
#define G19(i) "v_add_f32_sdwa %" i ", %" i ", %9 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD\n"
#define G9(i) "v_add_f32_dpp %" i ", %" i ", %9 row_shr:1 row_mask:0xf bank_mask:0x5\n"


#define BC3 " row_newbcast:3 row_mask:0xf bank_mask:0xf\n"
#define BC5 " row_newbcast:5 row_mask:0xf bank_mask:0xf\n"

// 64 VALU instructions per loop iteration in every stream
template <int STREAM>
__global__ void probe_kernel(float* out, long long* ticks, int iters) {
    // shader-clock and constant 100 MHz counters around the stream: the clock the part really runs at
    const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    float v0 = threadIdx.x * 1e-6f + 1.0f, v1 = v0 + 1, v2 = v0 + 2, v3 = v0 + 3, v4 = v0 + 4, v5 = v0 + 5, v6 = v0 + 6,
          v7 = v0 + 7;
    const float c = 0.999f, d = 1e-3f;
    asm volatile("s_mov_b64 s[20:21], 0x5555\n s_mov_b32 s22, 0\n s_mov_b64 vcc, 0x3333" ::: "s20", "s21", "s22", "vcc");
    for (int it = 0; it < iters; ++it) {
        if constexpr (STREAM == kFmaIndependent) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_fma_f32 %0, %0, %8, %9\n v_fma_f32 %1, %1, %8, %9\n v_fma_f32 %2, %2, %8, %9\n"
                             "v_fma_f32 %3, %3, %8, %9\n v_fma_f32 %4, %4, %8, %9\n v_fma_f32 %5, %5, %8, %9\n"
                             "v_fma_f32 %6, %6, %8, %9\n v_fma_f32 %7, %7, %8, %9\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
        } else if constexpr (STREAM == kFmaSgpr) {
            float sc = __builtin_amdgcn_readfirstlane(c);
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_fmac_f32 %0, %8, %9\n v_fmac_f32 %1, %8, %9\n v_fmac_f32 %2, %8, %9\n"
                             "v_fmac_f32 %3, %8, %9\n v_fmac_f32 %4, %8, %9\n v_fmac_f32 %5, %8, %9\n"
                             "v_fmac_f32 %6, %8, %9\n v_fmac_f32 %7, %8, %9\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "s"(sc), "v"(d));
        } else if constexpr (STREAM == kForwardMixSgpr) {
            float sc = __builtin_amdgcn_readfirstlane(c);
#pragma unroll
            for (int r = 0; r < 6; ++r)
                asm volatile("v_mul_f32 %2, %6, %9\n v_mul_f32 %3, %7, %9\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                             "v_mul_f32 %0, %2, %0\n v_mul_f32 %1, %3, %1\n v_fmac_f32 %0, %8, %9\n v_fmac_f32 %1, %8, %9\n"
                             "v_mul_f32 %4, %8, %0\n v_fmac_f32 %4, %8, %1\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "s"(sc), "v"(d));
            asm volatile("v_mov_b32 %0, %0\n v_mov_b32 %1, %1\n v_mov_b32 %2, %2\n v_mov_b32 %3, %3\n"
                         : "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7));
        } else if constexpr (STREAM == kG0) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G0)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG1) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G1)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG2) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G2)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG3) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G3)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG4) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G4)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG5) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G5)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG6) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G6)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG7) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G7)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG8) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G8)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG9) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G9)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG10) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G10)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kG11) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                asm volatile(GEN8(G11)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kG12) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G12)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kG13) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G13)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kG14) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G14)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kG15) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G15)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc", "s20", "s21", "s22");
        } else if constexpr (STREAM == kMixBatched) {
            // same 60 instructions as six forward-mix steps, batched by kind: 24 plain, 12 exp, 24 DPP
#pragma unroll
            for (int r = 0; r < 3; ++r)
                asm volatile("v_mul_f32 %0, %6, %8\n v_mul_f32 %1, %7, %8\n v_mul_f32 %2, %6, %8\n v_mul_f32 %3, %7, %8\n"
                             "v_mul_f32 %4, %6, %9\n v_mul_f32 %5, %7, %9\n v_mul_f32 %0, %0, %8\n v_mul_f32 %1, %1, %8\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
#pragma unroll
            for (int r = 0; r < 3; ++r)
                asm volatile("v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n v_exp_f32 %4, %4\n v_exp_f32 %5, %5\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
#pragma unroll
            for (int r = 0; r < 3; ++r)
                asm volatile("v_fmac_f32_dpp %0, %8, %9" BC3 "v_fmac_f32_dpp %1, %8, %9" BC3 "v_fmac_f32_dpp %2, %8, %9" BC3
                             "v_fmac_f32_dpp %3, %8, %9" BC3 "v_fmac_f32_dpp %4, %8, %9" BC5 "v_fmac_f32_dpp %5, %8, %9" BC5
                             "v_fmac_f32_dpp %6, %8, %9" BC5 "v_fmac_f32_dpp %7, %8, %9" BC5
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
            asm volatile("v_mov_b32 %0, %0\n v_mov_b32 %1, %1\n v_mov_b32 %2, %2\n v_mov_b32 %3, %3\n"
                         : "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7));
        } else if constexpr (STREAM == kMixAlt) {
            // strict alternation plain / DPP (independent): 32 + 32
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_mul_f32 %0, %0, %8\n v_fmac_f32_dpp %1, %8, %9" BC3 "v_mul_f32 %2, %2, %8\n v_fmac_f32_dpp %3, %8, %9" BC3
                             "v_mul_f32 %4, %4, %8\n v_fmac_f32_dpp %5, %8, %9" BC5 "v_mul_f32 %6, %6, %8\n v_fmac_f32_dpp %7, %8, %9" BC5
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
        } else if constexpr (STREAM == kMixAlt2) {
            // the same 32 + 32 in runs of four
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_mul_f32 %0, %0, %8\n v_mul_f32 %2, %2, %8\n v_mul_f32 %4, %4, %8\n v_mul_f32 %6, %6, %8\n"
                             "v_fmac_f32_dpp %1, %8, %9" BC3 "v_fmac_f32_dpp %3, %8, %9" BC3 "v_fmac_f32_dpp %5, %8, %9" BC5 "v_fmac_f32_dpp %7, %8, %9" BC5
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
        } else if constexpr (STREAM == kG16) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G16)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG17) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G17)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG18) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G18)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kG19) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile(GEN8(G19)
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d) : "vcc");
        } else if constexpr (STREAM == kFmaDependent) {
#pragma unroll
            for (int r = 0; r < 64; ++r) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v0) : "v"(c), "v"(d));
        } else if constexpr (STREAM == kExp) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_exp_f32 %0, %8\n v_exp_f32 %1, %8\n v_exp_f32 %2, %8\n v_exp_f32 %3, %8\n"
                             "v_exp_f32 %4, %8\n v_exp_f32 %5, %8\n v_exp_f32 %6, %8\n v_exp_f32 %7, %8\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(d));
        } else if constexpr (STREAM == kExpDependent) {
#pragma unroll
            for (int r = 0; r < 64; ++r) asm volatile("v_exp_f32 %0, %0" : "+v"(v0));
        } else if constexpr (STREAM == kDppBroadcast) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_fmac_f32_dpp %0, %8, %9" BC3 "v_fmac_f32_dpp %1, %8, %9" BC3 "v_fmac_f32_dpp %2, %8, %9" BC3
                             "v_fmac_f32_dpp %3, %8, %9" BC3 "v_fmac_f32_dpp %4, %8, %9" BC3 "v_fmac_f32_dpp %5, %8, %9" BC3
                             "v_fmac_f32_dpp %6, %8, %9" BC3 "v_fmac_f32_dpp %7, %8, %9" BC3
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
        } else if constexpr (STREAM == kLaneSwap32) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %2, %3\n v_permlane32_swap_b32 %4, %5\n"
                             "v_permlane32_swap_b32 %6, %7\n v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %2, %3\n"
                             "v_permlane32_swap_b32 %4, %5\n v_permlane32_swap_b32 %6, %7\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7));
        } else if constexpr (STREAM == kForwardMix || STREAM == kForwardMixPlain) {
            // the forward scan step for two states: multiply, exp2, multiply, two FMAs whose B / C
            // operand is a DPP row broadcast (or, "plain", an ordinary register); 6 steps + 4 moves
#pragma unroll
            for (int r = 0; r < 6; ++r) {
                if constexpr (STREAM == kForwardMix)
                    asm volatile("v_mul_f32 %2, %6, %8\n v_mul_f32 %3, %7, %8\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                                 "v_mul_f32 %0, %2, %0\n v_mul_f32 %1, %3, %1\n"
                                 "v_fmac_f32_dpp %0, %8, %9" BC3 "v_fmac_f32_dpp %1, %8, %9" BC3
                                 "s_nop 0\n v_mul_f32_dpp %4, %9, %0" BC5 "v_fmac_f32_dpp %4, %8, %1" BC5
                                 : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                                 : "v"(c), "v"(d));
                else
                    asm volatile("v_mul_f32 %2, %6, %8\n v_mul_f32 %3, %7, %8\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                                 "v_mul_f32 %0, %2, %0\n v_mul_f32 %1, %3, %1\n v_fmac_f32 %0, %8, %9\n v_fmac_f32 %1, %8, %9\n"
                                 "v_mul_f32 %4, %9, %0\n v_fmac_f32 %4, %8, %1\n"
                                 : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                                 : "v"(c), "v"(d));
            }
            asm volatile("v_mov_b32 %0, %0\n v_mov_b32 %1, %1\n v_mov_b32 %2, %2\n v_mov_b32 %3, %3\n"
                         : "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7));
        } else {
            // the backward scan step for two states as first written: recompute (multiply, exp2,
            // multiply, broadcast FMA), reverse recurrence and its products, and a channel reduction
            // that starts with lane swaps; 2 steps of 32 instructions
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                if constexpr (STREAM == kBackwardMix)
                    asm volatile(
                        "v_mul_f32 %2, %0, %8\n v_mul_f32 %3, %1, %8\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                        "v_mul_f32 %4, %2, %4\n v_mul_f32 %5, %3, %5\n"
                        "v_fmac_f32_dpp %4, %8, %9" BC3 "v_fmac_f32_dpp %5, %8, %9" BC3 "v_fmac_f32_dpp %6, %8, %9" BC5
                        "v_fmac_f32_dpp %7, %8, %9" BC5
                        "v_mul_f32 %0, %2, %6\n v_mul_f32 %1, %3, %7\n v_mul_f32 %2, %0, %4\n v_mul_f32 %3, %1, %5\n"
                        "v_fmac_f32 %4, %2, %9\n v_fmac_f32 %5, %3, %9\n v_fmac_f32 %0, %2, %8\n v_fmac_f32 %1, %3, %8\n"
                        "v_mul_f32_dpp %2, %8, %6" BC5 "v_fmac_f32_dpp %2, %9, %7" BC5
                        "v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %6, %4\n v_permlane32_swap_b32 %7, %5\n"
                        "v_mul_f32 %2, %0, %6\n v_mul_f32 %3, %0, %7\n v_fmac_f32 %2, %1, %4\n v_fmac_f32 %3, %1, %5\n s_nop 1\n"
                        "v_permlane16_swap_b32 %2, %3\n v_add_f32 %2, %2, %3\n s_nop 1\n"
                        "v_add_f32_dpp %3, %2, %2 row_mirror row_mask:0xf bank_mask:0x3\n"
                        : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                        : "v"(c), "v"(d));
                else
                    asm volatile(
                        "v_mul_f32 %2, %0, %8\n v_mul_f32 %3, %1, %8\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n"
                        "v_mul_f32 %4, %2, %4\n v_mul_f32 %5, %3, %5\n"
                        "v_fmac_f32 %4, %8, %9\n v_fmac_f32 %5, %8, %9\n v_fmac_f32 %6, %8, %9\n v_fmac_f32 %7, %8, %9\n"
                        "v_mul_f32 %0, %2, %6\n v_mul_f32 %1, %3, %7\n v_mul_f32 %2, %0, %4\n v_mul_f32 %3, %1, %5\n"
                        "v_fmac_f32 %4, %2, %9\n v_fmac_f32 %5, %3, %9\n v_fmac_f32 %0, %2, %8\n v_fmac_f32 %1, %3, %8\n"
                        "v_mul_f32 %2, %8, %6\n v_fmac_f32 %2, %9, %7\n"
                        "v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %6, %4\n v_permlane32_swap_b32 %7, %5\n"
                        "v_mul_f32 %2, %0, %6\n v_mul_f32 %3, %0, %7\n v_fmac_f32 %2, %1, %4\n v_fmac_f32 %3, %1, %5\n s_nop 1\n"
                        "v_permlane16_swap_b32 %2, %3\n v_add_f32 %2, %2, %3\n s_nop 1\n"
                        "v_add_f32_dpp %3, %2, %2 row_mirror row_mask:0xf bank_mask:0x3\n"
                        : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                        : "v"(c), "v"(d));
            }
        }
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7;
    if (blockIdx.x == gridDim.x / 2 && threadIdx.x == 0) {
        ticks[0] = __builtin_readcyclecounter() - c0;
        ticks[1] = wall_clock64() - w0;
    }
}

template <int STREAM>
static int run(const char* name, float* out, long long* ticks, double clock_hz) {
    const int iters = 2000;
    double mhz3 = 0.0, mhz8 = 0.0;
    printf("%-34s", name);
    for (int waves_per_simd : {1, 2, 3, 4, 8}) {
        dim3 block(64 * 4 * waves_per_simd), grid(256);
        if (block.x > 1024) {
            grid.x = 256 * (block.x / 1024);
            block.x = 1024;
        }
        hipEvent_t e0, e1;
        CK(hipEventCreate(&e0));
        CK(hipEventCreate(&e1));
        float best = 1e30f;
        for (int rep = 0; rep < 3; ++rep) {
            CK(hipEventRecord(e0));
            hipLaunchKernelGGL(probe_kernel<STREAM>, grid, block, 0, 0, out, ticks, iters);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (rep > 0 && ms < best) best = ms;
        }
        CK(hipEventDestroy(e0));
        CK(hipEventDestroy(e1));
        printf(" %6.2f", best * 1e-3 * clock_hz / (64.0 * iters * waves_per_simd));
        long long t[2];
        CK(hipMemcpy(t, ticks, sizeof(t), hipMemcpyDeviceToHost));
        if (waves_per_simd == 3 && t[1] > 0) mhz3 = 100.0 * (double)t[0] / (double)t[1];
        if (waves_per_simd == 8 && t[1] > 0) mhz8 = 100.0 * (double)t[0] / (double)t[1];
    }
    printf("   | %5.0f %5.0f MHz\n", mhz3, mhz8);
    return 0;
}

int main() {
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const double clock_hz = prop.clockRate * 1e3;  // the nominal shader clock; the part may run below it
    float* out;
    long long* ticks;
    CK(hipMalloc(&out, 4 << 20));
    CK(hipMalloc(&ticks, 2 * sizeof(long long)));
    printf("%s, %d CUs, nominal shader clock %.0f MHz\n", prop.gcnArchName, prop.multiProcessorCount, clock_hz / 1e6);
    printf("clocks per wave64 VALU instruction and SIMD (kernel time x nominal clock), with 1 / 2 / 3 / 4 / 8 waves on\n"
           "the SIMD; last columns: shader clock read inside the kernel (cycle counter / 100 MHz counter) at 3 and at 8 waves\n");
    int rc = 0;
    rc |= run<kFmaIndependent>("v_fma_f32, 8 independent chains", out, ticks, clock_hz);
    rc |= run<kFmaSgpr>("v_fmac_f32 with an SGPR operand", out, ticks, clock_hz);
    rc |= run<kForwardMixSgpr>("forward step mix, SGPR operands", out, ticks, clock_hz);
    rc |= run<kG0>("v_fmac_f32 inline constant 1.0", out, ticks, clock_hz);
    rc |= run<kG1>("v_mul_f32 literal", out, ticks, clock_hz);
    rc |= run<kG2>("v_lshlrev_b32 inline 16", out, ticks, clock_hz);
    rc |= run<kG3>("v_and_b32 literal", out, ticks, clock_hz);
    rc |= run<kG4>("v_cndmask_b32 vcc", out, ticks, clock_hz);
    rc |= run<kG5>("v_add_u32 vgprs", out, ticks, clock_hz);
    rc |= run<kG6>("v_add_f32 vgprs", out, ticks, clock_hz);
    rc |= run<kG7>("v_mov_b32", out, ticks, clock_hz);
    rc |= run<kG8>("v_cmp_lt_f32 -> vcc", out, ticks, clock_hz);
    rc |= run<kG9>("v_add_f32_dpp row_shr bank-masked", out, ticks, clock_hz);
    rc |= run<kG10>("v_cndmask_b32_e64 sgpr-pair mask", out, ticks, clock_hz);
    rc |= run<kG11>("v_cmp + v_cndmask pairs", out, ticks, clock_hz);
    rc |= run<kG12>("v_readlane_b32", out, ticks, clock_hz);
    rc |= run<kG13>("v_max_f32", out, ticks, clock_hz);
    rc |= run<kG14>("v_cvt_pk_bf16_f32", out, ticks, clock_hz);
    rc |= run<kG15>("v_writelane_b32", out, ticks, clock_hz);
    rc |= run<kMixBatched>("forward mix batched by kind", out, ticks, clock_hz);
    rc |= run<kMixAlt>("plain / DPP alternating", out, ticks, clock_hz);
    rc |= run<kMixAlt2>("plain / DPP in runs of four", out, ticks, clock_hz);
    rc |= run<kG16>("v_add_f32_dpp quad_perm", out, ticks, clock_hz);
    rc |= run<kG17>("v_add_f32_dpp row_mirror", out, ticks, clock_hz);
    rc |= run<kG18>("v_mov_b32_dpp quad_perm", out, ticks, clock_hz);
    rc |= run<kG19>("v_add_f32_sdwa (dword sel)", out, ticks, clock_hz);
    rc |= run<kFmaDependent>("v_fma_f32, one dependent chain", out, ticks, clock_hz);
    rc |= run<kExp>("v_exp_f32, independent", out, ticks, clock_hz);
    rc |= run<kExpDependent>("v_exp_f32, one dependent chain", out, ticks, clock_hz);
    rc |= run<kDppBroadcast>("v_fmac_f32_dpp row_newbcast", out, ticks, clock_hz);
    rc |= run<kLaneSwap32>("v_permlane32_swap_b32", out, ticks, clock_hz);
    rc |= run<kForwardMix>("forward step mix, DPP broadcast", out, ticks, clock_hz);
    rc |= run<kForwardMixPlain>("forward step mix, plain operands", out, ticks, clock_hz);
    rc |= run<kBackwardMix>("backward step mix, DPP broadcast", out, ticks, clock_hz);
    rc |= run<kBackwardMixPlain>("backward step mix, plain operands", out, ticks, clock_hz);
    CK(hipFree(out));
    CK(hipFree(ticks));
    return rc;
}
