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
    kBackwardMix, kBackwardMixPlain
};

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
    for (int it = 0; it < iters; ++it) {
        if constexpr (STREAM == kFmaIndependent) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
                asm volatile("v_fma_f32 %0, %0, %8, %9\n v_fma_f32 %1, %1, %8, %9\n v_fma_f32 %2, %2, %8, %9\n"
                             "v_fma_f32 %3, %3, %8, %9\n v_fma_f32 %4, %4, %8, %9\n v_fma_f32 %5, %5, %8, %9\n"
                             "v_fma_f32 %6, %6, %8, %9\n v_fma_f32 %7, %7, %8, %9\n"
                             : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7)
                             : "v"(c), "v"(d));
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
