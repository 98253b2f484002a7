// Shared device helpers for the gfx950 selective-scan kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>

#include "../../include/mambapy_amd.h"

namespace mpa {

constexpr int kWave = 64;             // CDNA wavefront width
constexpr int kTile = MPA_CKPT_STEPS; // time steps staged in LDS per iteration
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
    return v;
}
// round-to-nearest-even on the hardware converter (v_cvt_pk_bf16_f32)
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    const __bf16 r = static_cast<__bf16>(v);
    return bf16_t{__builtin_bit_cast(uint16_t, r)};
}

template <typename T>
__device__ __forceinline__ float load_as_float(const void* p, int64_t i) {
    return to_float(static_cast<const T*>(p)[i]);
}
template <typename T>
__device__ __forceinline__ void store_from_float(void* p, int64_t i, float v) {
    static_cast<T*>(p)[i] = from_float<T>(v);
}

// 2^x on the transcendental unit (v_exp_f32)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float softplus_f(float v) {
    // log(1 + e^v) = max(v, 0) + log1p(e^-|v|), free of branches on the hardware exp2 / log2
    // units (a library log1p is ~110 instructions and a branch).  log1p(e), 0 < e <= 1: the
    // cubic series below 2^-6 (truncation < 1e-6 relative), log2(1 + e) above (the rounding
    // of 1 + e costs < 4e-6 relative).  Above v = 20 the second term vanishes in fp32, which is
    // torch.nn.functional.softplus' linear branch.
    const float e = fast_exp2(-fabsf(v) * kLog2e);
    const float series = e * __builtin_fmaf(e, __builtin_fmaf(e, 0.33333334f, -0.5f), 1.0f);
    const float lg = __builtin_amdgcn_logf(1.0f + e) * kLn2;
    return fmaxf(v, 0.0f) + (e < 0.015625f ? series : lg);
}
__device__ __forceinline__ float sigmoid_f(float v) {
    return __builtin_amdgcn_rcpf(1.0f + fast_exp2(-v * kLog2e));
}

// Element at (wave-uniform pointer) + (32-bit per-lane BYTE offset) + (wave-uniform byte offset),
// through the buffer instructions: one instruction per access (scalar descriptor, one vector
// register of offset, one scalar register of offset), no 64-bit address arithmetic or address
// registers per lane.  `bytes` is the size of the window that starts at the pointer: loads
// beyond it return zero and stores beyond it are dropped by the hardware, so a caller that
// passes "bytes left in the tensor" needs no clamping to keep ragged tiles inside the
// allocation.  The default window is the maximum (no bounds check).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes = 0xffffffffu) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
// bytes from element offset `at` to the end of a tensor of `end` elements, as a buffer window
__device__ __forceinline__ uint32_t window_bytes(int64_t end, int64_t at, int es) {
    const int64_t left = (end - at) * es;
    return left <= 0 ? 0u : left > 0xffffffffll ? 0xffffffffu : (uint32_t)left;
}
__device__ __forceinline__ float ld_off(const float* base, uint32_t voff, uint32_t soff = 0,
                                        uint32_t bytes = 0xffffffffu) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(make_rsrc(base, bytes), voff, soff, 0));
}
__device__ __forceinline__ bf16_t ld_off(const bf16_t* base, uint32_t voff, uint32_t soff = 0,
                                         uint32_t bytes = 0xffffffffu) {
    return __builtin_bit_cast(bf16_t, __builtin_amdgcn_raw_buffer_load_b16(make_rsrc(base, bytes), voff, soff, 0));
}
__device__ __forceinline__ void st_off(float* base, uint32_t voff, float v, uint32_t soff = 0) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), make_rsrc(base), voff, soff, 0);
}
__device__ __forceinline__ void st_off(bf16_t* base, uint32_t voff, bf16_t v, uint32_t soff = 0) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), make_rsrc(base), voff, soff, 0);
}
// A delta element as loaded (see the service waves): float32 bits, or bfloat16 bits in the low half;
// `shift` is 16 for the latter, 0 for the former (wave-uniform, one instruction either way).
__device__ __forceinline__ uint32_t ld_bits32(const void* base, uint32_t voff, uint32_t soff, uint32_t bytes) {
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(make_rsrc(base, bytes), voff, soff, 0);
}
__device__ __forceinline__ uint32_t ld_bits16(const void* base, uint32_t voff, uint32_t soff, uint32_t bytes) {
    return (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(make_rsrc(base, bytes), voff, soff, 0);
}
__device__ __forceinline__ float bits_to_float(uint32_t bits, uint32_t shift) { return __uint_as_float(bits << shift); }
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st_off(float2* base, uint32_t voff, float2 v, uint32_t soff = 0) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), make_rsrc(base), voff, soff, 0);
}
__device__ __forceinline__ void st_off(float4* base, uint32_t voff, float4 v, uint32_t soff = 0) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), make_rsrc(base), voff, soff, 0);
}

__device__ __forceinline__ int wave_id() {
    // threadIdx.x / 64, told to the compiler as wave-uniform
    return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
}

typedef float f16v __attribute__((ext_vector_type(16)));

// COUNT consecutive floats through the scalar cache into SGPRs (the address is wave-uniform)
template <int COUNT>
__device__ __forceinline__ void scalar_load(const float* src, float (&dst)[COUNT]) {
    static_assert(COUNT % 16 == 0, "scalar_load moves multiples of 16 floats");
    const uintptr_t a = reinterpret_cast<uintptr_t>(src);
#pragma unroll
    for (int j = 0; j < COUNT / 16; ++j) {
        const f16v v = *reinterpret_cast<const __attribute__((address_space(4))) f16v*>(a + 64 * j);
#pragma unroll
        for (int k = 0; k < 16; ++k) dst[16 * j + k] = v[k];
    }
}

// acc + v[lane T of the reader's row of 16 lanes] * x in ONE instruction: the DPP control
// row_newbcast broadcasts lane T of every row to the 16 lanes of that row on the way into the
// multiplier.  A register that holds 16 wave-uniform values (one per lane of a row, the same
// in all four rows) thus feeds 16 different FMAs without a move or a scalar register.
template <int T>
__device__ __forceinline__ float fmac_bcast(float acc, float v, float x) {
    static_assert(T >= 0 && T < 16, "lane inside a row");
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(acc)
        : "v"(v), "v"(x), "n"(T));
    return acc;
}
// v[lane T of the reader's row] * x (same broadcast, no accumulator)
template <int T>
__device__ __forceinline__ float mul_bcast(float v, float x) {
    static_assert(T >= 0 && T < 16, "lane inside a row");
    float r;
    asm("v_mul_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v), "v"(x), "n"(T));
    return r;
}

inline int check_launch() { return hipGetLastError() == hipSuccess ? MPA_OK : MPA_ERR_LAUNCH; }

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline size_t dtype_size(int dt) { return dt == MPA_BF16 ? 2 : 4; }

// states owned by one lane of a scan wave, chosen from the problem size so that the launch
// fills the 1024 SIMDs of the chip (the only parallel axes are batch*dim and d_state)
int pick_states_per_lane(int64_t batch, int64_t dim, int64_t dstate, int ns_max, int pinned);
int padded_states(int64_t n);
int validate_shape(const mpa_sscan_shape* s);
// B and C repacked as float32 for scalar loads (see pack_bc_kernel in sscan_fwd.hip)
size_t bcpack_floats(const mpa_sscan_shape* s);
int launch_pack_bc(const mpa_sscan_shape* s, const void* B, const void* C, float* out, int ns,
                   int steps_per_subtile, hipStream_t st);

// Kernels may use more LDS than the 64 KB a static __shared__ array can hold (gfx950 has
// 160 KB per CU), so they take dynamic LDS; the limit is raised once per kernel and device (the
// attribute belongs to the kernel's code object on the device that is current).
template <typename K>
inline int allow_dynamic_lds(K kernel, size_t bytes) {
    if (bytes > 160 * 1024) return MPA_ERR_BAD_SHAPE;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               static_cast<int>(bytes)) == hipSuccess
               ? MPA_OK
               : MPA_ERR_LAUNCH;
}
// One per launch site: remembers on which devices the limit of that site's kernel has been raised.
struct LdsLimitOnce {
    static constexpr int kMaxDevices = 64;
    std::atomic<bool> done[kMaxDevices] = {};
    template <typename K>
    int ensure(K kernel, size_t bytes) {
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MPA_ERR_LAUNCH;
        if (done[dev].load(std::memory_order_acquire)) return MPA_OK;
        const int rc = allow_dynamic_lds(kernel, bytes);
        if (rc == MPA_OK) done[dev].store(true, std::memory_order_release);
        return rc;
    }
};

}  // namespace mpa
