// Shared pieces of libpromptcache_blocks.so (gfx950 only): the building-block kernels of decoder designs whose tensors are
// plain row-major bf16 or fp32 (no fragment images, no split planes) with an fp32 residual stream.
//
// Every kernel is a template over the element type E of weights, activations and cached keys: `bf16_t` (matrix products on
// v_mfma_f32_16x16x32_bf16, fp32 accumulation) or `float` (v_mfma_f32_16x16x4_f32: true fp32 products).  One "k-step" is 32
// k elements in both cases, so the tiling code does not branch on the type.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/promptcache_blocks.h"

#define PCB_EXPORT extern "C" __attribute__((visibility("default")))

void pcb_set_error(const char* fmt, ...);

#define PCB_REQUIRE(cond, code, ...)    \
    do {                                \
        if (!(cond)) {                  \
            pcb_set_error(__VA_ARGS__); \
            return (code);              \
        }                               \
    } while (0)

static inline int pcb_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        pcb_set_error("%s: %s", what, hipGetErrorString(e));
        return PCB_ERR_HIP_BASE - (int)e;
    }
    return PCB_OK;
}

static inline int pcb_ceil_div(int a, int b) { return (a + b - 1) / b; }

#ifdef __HIPCC__
namespace pcb {

struct bf16_t {
    uint16_t bits;
};

typedef float f4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float to_f32(float v) { return v; }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename E>
__device__ __forceinline__ E from_f32(float f);
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) {
    bf16_t r;
    r.bits = bf16_bits(f);
    return r;
}
template <>
__device__ __forceinline__ float from_f32<float>(float f) {
    return f;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---- MFMA operand fragments of one 32-element k-step -----------------------------------------------------------------
// A 16 x 32 operand tile (16 rows of the A matrix, or 16 columns of B given as rows of B^T) is held by a wave as: lane l owns
// row (l & 15) and the 8 k elements lane_k<E>(l >> 4, e), e = 0..7.  bf16: 8 consecutive elements (one MFMA);
// fp32: elements 4*e + group (eight 16x16x4 MFMAs).  A and B use the same map, so any k permutation cancels.
template <typename E>
struct Frag;
template <>
struct Frag<bf16_t> {
    u32x4 v;
};
template <>
struct Frag<float> {
    float v[8];
};

template <typename E>
__device__ __forceinline__ int lane_k(int group, int e);
template <>
__device__ __forceinline__ int lane_k<bf16_t>(int group, int e) {
    return 8 * group + e;
}
template <>
__device__ __forceinline__ int lane_k<float>(int group, int e) {
    return 4 * e + group;
}

// p points at k element 0 of this k-step in the lane's row; `valid` elements from there exist (<= 0: none).
// `vec`: p + 8*group is 16-byte aligned and the row may be read with one 16-byte load (bf16 only).
__device__ __forceinline__ Frag<bf16_t> load_frag(const bf16_t* p, int group, int valid, bool vec) {
    Frag<bf16_t> f;
    if (vec && valid >= 32) {
        f.v = *reinterpret_cast<const u32x4*>(p + 8 * group);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k0 = 8 * group + 2 * e;
            const uint32_t lo = k0 < valid ? p[k0].bits : 0u;
            const uint32_t hi = k0 + 1 < valid ? p[k0 + 1].bits : 0u;
            w[e] = lo | (hi << 16);
        }
        f.v = u32x4{w[0], w[1], w[2], w[3]};
    }
    return f;
}
__device__ __forceinline__ Frag<float> load_frag(const float* p, int group, int valid, bool) {
    Frag<float> f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int k = 4 * e + group;
        f.v[e] = k < valid ? p[k] : 0.0f;
    }
    return f;
}

__device__ __forceinline__ f4 mma(const Frag<bf16_t>& a, const Frag<bf16_t>& b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a.v), __builtin_bit_cast(bf8, b.v), c, 0, 0, 0);
}
__device__ __forceinline__ f4 mma(const Frag<float>& a, const Frag<float>& b, f4 c) {
#pragma unroll
    for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[e], b.v[e], c, 0, 0, 0);
    return c;
}
// result tile: lane l holds column (l & 15), rows 4 * (l >> 4) + r, r = 0..3

}  // namespace pcb
#endif
