// Shared device helpers for the gated delta-rule kernels (gfx950 / CDNA4, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gdn_hip.h"

namespace gdn {

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

constexpr float L2NORM_EPS = 1e-6f;
constexpr int WAVE = 64;

template <typename T>
__device__ __forceinline__ float to_f32(T x) {
    return static_cast<float>(x);
}

template <typename T>
__device__ __forceinline__ T from_f32(float x) {
    return static_cast<T>(x);
}

// Sum over the 64 lanes of a wave, result in every lane.
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, WAVE);
    return x;
}

// Load / store 4 consecutive elements as fp32.
template <typename T>
__device__ __forceinline__ f32x4 load4(const T* p);

template <>
__device__ __forceinline__ f32x4 load4<float>(const float* p) {
    return *reinterpret_cast<const f32x4*>(p);
}

template <>
__device__ __forceinline__ f32x4 load4<bf16_t>(const bf16_t* p) {
    bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
    f32x4 r;
    r.x = (float)x.x;
    r.y = (float)x.y;
    r.z = (float)x.z;
    r.w = (float)x.w;
    return r;
}

template <typename T>
__device__ __forceinline__ void store4(T* p, f32x4 x);

template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4 x) {
    *reinterpret_cast<f32x4*>(p) = x;
}

template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4 x) {
    bf16x4 r;
    r.x = (bf16_t)x.x;
    r.y = (bf16_t)x.y;
    r.z = (bf16_t)x.z;
    r.w = (bf16_t)x.w;
    *reinterpret_cast<bf16x4*>(p) = r;
}

// Packed sequences: first token and length of sequence n from cu_seqlens, which lives on the device and is
// never seen by the host-side checks: clamped into [0, total] and made non-negative, so that a malformed
// prefix (decreasing, or running past the packed token count) gives short or empty sequences and never
// an address outside the tensors.
__device__ __forceinline__ void packed_bounds(const int32_t* cu, int n, int total, int& t0, int& len) {
    t0 = min(max(cu[n], 0), total);
    len = min(max(cu[n + 1], t0), total) - t0;
}

// beta / g are per (token, head) scalars; beta may be bf16 or fp32, NULL means 1.
__device__ __forceinline__ float load_beta(const void* beta, int beta_dtype, int64_t idx) {
    if (beta == nullptr) return 1.0f;
    if (beta_dtype == GDN_BF16) return (float)reinterpret_cast<const bf16_t*>(beta)[idx];
    return reinterpret_cast<const float*>(beta)[idx];
}

}  // namespace gdn
