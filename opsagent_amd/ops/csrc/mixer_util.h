// Element access helpers shared by the sequence-mixer and decoder-block
// kernels: activations and weights are bf16 (dt = 0) or float32 (dt = 1).
#pragma once

#include "common.h"

#include <algorithm>
#include <cstdlib>

typedef uint16_t bf16s;  // bf16 storage

__device__ __forceinline__ float ldf(const float* p, int64_t i) { return p[i]; }
__device__ __forceinline__ float ldf(const bf16s* p, int64_t i) { return bf16_to_f32(p[i]); }
__device__ __forceinline__ void stf(float* p, int64_t i, float v) { p[i] = v; }
__device__ __forceinline__ void stf(bf16s* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }

// 8 consecutive elements at once (16-byte aligned for bf16, 32 for float32)
__device__ __forceinline__ void ld8(const float* p, int64_t i, float* o) {
    const float4 a = *reinterpret_cast<const float4*>(p + i);
    const float4 b = *reinterpret_cast<const float4*>(p + i + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void ld8(const bf16s* p, int64_t i, float* o) {
    const uint4 a = *reinterpret_cast<const uint4*>(p + i);
    o[0] = bf16_lo(a.x); o[1] = bf16_hi(a.x); o[2] = bf16_lo(a.y); o[3] = bf16_hi(a.y);
    o[4] = bf16_lo(a.z); o[5] = bf16_hi(a.z); o[6] = bf16_lo(a.w); o[7] = bf16_hi(a.w);
}
__device__ __forceinline__ void st8(float* p, int64_t i, const float* v) {
    *reinterpret_cast<float4*>(p + i) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void st8(bf16s* p, int64_t i, const float* v) {
    uint4 a;
    a.x = pack_bf16x2(v[0], v[1]); a.y = pack_bf16x2(v[2], v[3]);
    a.z = pack_bf16x2(v[4], v[5]); a.w = pack_bf16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p + i) = a;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) {
    return fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z)));
}

static inline int grid_for(int64_t total) {
    return (int)std::max<int64_t>(1, std::min<int64_t>(4096, CEIL_DIV(total, 256)));
}
