// Shared by the kernels of the Mamba-2 block stages (forward and backward): activation functions and the 16-byte
// (bf16) or 32-byte (float) piece of eight consecutive channels a thread moves at a time.
#pragma once
#include "ssd_device.h"

namespace ssd {

__device__ inline float silu(float v) { return v * __builtin_amdgcn_rcpf(1.f + __expf(-v)); }
__device__ inline float softplus(float v) { return v > 20.f ? v : log1pf(__expf(v)); }

template <typename T> struct Pack8;  // eight consecutive channels
template <> struct Pack8<__bf16> {
    uint4 u;
    __device__ inline float get(int i) const {
        const unsigned w = (&u.x)[i >> 1];
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    static __device__ inline Pack8 load(const __bf16 *p) { return Pack8{*reinterpret_cast<const uint4 *>(p)}; }
    static __device__ inline void store(__bf16 *p, const float (&v)[8]) {
        uint4 o;
        o.x = pack_bf16x2(v[0], v[1]);
        o.y = pack_bf16x2(v[2], v[3]);
        o.z = pack_bf16x2(v[4], v[5]);
        o.w = pack_bf16x2(v[6], v[7]);
        *reinterpret_cast<uint4 *>(p) = o;
    }
};
template <> struct Pack8<float> {
    float4 a, b;
    __device__ inline float get(int i) const { return i < 4 ? (&a.x)[i] : (&b.x)[i - 4]; }
    static __device__ inline Pack8 load(const float *p) {
        return Pack8{*reinterpret_cast<const float4 *>(p), *reinterpret_cast<const float4 *>(p + 4)};
    }
    static __device__ inline void store(float *p, const float (&v)[8]) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};

// derivative of silu: s (1 + v (1 - s)), s = sigmoid(v)
__device__ inline float dsilu(float v) {
    const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-v));
    return sg * (1.f + v * (1.f - sg));
}
__device__ inline float sigmoidf(float v) { return __builtin_amdgcn_rcpf(1.f + __expf(-v)); }

}  // namespace ssd
