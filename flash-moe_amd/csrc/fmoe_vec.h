// 16-byte packet arithmetic shared by the row-streaming kernels: a packet is 4 fp32 or 8 bf16 / fp16 elements.
#pragma once

#include "fmoe_common.h"

namespace fmoe {

// dot of two 16-byte packets, accumulated into acc
template <typename T> __device__ inline float dot16(u32x4_t a, u32x4_t b, float acc);
template <> __device__ inline float dot16<float>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_fmaf(__uint_as_float(a[i]), __uint_as_float(b[i]), acc);
    return acc;
}
template <> __device__ inline float dot16<bf16_t>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // element first into a scalar: bit-casting the subscript expression itself reads element 0
        const uint32_t ai = a[i], bi = b[i];
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, ai), __builtin_bit_cast(bf16x2_t, bi), acc, false);
    }
    return acc;
}
template <> __device__ inline float dot16<f16_t>(u32x4_t a, u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t ai = a[i], bi = b[i];
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, ai), __builtin_bit_cast(f16x2_t, bi), acc, false);
    }
    return acc;
}

// acc[0..kVec) += s * packet
template <typename T> __device__ inline void axpy16(float s, u32x4_t w, float* acc);
template <> __device__ inline void axpy16<float>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(s, __uint_as_float(w[i]), acc[i]);
}
template <> __device__ inline void axpy16<bf16_t>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc[2 * i] = __builtin_fmaf(s, __uint_as_float(w[i] << 16), acc[2 * i]);
        acc[2 * i + 1] = __builtin_fmaf(s, __uint_as_float(w[i] & 0xffff0000u), acc[2 * i + 1]);
    }
}
template <> __device__ inline void axpy16<f16_t>(float s, u32x4_t w, float* acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t wi = w[i];
        f16x2_t p = __builtin_bit_cast(f16x2_t, wi);
        acc[2 * i] = __builtin_fmaf(s, (float)p[0], acc[2 * i]);
        acc[2 * i + 1] = __builtin_fmaf(s, (float)p[1], acc[2 * i + 1]);
    }
}

template <typename T> __device__ inline u32x4_t pack16(const float* v);
template <> __device__ inline u32x4_t pack16<float>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __float_as_uint(v[i]);
    return r;
}
template <> __device__ inline u32x4_t pack16<bf16_t>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bf16x2_t p = {(bf16_t)v[2 * i], (bf16_t)v[2 * i + 1]};
        r[i] = __builtin_bit_cast(uint32_t, p);
    }
    return r;
}
template <> __device__ inline u32x4_t pack16<f16_t>(const float* v) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f16x2_t p = {(f16_t)v[2 * i], (f16_t)v[2 * i + 1]};
        r[i] = __builtin_bit_cast(uint32_t, p);
    }
    return r;
}

// the elements of a packet as fp32
template <typename T> __device__ inline void unpack16(u32x4_t w, float* v);
template <> __device__ inline void unpack16<float>(u32x4_t w, float* v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(w[i]);
}
template <> __device__ inline void unpack16<bf16_t>(u32x4_t w, float* v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <> __device__ inline void unpack16<f16_t>(u32x4_t w, float* v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t wi = w[i];
        const f16x2_t p = __builtin_bit_cast(f16x2_t, wi);
        v[2 * i] = (float)p[0];
        v[2 * i + 1] = (float)p[1];
    }
}

}  // namespace fmoe
