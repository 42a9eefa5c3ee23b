// Device helpers shared by the quantise / dequantise / decode kernels.
#pragma once
#include "common.h"

// ---- bit-field helpers over register arrays (indices are constants once loops are unrolled) ----
template <int W>
__device__ static inline uint32_t get_code(const uint32_t* w, int i) {
    const int bit = i * W, k = bit >> 5, sh = bit & 31;
    uint32_t v = w[k] >> sh;
    if (sh + W > 32) v |= w[k + 1] << (32 - sh);
    return v & ((1u << W) - 1u);
}
template <int W>
__device__ static inline void put_code(uint32_t* w, int i, uint32_t c) {
    const int bit = i * W, k = bit >> 5, sh = bit & 31;
    w[k] |= c << sh;
    if (sh + W > 32) w[k + 1] |= c >> (32 - sh);
}

// V layout: word k (of 2W) of dim j lives in a unit of U bytes
template <int W>
__device__ static inline size_t v_word_offset(int k, int j) {
    constexpr int U = (W == 3) ? 8 : 16;
    constexpr int WPU = U / 4;
    return ((size_t)(k / WPU) * HD + j) * U + (size_t)(k % WPU) * 4;
}

template <int DT>
__device__ static inline void load_row(const void* base, size_t elem_off, float* x) {
    if constexpr (DT == ODMKV_F32) {
        const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + elem_off);
#pragma unroll
        for (int c = 0; c < 32; ++c) {
            const float4 v = p[c];
            x[4 * c] = v.x; x[4 * c + 1] = v.y; x[4 * c + 2] = v.z; x[4 * c + 3] = v.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + elem_off);
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const uint4 v = p[c];
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[8 * c + 2 * e] = Elem<DT>::to_f32((uint16_t)(w[e] & 0xffffu));
                x[8 * c + 2 * e + 1] = Elem<DT>::to_f32((uint16_t)(w[e] >> 16));
            }
        }
    }
}

// index of the centroid nearest to y among K = 2^W sorted centroids in LDS (lower index on a tie)
template <int W>
__device__ static inline uint32_t nearest_code(float y, const float* cb) {
    constexpr int K = 1 << W;
    int pos = 0;
#pragma unroll
    for (int s = K / 2; s >= 1; s >>= 1)
        if (cb[pos + s - 1] < y) pos += s;       // pos = min(#centroids below y, K-1)
    pos = pos < 1 ? 1 : pos;
    const float dl = fabsf(y - cb[pos - 1]);
    const float dh = fabsf(y - cb[pos]);
    return dh < dl ? (uint32_t)pos : (uint32_t)(pos - 1);
}

template <int DT>
__device__ static inline void store8(void* base, size_t elem_off, const float* v) {
    if constexpr (DT == ODMKV_F32) {
        float4* p = reinterpret_cast<float4*>(reinterpret_cast<float*>(base) + elem_off);
        p[0] = make_float4(v[0], v[1], v[2], v[3]);
        p[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint4 pk;
        pk.x = Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
        pk.y = Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
        pk.z = Elem<DT>::from_f32(v[4]) | ((uint32_t)Elem<DT>::from_f32(v[5]) << 16);
        pk.w = Elem<DT>::from_f32(v[6]) | ((uint32_t)Elem<DT>::from_f32(v[7]) << 16);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(base) + elem_off) = pk;
    }
}

