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

// ---- tile layouts (see include/odmkv.h) ----------------------------------------------------------
// Every tile buffer is W (codes) or 16 (exact rows) chunks of 16 bytes per lane; chunk c of lane l sits
// at byte (c*64 + l)*16 of the tile.  Lane l = 16j + n.
//   key codes:    the lane's 128 codes are  code 32b + i   = dim 32j + i   of slot key_slot(n, b)
//   value codes:  the lane's 128 codes are  code 64k + 8m + e = slot 32k + 8j + e  of dim 16m + n
//   exact keys:   chunk 4b + k of the lane  = dims 32j + 8k .. + 7 of slot key_slot(n, b)
//   exact values: chunk 8k + m of the lane  = slots 32k + 8j .. + 7 of dim 16m + n
// Both halves of a lane's code bytes (and chunks 0-7 / 8-15 of its exact rows) belong to the same 32 slots,
// 32h .. 32h + 31: half a tile is a unit of work of its own.
// slot of key block b (0..3), column n (0..15): the two blocks of a half interleave, so that a lane's two
// softmax weights of a half sit next to each other in slot order
__host__ __device__ static inline int key_slot(int n, int b) { return 32 * (b >> 1) + 8 * (n >> 2) + 2 * (n & 3) + (b & 1); }
// index (in 16-bit elements) of element (slot, dim) inside an exact tile
__host__ __device__ static inline int exact_k_index(int slot, int dim) {
    const int b = 2 * (slot >> 5) + (slot & 1), n = 4 * ((slot >> 3) & 3) + ((slot >> 1) & 3);
    const int j = dim >> 5, k = (dim >> 3) & 3, e = dim & 7;
    return (((4 * b + k) * TILE) + 16 * j + n) * 8 + e;
}
__host__ __device__ static inline int exact_v_index(int slot, int dim) {
    const int k = slot >> 5, j = (slot >> 3) & 3, e = slot & 7, m = dim >> 4, n = dim & 15;
    return (((8 * k + m) * TILE) + 16 * j + n) * 8 + e;
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

