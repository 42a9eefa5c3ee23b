// Shared host/device helpers for libodmkv (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/odmkv.h"

#define HD ODMKV_HEAD_DIM       // 128
#define TILE ODMKV_TILE         // 64
#define WAVE 64

// ---- error slot -------------------------------------------------------------------------------
void odmkv_set_error(const char* fmt, ...);

#define ODMKV_CHECK_ARG(cond, ...)                 \
    do {                                           \
        if (!(cond)) {                             \
            odmkv_set_error(__VA_ARGS__);          \
            return ODMKV_EINVAL;                   \
        }                                          \
    } while (0)

#define ODMKV_CHECK_HIP(expr)                                                        \
    do {                                                                             \
        hipError_t e_ = (expr);                                                      \
        if (e_ != hipSuccess) {                                                      \
            odmkv_set_error("%s failed: %s", #expr, hipGetErrorString(e_));          \
            return ODMKV_EHIP;                                                       \
        }                                                                            \
    } while (0)

#define ODMKV_CHECK_LAUNCH(name)                                                     \
    do {                                                                             \
        hipError_t e_ = hipGetLastError();                                           \
        if (e_ != hipSuccess) {                                                      \
            odmkv_set_error("launch of %s failed: %s", name, hipGetErrorString(e_)); \
            return ODMKV_EHIP;                                                       \
        }                                                                            \
    } while (0)

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
// pack.hip: byte offset, inside the pack workspace, of the list of tiles the fp16 quantiser hands to the exact one
size_t pack_redo_offset(int nseg, int T);

// level index of a bit width: 0 -> evicted, 2,3,4,8 -> 1..4, 16 -> 5; anything else -> -1
__host__ __device__ static inline int level_slot(int bits) {
    switch (bits) {
        case 0: return 0;
        case 2: return 1;
        case 3: return 2;
        case 4: return 3;
        case 8: return 4;
        case 16: return 5;
        default: return -1;
    }
}
__host__ __device__ static inline int width_of(int li) { return li == 0 ? 2 : li == 1 ? 3 : li == 2 ? 4 : 8; }
// offset of width li's table inside the concatenated codebook array (4 + 8 + 16 + 256 floats)
__host__ __device__ static inline int codebook_offset(int li) { return li == 0 ? 0 : li == 1 ? 4 : li == 2 ? 12 : 28; }
#define CODEBOOK_FLOATS 284

// ---- element loads ----------------------------------------------------------------------------
template <int DT> struct Elem;
template <> struct Elem<ODMKV_F16> {
    typedef uint16_t raw;
    __device__ static inline float to_f32(uint16_t v) { return __half2float(__ushort_as_half(v)); }
    __device__ static inline uint16_t from_f32(float f) { return __half_as_ushort(__float2half_rn(f)); }
};
template <> struct Elem<ODMKV_BF16> {
    typedef uint16_t raw;
    __device__ static inline float to_f32(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
    __device__ static inline uint16_t from_f32(float f) {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);   // quiet NaN
        u += 0x7fffu + ((u >> 16) & 1u);                                            // round to nearest even
        return (uint16_t)(u >> 16);
    }
};
template <> struct Elem<ODMKV_F32> {
    typedef float raw;
    __device__ static inline float to_f32(float v) { return v; }
    __device__ static inline float from_f32(float f) { return f; }
};

// wave-wide reductions (64 lanes) through cross-lane shuffles
__device__ static inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ static inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
