// Row-wise TurboQuant-MSE quantise / dequantise without the packed store (one lane per row).
// Same arithmetic, in the same order, as the tile kernels of the packed store.
#include "quant.h"

template <int W, int DT>
__global__ __launch_bounds__(64) void quantize_rows_kernel(const void* x, int64_t N, int64_t stride_n,
                                                           const float* __restrict__ pi, const float* __restrict__ cbg,
                                                           uint8_t* __restrict__ codes, float* __restrict__ norms) {
    __shared__ float cb[1 << W];
    const int lane = threadIdx.x;
    for (int i = lane; i < (1 << W); i += WAVE) cb[i] = cbg[i];
    __syncthreads();
    const int64_t n = (int64_t)blockIdx.x * WAVE + lane;
    const bool valid = n < N;
    float u[HD];
    if (valid) load_row<DT>(x, (size_t)n * stride_n, u);
    else {
#pragma unroll
        for (int j = 0; j < HD; ++j) u[j] = 0.0f;
    }
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < HD; ++j) ss = __fmaf_rn(u[j], u[j], ss);
    const float norm = sqrtf(ss);
    const float den = norm + 1e-10f;
#pragma unroll
    for (int j = 0; j < HD; ++j) u[j] = u[j] / den;
    if (valid) norms[n] = norm;
#pragma unroll 1
    for (int i0 = 0; i0 < HD; i0 += 8) {
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        const float* __restrict__ rows = pi + (size_t)i0 * HD;
#pragma unroll
        for (int j = 0; j < HD; ++j) {
#pragma unroll
            for (int b = 0; b < 8; ++b) acc[b] = __fmaf_rn(u[j], rows[b * HD + j], acc[b]);
        }
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) w0 |= nearest_code<W>(acc[b], cb) << (8 * b);
#pragma unroll
        for (int b = 0; b < 4; ++b) w1 |= nearest_code<W>(acc[4 + b], cb) << (8 * b);
        if (valid) *reinterpret_cast<uint2*>(codes + (size_t)n * HD + i0) = make_uint2(w0, w1);
    }
}

template <int W>
__global__ __launch_bounds__(64) void dequantize_rows_kernel(const uint8_t* __restrict__ codes,
                                                             const float* __restrict__ norms, int64_t N,
                                                             const float* __restrict__ pi, const float* __restrict__ cbg,
                                                             float* __restrict__ out) {
    __shared__ float cb[1 << W];
    const int lane = threadIdx.x;
    for (int i = lane; i < (1 << W); i += WAVE) cb[i] = cbg[i];
    __syncthreads();
    const int64_t n = (int64_t)blockIdx.x * WAVE + lane;
    if (n >= N) return;
    float y[HD];
    const uint4* src = reinterpret_cast<const uint4*>(codes + (size_t)n * HD);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint4 v = src[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 16; ++e) y[16 * c + e] = cb[((w[e >> 2] >> (8 * (e & 3))) & 0xffu) & ((1u << W) - 1u)];
    }
    const float norm = norms[n];
#pragma unroll 1
    for (int j0 = 0; j0 < HD; j0 += 8) {
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < HD; ++i) {
#pragma unroll
            for (int b = 0; b < 8; ++b) acc[b] = __fmaf_rn(y[i], pi[i * HD + j0 + b], acc[b]);
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[b] = acc[b] * norm;
        store8<ODMKV_F32>(out, (size_t)n * HD + j0, acc);
    }
}

template <int W>
static int launch_quantize_rows(const void* x, int dtype, int64_t N, int64_t stride_n, const float* pi,
                                const float* cb, uint8_t* codes, float* norms, hipStream_t st) {
    dim3 grid((unsigned)((N + WAVE - 1) / WAVE)), block(64);
    if (dtype == ODMKV_F16) hipLaunchKernelGGL((quantize_rows_kernel<W, ODMKV_F16>), grid, block, 0, st, x, N, stride_n, pi, cb, codes, norms);
    else if (dtype == ODMKV_BF16) hipLaunchKernelGGL((quantize_rows_kernel<W, ODMKV_BF16>), grid, block, 0, st, x, N, stride_n, pi, cb, codes, norms);
    else hipLaunchKernelGGL((quantize_rows_kernel<W, ODMKV_F32>), grid, block, 0, st, x, N, stride_n, pi, cb, codes, norms);
    ODMKV_CHECK_LAUNCH("quantize_rows_kernel");
    return 0;
}

extern "C" int odmkv_quantize_rows(const void* x, int dtype, int64_t N, int64_t stride_n, int bits,
                                   const float* pi, const float* cb, uint8_t* codes, float* norms,
                                   void* stream) {
    ODMKV_CHECK_ARG(x && pi && cb && codes && norms, "quantize_rows: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "quantize_rows: bad dtype %d", dtype);
    ODMKV_CHECK_ARG(bits == 2 || bits == 3 || bits == 4 || bits == 8, "quantize_rows: width %d not in {2,3,4,8}", bits);
    ODMKV_CHECK_ARG(N >= 0 && N < ((int64_t)1 << 37), "quantize_rows: bad row count");
    const int align = dtype == ODMKV_F32 ? 4 : 8;
    ODMKV_CHECK_ARG(stride_n % align == 0 && stride_n >= HD && ((uintptr_t)x & 15) == 0 && ((uintptr_t)codes & 15) == 0,
                    "quantize_rows: rows must be 16-byte aligned");
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
        case 2: return launch_quantize_rows<2>(x, dtype, N, stride_n, pi, cb, codes, norms, st);
        case 3: return launch_quantize_rows<3>(x, dtype, N, stride_n, pi, cb, codes, norms, st);
        case 4: return launch_quantize_rows<4>(x, dtype, N, stride_n, pi, cb, codes, norms, st);
        default: return launch_quantize_rows<8>(x, dtype, N, stride_n, pi, cb, codes, norms, st);
    }
}

extern "C" int odmkv_dequantize_rows(const uint8_t* codes, const float* norms, int64_t N, int bits,
                                     const float* pi, const float* cb, float* out, void* stream) {
    ODMKV_CHECK_ARG(codes && norms && pi && cb && out, "dequantize_rows: null pointer");
    ODMKV_CHECK_ARG(bits == 2 || bits == 3 || bits == 4 || bits == 8, "dequantize_rows: width %d not in {2,3,4,8}", bits);
    ODMKV_CHECK_ARG(N >= 0 && N < ((int64_t)1 << 37), "dequantize_rows: bad row count");
    ODMKV_CHECK_ARG(((uintptr_t)codes & 15) == 0 && ((uintptr_t)out & 15) == 0, "dequantize_rows: buffers must be 16-byte aligned");
    if (N == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)((N + WAVE - 1) / WAVE)), block(64);
    switch (bits) {
        case 2: hipLaunchKernelGGL((dequantize_rows_kernel<2>), grid, block, 0, st, codes, norms, N, pi, cb, out); break;
        case 3: hipLaunchKernelGGL((dequantize_rows_kernel<3>), grid, block, 0, st, codes, norms, N, pi, cb, out); break;
        case 4: hipLaunchKernelGGL((dequantize_rows_kernel<4>), grid, block, 0, st, codes, norms, N, pi, cb, out); break;
        default: hipLaunchKernelGGL((dequantize_rows_kernel<8>), grid, block, 0, st, codes, norms, N, pi, cb, out); break;
    }
    ODMKV_CHECK_LAUNCH("dequantize_rows_kernel");
    return 0;
}
