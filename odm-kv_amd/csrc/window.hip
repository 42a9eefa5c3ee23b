// Observation-window attention mass: p[h,t] = mean over the W window queries and the G query heads of a
// kv-head of softmax_t(q . k_t * scaling), causal inside the window, over the core tokens t >= n_sink.
//
// This is the per-query form of the scorer's attention estimate (the reference scores with ONE query per
// head, the mean query: kvquant/scorer.py:285-318; here every query of the last W positions votes).  It is a
// true dense contraction, [G W, 128] x [128, T] per kv-head, and runs on the 16-bit matrix instructions
// (v_mfma_f32_32x32x16_f16 / _bf16) with exact products of the model's own 16-bit values and fp32 sums.
//
// Two passes over K, the logits are never stored:
//   pass 1  rows of the matrix product = tokens, columns = queries: a lane owns a query and keeps that
//           query's running (max, sum) over the tokens it sees; per-wave results go to `stats`
//   stats   merge per query -> M + log2 Z
//   pass 2  rows = queries, columns = tokens: a lane owns a token and sums exp2(s - M - log2 Z) over the queries
// The same two operand fragments serve both passes; only their roles (A or B) swap.  The queries of a
// kv-head (up to 256 at a time) sit in LDS, a wave holds its 64 tokens in registers (each lane the half row it
// contracts) and every 16-byte LDS read of a query fragment feeds two matrix instructions.
#include "common.h"

#define WIN_CHUNK 256        // tokens per workgroup (4 waves x 64)
#define WIN_ROWS 256         // queries staged in LDS at a time
#define WIN_QROW 136         // 16-bit entries per LDS row: 128 + 8, 16-byte reads of consecutive rows on distinct banks

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct WinArgs {
    const void* K;
    const void* Q;        // [Hq, W, 128], same 16-bit type as K; the queries of kv-head h are rows h G W .. (h+1) G W
    int64_t sH, sT;
    int Hkv, G, W, R, T, Tc, n_sink, nchunks, nstat, qpos0;
    float c;              // scaling * log2(e): logits in base-2 units
    float* stats;         // [Hkv R][nstat][2]
    float* mz;            // [Hkv R]: maximum + log2(sum), both in base-2 units
    float* p;             // [Hkv][Tc]
};

template <int DT>
__device__ static inline f32x16 win_mfma(uint4 a, uint4 b, f32x16 c) {
    if constexpr (DT == ODMKV_F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// merge two (max, sum) pairs kept in base-2 units
__device__ static inline void ms2_merge(float& m, float& s, float m2, float s2) {
    const float mn = fmaxf(m, m2);
    if (mn == -INFINITY) { m = mn; s = 0.0f; return; }
    s = s * __builtin_amdgcn_exp2f(m - mn) + s2 * __builtin_amdgcn_exp2f(m2 - mn);
    m = mn;
}

// index (0..31) inside a 32-row block of accumulator register r of a lane in wave half `half`
__device__ static inline int acc_row(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

template <int DT, int PASS>
__global__ __launch_bounds__(256) void window_kernel(WinArgs a) {
    extern __shared__ __align__(16) uint16_t q_s[];                 // [WIN_ROWS][WIN_QROW]
    __shared__ float ml_s[WIN_ROWS];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, col = lane & 31, half = lane >> 5;
    const int t0 = chunk * WIN_CHUNK + wave * 64;                    // first of this wave's 64 core tokens
    const bool active = t0 < a.Tc;                                  // wave-uniform
    // keys at or before every window query need no causal test: only the last tokens do
    const bool need_mask = a.n_sink + t0 + 63 > a.qpos0;
    const bool tail = t0 + 64 > a.Tc;                               // some of the wave's tokens lie past the end
    // Operand fragments: the matrix instruction contracts over 16 elements per step, 8 from either half of
    // the wave; which 8 is free as long as both operands agree.  Here half h of the wave takes elements
    // 64 h + 8 st .. + 7 in step st, so a lane reads one contiguous 128-byte half row of its token (a whole
    // cache line, used by that lane alone) and nothing it does not use.
    uint4 k0[8], k1[8];                                             // half rows of tokens t0 + col and t0 + 32 + col
    if (active) {                                                   // rows past the end repeat the last row and are masked
        const uint4* p0 = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.K) + (size_t)h * a.sH +
                                                          (size_t)(a.n_sink + min(t0 + col, a.Tc - 1)) * a.sT + 64 * half);
        const uint4* p1 = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.K) + (size_t)h * a.sH +
                                                          (size_t)(a.n_sink + min(t0 + 32 + col, a.Tc - 1)) * a.sT + 64 * half);
#pragma unroll
        for (int i = 0; i < 8; ++i) { k0[i] = p0[i]; k1[i] = p1[i]; }
    }
    float pacc0 = 0.0f, pacc1 = 0.0f;
    const uint4* qsrc = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.Q) + (size_t)h * a.R * HD);
    for (int rg = 0; rg < a.R; rg += WIN_ROWS) {
        const int nr = min(WIN_ROWS, a.R - rg), nrb = (nr + 31) >> 5;
        __syncthreads();                                            // the previous group's reads are done
        {
            // all of a thread's 16-byte pieces are requested before the first is stored (one round trip to
            // the caches instead of sixteen)
            uint4 stage[WIN_ROWS * 16 / 256];
#pragma unroll
            for (int i = 0; i < WIN_ROWS * 16 / 256; ++i) {
                const int e = tid + 256 * i, row = e >> 4, pc = e & 15;
                stage[i] = row < nr ? qsrc[(size_t)(rg + row) * 16 + pc] : make_uint4(0u, 0u, 0u, 0u);
            }
#pragma unroll
            for (int i = 0; i < WIN_ROWS * 16 / 256; ++i) {
                const int e = tid + 256 * i, row = e >> 4, pc = e & 15;
                if (row < nrb * 32) *reinterpret_cast<uint4*>(q_s + (size_t)row * WIN_QROW + pc * 8) = stage[i];
            }
        }
        if (PASS == 2) {
            // queries beyond the last take weight 0: exp2(0 - inf)
            for (int e = tid; e < nrb * 32; e += 256) ml_s[e] = e < nr ? a.mz[(size_t)h * a.R + rg + e] : INFINITY;
        }
        __syncthreads();
        if (!active) {
            if (PASS == 1) {                                        // neutral entries for the merge
                for (int e = lane; e < nr; e += 64) {
                    float* st = a.stats + (((size_t)h * a.R + rg + e) * a.nstat + chunk * 4 + wave) * 2;
                    st[0] = -INFINITY; st[1] = 0.0f;
                }
            }
            continue;
        }
#pragma unroll 1
        for (int rb = 0; rb < nrb; ++rb) {
            f32x16 acc0, acc1;
#pragma unroll
            for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
            const uint16_t* qrow = q_s + (size_t)(rb * 32 + col) * WIN_QROW + 64 * half;
#pragma unroll
            for (int st = 0; st < 8; ++st) {
                const uint4 qv = *reinterpret_cast<const uint4*>(qrow + 8 * st);
                const uint4 ka = k0[st], kb = k1[st];
                if (PASS == 1) { acc0 = win_mfma<DT>(ka, qv, acc0); acc1 = win_mfma<DT>(kb, qv, acc1); }
                else { acc0 = win_mfma<DT>(qv, ka, acc0); acc1 = win_mfma<DT>(qv, kb, acc1); }
            }
            if (PASS == 1) {
                // this lane's query: row rho of the kv-head; its position decides which of the last keys it sees
                const int rho = rg + rb * 32 + col;
                const int qpos = a.qpos0 + rho % a.W;
                float mx = -INFINITY, z = 0.0f;
                if (!need_mask && !tail) {
                    // every token of the wave is a key every query sees: the maximum is taken on the raw
                    // products (the scale is positive) and the scale folds into the exponent
                    float mr = acc0[0];
#pragma unroll
                    for (int r = 0; r < 16; ++r) mr = fmaxf(mr, fmaxf(acc0[r], acc1[r]));
                    mx = mr * a.c;
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        z += __builtin_amdgcn_exp2f(__fmaf_rn(acc0[r], a.c, -mx)) + __builtin_amdgcn_exp2f(__fmaf_rn(acc1[r], a.c, -mx));
                } else {
                    float s0[16], s1[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int ta = t0 + acc_row(r, half), tb = ta + 32;
                        const bool va = ta < a.Tc && a.n_sink + ta <= qpos;
                        const bool vb = tb < a.Tc && a.n_sink + tb <= qpos;
                        s0[r] = va ? acc0[r] * a.c : -INFINITY;
                        s1[r] = vb ? acc1[r] * a.c : -INFINITY;
                        mx = fmaxf(mx, fmaxf(s0[r], s1[r]));
                    }
                    if (mx > -INFINITY) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) z += __builtin_amdgcn_exp2f(s0[r] - mx) + __builtin_amdgcn_exp2f(s1[r] - mx);
                    }
                }
                // the other half of the wave holds the same query's other tokens
                const float m2 = __shfl_xor(mx, 32, WAVE), z2 = __shfl_xor(z, 32, WAVE);
                ms2_merge(mx, z, m2, z2);
                if (half == 0 && rho < a.R) {
                    float* st = a.stats + (((size_t)h * a.R + rho) * a.nstat + chunk * 4 + wave) * 2;
                    st[0] = mx; st[1] = z;
                }
            } else {
                const int ta = t0 + col, tb = ta + 32;               // this lane's tokens
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = rb * 32 + acc_row(r, half);
                    const float ml = ml_s[row];                     // M + log2 Z: exp2(s - ml) = exp2(s - M) / Z
                    float ea = __builtin_amdgcn_exp2f(__fmaf_rn(acc0[r], a.c, -ml));
                    float eb = __builtin_amdgcn_exp2f(__fmaf_rn(acc1[r], a.c, -ml));
                    if (need_mask) {
                        const int qpos = a.qpos0 + (rg + row) % a.W;
                        if (a.n_sink + ta > qpos) ea = 0.0f;
                        if (a.n_sink + tb > qpos) eb = 0.0f;
                    }
                    pacc0 += ea; pacc1 += eb;
                }
            }
        }
    }
    if (PASS == 2 && active) {
        pacc0 += __shfl_xor(pacc0, 32, WAVE);
        pacc1 += __shfl_xor(pacc1, 32, WAVE);
        const int t = t0 + 32 * half + col;                         // the upper half stores the second block
        if (t < a.Tc) a.p[(size_t)h * a.Tc + t] = (half ? pacc1 : pacc0) / (float)a.R;
    }
}

// merge a query's per-wave statistics into (maximum, reciprocal sum)
__global__ __launch_bounds__(64) void window_stats_kernel(WinArgs a) {
    const size_t row = blockIdx.x;
    const int lane = threadIdx.x;
    float m = -INFINITY, s = 0.0f;
    for (int e = lane; e < a.nstat; e += WAVE) {
        const float* st = a.stats + (row * a.nstat + e) * 2;
        ms2_merge(m, s, st[0], st[1]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float m2 = __shfl_xor(m, o, WAVE), s2 = __shfl_xor(s, o, WAVE);
        ms2_merge(m, s, m2, s2);
    }
    // M + log2 Z; a query that sees no key at all (cannot happen when the window lies behind the sinks) votes for nothing
    if (lane == 0) a.mz[row] = (m > -INFINITY && s > 0.0f) ? m + __builtin_amdgcn_logf(s) : INFINITY;
}

static inline int win_chunks(int Tc) { return (Tc + WIN_CHUNK - 1) / WIN_CHUNK; }

extern "C" size_t odmkv_window_attention_workspace_bytes(int Hkv, int Hq, int W, int T) {
    if (Hkv <= 0 || Hq <= 0 || W <= 0 || T <= 0) return 0;
    const size_t rows = (size_t)Hq * W, nstat = (size_t)win_chunks(T) * 4;
    return align_up(rows * nstat * 8, 256) + align_up(rows * 8, 256);
}

template <int DT>
static int run_window(WinArgs& a, hipStream_t st) {
    const int lds = WIN_ROWS * WIN_QROW * (int)sizeof(uint16_t);
    ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&window_kernel<DT, 1>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&window_kernel<DT, 2>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    dim3 grid(a.nchunks, a.Hkv), block(256);
    hipLaunchKernelGGL((window_kernel<DT, 1>), grid, block, lds, st, a);
    ODMKV_CHECK_LAUNCH("window_kernel<1>");
    hipLaunchKernelGGL(window_stats_kernel, dim3(a.Hkv * a.R), dim3(64), 0, st, a);
    ODMKV_CHECK_LAUNCH("window_stats_kernel");
    hipLaunchKernelGGL((window_kernel<DT, 2>), grid, block, lds, st, a);
    ODMKV_CHECK_LAUNCH("window_kernel<2>");
    return 0;
}

extern "C" int odmkv_window_attention(const void* K, int dtype, int Hkv, int T, int64_t stride_h, int64_t stride_t,
                                      const void* Q, int Hq, int W, int q_pos0, int n_sink, float scaling,
                                      float* p, void* workspace, size_t workspace_bytes, void* stream) {
    ODMKV_CHECK_ARG(K && Q && p && workspace, "window_attention: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16,
                    "window_attention: keys and queries must be float16 or bfloat16 (dtype %d)", dtype);
    ODMKV_CHECK_ARG(Hkv > 0 && Hq > 0 && Hq % Hkv == 0, "window_attention: bad head counts Hkv=%d Hq=%d", Hkv, Hq);
    ODMKV_CHECK_ARG(W >= 1 && W <= 4096, "window_attention: bad window %d", W);
    ODMKV_CHECK_ARG(n_sink >= 0 && T > n_sink, "window_attention: need T > n_sink (T=%d, n_sink=%d)", T, n_sink);
    ODMKV_CHECK_ARG(q_pos0 >= n_sink, "window_attention: the window must lie behind the sinks (q_pos0=%d, n_sink=%d)", q_pos0, n_sink);
    ODMKV_CHECK_ARG(stride_h % 8 == 0 && stride_t % 8 == 0 && stride_t >= HD, "window_attention: strides must keep rows 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)Q & 15) == 0, "window_attention: K and Q must be 16-byte aligned");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_window_attention_workspace_bytes(Hkv, Hq, W, T), "window_attention: workspace too small");
    WinArgs a;
    a.K = K; a.Q = Q; a.sH = stride_h; a.sT = stride_t;
    a.Hkv = Hkv; a.G = Hq / Hkv; a.W = W; a.R = a.G * W; a.T = T; a.Tc = T - n_sink; a.n_sink = n_sink;
    a.nchunks = win_chunks(a.Tc); a.nstat = a.nchunks * 4; a.qpos0 = q_pos0;
    a.c = scaling * 1.4426950408889634f;
    const size_t rows = (size_t)Hq * W;
    a.stats = (float*)workspace;                          // the workspace is sized for the chunks of all T tokens
    a.mz = (float*)((char*)workspace + align_up(rows * (size_t)win_chunks(T) * 4 * 8, 256));
    a.p = p;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODMKV_F16) return run_window<ODMKV_F16>(a, st);
    return run_window<ODMKV_BF16>(a, st);
}
