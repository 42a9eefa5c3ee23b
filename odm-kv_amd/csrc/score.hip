// ODM risk score  s = (p + eps)^2 * (|v|^2 + |k|^2/d * |v - obar|^2)  for one layer of one sequence.
//
// K and V are each streamed from HBM once for the sums that need them (V a second time for
// |v - obar|^2, which is computed directly rather than expanded, to avoid cancellation).
// A row of 128 elements is handled by 16 lanes x 8 elements, so a wavefront reads four rows
// (1 KB contiguous for a dense cache) per load instruction.  All reductions run in a fixed
// order (shuffle butterflies, then ordered sums over chunk partials): results do not depend
// on scheduling.
#include "common.h"

#define ROWS_PER_WG 256     // rows of one kv-head handled by a 256-thread workgroup
#define LANES_PER_ROW 16

struct ScoreArgs {
    const void* K;
    const void* V;
    int64_t sH, sT;
    int Hkv, Hq, G, Gl, T, Tc, n_sink, nchunks;   // Gl: heads the logits pass covers (0 when p is given)
    float eps;
    const float* mu;      // [Hq, 128]
    const float* attn;    // [Hkv, T] or null
    const float* cov;     // [Hq, 128, 128] query covariance (expected-attention score only) or null
    int round_dt;         // -1, or ODMKV_F16 / ODMKV_BF16: round logits, softmax and group mean like a model of that dtype
    int use_vnorm;        // expected-attention score: multiply (p + eps) by |v|
    int ea_cpw;           // expected-attention score: 256-token chunks a workgroup walks
    int nstat;            // softmax statistics entries per query head (one per chunk, or one per wave and chunk)
    float* scores;        // [Hkv, T]
    float* logits;        // [Hq, Tc]
    float* kn2;           // [Hkv, Tc]
    float* p;             // [Hkv, Tc]
    float* stats;         // [Hq, nchunks, 2]
    float* mz;            // [Hq, 2]
    float* opart;         // [Hkv, nchunks, 128]
    float* psum;          // [Hkv, nchunks]
    float* obar;          // [Hkv, 128]
};

template <int DT>
__device__ static inline void load8(const void* base, size_t elem_off, float* x) {
    if constexpr (DT == ODMKV_F32) {
        const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + elem_off);
        const float4 a = p[0], b = p[1];
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    } else {
        const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + elem_off);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[2 * e] = Elem<DT>::to_f32((uint16_t)(w[e] & 0xffffu));
            x[2 * e + 1] = Elem<DT>::to_f32((uint16_t)(w[e] >> 16));
        }
    }
}

// the same 8 elements as raw registers (so that a later trip's rows can be requested before the current
// trip's are converted and used), and their conversion
template <int DT> struct Raw8 { uint4 a; };
template <> struct Raw8<ODMKV_F32> { float4 a, b; };
template <int DT>
__device__ static inline void load8_raw(const void* base, size_t elem_off, Raw8<DT>& r) {
    if constexpr (DT == ODMKV_F32) {
        const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + elem_off);
        r.a = p[0]; r.b = p[1];
    } else {
        r.a = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + elem_off);
    }
}
template <int DT>
__device__ static inline void cvt8(const Raw8<DT>& r, float* x) {
    if constexpr (DT == ODMKV_F32) {
        x[0] = r.a.x; x[1] = r.a.y; x[2] = r.a.z; x[3] = r.a.w; x[4] = r.b.x; x[5] = r.b.y; x[6] = r.b.z; x[7] = r.b.w;
    } else {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[2 * e] = Elem<DT>::to_f32((uint16_t)(w[e] & 0xffffu));
            x[2 * e + 1] = Elem<DT>::to_f32((uint16_t)(w[e] >> 16));
        }
    }
}

// sum over the 16 lanes that share a row, by data-parallel-primitive moves (no LDS traffic): inside the
// quad, then the neighbouring quad, then the other half of the 16-lane row.  Every lane ends with the
// total; the order of the additions is fixed per lane (only lane 0 of the row is used).
template <int CTRL>
__device__ static inline float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ static inline float group16_sum(float v) {
    v += dpp_move<0xB1>(v);     // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);     // quad_perm [2,3,0,1]
    v += dpp_move<0x124>(v);    // row_ror 4
    v += dpp_move<0x128>(v);    // row_ror 8
    return v;
}
// workgroup barrier that orders LDS traffic only: global loads requested before it stay in flight
// (__syncthreads would first wait for every outstanding load of the wavefront, the rows from memory included)
__device__ static inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
#define SC_UNROLL 4            // rows in flight per lane group: their loads are issued before any is used
#define SC_UNROLL_V 4          // the same for the two passes over V

// merge two online-softmax states
// x as a model of 16-bit dtype `dt` would hold it (-1: unchanged)
__device__ static inline float round_model(float x, int dt) {
    return dt == ODMKV_F16 ? __half2float(__float2half_rn(x))
         : dt == ODMKV_BF16 ? Elem<ODMKV_BF16>::to_f32(Elem<ODMKV_BF16>::from_f32(x)) : x;
}

__device__ static inline void ms_merge(float& m, float& s, float m2, float s2) {
    const float mn = fmaxf(m, m2);
    if (mn == -INFINITY) { m = mn; s = 0.0f; return; }
    s = s * __expf(m - mn) + s2 * __expf(m2 - mn);
    m = mn;
}

// ---- pass 1 over K: logits of every query head, |k|^2, per-chunk softmax statistics ----
template <int DT, int GMAX>
__global__ __launch_bounds__(256) void score_logits_kernel(ScoreArgs a) {
    __shared__ float mu_s[GMAX * HD];
    __shared__ float red_m[4][GMAX], red_s[4][GMAX];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, part = lane & 15, rsub = lane >> 4;
    for (int e = tid; e < a.Gl * HD; e += 256) mu_s[e] = a.mu[(size_t)h * a.G * HD + e];
    __syncthreads();
    float mu_r[GMAX][8];
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) mu_r[g][e] = g < a.Gl ? mu_s[g * HD + part * 8 + e] : 0.0f;
    float m[GMAX], s[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) { m[g] = -INFINITY; s[g] = 0.0f; }
    const float inv_sqrt_d = 0.08838834764831845f;    // 1 / sqrt(128): a multiplication, one rounding like the division
    const int t0 = chunk * ROWS_PER_WG;
    // A group of 16 lanes takes four consecutive rows per trip (all four requested before any is
    // used).  The row sums leave the reduction in every lane of the group, so lane u < 4 of the group
    // owns row u: it stores the row's results (the 16 owners of a wave write 16 consecutive floats)
    // and keeps the running softmax statistics of its rows.
    static_assert(SC_UNROLL == 4, "four rows per lane group and trip");
    const bool owner = part < SC_UNROLL;
    // rows of the next trip are requested before the current trip's are used; rows past the end repeat the
    // last row (never stored)
    auto request = [&](int it0, Raw8<DT>* raw) {
        const int tb = t0 + it0 * 16 + (wave * 4 + rsub) * SC_UNROLL;
#pragma unroll
        for (int u = 0; u < SC_UNROLL; ++u)
            load8_raw<DT>(a.K, (size_t)h * a.sH + (size_t)(a.n_sink + min(tb + u, a.Tc - 1)) * a.sT + part * 8, raw[u]);
    };
    Raw8<DT> raw[SC_UNROLL], nraw[SC_UNROLL];
    request(0, raw);
#pragma unroll                 // straight-line code: the wait before a trip's first use counts only that trip's loads
    for (int it0 = 0; it0 < ROWS_PER_WG / 16; it0 += SC_UNROLL) {
        const int tb = t0 + it0 * 16 + (wave * 4 + rsub) * SC_UNROLL;
        if (it0 + SC_UNROLL < ROWS_PER_WG / 16) request(it0 + SC_UNROLL, nraw);
        float xs[SC_UNROLL][8];
#pragma unroll
        for (int u = 0; u < SC_UNROLL; ++u) cvt8<DT>(raw[u], xs[u]);
        float kn_own = 0.0f, d_own[GMAX];
#pragma unroll
        for (int g = 0; g < GMAX; ++g) d_own[g] = 0.0f;
#pragma unroll
        for (int u = 0; u < SC_UNROLL; ++u) {
            const float* x = xs[u];
            float kn = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) kn = __fmaf_rn(x[e], x[e], kn);
            kn = group16_sum(kn);
            kn_own = part == u ? kn : kn_own;
#pragma unroll
            for (int g = 0; g < GMAX; ++g) {
                if (g < a.Gl) {
                    float d = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) d = __fmaf_rn(x[e], mu_r[g][e], d);
                    d = group16_sum(d);
                    // a 16-bit model rounds the product and, again, the division by sqrt(d) (kvquant/scorer.py:309-310)
                    d = a.round_dt < 0 ? d * inv_sqrt_d : round_model(round_model(d, a.round_dt) / 11.313708498984761f, a.round_dt);
                    d_own[g] = part == u ? d : d_own[g];
                }
            }
        }
        const int t = tb + part;
        if (owner && t < a.Tc) {
            a.kn2[(size_t)h * a.Tc + t] = kn_own;
#pragma unroll
            for (int g = 0; g < GMAX; ++g) {
                if (g < a.Gl) {
                    a.logits[((size_t)h * a.G + g) * a.Tc + t] = d_own[g];
                    ms_merge(m[g], s[g], d_own[g], 1.0f);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < SC_UNROLL; ++u) raw[u] = nraw[u];
    }
    // only the owner lanes hold statistics; butterfly over the wave, then over the 4 waves
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        if (g < a.Gl) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float m2 = __shfl_xor(m[g], o, WAVE), s2 = __shfl_xor(s[g], o, WAVE);
                ms_merge(m[g], s[g], m2, s2);
            }
            if (lane == 0) { red_m[wave][g] = m[g]; red_s[wave][g] = s[g]; }
        }
    }
    __syncthreads();
    if (tid < a.Gl) {
        float mm = red_m[0][tid], ss = red_s[0][tid];
        for (int w = 1; w < 4; ++w) ms_merge(mm, ss, red_m[w][tid], red_s[w][tid]);
        float* st = a.stats + (((size_t)h * a.G + tid) * a.nchunks + chunk) * 2;
        st[0] = mm; st[1] = ss;
    }
}

// ---- pass 1 over 16-bit K on the matrix cores ----
// v_mfma_f32_16x16x32_{f16,bf16}: D[16x16] += A[16x32] . B[32x16]; lane (n = lane % 16, j = lane / 16) supplies
// A[n][8j+e] and B[8j+e][n] and holds D[4j+r][n].  B = 16 tokens x 32 dims of K exactly as they lie in memory (a
// lane's 16 bytes), A = the mean queries of four heads, head (row % 4) in every row, as 16-bit pieces whose sum
// is the fp32 value (fp16: high + low of the vector scaled by a power of two into fp16's range; bf16: three
// pieces).  A wave takes 64 tokens as four groups of 16; after the products lane (j, n) keeps group j's
// accumulator: the logits of four heads for token 16j + n.  |k|^2 is the diagonal of K_g . K_g^T, the same
// registers as both operands.  All of a workgroup's rows are requested before anything is computed.
typedef _Float16 sc_h8 __attribute__((ext_vector_type(8)));
typedef __bf16 sc_b8 __attribute__((ext_vector_type(8)));
typedef float sc_f4 __attribute__((ext_vector_type(4)));
template <int DT>
__device__ static __forceinline__ sc_f4 sc_mfma(const uint4& a, const uint4& b, const sc_f4& c) {
    if constexpr (DT == ODMKV_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sc_h8, a), __builtin_bit_cast(sc_h8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sc_b8, a), __builtin_bit_cast(sc_b8, b), c, 0, 0, 0);
}

template <int DT, int GMAX>
__global__ __launch_bounds__(256) void score_logits16_kernel(ScoreArgs a) {
    static_assert(DT == ODMKV_F16 || DT == ODMKV_BF16, "16-bit keys");
    static_assert(ROWS_PER_WG == 256, "four waves of 64 tokens");
    constexpr int NP = DT == ODMKV_F16 ? 2 : 3;     // 16-bit pieces of a mean query
    constexpr int HB = GMAX / 4;                    // blocks of four heads
    __shared__ uint4 mu_op[HB][4][NP][16];          // [head block][32-dim block][piece][4 j + head % 4]: 8 elements
    __shared__ float unscale[GMAX];                 // 2^exponent / sqrt(d) per head
    __shared__ float red_m[4][GMAX], red_s[4][GMAX];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, n = lane & 15, j = lane >> 4;
    const int t0 = chunk * ROWS_PER_WG + wave * 64;
    // The mean queries first: loads return in the order of their requests, and these few kilobytes come out of the
    // L2 while the keys come from memory; requested behind the keys they would arrive no earlier than the keys, and
    // the two barriers of the split below would start only then.
    const int mg = tid >> 5, msub = tid & 31;       // 8 heads x 32 threads x 4 dims: the largest entry per head
    float4 mu_max = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (mg < a.Gl) mu_max = *reinterpret_cast<const float4*>(a.mu + ((size_t)h * a.G + mg) * HD + 4 * msub);
    const int shb = tid >> 6, si = (tid >> 4) & 3, sjj = (tid >> 2) & 3, sg = 4 * shb + (tid & 3);   // the split's share
    float4 mu_a = make_float4(0.0f, 0.0f, 0.0f, 0.0f), mu_b = mu_a;
    if (tid < HB * 64 && sg < a.Gl) {
        const float* src = a.mu + ((size_t)h * a.G + sg) * HD + 32 * si + 8 * sjj;
        mu_a = *reinterpret_cast<const float4*>(src); mu_b = *reinterpret_cast<const float4*>(src + 4);
    }
    // the keys: group q's token n, dims 32 i + 8 j .. + 7 (rows past the end repeat the last row, never stored)
    uint4 kx[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint16_t* row = reinterpret_cast<const uint16_t*>(a.K) + (size_t)h * a.sH
                              + (size_t)(a.n_sink + min(t0 + 16 * q + n, a.Tc - 1)) * a.sT + 8 * j;
#pragma unroll
        for (int i = 0; i < 4; ++i) kx[q][i] = *reinterpret_cast<const uint4*>(row + 32 * i);
    }
    // per head: the power of two that brings the largest entry below 1 (fp16 pieces; bf16 has fp32's range)
    {
        const int g = mg, sub = msub;
        float mx = fmaxf(fmaxf(fabsf(mu_max.x), fabsf(mu_max.y)), fmaxf(fabsf(mu_max.z), fabsf(mu_max.w)));
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, WAVE));
        if (sub == 0 && g < GMAX) {
            int ex = 0;
            if (DT == ODMKV_F16 && mx > 0.0f && mx < INFINITY) { (void)frexpf(mx, &ex); ex = max(-100, min(112, ex)); }
            unscale[g] = ldexpf(0.08838834764831845f, ex);     // 1 / sqrt(128) times the scale taken out below
            red_m[0][g] = ldexpf(1.0f, -ex);                   // (borrowed until the barrier after the split)
        }
    }
    lds_barrier();
    if (tid < HB * 64) {
        const int hb = shb, i = si, g = sg;
        const float sc = g < a.Gl ? red_m[0][g] : 0.0f;
        float x[8] = {mu_a.x * sc, mu_a.y * sc, mu_a.z * sc, mu_a.w * sc, mu_b.x * sc, mu_b.y * sc, mu_b.z * sc, mu_b.w * sc};
#pragma unroll
        for (int pc = 0; pc < NP; ++pc) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const uint16_t b0 = Elem<DT>::from_f32(x[e]), b1 = Elem<DT>::from_f32(x[e + 1]);
                x[e] -= Elem<DT>::to_f32(b0); x[e + 1] -= Elem<DT>::to_f32(b1);       // exact: what the piece left over
                w[e >> 1] = (uint32_t)b0 | ((uint32_t)b1 << 16);
            }
            mu_op[hb][i][pc][tid & 15] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    lds_barrier();
    // |k|^2: lane (n / 4, n) holds the diagonal element of token n in component n % 4
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        sc_f4 gr = (sc_f4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i) gr = sc_mfma<DT>(kx[q][i], kx[q][i], gr);
        const int r = n & 3, t = t0 + 16 * q + n;
        const float kn = r == 0 ? gr[0] : r == 1 ? gr[1] : r == 2 ? gr[2] : gr[3];
        if (j == (n >> 2) && t < a.Tc) a.kn2[(size_t)h * a.Tc + t] = kn;
    }
    const int t = t0 + lane;                      // this lane's token: group j, column n
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
        if (4 * hb >= a.Gl) break;
        sc_f4 acc[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = (sc_f4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int pc = NP - 1; pc >= 0; --pc) {           // small pieces first
                const uint4 mu8 = mu_op[hb][i][pc][4 * j + (n & 3)];
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[q] = sc_mfma<DT>(mu8, kx[q][i], acc[q]);
            }
        const sc_f4 mine = j == 0 ? acc[0] : j == 1 ? acc[1] : j == 2 ? acc[2] : acc[3];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int g = 4 * hb + r;
            if (g < a.Gl) {
                const float d = t < a.Tc ? mine[r] * unscale[g] : -INFINITY;
                if (t < a.Tc) a.logits[((size_t)h * a.G + g) * a.Tc + t] = d;
                const float m = wave_max(d);
                const float s = wave_sum(d == -INFINITY ? 0.0f : __expf(d - m));
                if (lane == 0) { red_m[wave][g] = m; red_s[wave][g] = s; }
            }
        }
    }
    __syncthreads();
    if (tid < a.Gl) {
        float mm = red_m[0][tid], ss = red_s[0][tid];
        for (int w = 1; w < 4; ++w) ms_merge(mm, ss, red_m[w][tid], red_s[w][tid]);
        float* st = a.stats + (((size_t)h * a.G + tid) * a.nchunks + chunk) * 2;
        st[0] = mm; st[1] = ss;
    }
}

// ---- merge chunk statistics into (max, sum) per query head ----
__global__ __launch_bounds__(64) void score_stats_kernel(ScoreArgs a) {
    const int hq = blockIdx.x, lane = threadIdx.x;
    float m = -INFINITY, s = 0.0f;
    for (int c = lane; c < a.nstat; c += WAVE) {
        const float* st = a.stats + ((size_t)hq * a.nstat + c) * 2;
        ms_merge(m, s, st[0], st[1]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float m2 = __shfl_xor(m, o, WAVE), s2 = __shfl_xor(s, o, WAVE);
        ms_merge(m, s, m2, s2);
    }
    if (lane == 0) { a.mz[2 * hq] = m; a.mz[2 * hq + 1] = s; }
}

// ---- pass 1 over V: p, sum p, partial sums of p * v ----
// The two passes over V share one shape: a group of 16 lanes takes 16 consecutive rows (4 KB of a dense cache),
// lane `part` of the group owns row `part` (it reads and writes that row's scalars: 64 consecutive floats per
// wave), and all rows of a trip are requested before any is used.  16-bit rows: one trip of 16; fp32: two of 8.
template <int DT> struct VTrip { static constexpr int ROWS = DT == ODMKV_F32 ? 8 : 16; };

// lane `src` of this lane's group of 16 (a row of the data-parallel-primitive network)
__device__ static inline float group16_bcast(float v, int src) {
    return __shfl(v, (int)((threadIdx.x & 48u) | (unsigned)src), WAVE);
}

template <int DT, int GMAX>
__global__ __launch_bounds__(256) void score_pv_kernel(ScoreArgs a) {
    constexpr int U = VTrip<DT>::ROWS;
    __shared__ float osum[16][HD];
    __shared__ float psum_s[4];
    __shared__ float mz_s[2 * GMAX];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, part = lane & 15, grp = tid >> 4;
    const int tb = chunk * ROWS_PER_WG + grp * 16;
    Raw8<DT> raw[U];
    auto request = [&](int u0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            load8_raw<DT>(a.V, (size_t)h * a.sH + (size_t)(a.n_sink + min(tb + u0 + u, a.Tc - 1)) * a.sT + part * 8, raw[u]);
    };
    // The small operands first (the row's logits, the block statistics): loads return in the order of their
    // requests, these come out of the L2 and the rows of V from memory; behind V they would arrive with V, and the
    // merge of the statistics, a barrier and the weights would start only then.
    const int t = tb + part;                       // the lane's own row
    float lg[GMAX];
    if (a.attn == nullptr && t < a.Tc) {
#pragma unroll
        for (int g = 0; g < GMAX; ++g)
            if (g < a.G) lg[g] = a.logits[((size_t)h * a.G + g) * a.Tc + t];
    }
    constexpr int NPRE = 4;                        // statistics entries per lane and head requested ahead (256 blocks)
    float2 pre[GMAX / 4][NPRE];
#pragma unroll
    for (int gi = 0; gi < GMAX / 4; ++gi)
#pragma unroll
        for (int k = 0; k < NPRE; ++k) {
            const int g = wave + 4 * gi, c = lane + WAVE * k;
            pre[gi][k] = make_float2(-INFINITY, 0.0f);
            if (a.attn == nullptr && g < a.G && c < a.nstat)
                pre[gi][k] = *reinterpret_cast<const float2*>(a.stats + ((size_t)(h * a.G + g) * a.nstat + c) * 2);
        }
    request(0);
    // (max, sum) of every query head of the group over all chunks: each workgroup merges the chunk statistics
    // again (a kilobyte per head out of the L2) instead of waiting for a launch that does
    if (a.attn == nullptr) {
#pragma unroll
        for (int gi = 0; gi < GMAX / 4; ++gi) {
            const int g = wave + 4 * gi;
            if (g >= a.G) break;
            float m = -INFINITY, sm = 0.0f;
#pragma unroll
            for (int k = 0; k < NPRE; ++k) ms_merge(m, sm, pre[gi][k].x, pre[gi][k].y);
            for (int c = lane + WAVE * NPRE; c < a.nstat; c += WAVE) {
                const float2 e = *reinterpret_cast<const float2*>(a.stats + ((size_t)(h * a.G + g) * a.nstat + c) * 2);
                ms_merge(m, sm, e.x, e.y);
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float m2 = __shfl_xor(m, o, WAVE), s2 = __shfl_xor(sm, o, WAVE);
                ms_merge(m, sm, m2, s2);
            }
            if (lane == 0) { mz_s[2 * g] = m; mz_s[2 * g + 1] = 1.0f / sm; }     // reciprocal of the sum
        }
        lds_barrier();
    }
    // the weight of the lane's own row
    float pt = 0.0f;
    if (t < a.Tc) {
        if (a.attn != nullptr) {
            pt = a.attn[(size_t)h * a.T + a.n_sink + t];
        } else {
            float Mg[GMAX], Zg[GMAX];
#pragma unroll
            for (int g = 0; g < GMAX; ++g) {
                if (g < a.G) { Mg[g] = mz_s[2 * g]; Zg[g] = mz_s[2 * g + 1]; }
            }
            const float inv_g = 1.0f / (float)a.G;
            float acc = 0.0f;
            if (a.round_dt < 0) {
#pragma unroll
                for (int g = 0; g < GMAX; ++g)
                    if (g < a.G) acc = __fmaf_rn(__expf(lg[g] - Mg[g]), Zg[g], acc);
                pt = acc * inv_g;
            } else {
                // the softmax of every query head and the mean over the group, each rounded to the model's
                // dtype (kvquant/scorer.py:314-315)
#pragma unroll
                for (int g = 0; g < GMAX; ++g)
                    if (g < a.G) acc += round_model(expf(lg[g] - Mg[g]) * Zg[g], a.round_dt);
                pt = round_model(acc * inv_g, a.round_dt);
            }
        }
        a.p[(size_t)h * a.Tc + t] = pt;
    }
    float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int u0 = 0; u0 < 16; u0 += U) {
        if (u0 > 0) request(u0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float pu = group16_bcast(pt, u0 + u);       // 0 for rows past the end
            float x[8];
            cvt8<DT>(raw[u], x);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = __fmaf_rn(pu, x[e], o[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) osum[grp][part * 8 + e] = o[e];
    const float ps = wave_sum(pt);
    if (lane == 0) psum_s[wave] = ps;
    __syncthreads();
    if (tid < HD) {
        float acc = 0.0f;
        for (int g = 0; g < 16; ++g) acc += osum[g][tid];
        a.opart[((size_t)h * a.nchunks + chunk) * HD + tid] = acc;
    }
    if (tid == 0) a.psum[(size_t)h * a.nchunks + chunk] = (psum_s[0] + psum_s[1]) + (psum_s[2] + psum_s[3]);
}

__global__ __launch_bounds__(1024) void score_obar_kernel(ScoreArgs a) {
    // 8 groups of 128 threads take every eighth chunk, then the groups are added in order
    __shared__ float part_o[8][HD];
    __shared__ float part_p[8];
    const int h = blockIdx.x, j = threadIdx.x & (HD - 1), grp = threadIdx.x >> 7;
    float acc = 0.0f, P = 0.0f;
#pragma unroll 8
    for (int c = grp; c < a.nchunks; c += 8) {
        acc += a.opart[((size_t)h * a.nchunks + c) * HD + j];
        P += a.psum[(size_t)h * a.nchunks + c];
    }
    part_o[grp][j] = acc;
    if (j == 0) part_p[grp] = P;
    __syncthreads();
    if (grp == 0) {
        float o = 0.0f, p = 0.0f;
#pragma unroll
        for (int g = 0; g < 8; ++g) { o += part_o[g][j]; p += part_p[g]; }
        a.obar[h * HD + j] = o / fmaxf(p, 1e-8f);
    }
}

// ---- pass 2 over V: |v|^2, |v - obar|^2, the score, and its global maximum ----
template <int DT>
__global__ __launch_bounds__(256) void score_final_kernel(ScoreArgs a) {
    constexpr int U = VTrip<DT>::ROWS;
    __shared__ unsigned int wmax[4];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, part = lane & 15, grp = tid >> 4;
    const int tb = chunk * ROWS_PER_WG + grp * 16;
    Raw8<DT> raw[U];
    auto request = [&](int u0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            load8_raw<DT>(a.V, (size_t)h * a.sH + (size_t)(a.n_sink + min(tb + u0 + u, a.Tc - 1)) * a.sT + part * 8, raw[u]);
    };
    // the row's scalars and the mean output first (loads return in the order of their requests: behind the rows,
    // the first row could not be used before the last had arrived)
    const int t = tb + part;                       // the lane's own row
    const bool ok = t < a.Tc;
    const float pin = ok ? a.p[(size_t)h * a.Tc + t] : 0.0f;
    const float knin = ok ? a.kn2[(size_t)h * a.Tc + t] : 0.0f;
    float ob[8];
    {
        const float4 o0 = *reinterpret_cast<const float4*>(a.obar + h * HD + part * 8);
        const float4 o1 = *reinterpret_cast<const float4*>(a.obar + h * HD + part * 8 + 4);
        ob[0] = o0.x; ob[1] = o0.y; ob[2] = o0.z; ob[3] = o0.w; ob[4] = o1.x; ob[5] = o1.y; ob[6] = o1.z; ob[7] = o1.w;
    }
    request(0);
    float vn_own = 0.0f, ir_own = 0.0f;
#pragma unroll
    for (int u0 = 0; u0 < 16; u0 += U) {
        if (u0 > 0) request(u0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float x[8];
            cvt8<DT>(raw[u], x);
            float vn = 0.0f, ir = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                vn = __fmaf_rn(x[e], x[e], vn);
                const float dlt = x[e] - ob[e];
                ir = __fmaf_rn(dlt, dlt, ir);
            }
            vn = group16_sum(vn);
            ir = group16_sum(ir);
            vn_own = part == u0 + u ? vn : vn_own;
            ir_own = part == u0 + u ? ir : ir_own;
        }
    }
    float best = 0.0f;
    if (ok) {
        // (p + eps)^2 is formed on the tensor of the model's dtype in the reference (kvquant/scorer.py:403):
        // eps becomes a scalar of that dtype, the sum and the square are rounded to it
        const float pe = round_model(pin + round_model(a.eps, a.round_dt), a.round_dt);
        const float kterm = (knin * (1.0f / (float)HD)) * ir_own;      // 1/128: exact
        const float sc = round_model(pe * pe, a.round_dt) * (vn_own + kterm);
        a.scores[(size_t)h * a.T + a.n_sink + t] = sc;
        best = sc;
    }
    best = wave_max(best);
    if (lane == 0) wmax[wave] = __float_as_uint(best);
    __syncthreads();
    if (tid == 0)       // non-negative floats order like their bit patterns; the partial sums of p have been consumed
        reinterpret_cast<unsigned int*>(a.psum)[(size_t)h * a.nchunks + chunk] = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
}

// the sinks take the largest score of the layer: every workgroup of the last pass left its own maximum (one
// store each; a single word updated atomically by a thousand workgroups kept that pass waiting on the updates)
__global__ __launch_bounds__(64) void score_pad_kernel(ScoreArgs a) {
    const int h = blockIdx.x, i = threadIdx.x;
    const unsigned int* part = reinterpret_cast<const unsigned int*>(a.psum);
    unsigned int mx = 0u;
#pragma unroll 8
    for (int c = i; c < a.Hkv * a.nchunks; c += WAVE) mx = max(mx, part[c]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, (unsigned int)__shfl_xor((int)mx, o, WAVE));
    if (i < a.n_sink) a.scores[(size_t)h * a.T + i] = __uint_as_float(mx);
}

// ------------------------------------------------------------------------------------------------
// Expected-attention score (ExpectedAttentionScorer.score_prefill, kvquant/scorer.py:204-257):
//
//   logit[q,t] = mu[q] . k[t] / sqrt(d)  +  k[t]^T Cov[q] k[t] / (2 d)
//   p[h,t]     = mean over the group of softmax_t(logit[q,:]);   s = (p + eps) * |v|   (or p alone)
//
// The quadratic form is a true dense contraction, [T,128] x [128,128] per query head, and runs on
// the fp32 matrix cores (v_mfma_f32_32x32x2_f32): a wave takes 32 tokens, D = Cov/(2d) . K^T with the
// accumulator preset to mu[c]/sqrt(d), so that logit[t] = sum_c K[t][c] * D[c][t] holds both terms.  Cov/(2d) stays in LDS (64 KB) for the workgroup's life; K is read from HBM by the
// first head of a group and from the caches by the others.
// ------------------------------------------------------------------------------------------------
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define EA_MAX_CHUNKS_PER_WG 4   // most 256-token chunks a workgroup walks with one copy of the covariance

// the 128 elements of one token's row, as raw registers
template <int DT> struct RowRegs;
template <> struct RowRegs<ODMKV_F32> {
    float4 r[32];
    __device__ inline void load(const void* base, size_t off) {
        const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + off);
#pragma unroll
        for (int i = 0; i < 32; ++i) r[i] = p[i];
    }
    __device__ inline float at(int e) const {            // e is a compile-time constant where this is used
        const float4 v = r[e >> 2];
        return (e & 3) == 0 ? v.x : (e & 3) == 1 ? v.y : (e & 3) == 2 ? v.z : v.w;
    }
    // element 2 s + half
    __device__ inline float pair_elem(int s, int half) const { return half ? at(2 * s + 1) : at(2 * s); }
    // the four elements e0 + 4 half + 0..3 (e0 a multiple of 8)
    __device__ inline void quad(int e0, int half, float* x) const {
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = half ? at(e0 + 4 + j) : at(e0 + j);
    }
};
template <int DT> struct RowRegs {
    uint4 r[16];
    __device__ inline void load(const void* base, size_t off) {
        const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + off);
#pragma unroll
        for (int i = 0; i < 16; ++i) r[i] = p[i];
    }
    __device__ inline uint32_t dword(int i) const {
        const uint4 v = r[i >> 2];
        return (i & 3) == 0 ? v.x : (i & 3) == 1 ? v.y : (i & 3) == 2 ? v.z : v.w;
    }
    __device__ inline float pair_elem(int s, int half) const {
        const uint32_t w = dword(s);
        return Elem<DT>::to_f32((uint16_t)(half ? (w >> 16) : (w & 0xffffu)));
    }
    __device__ inline void quad(int e0, int half, float* x) const {
        const uint32_t w0 = half ? dword(e0 / 2 + 2) : dword(e0 / 2);
        const uint32_t w1 = half ? dword(e0 / 2 + 3) : dword(e0 / 2 + 1);
        x[0] = Elem<DT>::to_f32((uint16_t)(w0 & 0xffffu)); x[1] = Elem<DT>::to_f32((uint16_t)(w0 >> 16));
        x[2] = Elem<DT>::to_f32((uint16_t)(w1 & 0xffffu)); x[3] = Elem<DT>::to_f32((uint16_t)(w1 >> 16));
    }
};

// Operand roles: the matrix rows are the covariance's output columns c, the matrix columns the 32
// tokens (D[c][t] = sum_e Cov[e][c] K[t][e]; the quadratic form only sees the symmetric part of
// Cov, so Cov[e][c] stands for Cov[c][e]).  A lane then ends with token lane % 32 and the 64
// columns c = 32 cb + 8 q + 4 (lane / 32) + j: logit[t] = sum_c K[t][c] D[c][t] takes the lane's own
// row, which it still holds in registers, and one exchange between the two halves of the wave.
template <int DT>
__global__ __launch_bounds__(256) void ea_logits_kernel(ScoreArgs a) {
    extern __shared__ __align__(16) float cov_s[];      // [128][128], already divided by 2 d
    __shared__ __align__(16) float mu_s[HD];            // mu / sqrt(d)
    __shared__ float red_m[4], red_s[4];
    const int hq = blockIdx.y, h = hq / a.G, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, col = lane & 31, half = lane >> 5;
    {
        const float4* src = reinterpret_cast<const float4*>(a.cov + (size_t)hq * HD * HD);
        float4* dst = reinterpret_cast<float4*>(cov_s);
        const float sc = 1.0f / (2.0f * HD);            // a power of two: exact
        for (int e = tid; e < HD * HD / 4; e += 256) {
            float4 v = src[e];
            v.x *= sc; v.y *= sc; v.z *= sc; v.w *= sc;
            dst[e] = v;
        }
        if (tid < HD) mu_s[tid] = a.mu[(size_t)hq * HD + tid] / 11.313708498984761f;
    }
    // sub-tile i of this wave (two per chunk): tokens t0(i) .. t0(i) + 31
    auto t0_of = [&](int i) { return (blockIdx.x * a.ea_cpw + (i >> 1)) * ROWS_PER_WG + (wave * 2 + (i & 1)) * 32; };
    auto row_of = [&](int i) {                          // rows past the end repeat the last row and are not stored
        return (size_t)h * a.sH + (size_t)(a.n_sink + min(t0_of(i) + col, a.Tc - 1)) * a.sT;
    };
    RowRegs<DT> cur;
    cur.load(a.K, row_of(0));
    __syncthreads();
    const float* cbase = cov_s + half * HD + col;
    for (int cc = 0; cc < a.ea_cpw; ++cc) {
        const int chunk = blockIdx.x * a.ea_cpw + cc;
        if (chunk >= a.nchunks) break;                  // the same for every thread of the workgroup
        float m = -INFINITY, s = 0.0f;
        for (int sub = 0; sub < 2; ++sub) {
            const int it = cc * 2 + sub;
            const int t0 = t0_of(it);
            RowRegs<DT> nxt;
            if constexpr (DT != ODMKV_F32) {            // the next sub-tile's row travels under this one's products
                if (it < 2 * a.ea_cpw - 1) nxt.load(a.K, row_of(it + 1));
            }
            if (t0 < a.Tc) {                            // wave-uniform
                f32x16 acc[4];
#pragma unroll
                for (int cb = 0; cb < 4; ++cb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 mv = *reinterpret_cast<const float4*>(mu_s + 32 * cb + 8 * q + 4 * half);
                        acc[cb][4 * q] = mv.x; acc[cb][4 * q + 1] = mv.y; acc[cb][4 * q + 2] = mv.z; acc[cb][4 * q + 3] = mv.w;
                    }
#pragma unroll
                for (int st = 0; st < 64; ++st) {
                    const float kv = cur.pair_elem(st, half);
#pragma unroll
                    for (int cb = 0; cb < 4; ++cb)
                        acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(cbase[st * 2 * HD + cb * 32], kv, acc[cb], 0, 0, 0);
                }
                float lg = 0.0f;
#pragma unroll
                for (int cb = 0; cb < 4; ++cb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float x[4];
                        cur.quad(32 * cb + 8 * q, half, x);
#pragma unroll
                        for (int j = 0; j < 4; ++j) lg = __fmaf_rn(x[j], acc[cb][4 * q + j], lg);
                    }
                lg += __shfl_xor(lg, 32, WAVE);
                const int t = t0 + col;
                if (half == 0 && t < a.Tc) {
                    a.logits[(size_t)hq * a.Tc + t] = lg;
                    ms_merge(m, s, lg, 1.0f);
                }
            }
            if constexpr (DT != ODMKV_F32) cur = nxt;
            else if (it < 2 * a.ea_cpw - 1) cur.load(a.K, row_of(it + 1));
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float m2 = __shfl_xor(m, o, WAVE), s2 = __shfl_xor(s, o, WAVE);
            ms_merge(m, s, m2, s2);
        }
        if (lane == 0) { red_m[wave] = m; red_s[wave] = s; }
        __syncthreads();
        if (tid == 0) {
            float mm = red_m[0], ss = red_s[0];
            for (int w = 1; w < 4; ++w) ms_merge(mm, ss, red_m[w], red_s[w]);
            float* st = a.stats + ((size_t)hq * a.nchunks + chunk) * 2;
            st[0] = mm; st[1] = ss;
        }
        __syncthreads();
    }
}

// ---- the same contraction for 16-bit keys, on the 16-bit matrix instructions ----------------------
// K is exact in its own 16-bit type; Cov/(2d) is split into pieces of that type (two fp16 pieces after
// scaling the head's largest entry to 2^14, or three bf16 pieces), so the products are exact and the
// sum carries 22-24 bits of every covariance entry relative to the largest: the logits agree with the
// fp32 kernel to ~1e-6.  v_mfma_f32_32x32x16_{f16,bf16}: operand A = 8 consecutive entries of row c of
// a piece (one 16-byte LDS read), operand B = 8 consecutive elements of the lane's token row; a wave
// takes 64 tokens at a time.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#define EA_ROW 136           // 16-bit entries per LDS row of a piece: 128 + 8, so that 16-byte reads of
                             // consecutive rows fall on distinct banks

template <int DT> struct Piece;
template <> struct Piece<ODMKV_F16> {
    static constexpr int NP = 2;
    __device__ static inline f32x16 mfma(uint4 a, uint4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct Piece<ODMKV_BF16> {
    static constexpr int NP = 3;
    __device__ static inline f32x16 mfma(uint4 a, uint4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// x -> NP values of the 16-bit type whose sum approximates x (each the rounding of what is left)
template <int DT>
__device__ static inline void split_pieces(float x, uint16_t* out) {
#pragma unroll
    for (int p = 0; p < Piece<DT>::NP; ++p) {
        out[p] = Elem<DT>::from_f32(x);
        x -= Elem<DT>::to_f32(out[p]);
    }
}

template <int DT, int NW>
__global__ __launch_bounds__(NW * 64) void ea_logits16_kernel(ScoreArgs a) {
    constexpr int NP = Piece<DT>::NP, NT = NW * 64, CPI = NW / 4;      // CPI: 256-token chunks per iteration
    constexpr int PER = HD * HD / 4 / NT;
    extern __shared__ __align__(16) uint16_t piece_s[];               // [NP][128][EA_ROW]
    __shared__ __align__(16) float mu_s[HD];                          // mu / sqrt(d), scaled like the pieces
    __shared__ float red_a[NW];
    const int hq = blockIdx.y, h = hq / a.G, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, col = lane & 31, half = lane >> 5;
    int kexp = 0;
    {
        const float4* src = reinterpret_cast<const float4*>(a.cov + (size_t)hq * HD * HD);
        float4 v[PER];
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            v[i] = src[tid + NT * i];
            amax = fmaxf(fmaxf(amax, fmaxf(fabsf(v[i].x), fabsf(v[i].y))), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
        }
        amax = wave_max(amax);
        if (lane == 0) red_a[wave] = amax;
        __syncthreads();
        amax = red_a[0];
#pragma unroll
        for (int w = 1; w < NW; ++w) amax = fmaxf(amax, red_a[w]);
        if (DT == ODMKV_F16 && amax > 0.0f && amax < INFINITY) {     // fp16 pieces: largest entry of Cov/(2d) -> [2^13, 2^14)
            int ex;
            (void)frexpf(amax, &ex);
            kexp = max(-60, min(60, 14 + 8 - ex));
        }
        const float sc = ldexpf(1.0f, kexp - 8);                     // includes the 1 / (2 d)
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e4 = tid + NT * i, row = e4 >> 5, c0 = (e4 & 31) * 4;
            uint16_t px[NP], py[NP], pz[NP], pw[NP];
            split_pieces<DT>(v[i].x * sc, px); split_pieces<DT>(v[i].y * sc, py);
            split_pieces<DT>(v[i].z * sc, pz); split_pieces<DT>(v[i].w * sc, pw);
#pragma unroll
            for (int p = 0; p < NP; ++p)
                *reinterpret_cast<uint2*>(piece_s + ((size_t)p * HD + row) * EA_ROW + c0) =
                    make_uint2((uint32_t)px[p] | ((uint32_t)py[p] << 16), (uint32_t)pz[p] | ((uint32_t)pw[p] << 16));
        }
        if (tid < HD) mu_s[tid] = a.mu[(size_t)hq * HD + tid] / 11.313708498984761f * ldexpf(1.0f, kexp);
    }
    const float unscale = ldexpf(1.0f, -kexp);
    __syncthreads();
    const uint16_t* abase = piece_s + (size_t)col * EA_ROW + 8 * half;
    for (int itn = 0; itn < a.ea_cpw; ++itn) {
        const int chunk0 = (blockIdx.x * a.ea_cpw + itn) * CPI;
        if (chunk0 >= a.nchunks) break;                               // the same for every thread of the workgroup
        const int t0 = (chunk0 + (wave >> 2)) * ROWS_PER_WG + (wave & 3) * 64;
        float m = -INFINITY, s = 0.0f;
        if (t0 < a.Tc) {                                              // wave-uniform
            // Two blocks of 32 tokens share every A operand: one 16-byte LDS read feeds two matrix
            // instructions (with one read per instruction the LDS pipe, 128 bytes per clock and compute
            // unit, is exactly as fast as the matrix pipes and sets the time).  The 32-column blocks of the
            // covariance go one after the other, so that only two accumulator blocks are live.
            RowRegs<DT> r0, r1;                                       // rows past the end repeat the last row and are not stored
            r0.load(a.K, (size_t)h * a.sH + (size_t)(a.n_sink + min(t0 + col, a.Tc - 1)) * a.sT);
            r1.load(a.K, (size_t)h * a.sH + (size_t)(a.n_sink + min(t0 + 32 + col, a.Tc - 1)) * a.sT);
            float lg0 = 0.0f, lg1 = 0.0f;
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) {
                f32x16 acc0, acc1;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 mv = *reinterpret_cast<const float4*>(mu_s + 32 * cb + 8 * q + 4 * half);
                    acc0[4 * q] = mv.x; acc0[4 * q + 1] = mv.y; acc0[4 * q + 2] = mv.z; acc0[4 * q + 3] = mv.w;
                }
                acc1 = acc0;
#pragma unroll
                for (int st = 0; st < 8; ++st) {
                    const uint4 b0 = half ? r0.r[2 * st + 1] : r0.r[2 * st];
                    const uint4 b1 = half ? r1.r[2 * st + 1] : r1.r[2 * st];
#pragma unroll
                    for (int p = 0; p < NP; ++p) {
                        const uint4 av = *reinterpret_cast<const uint4*>(abase + ((size_t)p * HD + 32 * cb) * EA_ROW + 16 * st);
                        acc0 = Piece<DT>::mfma(av, b0, acc0);
                        acc1 = Piece<DT>::mfma(av, b1, acc1);
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float x0[4], x1[4];
                    r0.quad(32 * cb + 8 * q, half, x0);
                    r1.quad(32 * cb + 8 * q, half, x1);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        lg0 = __fmaf_rn(x0[j], acc0[4 * q + j], lg0);
                        lg1 = __fmaf_rn(x1[j], acc1[4 * q + j], lg1);
                    }
                }
            }
            lg0 += __shfl_xor(lg0, 32, WAVE);
            lg1 += __shfl_xor(lg1, 32, WAVE);
            const float lg = (half ? lg1 : lg0) * unscale;            // the upper half of the wave stores the second block
            const int t = t0 + 32 * half + col;
            if (t < a.Tc) {
                a.logits[(size_t)hq * a.Tc + t] = lg;
                ms_merge(m, s, lg, 1.0f);
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float m2 = __shfl_xor(m, o, WAVE), s2 = __shfl_xor(s, o, WAVE);
            ms_merge(m, s, m2, s2);
        }
        // one entry per wave and chunk: the waves of a workgroup never wait for each other in this loop
        const int chunk = chunk0 + (wave >> 2);
        if (lane == 0 && chunk < a.nchunks) {
            float* st = a.stats + ((size_t)hq * a.nstat + chunk * 4 + (wave & 3)) * 2;
            st[0] = m; st[1] = s;
        }
    }
}

// p from the logits, then (p + eps) * |v| (or p alone), and the running maximum
template <int DT, int GMAX>
__global__ __launch_bounds__(256) void ea_final_kernel(ScoreArgs a) {
    __shared__ unsigned int wmax[4];
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, part = lane & 15, rsub = lane >> 4;
    float Mg[GMAX], Zg[GMAX];
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
        Mg[g] = g < a.G ? a.mz[2 * (h * a.G + g)] : 0.0f;
        Zg[g] = g < a.G ? 1.0f / a.mz[2 * (h * a.G + g) + 1] : 1.0f;   // reciprocal of the sum
    }
    const float inv_g = 1.0f / (float)a.G;
    float best = 0.0f;
    const int t0 = chunk * ROWS_PER_WG;
    for (int it0 = 0; it0 < ROWS_PER_WG / 16; it0 += SC_UNROLL_V) {
        float xs[SC_UNROLL_V][8], lg[SC_UNROLL_V][GMAX];
#pragma unroll
        for (int u = 0; u < SC_UNROLL_V; ++u) {
            const int t = t0 + (it0 + u) * 16 + wave * 4 + rsub;
#pragma unroll
            for (int e = 0; e < 8; ++e) xs[u][e] = 0.0f;
            if (t < a.Tc) {
                if (a.use_vnorm) load8<DT>(a.V, (size_t)h * a.sH + (size_t)(a.n_sink + t) * a.sT + part * 8, xs[u]);
#pragma unroll
                for (int g = 0; g < GMAX; ++g)
                    if (g < a.G && part == 0) lg[u][g] = a.logits[((size_t)h * a.G + g) * a.Tc + t];
            }
        }
#pragma unroll
        for (int u = 0; u < SC_UNROLL_V; ++u) {
            const int t = t0 + (it0 + u) * 16 + wave * 4 + rsub;
            float vn = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) vn = __fmaf_rn(xs[u][e], xs[u][e], vn);
            vn = group16_sum(vn);
            if (t < a.Tc && part == 0) {
                float acc = 0.0f;
#pragma unroll
                for (int g = 0; g < GMAX; ++g)
                    if (g < a.G) acc = __fmaf_rn(__expf(lg[u][g] - Mg[g]), Zg[g], acc);
                const float pt = acc * inv_g;
                const float sc = a.use_vnorm ? (pt + a.eps) * sqrtf(vn) : pt;
                a.scores[(size_t)h * a.T + a.n_sink + t] = sc;
                best = fmaxf(best, sc);
            }
        }
    }
    best = wave_max(best);
    if (lane == 0) wmax[wave] = __float_as_uint(best);
    __syncthreads();
    if (tid == 0)
        reinterpret_cast<unsigned int*>(a.psum)[(size_t)h * a.nchunks + chunk] = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
}

static inline int n_chunks(int Tc) { return (Tc + ROWS_PER_WG - 1) / ROWS_PER_WG; }

struct ScoreLayout { size_t logits, kn2, p, stats, mz, opart, psum, obar, total; };
static ScoreLayout score_layout(int Hkv, int Hq, int T) {
    ScoreLayout L;
    const size_t Tc = T, nc = n_chunks(T);
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
    L.logits = take((size_t)Hq * Tc * 4);
    L.kn2 = take((size_t)Hkv * Tc * 4);
    L.p = take((size_t)Hkv * Tc * 4);
    L.stats = take((size_t)Hq * nc * 4 * 8);        // up to one entry per wave and chunk
    L.mz = take((size_t)Hq * 8);
    L.opart = take((size_t)Hkv * nc * HD * 4);
    L.psum = take((size_t)Hkv * nc * 4);
    L.obar = take((size_t)Hkv * HD * 4);
    L.total = off;
    return L;
}

extern "C" size_t odmkv_score_workspace_bytes(int Hkv, int Hq, int T) {
    if (Hkv <= 0 || Hq <= 0 || T <= 0) return 0;
    return score_layout(Hkv, Hq, T).total;
}

template <int DT>
static int run_score(ScoreArgs& a, hipStream_t st) {
    dim3 grid(a.nchunks, a.Hkv), block(256);
    if constexpr (DT != ODMKV_F32) {
        // 16-bit keys feed the matrix cores as they lie in memory; the mode that rounds like a 16-bit model and
        // the call that brings its own attention weights keep the kernel that forms every product in fp32
        if (a.round_dt < 0 && a.Gl > 0) {
            if (a.G <= 4) hipLaunchKernelGGL((score_logits16_kernel<DT, 4>), grid, block, 0, st, a);
            else hipLaunchKernelGGL((score_logits16_kernel<DT, 8>), grid, block, 0, st, a);
        } else if (a.G <= 4) hipLaunchKernelGGL((score_logits_kernel<DT, 4>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((score_logits_kernel<DT, 8>), grid, block, 0, st, a);
    } else if (a.G <= 4) hipLaunchKernelGGL((score_logits_kernel<DT, 4>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((score_logits_kernel<DT, 8>), grid, block, 0, st, a);
    ODMKV_CHECK_LAUNCH("score_logits_kernel");
    if (a.G <= 4) hipLaunchKernelGGL((score_pv_kernel<DT, 4>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((score_pv_kernel<DT, 8>), grid, block, 0, st, a);
    ODMKV_CHECK_LAUNCH("score_pv_kernel");
    hipLaunchKernelGGL(score_obar_kernel, dim3(a.Hkv), dim3(1024), 0, st, a);
    ODMKV_CHECK_LAUNCH("score_obar_kernel");
    hipLaunchKernelGGL((score_final_kernel<DT>), grid, block, 0, st, a);
    ODMKV_CHECK_LAUNCH("score_final_kernel");
    if (a.n_sink > 0) {
        hipLaunchKernelGGL(score_pad_kernel, dim3(a.Hkv), dim3(64), 0, st, a);
        ODMKV_CHECK_LAUNCH("score_pad_kernel");
    }
    return 0;
}

extern "C" int odmkv_score(const void* K, const void* V, int dtype, int Hkv, int T,
                           int64_t stride_h, int64_t stride_t,
                           const float* mu, int Hq, const float* attn, int n_sink, float eps,
                           float* scores, void* workspace, size_t workspace_bytes, void* stream) {
    return odmkv_score_model_dtype(K, V, dtype, Hkv, T, stride_h, stride_t, mu, Hq, attn, n_sink, eps, -1,
                                   scores, workspace, workspace_bytes, stream);
}

extern "C" int odmkv_score_model_dtype(const void* K, const void* V, int dtype, int Hkv, int T,
                                       int64_t stride_h, int64_t stride_t,
                                       const float* mu, int Hq, const float* attn, int n_sink, float eps,
                                       int round_dtype, float* scores, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    ODMKV_CHECK_ARG(K && V && scores && workspace, "score: null pointer");
    ODMKV_CHECK_ARG(round_dtype == -1 || round_dtype == ODMKV_F16 || round_dtype == ODMKV_BF16,
                    "score: rounding dtype %d (-1, fp16 or bf16)", round_dtype);
    ODMKV_CHECK_ARG(mu || attn, "score: need the mean query or attention weights");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "score: bad dtype %d", dtype);
    ODMKV_CHECK_ARG(Hkv > 0 && Hq > 0 && Hq % Hkv == 0 && Hq / Hkv <= ODMKV_MAX_GROUP,
                    "score: bad head counts Hkv=%d Hq=%d", Hkv, Hq);
    ODMKV_CHECK_ARG(n_sink >= 0 && n_sink <= 64 && T > n_sink, "score: need T > n_sink (T=%d, n_sink=%d)", T, n_sink);
    ODMKV_CHECK_ARG(!(attn && n_sink != 0), "score: attention-weight mode takes n_sink = 0");
    const int align = dtype == ODMKV_F32 ? 4 : 8;
    ODMKV_CHECK_ARG(stride_h % align == 0 && stride_t % align == 0 && stride_t >= HD,
                    "score: strides must keep rows 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)V & 15) == 0, "score: K/V must be 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)mu & 15) == 0, "score: the mean queries must be 16-byte aligned");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_score_workspace_bytes(Hkv, Hq, T), "score: workspace too small");
    const ScoreLayout L = score_layout(Hkv, Hq, T);
    char* ws = (char*)workspace;
    ScoreArgs a;
    a.K = K; a.V = V; a.sH = stride_h; a.sT = stride_t;
    a.Hkv = Hkv; a.Hq = Hq; a.G = Hq / Hkv; a.Gl = attn ? 0 : Hq / Hkv; a.T = T; a.Tc = T - n_sink; a.n_sink = n_sink;
    a.nchunks = n_chunks(a.Tc); a.eps = eps; a.mu = mu; a.attn = attn; a.scores = scores;
    a.cov = nullptr; a.use_vnorm = 0; a.ea_cpw = 1; a.nstat = a.nchunks; a.round_dt = round_dtype;
    a.logits = (float*)(ws + L.logits); a.kn2 = (float*)(ws + L.kn2); a.p = (float*)(ws + L.p);
    a.stats = (float*)(ws + L.stats); a.mz = (float*)(ws + L.mz); a.opart = (float*)(ws + L.opart);
    a.psum = (float*)(ws + L.psum); a.obar = (float*)(ws + L.obar);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODMKV_F16) return run_score<ODMKV_F16>(a, st);
    if (dtype == ODMKV_BF16) return run_score<ODMKV_BF16>(a, st);
    return run_score<ODMKV_F32>(a, st);
}

template <int DT>
static int run_expected(ScoreArgs& a, hipStream_t st) {
    dim3 grid(a.nchunks, a.Hkv), block(256);
    if (a.cov) {
        // A workgroup prepares its head's covariance (64 KB) once: give it as many chunks as still leaves
        // `per_cu` workgroups for every compute unit.
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) == hipSuccess) {
            int v = 0;
            if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
        }
        auto pick = [&](int cpi, int max_cpw, int per_cu) {
            int cpw = max_cpw;
            while (cpw > 1 && (long)((a.nchunks + cpi * cpw - 1) / (cpi * cpw)) * a.Hq < (long)per_cu * cus) cpw >>= 1;
            a.ea_cpw = cpw;
            return dim3((a.nchunks + cpi * cpw - 1) / (cpi * cpw), a.Hq);
        };
        // the attribute belongs to the function on the current device: set on every call (layers of one
        // model may live on several devices)
        if constexpr (DT == ODMKV_F32) {
            const int lds = HD * HD * (int)sizeof(float);
            ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ea_logits_kernel<DT>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            const dim3 g2 = pick(1, EA_MAX_CHUNKS_PER_WG, 2);
            hipLaunchKernelGGL((ea_logits_kernel<DT>), g2, block, lds, st, a);
        } else {
            constexpr int NW = DT == ODMKV_F16 ? 4 : 8;        // three bf16 pieces leave room for one workgroup: eight waves
            const int lds = Piece<DT>::NP * HD * EA_ROW * (int)sizeof(uint16_t);
            ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&ea_logits16_kernel<DT, NW>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            const dim3 g2 = pick(NW / 4, 8, DT == ODMKV_F16 ? 2 : 1);
            a.nstat = a.nchunks * 4;
            hipLaunchKernelGGL((ea_logits16_kernel<DT, NW>), g2, dim3(NW * 64), lds, st, a);
        }
        ODMKV_CHECK_LAUNCH("ea_logits_kernel");
    } else {
        if (a.G <= 4) hipLaunchKernelGGL((score_logits_kernel<DT, 4>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((score_logits_kernel<DT, 8>), grid, block, 0, st, a);
        ODMKV_CHECK_LAUNCH("score_logits_kernel");
    }
    hipLaunchKernelGGL(score_stats_kernel, dim3(a.Hq), dim3(64), 0, st, a);
    ODMKV_CHECK_LAUNCH("score_stats_kernel");
    if (a.G <= 4) hipLaunchKernelGGL((ea_final_kernel<DT, 4>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((ea_final_kernel<DT, 8>), grid, block, 0, st, a);
    ODMKV_CHECK_LAUNCH("ea_final_kernel");
    if (a.n_sink > 0) {
        hipLaunchKernelGGL(score_pad_kernel, dim3(a.Hkv), dim3(64), 0, st, a);
        ODMKV_CHECK_LAUNCH("score_pad_kernel");
    }
    return 0;
}

extern "C" int odmkv_score_expected(const void* K, const void* V, int dtype, int Hkv, int T,
                                    int64_t stride_h, int64_t stride_t,
                                    const float* mu, const float* cov, int Hq, int n_sink, float eps,
                                    int use_vnorm, float* scores, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    ODMKV_CHECK_ARG(K && V && scores && workspace && mu, "score_expected: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "score_expected: bad dtype %d", dtype);
    ODMKV_CHECK_ARG(Hkv > 0 && Hq > 0 && Hq % Hkv == 0 && Hq / Hkv <= ODMKV_MAX_GROUP,
                    "score_expected: bad head counts Hkv=%d Hq=%d", Hkv, Hq);
    ODMKV_CHECK_ARG(n_sink >= 0 && n_sink <= 64 && T > n_sink, "score_expected: need T > n_sink (T=%d, n_sink=%d)", T, n_sink);
    const int align = dtype == ODMKV_F32 ? 4 : 8;
    ODMKV_CHECK_ARG(stride_h % align == 0 && stride_t % align == 0 && stride_t >= HD,
                    "score_expected: strides must keep rows 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)V & 15) == 0, "score_expected: K/V must be 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)cov & 15) == 0, "score_expected: the covariance must be 16-byte aligned");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_score_workspace_bytes(Hkv, Hq, T), "score_expected: workspace too small");
    const ScoreLayout L = score_layout(Hkv, Hq, T);
    char* ws = (char*)workspace;
    ScoreArgs a;
    a.K = K; a.V = V; a.sH = stride_h; a.sT = stride_t;
    a.Hkv = Hkv; a.Hq = Hq; a.G = Hq / Hkv; a.Gl = a.G; a.T = T; a.Tc = T - n_sink; a.n_sink = n_sink;
    a.nchunks = n_chunks(a.Tc); a.eps = eps; a.mu = mu; a.attn = nullptr; a.scores = scores;
    a.cov = cov; a.use_vnorm = use_vnorm ? 1 : 0; a.ea_cpw = 1; a.nstat = a.nchunks; a.round_dt = -1;
    a.logits = (float*)(ws + L.logits); a.kn2 = (float*)(ws + L.kn2); a.p = (float*)(ws + L.p);
    a.stats = (float*)(ws + L.stats); a.mz = (float*)(ws + L.mz); a.opart = (float*)(ws + L.opart);
    a.psum = (float*)(ws + L.psum); a.obar = (float*)(ws + L.obar);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODMKV_F16) return run_expected<ODMKV_F16>(a, st);
    if (dtype == ODMKV_BF16) return run_expected<ODMKV_BF16>(a, st);
    return run_expected<ODMKV_F32>(a, st);
}
