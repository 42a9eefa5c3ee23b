// Decode-time flush of the exact token buffer, on the device: read the newest exact tokens of every
// (sequence, kv-head) out of the store, score them with the current query (attention over the buffer, then the
// risk score given attention weights), and turn the scores into bit levels by rank with level shares fixed per
// kv-head.  Stands where the reference runs a chain of torch operations per flush
// (kvquant/adaptive_backend_press.py:464-665: _flush_decode_buffer, _flush_attention,
// _allocate_bits_via_cached_ratios).
#include "quant.h"

#define FLUSH_THREADS 256
#define FLUSH_MAX_TOKENS 2048        // buffered tokens per (sequence, kv-head) the scoring kernel takes
#define RANK_MAX_TOKENS 4096         // tokens per kv-head (all sequences) the ranking kernel sorts

// ------------------------------------------------------------------------------------------------
// the last n_tail tokens of every exact segment as dense rows [B*Hkv, n_tail, 128] of the store's exact type
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(HD) void exact_tail_kernel(odmkv_packed_t s, int n_tail, uint16_t* K, uint16_t* V) {
    const int i = blockIdx.x, bh = blockIdx.y, dim = threadIdx.x;
    const int count = s.seg_count[4][bh];
    const size_t o = ((size_t)bh * n_tail + i) * HD + dim;
    const int idx = count - n_tail + i;
    if (idx < 0) { K[o] = 0; V[o] = 0; return; }       // fewer tokens than asked for: the host checks its own mirror first
    const size_t tile = (size_t)s.seg_tile[4][bh] + (idx >> 6);
    const int slot = idx & 63;
    K[o] = s.kexact[tile * (TILE * HD) + exact_k_index(slot, dim)];
    V[o] = s.vexact[tile * (TILE * HD) + exact_v_index(slot, dim)];
}

extern "C" int odmkv_exact_tail(const odmkv_packed_t* store, int n_tail, void* K, void* V, void* stream) {
    ODMKV_CHECK_ARG(store && K && V, "exact_tail: null pointer");
    ODMKV_CHECK_ARG(n_tail > 0 && store->B > 0 && store->Hkv > 0, "exact_tail: bad shape n_tail=%d", n_tail);
    hipLaunchKernelGGL(exact_tail_kernel, dim3(n_tail, store->B * store->Hkv), dim3(HD), 0, (hipStream_t)stream,
                       *store, n_tail, reinterpret_cast<uint16_t*>(K), reinterpret_cast<uint16_t*>(V));
    ODMKV_CHECK_LAUNCH("exact_tail_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// attention of one query per (sequence, kv-head) over its n buffered keys, and the score of every buffered token
//   a_t = softmax_t(q . k_t * scaling)
//   mode 0: p_hat = a / max(sum a, 1e-8); o = sum_t p_hat_t v_t;
//           s_t = (a_t + eps)^2 * (|v_t|^2 + |k_t|^2 / d * |v_t - o|^2)        (kvquant/scorer.py:406-416)
//   mode 1: s_t = a_t^2 * |v_t|^2                                              (adaptive_backend_press.py, no scorer)
// One workgroup per (sequence, kv-head); a group of 16 lanes takes a row, a lane 8 of its dims.
// ------------------------------------------------------------------------------------------------
struct FlushScoreArgs {
    const void* K; const void* V;
    const float* q;
    float scaling, eps;
    int n, mode;
    float* attn; float* scores; float* minmax;
};

__device__ static inline float group16_total(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

template <int DT>
__device__ static inline void row8(const void* base, size_t elem, float* x) {
    if constexpr (DT == ODMKV_F32) {
        const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + elem);
        const float4 b = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + elem + 4);
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    } else {
        const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + elem);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[2 * e] = Elem<DT>::to_f32((uint16_t)(w[e] & 0xffffu));
            x[2 * e + 1] = Elem<DT>::to_f32((uint16_t)(w[e] >> 16));
        }
    }
}

template <int DT>
__global__ __launch_bounds__(FLUSH_THREADS) void flush_score_kernel(FlushScoreArgs a) {
    __shared__ float lg[FLUSH_MAX_TOKENS], kn2[FLUSH_MAX_TOKENS], vn2[FLUSH_MAX_TOKENS];
    __shared__ float opart[FLUSH_THREADS / 16][HD];
    __shared__ float obar[HD];
    __shared__ float red[FLUSH_THREADS / 64], red2[FLUSH_THREADS / 64];
    const int bh = blockIdx.x, tid = threadIdx.x, grp = tid >> 4, part = tid & 15, wave = tid >> 6, lane = tid & 63;
    const size_t base = (size_t)bh * a.n * HD;
    float qr[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qr[e] = a.q[(size_t)bh * HD + part * 8 + e];
    // pass 1: logits and squared norms
    for (int t = grp; t < a.n; t += FLUSH_THREADS / 16) {
        float k[8], v[8];
        row8<DT>(a.K, base + (size_t)t * HD + part * 8, k);
        row8<DT>(a.V, base + (size_t)t * HD + part * 8, v);
        float d = 0.0f, kk = 0.0f, vv = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { d = __fmaf_rn(k[e], qr[e], d); kk = __fmaf_rn(k[e], k[e], kk); vv = __fmaf_rn(v[e], v[e], vv); }
        d = group16_total(d); kk = group16_total(kk); vv = group16_total(vv);
        if (part == 0) { lg[t] = d * a.scaling; kn2[t] = kk; vn2[t] = vv; }
    }
    __syncthreads();
    // softmax over the buffer
    float m = -INFINITY;
    for (int t = tid; t < a.n; t += FLUSH_THREADS) m = fmaxf(m, lg[t]);
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float z = 0.0f;
    for (int t = tid; t < a.n; t += FLUSH_THREADS) { const float e = expf(lg[t] - m); lg[t] = e; z += e; }
    z = wave_sum(z);
    if (lane == 0) red2[wave] = z;
    __syncthreads();
    z = (red2[0] + red2[1]) + (red2[2] + red2[3]);
    float psum = 0.0f;
    for (int t = tid; t < a.n; t += FLUSH_THREADS) {
        const float p = lg[t] / z;
        lg[t] = p;
        psum += p;
        if (a.attn) a.attn[(size_t)bh * a.n + t] = p;
    }
    __syncthreads();                       // red is read above by everybody before it is written again
    psum = wave_sum(psum);
    if (lane == 0) red[wave] = psum;
    __syncthreads();
    const float inv_p = 1.0f / fmaxf((red[0] + red[1]) + (red[2] + red[3]), 1e-8f);
    float lo = INFINITY, hi = -INFINITY;
    bool nan_seen = false;          // a NaN score makes the whole flush's range NaN, as torch's min() / max() do
    if (a.mode == 0) {
        // pass 2: o = sum_t p_hat_t v_t
        float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int t = grp; t < a.n; t += FLUSH_THREADS / 16) {
            float v[8];
            row8<DT>(a.V, base + (size_t)t * HD + part * 8, v);
            const float ph = lg[t] * inv_p;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = __fmaf_rn(ph, v[e], o[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) opart[grp][part * 8 + e] = o[e];
        __syncthreads();
        if (tid < HD) {
            float acc = 0.0f;
            for (int g = 0; g < FLUSH_THREADS / 16; ++g) acc += opart[g][tid];
            obar[tid] = acc;
        }
        __syncthreads();
        float ob[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) ob[e] = obar[part * 8 + e];
        // pass 3: |v_t - o|^2 and the score
        for (int t = grp; t < a.n; t += FLUSH_THREADS / 16) {
            float v[8];
            row8<DT>(a.V, base + (size_t)t * HD + part * 8, v);
            float ir = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) { const float dlt = v[e] - ob[e]; ir = __fmaf_rn(dlt, dlt, ir); }
            ir = group16_total(ir);
            if (part == 0) {
                const float pe = lg[t] + a.eps;
                const float sc = (pe * pe) * (vn2[t] + (kn2[t] * (1.0f / (float)HD)) * ir);
                a.scores[(size_t)bh * a.n + t] = sc;
                lo = fminf(lo, sc); hi = fmaxf(hi, sc);
                nan_seen |= sc != sc;
            }
        }
    } else {
        for (int t = tid; t < a.n; t += FLUSH_THREADS) {
            const float sc = (lg[t] * lg[t]) * vn2[t];
            a.scores[(size_t)bh * a.n + t] = sc;
            lo = fminf(lo, sc); hi = fmaxf(hi, sc);
            nan_seen |= sc != sc;
        }
    }
    lo = -wave_max(-lo); hi = wave_max(hi);
    if (__builtin_amdgcn_ballot_w64(nan_seen) != 0) { lo = NAN; hi = NAN; }       // (fminf / fmaxf drop NaN operands)
    __syncthreads();
    if (lane == 0) { red[wave] = lo; red2[wave] = hi; }
    __syncthreads();
    if (tid == 0) {
        const bool bad = red[0] != red[0] || red[1] != red[1] || red[2] != red[2] || red[3] != red[3];
        a.minmax[2 * bh] = bad ? NAN : fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
        a.minmax[2 * bh + 1] = bad ? NAN : fmaxf(fmaxf(red2[0], red2[1]), fmaxf(red2[2], red2[3]));
    }
}

extern "C" int odmkv_flush_score(const void* K, const void* V, int dtype, int BH, int n, const float* q, float scaling,
                                 float eps, int mode, float* attn, float* scores, float* minmax, void* stream) {
    ODMKV_CHECK_ARG(K && V && q && scores && minmax, "flush_score: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "flush_score: bad dtype %d", dtype);
    ODMKV_CHECK_ARG(BH > 0 && n > 0 && n <= FLUSH_MAX_TOKENS, "flush_score: %d buffered tokens per head (1..%d)", n, FLUSH_MAX_TOKENS);
    ODMKV_CHECK_ARG(mode == 0 || mode == 1, "flush_score: mode %d", mode);
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)V & 15) == 0, "flush_score: K/V must be 16-byte aligned");
    FlushScoreArgs a{K, V, q, scaling, eps, n, mode, attn, scores, minmax};
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODMKV_F16) hipLaunchKernelGGL(flush_score_kernel<ODMKV_F16>, dim3(BH), dim3(FLUSH_THREADS), 0, st, a);
    else if (dtype == ODMKV_BF16) hipLaunchKernelGGL(flush_score_kernel<ODMKV_BF16>, dim3(BH), dim3(FLUSH_THREADS), 0, st, a);
    else hipLaunchKernelGGL(flush_score_kernel<ODMKV_F32>, dim3(BH), dim3(FLUSH_THREADS), 0, st, a);
    ODMKV_CHECK_LAUNCH("flush_score_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// levels by rank: the scores of all (sequence, kv-head) are min-max normalised over the whole flush
// (x - lo) / max(hi - lo, 1e-30), 0.5 everywhere when hi - lo <= 1e-8), then every kv-head's tokens (its rows of all
// sequences, row after row) are sorted ascending, equal scores in index order, and the token of rank r gets
// by_rank[h][r] (adaptive_backend_press.py:198-241 with the shares cached at prefill).
// One workgroup per kv-head, a bitonic sort of (score, index) pairs in LDS.
// Scores that are not finite follow torch: a NaN anywhere in the flush makes the range NaN and every key 0.5 (ranks in
// index order); an infinite score makes the spread infinite, its own key NaN and every finite key 0; NaN keys sort
// behind every number, among themselves in index order.  The keys are compared as integers whose order is that of the
// floats with NaN on top and the sort's padding above NaN, so the comparison is a total order whatever the scores.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(FLUSH_THREADS) void flush_rank_kernel(const float* scores, const float* minmax, int B, int H,
                                                                   int n, const int32_t* by_rank, int32_t* bits) {
    __shared__ uint32_t key[RANK_MAX_TOKENS];
    __shared__ uint32_t idx[RANK_MAX_TOKENS];
    __shared__ float red[FLUSH_THREADS / 64], red2[FLUSH_THREADS / 64];
    const int h = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    float lo = INFINITY, hi = -INFINITY;
    bool nan_seen = false;
    for (int i = tid; i < B * H; i += FLUSH_THREADS) {
        const float l = minmax[2 * i], u = minmax[2 * i + 1];
        nan_seen |= l != l || u != u;
        lo = fminf(lo, l); hi = fmaxf(hi, u);
    }
    lo = -wave_max(-lo); hi = wave_max(hi);
    if (__builtin_amdgcn_ballot_w64(nan_seen) != 0) { lo = NAN; hi = NAN; }
    if (lane == 0) { red[wave] = lo; red2[wave] = hi; }
    __syncthreads();
    const bool bad = red[0] != red[0] || red[1] != red[1] || red[2] != red[2] || red[3] != red[3];
    lo = fminf(fminf(red[0], red[1]), fminf(red[2], red[3]));
    hi = fmaxf(fmaxf(red2[0], red2[1]), fmaxf(red2[2], red2[3]));
    const float spread = bad ? NAN : hi - lo;               // NaN: the comparison below fails and every key is 0.5
    const int N = B * n;
    int P = 1;
    while (P < N) P <<= 1;
    for (int i = tid; i < P; i += FLUSH_THREADS) {
        if (i < N) {
            const int b = i / n, t = i % n;
            const float x = scores[((size_t)b * H + h) * n + t];
            const float y = (spread > 1e-8f ? (x - lo) / fmaxf(spread, 1e-30f) : 0.5f) + 0.0f;      // (-0 -> +0)
            const uint32_t u = __float_as_uint(y);
            key[i] = y != y ? 0xfffffffeu : (u & 0x80000000u) ? ~u : (u | 0x80000000u);
        } else {
            key[i] = 0xffffffffu;                          // padding: above every token, NaN keys included
        }
        idx[i] = (uint32_t)i;
    }
    __syncthreads();
    for (int k = 2; k <= P; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < P; i += FLUSH_THREADS) {
                const int l = i ^ j;
                if (l > i) {
                    const bool up = (i & k) == 0;
                    const uint32_t a0 = key[i], a1 = key[l];
                    const uint32_t i0 = idx[i], i1 = idx[l];
                    const bool gt = a0 > a1 || (a0 == a1 && i0 > i1);       // (score, index) pairs: a total order, so the sort is stable
                    if (gt == up) { key[i] = a1; key[l] = a0; idx[i] = i1; idx[l] = i0; }
                }
            }
            __syncthreads();
        }
    }
    for (int r = tid; r < N; r += FLUSH_THREADS) {
        const int i = (int)idx[r], b = i / n, t = i % n;
        if (i < N) bits[((size_t)b * H + h) * n + t] = by_rank[(size_t)h * N + r];      // (always: the padding sorts last)
    }
}

extern "C" int odmkv_flush_rank(const float* scores, const float* minmax, int B, int H, int n, const int32_t* by_rank,
                                int32_t* bits, void* stream) {
    ODMKV_CHECK_ARG(scores && minmax && by_rank && bits, "flush_rank: null pointer");
    ODMKV_CHECK_ARG(B > 0 && H > 0 && n > 0 && (long long)B * n <= RANK_MAX_TOKENS,
                    "flush_rank: %d x %d tokens per kv-head (at most %d)", B, n, RANK_MAX_TOKENS);
    hipLaunchKernelGGL(flush_rank_kernel, dim3(H), dim3(FLUSH_THREADS), 0, (hipStream_t)stream, scores, minmax, B, H, n, by_rank, bits);
    ODMKV_CHECK_LAUNCH("flush_rank_kernel");
    return 0;
}
