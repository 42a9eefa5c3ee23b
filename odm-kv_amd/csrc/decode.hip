// Fused LUT decode attention over the packed mixed-width KV store.
//
// Three launches per call:
//   1. prep:   q' = scaling * Pi_k q (queries in the rotated basis of the quantised keys) and
//              qs = scaling * q (for the exact fp16 tokens)
//   2. main:   one workgroup per work item (a run of tiles of one (sequence, kv-head, level));
//              each wavefront streams tiles: lane = token for the key side (codes -> centroid
//              lookup -> dot with the G query heads sharing this kv-head), an online softmax
//              per query head, then lane = dim for the value side, accumulating
//              sum_t p_t |v_t| centroid[code] in the rotated basis.  Partial (acc, m, l) per
//              item go to the workspace.
//   3. merge:  log-sum-exp merge of a kv-head's items per query head, rotate the quantised
//              part back (acc . Pi_v), add the exact part, normalise.
// Packed bytes are read exactly once; evicted tokens do not exist in the store.
#include "quant.h"

#define PSTRIDE 132          // floats per (item, head) partial: 128 acc + m + l + 2 pad
#define NWAVES 4

struct DecodeArgs {
    odmkv_packed_t s;
    const float* q;
    int Hq, G;
    float scaling;
    const int32_t* items;
    const int32_t* item_range;
    const float* pi_k;
    const float* pi_v;
    const float* cb;
    float* qrot;      // [B*Hq, 128]
    float* qs;        // [B*Hq, 128]
    float* partial;   // [n_items, GP, PSTRIDE]
    float* out;
    float* lse;
};

__global__ __launch_bounds__(128) void decode_prep_kernel(DecodeArgs a) {
    __shared__ float qsh[HD];
    const int bq = blockIdx.x, i = threadIdx.x;
    const float qi = a.q[(size_t)bq * HD + i];
    qsh[i] = qi;
    __syncthreads();
    const float* row = a.pi_k + (size_t)i * HD;
    float acc = 0.0f;
#pragma unroll 8
    for (int j = 0; j < HD; ++j) acc = __fmaf_rn(row[j], qsh[j], acc);
    a.qrot[(size_t)bq * HD + i] = acc * a.scaling;
    a.qs[(size_t)bq * HD + i] = qi * a.scaling;
}

// online-softmax update shared by both tile kinds: logits -> p (this lane's token), rescale
template <int GP>
__device__ static inline void softmax_step(const float (&logit)[GP], float (&m)[GP], float (&l)[GP],
                                           float (&acc)[GP][2], float (&p)[GP]) {
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        const float mt = wave_max(logit[g]);
        const float mn = fmaxf(m[g], mt);
        const float alpha = __expf(m[g] - mn);        // m = -inf on the first tile -> 0
        p[g] = __expf(logit[g] - mn);                 // padded lanes carry -inf -> 0
        l[g] = __fmaf_rn(l[g], alpha, p[g]);
        acc[g][0] *= alpha;
        acc[g][1] *= alpha;
        m[g] = mn;
    }
}

template <int W, int GP>
__device__ static inline void tile_quant(const DecodeArgs& a, int li, int tile, int nvalid, int lane,
                                         const float* qT, const float* cb, float* pw,
                                         float (&m)[GP], float (&l)[GP], float (&acc)[GP][2]) {
    const size_t slot = (size_t)tile * TILE + lane;
    // ---- keys: lane = token ----
    uint32_t kw[4 * W];
    const uint8_t* ksrc = a.s.kcodes[li] + (size_t)tile * (TILE * 16 * W);
#pragma unroll
    for (int c = 0; c < W; ++c) {
        const uint4 v = *reinterpret_cast<const uint4*>(ksrc + ((size_t)c * TILE + lane) * 16);
        kw[4 * c] = v.x; kw[4 * c + 1] = v.y; kw[4 * c + 2] = v.z; kw[4 * c + 3] = v.w;
    }
    const float kn = a.s.knorm[li][slot];
    const float vn = a.s.vnorm[li][slot];
    // ---- values: lane = dim (lane, lane + 64), issued early so the loads overlap the key math ----
    uint32_t vw[2][2 * W];
    const uint8_t* vsrc = a.s.vcodes[li] + (size_t)tile * (HD * 8 * W);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int k = 0; k < 2 * W; ++k)
            vw[h][k] = *reinterpret_cast<const uint32_t*>(vsrc + v_word_offset<W>(k, lane + 64 * h));

    float dot[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) dot[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < HD; ++i) {
        const float val = cb[get_code<W>(kw, i)];
#pragma unroll
        for (int g = 0; g < GP; ++g) dot[g] = __fmaf_rn(val, qT[i * GP + g], dot[g]);
    }
    float logit[GP], p[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) logit[g] = lane < nvalid ? dot[g] * kn : -INFINITY;
    softmax_step<GP>(logit, m, l, acc, p);
#pragma unroll
    for (int g = 0; g < GP; ++g) pw[lane * GP + g] = lane < nvalid ? p[g] * vn : 0.0f;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < TILE; ++t) {
        const float v0 = cb[get_code<W>(vw[0], t)];
        const float v1 = cb[get_code<W>(vw[1], t)];
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const float pg = pw[t * GP + g];
            acc[g][0] = __fmaf_rn(pg, v0, acc[g][0]);
            acc[g][1] = __fmaf_rn(pg, v1, acc[g][1]);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

__device__ static inline float half_bits_to_f32(uint16_t v, int bf16) {
    return bf16 ? __uint_as_float(((uint32_t)v) << 16) : __half2float(__ushort_as_half(v));
}

template <int GP>
__device__ static inline void tile_exact(const DecodeArgs& a, int tile, int nvalid, int lane,
                                         const float* qT, float* pw,
                                         float (&m)[GP], float (&l)[GP], float (&acc)[GP][2]) {
    const int bf = a.s.exact_dtype == ODMKV_BF16;
    const uint16_t* ksrc = a.s.kexact + (size_t)tile * TILE * HD;
    const uint16_t* vsrc = a.s.vexact + (size_t)tile * TILE * HD;
    float dot[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) dot[g] = 0.0f;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const uint4 v = *reinterpret_cast<const uint4*>(ksrc + ((size_t)c * TILE + lane) * 8);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float val = half_bits_to_f32((uint16_t)((w[e >> 1] >> (16 * (e & 1))) & 0xffffu), bf);
#pragma unroll
            for (int g = 0; g < GP; ++g) dot[g] = __fmaf_rn(val, qT[(8 * c + e) * GP + g], dot[g]);
        }
    }
    float logit[GP], p[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) logit[g] = lane < nvalid ? dot[g] : -INFINITY;
    softmax_step<GP>(logit, m, l, acc, p);
#pragma unroll
    for (int g = 0; g < GP; ++g) pw[lane * GP + g] = lane < nvalid ? p[g] : 0.0f;
    __builtin_amdgcn_wave_barrier();
#pragma unroll 4
    for (int tg = 0; tg < TILE / 4; ++tg) {
        const uint2 r0 = *reinterpret_cast<const uint2*>(vsrc + ((size_t)tg * HD + lane) * 4);
        const uint2 r1 = *reinterpret_cast<const uint2*>(vsrc + ((size_t)tg * HD + lane + 64) * 4);
        const uint32_t w0[2] = {r0.x, r0.y}, w1[2] = {r1.x, r1.y};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // padded tokens hold stale bytes: their p is 0, but 0 * inf would poison the sum
            const bool live = 4 * tg + e < nvalid;
            const float v0 = live ? half_bits_to_f32((uint16_t)((w0[e >> 1] >> (16 * (e & 1))) & 0xffffu), bf) : 0.0f;
            const float v1 = live ? half_bits_to_f32((uint16_t)((w1[e >> 1] >> (16 * (e & 1))) & 0xffffu), bf) : 0.0f;
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                const float pg = pw[(4 * tg + e) * GP + g];
                acc[g][0] = __fmaf_rn(pg, v0, acc[g][0]);
                acc[g][1] = __fmaf_rn(pg, v1, acc[g][1]);
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
}

template <int GP>
__global__ __launch_bounds__(256) void decode_main_kernel(DecodeArgs a) {
    __shared__ float qT[HD * GP];                 // [dim][head]
    __shared__ float cb[256];
    __shared__ float pw_all[NWAVES][TILE * GP];   // per-wave p * |v|
    __shared__ float wm[NWAVES][GP], wl[NWAVES][GP];
    __shared__ float wacc[NWAVES][GP][HD];

    const int item = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int bh = a.items[4 * item + 0];
    const int li = a.items[4 * item + 1];
    const int tile0 = a.items[4 * item + 2];
    const int ntiles = a.items[4 * item + 3];
    const int b = bh / a.s.Hkv, hkv = bh % a.s.Hkv;

    // queries of this kv-head's group, transposed to [dim][head]; unused heads are zero
    const float* qsrc = (li == 4 ? a.qs : a.qrot) + ((size_t)b * a.Hq + (size_t)hkv * a.G) * HD;
    for (int e = tid; e < HD * GP; e += 256) {
        const int i = e / GP, g = e % GP;
        qT[e] = g < a.G ? qsrc[(size_t)g * HD + i] : 0.0f;
    }
    if (li < 4) {
        const int n = 1 << width_of(li);
        for (int e = tid; e < n; e += 256) cb[e] = a.cb[codebook_offset(li) + e];
    }
    __syncthreads();

    float m[GP], l[GP], acc[GP][2];
#pragma unroll
    for (int g = 0; g < GP; ++g) { m[g] = -INFINITY; l[g] = 0.0f; acc[g][0] = 0.0f; acc[g][1] = 0.0f; }

    const int seg_first = a.s.seg_tile[li][bh];
    const int count = a.s.seg_count[li][bh];
    float* pw = pw_all[wave];
    for (int tt = wave; tt < ntiles; tt += NWAVES) {
        const int tile = tile0 + tt;
        const int nvalid = min(count - (tile - seg_first) * TILE, TILE);
        if (nvalid <= 0) break;                                  // tiles are filled front to back
        switch (li) {
            case 0: tile_quant<2, GP>(a, 0, tile, nvalid, lane, qT, cb, pw, m, l, acc); break;
            case 1: tile_quant<3, GP>(a, 1, tile, nvalid, lane, qT, cb, pw, m, l, acc); break;
            case 2: tile_quant<4, GP>(a, 2, tile, nvalid, lane, qT, cb, pw, m, l, acc); break;
            case 3: tile_quant<8, GP>(a, 3, tile, nvalid, lane, qT, cb, pw, m, l, acc); break;
            default: tile_exact<GP>(a, tile, nvalid, lane, qT, pw, m, l, acc); break;
        }
    }

    // ---- combine the four wavefronts ----
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        const float ls = wave_sum(l[g]);
        if (lane == 0) { wm[wave][g] = m[g]; wl[wave][g] = ls; }
        wacc[wave][g][lane] = acc[g][0];
        wacc[wave][g][lane + 64] = acc[g][1];
    }
    __syncthreads();
    float* dst = a.partial + (size_t)item * GP * PSTRIDE;
    for (int e = tid; e < GP * HD; e += 256) {
        const int g = e / HD, j = e % HD;
        float M = wm[0][g];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w) M = fmaxf(M, wm[w][g]);
        float s = 0.0f, L = 0.0f;
        if (M > -INFINITY) {
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                const float f = __expf(wm[w][g] - M);
                s = __fmaf_rn(wacc[w][g][j], f, s);
                L = __fmaf_rn(wl[w][g], f, L);
            }
        }
        dst[g * PSTRIDE + j] = s;
        if (j == 0) { dst[g * PSTRIDE + HD] = M; dst[g * PSTRIDE + HD + 1] = L; }
    }
}

template <int GP>
__global__ __launch_bounds__(128) void decode_merge_kernel(DecodeArgs a) {
    __shared__ float rot[HD];
    const int bq = blockIdx.x, j = threadIdx.x;
    const int b = bq / a.Hq, hq = bq % a.Hq;
    const int bh = b * a.s.Hkv + hq / a.G, g = hq % a.G;
    const int i0 = a.item_range[bh], i1 = a.item_range[bh + 1];
    float M = -INFINITY;
    for (int it = i0; it < i1; ++it) M = fmaxf(M, a.partial[((size_t)it * GP + g) * PSTRIDE + HD]);
    float L = 0.0f, arot = 0.0f, aex = 0.0f;
    if (M > -INFINITY) {
        for (int it = i0; it < i1; ++it) {
            const float* p = a.partial + ((size_t)it * GP + g) * PSTRIDE;
            const float f = __expf(p[HD] - M);
            L = __fmaf_rn(p[HD + 1], f, L);
            if (a.items[4 * it + 1] == 4) aex = __fmaf_rn(p[j], f, aex);
            else arot = __fmaf_rn(p[j], f, arot);
        }
    }
    rot[j] = arot;
    __syncthreads();
    float o = aex;
#pragma unroll 8
    for (int i = 0; i < HD; ++i) o = __fmaf_rn(rot[i], a.pi_v[(size_t)i * HD + j], o);
    a.out[(size_t)bq * HD + j] = L > 0.0f ? o / L : 0.0f;
    if (a.lse && j == 0) a.lse[bq] = L > 0.0f ? M + __logf(L) : -INFINITY;
}

static inline int group_pad(int G) { return G <= 4 ? 4 : 8; }

// ---- measurement hooks: event pairs around the main kernel ----
#include <vector>
static std::vector<hipEvent_t> g_prof_events;   // 2 per record
static int g_prof_used = 0;
static bool g_prof_on = false;

extern "C" int odmkv_profile_enable(int max_records) {
    ODMKV_CHECK_ARG(max_records > 0 && max_records <= (1 << 20), "profile_enable: bad record count %d", max_records);
    if (g_prof_on) odmkv_profile_disable();
    g_prof_events.resize((size_t)2 * max_records);
    for (auto& e : g_prof_events) ODMKV_CHECK_HIP(hipEventCreate(&e));
    g_prof_used = 0;
    g_prof_on = true;
    return 0;
}

extern "C" int odmkv_profile_collect(float* ms, int capacity, int* n_out) {
    ODMKV_CHECK_ARG(ms && n_out && capacity >= 0, "profile_collect: bad arguments");
    int n = 0;
    for (int r = 0; r < g_prof_used && n < capacity; ++r, ++n) {
        ODMKV_CHECK_HIP(hipEventSynchronize(g_prof_events[2 * r + 1]));
        ODMKV_CHECK_HIP(hipEventElapsedTime(&ms[n], g_prof_events[2 * r], g_prof_events[2 * r + 1]));
    }
    *n_out = n;
    g_prof_used = 0;
    return 0;
}

extern "C" int odmkv_profile_disable(void) {
    for (auto& e : g_prof_events) hipEventDestroy(e);
    g_prof_events.clear();
    g_prof_used = 0;
    g_prof_on = false;
    return 0;
}

extern "C" size_t odmkv_decode_workspace_bytes(int B, int Hq, int n_items) {
    size_t q = align_up((size_t)B * Hq * HD * sizeof(float), 256);
    return 2 * q + align_up((size_t)n_items * ODMKV_MAX_GROUP * PSTRIDE * sizeof(float), 256);
}

extern "C" int odmkv_decode_attn(const float* q, int B, int Hq, float scaling,
                                 const odmkv_packed_t* store,
                                 const int32_t* items, int n_items, const int32_t* item_range,
                                 const float* pi_k, const float* pi_v, const float* codebooks,
                                 float* out, float* lse, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    ODMKV_CHECK_ARG(q && store && item_range && pi_k && pi_v && codebooks && out && workspace, "decode_attn: null pointer");
    ODMKV_CHECK_ARG(n_items == 0 || items, "decode_attn: null work list");
    ODMKV_CHECK_ARG(B > 0 && Hq > 0 && store->B == B && store->Hkv > 0 && Hq % store->Hkv == 0,
                    "decode_attn: bad head counts B=%d Hq=%d store(B=%d,Hkv=%d)", B, Hq, store->B, store->Hkv);
    const int G = Hq / store->Hkv;
    ODMKV_CHECK_ARG(G <= ODMKV_MAX_GROUP, "decode_attn: GQA group %d exceeds %d", G, ODMKV_MAX_GROUP);
    ODMKV_CHECK_ARG(n_items >= 0, "decode_attn: negative item count");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_decode_workspace_bytes(B, Hq, n_items), "decode_attn: workspace too small");
    hipStream_t st = (hipStream_t)stream;
    DecodeArgs a;
    a.s = *store; a.q = q; a.Hq = Hq; a.G = G; a.scaling = scaling;
    a.items = items; a.item_range = item_range;
    a.pi_k = pi_k; a.pi_v = pi_v; a.cb = codebooks;
    const size_t qbytes = align_up((size_t)B * Hq * HD * sizeof(float), 256);
    a.qrot = (float*)workspace;
    a.qs = (float*)((char*)workspace + qbytes);
    a.partial = (float*)((char*)workspace + 2 * qbytes);
    a.out = out; a.lse = lse;
    hipLaunchKernelGGL(decode_prep_kernel, dim3(B * Hq), dim3(128), 0, st, a);
    ODMKV_CHECK_LAUNCH("decode_prep_kernel");
    const int GP = group_pad(G);
    if (n_items > 0) {
        const bool rec = g_prof_on && (size_t)(2 * g_prof_used + 1) < g_prof_events.size();
        if (rec) ODMKV_CHECK_HIP(hipEventRecord(g_prof_events[2 * g_prof_used], st));
        if (GP == 4) hipLaunchKernelGGL((decode_main_kernel<4>), dim3(n_items), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((decode_main_kernel<8>), dim3(n_items), dim3(256), 0, st, a);
        ODMKV_CHECK_LAUNCH("decode_main_kernel");
        if (rec) {
            ODMKV_CHECK_HIP(hipEventRecord(g_prof_events[2 * g_prof_used + 1], st));
            ++g_prof_used;
        }
    }
    if (GP == 4) hipLaunchKernelGGL((decode_merge_kernel<4>), dim3(B * Hq), dim3(128), 0, st, a);
    else hipLaunchKernelGGL((decode_merge_kernel<8>), dim3(B * Hq), dim3(128), 0, st, a);
    ODMKV_CHECK_LAUNCH("decode_merge_kernel");
    return 0;
}
