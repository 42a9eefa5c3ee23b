// Packed mixed-width KV store: level counts, position compaction, TurboQuant-MSE quantise + pack,
// exact-row gather, decode-time append, and dequantise-to-dense.
//
// One wavefront owns one 64-token tile.  During quantisation and dequantisation a lane owns one
// token: it keeps the 128 coordinates in registers and walks the rotation matrix through
// scalar (wave-uniform) loads, so the 128x128 rotation needs no LDS traffic and its fp32
// summation order is exactly the sequential one the CPU oracle uses.
#include "quant.h"

// ------------------------------------------------------------------------------------------------
// level counts
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void level_counts_kernel(const int32_t* __restrict__ bits, int T,
                                                           int32_t* __restrict__ counts) {
    __shared__ int c[6];
    const int bh = blockIdx.x;
    if (threadIdx.x < 6) c[threadIdx.x] = 0;
    __syncthreads();
    int local[6] = {0, 0, 0, 0, 0, 0};
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        const int s = level_slot(bits[(size_t)bh * T + t]);
#pragma unroll
        for (int k = 0; k < 6; ++k) local[k] += (s == k);
    }
#pragma unroll
    for (int k = 0; k < 6; ++k)
        if (local[k]) atomicAdd(&c[k], local[k]);
    __syncthreads();
    if (threadIdx.x < 6) counts[bh * 6 + threadIdx.x] = c[threadIdx.x];
}

extern "C" int odmkv_level_counts(const int32_t* bits, int B, int Hkv, int T, int32_t* counts,
                                  void* stream) {
    ODMKV_CHECK_ARG(bits && counts, "level_counts: null pointer");
    ODMKV_CHECK_ARG(B > 0 && Hkv > 0 && T >= 0, "level_counts: bad shape B=%d Hkv=%d T=%d", B, Hkv, T);
    hipLaunchKernelGGL(level_counts_kernel, dim3(B * Hkv), dim3(256), 0, (hipStream_t)stream, bits, T, counts);
    ODMKV_CHECK_LAUNCH("level_counts_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// compaction: ascending token positions per (bh, level), appended behind what is stored
// ------------------------------------------------------------------------------------------------
struct CompactArgs {
    const int32_t* bits;
    int T, pos_offset, nseg;
    int32_t* pos[5];
    const int32_t* seg_tile[5];
    int32_t* seg_count[5];
    int32_t* old_count;   // [5][nseg]
};

__global__ __launch_bounds__(256) void compact_kernel(CompactArgs a) {
    __shared__ int wave_tot[5][4];
    __shared__ int base[5];
    __shared__ int cap[5];
    const int bh = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < 5) {
        const int b0 = a.seg_count[tid][bh];
        base[tid] = b0;
        a.old_count[tid * a.nseg + bh] = b0;
        cap[tid] = (a.seg_tile[tid][bh + 1] - a.seg_tile[tid][bh]) * TILE;
    }
    __syncthreads();
    for (int c = 0; c < a.T; c += 256) {
        const int t = c + tid;
        const int s = (t < a.T) ? level_slot(a.bits[(size_t)bh * a.T + t]) : -1;
        int rank = 0;
#pragma unroll
        for (int L = 0; L < 5; ++L) {
            const unsigned long long m = __ballot(s == L + 1);
            if (lane == 0) wave_tot[L][wave] = __popcll(m);
            if (s == L + 1) rank = __popcll(m & ((1ull << lane) - 1ull));
        }
        __syncthreads();
        if (s >= 1) {
            const int L = s - 1;
            int off = base[L] + rank;
            for (int w = 0; w < wave; ++w) off += wave_tot[L][w];
            if (off < cap[L]) a.pos[L][(size_t)a.seg_tile[L][bh] * TILE + off] = t + a.pos_offset;
        }
        __syncthreads();
        if (tid < 5) base[tid] += wave_tot[tid][0] + wave_tot[tid][1] + wave_tot[tid][2] + wave_tot[tid][3];
        __syncthreads();
    }
    if (tid < 5) a.seg_count[tid][bh] = min(base[tid], cap[tid]);
}

// ------------------------------------------------------------------------------------------------
// quantise + pack one tile (blockIdx.y: 0 = keys, 1 = values)
// ------------------------------------------------------------------------------------------------
struct QuantArgs {
    const void* K;
    const void* V;
    int64_t sB, sH, sT;
    int Hkv, nseg, pos_offset;
    const float* pi_k;
    const float* pi_v;
    const float* cb;             // this width's centroids
    const int32_t* pos;          // this level
    const int32_t* seg_tile;
    const int32_t* seg_count;
    const int32_t* old_count;
    uint8_t* kcodes;
    uint8_t* vcodes;
    float* knorm;
    float* vnorm;
};

#define CODE_ROW 144   // LDS bytes per token row of codes (128 + padding, multiple of 16)

// which segment owns `tile`: the largest bh with seg_tile[bh] <= tile
__device__ static inline int find_segment(const int32_t* seg_tile, int nseg, int tile) {
    int lo = 0, hi = nseg;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (seg_tile[mid] <= tile) lo = mid; else hi = mid;
    }
    return lo;
}

template <int W, int DT>
__global__ __launch_bounds__(64) void quant_pack_kernel(QuantArgs a) {
    __shared__ __align__(16) uint8_t codes[TILE * CODE_ROW];
    __shared__ float cb[1 << W];
    const int lane = threadIdx.x;
    const int tile = blockIdx.x;
    const bool is_v = blockIdx.y != 0;

    const int bh = find_segment(a.seg_tile, a.nseg, tile);
    const int ts = (tile - a.seg_tile[bh]) * TILE;
    const int lo = max(a.old_count[bh] - ts, 0);
    const int hi = min(a.seg_count[bh] - ts, TILE);
    if (lo >= hi) return;                                   // nothing new in this tile (wave-uniform)

    for (int i = lane; i < (1 << W); i += WAVE) cb[i] = a.cb[i];
    const bool valid = lane >= lo && lane < hi;
    const size_t slot = (size_t)tile * TILE + lane;

    float x[HD];
    if (valid) {
        const int t = a.pos[slot] - a.pos_offset;
        const size_t off = (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT;
        load_row<DT>(is_v ? a.V : a.K, off, x);
    } else {
#pragma unroll
        for (int j = 0; j < HD; ++j) x[j] = 0.0f;
    }
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < HD; ++j) ss = __fmaf_rn(x[j], x[j], ss);
    const float norm = sqrtf(ss);
    const float den = norm + 1e-10f;
#pragma unroll
    for (int j = 0; j < HD; ++j) x[j] = x[j] / den;
    __syncthreads();                                        // codebook visible

    const float* __restrict__ pi = is_v ? a.pi_v : a.pi_k;
#pragma unroll 1
    for (int i0 = 0; i0 < HD; i0 += 8) {
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        const float* __restrict__ rows = pi + (size_t)i0 * HD;
#pragma unroll
        for (int j = 0; j < HD; ++j) {
#pragma unroll
            for (int b = 0; b < 8; ++b) acc[b] = __fmaf_rn(x[j], rows[b * HD + j], acc[b]);
        }
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) w0 |= nearest_code<W>(acc[b], cb) << (8 * b);
#pragma unroll
        for (int b = 0; b < 4; ++b) w1 |= nearest_code<W>(acc[4 + b], cb) << (8 * b);
        *reinterpret_cast<uint2*>(&codes[lane * CODE_ROW + i0]) = make_uint2(w0, w1);
    }
    __syncthreads();

    if (!is_v) {
        // token-major: this lane packs its own 128 codes
        if (valid) {
            uint32_t words[4 * W];
#pragma unroll
            for (int k = 0; k < 4 * W; ++k) words[k] = 0;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint4 v = *reinterpret_cast<const uint4*>(&codes[lane * CODE_ROW + 16 * c]);
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 16; ++e) put_code<W>(words, 16 * c + e, (w[e >> 2] >> (8 * (e & 3))) & 0xffu);
            }
            uint8_t* dst = a.kcodes + (size_t)tile * (TILE * 16 * W);
#pragma unroll
            for (int c = 0; c < W; ++c)
                *reinterpret_cast<uint4*>(dst + ((size_t)c * TILE + lane) * 16) =
                    make_uint4(words[4 * c], words[4 * c + 1], words[4 * c + 2], words[4 * c + 3]);
            a.knorm[slot] = norm;
        }
    } else {
        // dim-major: this lane packs the 64 tokens' codes of dims `lane` and `lane + 64`
        uint8_t* dst = a.vcodes + (size_t)tile * (HD * 8 * W);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int j = lane + 64 * half;
            uint32_t words[2 * W];
#pragma unroll
            for (int k = 0; k < 2 * W; ++k) words[k] = 0;
#pragma unroll
            for (int t = 0; t < TILE; ++t) {
                uint32_t c = codes[t * CODE_ROW + j];
                c = (t >= lo && t < hi) ? c : 0u;
                put_code<W>(words, t, c);
            }
            if (lo > 0) {
                // tokens below `lo` were packed earlier: keep their bits
                const int keep_bits = lo * W;
#pragma unroll
                for (int k = 0; k < 2 * W; ++k) {
                    const int nb = keep_bits - 32 * k;
                    if (nb > 0) {
                        const uint32_t old = *reinterpret_cast<const uint32_t*>(dst + v_word_offset<W>(k, j));
                        const uint32_t mask = nb >= 32 ? 0xffffffffu : ((1u << nb) - 1u);
                        words[k] = (old & mask) | (words[k] & ~mask);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 2 * W; ++k)
                *reinterpret_cast<uint32_t*>(dst + v_word_offset<W>(k, j)) = words[k];
        }
        if (valid) a.vnorm[slot] = norm;
    }
}

// ------------------------------------------------------------------------------------------------
// exact rows: gather into the tiled fp16/bf16 layout
// ------------------------------------------------------------------------------------------------
struct ExactArgs {
    const void* K;
    const void* V;
    int64_t sB, sH, sT;
    int Hkv, nseg, pos_offset;
    const int32_t* pos;
    const int32_t* seg_tile;
    const int32_t* seg_count;
    const int32_t* old_count;
    uint16_t* kexact;
    uint16_t* vexact;
};

template <int DT, int ODT>
__device__ static inline uint16_t to_store16(typename Elem<DT>::raw v) {
    if constexpr (DT == ODT) return v;
    else return Elem<ODT>::from_f32(Elem<DT>::to_f32(v));
}

template <int DT, int ODT>
__global__ __launch_bounds__(64) void exact_gather_kernel(ExactArgs a) {
    const int lane = threadIdx.x, tile = blockIdx.x;
    const int bh = find_segment(a.seg_tile, a.nseg, tile);
    const int ts = (tile - a.seg_tile[bh]) * TILE;
    const int lo = max(a.old_count[bh] - ts, 0);
    const int hi = min(a.seg_count[bh] - ts, TILE);
    if (lane < lo || lane >= hi) return;
    const size_t slot = (size_t)tile * TILE + lane;
    const int t = a.pos[slot] - a.pos_offset;
    const size_t off = (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT;
    const typename Elem<DT>::raw* kr = reinterpret_cast<const typename Elem<DT>::raw*>(a.K) + off;
    const typename Elem<DT>::raw* vr = reinterpret_cast<const typename Elem<DT>::raw*>(a.V) + off;
    uint16_t* kd = a.kexact + (size_t)tile * TILE * HD;
    uint16_t* vd = a.vexact + (size_t)tile * TILE * HD;
    for (int c = 0; c < 16; ++c) {
        uint16_t tmp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) tmp[e] = to_store16<DT, ODT>(kr[8 * c + e]);
        uint4 pk;
        pk.x = tmp[0] | ((uint32_t)tmp[1] << 16);
        pk.y = tmp[2] | ((uint32_t)tmp[3] << 16);
        pk.z = tmp[4] | ((uint32_t)tmp[5] << 16);
        pk.w = tmp[6] | ((uint32_t)tmp[7] << 16);
        *reinterpret_cast<uint4*>(kd + ((size_t)c * TILE + lane) * 8) = pk;
    }
    for (int j = 0; j < HD; ++j)
        vd[((size_t)(lane >> 2) * HD + j) * 4 + (lane & 3)] = to_store16<DT, ODT>(vr[j]);
}

// one new token per (b, h) behind the stored exact tokens
__global__ __launch_bounds__(128) void append_exact_kernel(odmkv_packed_t s, const uint16_t* __restrict__ k,
                                                           const uint16_t* __restrict__ v, int pos) {
    const int bh = blockIdx.x, j = threadIdx.x;
    const int cnt = s.seg_count[4][bh];
    const int cap = (s.seg_tile[4][bh + 1] - s.seg_tile[4][bh]) * TILE;
    if (cnt >= cap) return;                                  // full: the host sized it too small
    const int tile = s.seg_tile[4][bh] + cnt / TILE;
    const int l = cnt % TILE;
    uint16_t* kd = s.kexact + (size_t)tile * TILE * HD;
    uint16_t* vd = s.vexact + (size_t)tile * TILE * HD;
    kd[((size_t)(j >> 3) * TILE + l) * 8 + (j & 7)] = k[(size_t)bh * HD + j];
    vd[((size_t)(l >> 2) * HD + j) * 4 + (l & 3)] = v[(size_t)bh * HD + j];
    __syncthreads();
    if (j == 0) {
        s.pos[4][(size_t)tile * TILE + l] = pos;
        s.seg_count[4][bh] = cnt + 1;
    }
}

extern "C" int odmkv_append_exact(const odmkv_packed_t* store, const void* k, const void* v, int pos,
                                  void* stream) {
    ODMKV_CHECK_ARG(store && k && v, "append_exact: null pointer");
    ODMKV_CHECK_ARG(store->kexact && store->vexact && store->seg_tile[4] && store->seg_count[4] && store->pos[4],
                    "append_exact: store has no exact segments");
    hipLaunchKernelGGL(append_exact_kernel, dim3(store->B * store->Hkv), dim3(128), 0, (hipStream_t)stream,
                       *store, (const uint16_t*)k, (const uint16_t*)v, pos);
    ODMKV_CHECK_LAUNCH("append_exact_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// host entry: quantise + pack
// ------------------------------------------------------------------------------------------------
static int check_store(const odmkv_packed_t* s, const char* who) {
    ODMKV_CHECK_ARG(s != nullptr, "%s: null store", who);
    ODMKV_CHECK_ARG(s->B > 0 && s->Hkv > 0, "%s: bad store shape B=%d Hkv=%d", who, s->B, s->Hkv);
    ODMKV_CHECK_ARG(s->exact_dtype == ODMKV_F16 || s->exact_dtype == ODMKV_BF16, "%s: exact dtype must be fp16 or bf16", who);
    for (int li = 0; li < ODMKV_NQ + 1; ++li) {
        ODMKV_CHECK_ARG(s->n_tiles[li] >= 0, "%s: negative tile count", who);
        ODMKV_CHECK_ARG(s->seg_tile[li] && s->seg_count[li], "%s: missing segment table for level %d", who, li);
        if (s->n_tiles[li] == 0) continue;
        ODMKV_CHECK_ARG(s->pos[li], "%s: missing positions for level %d", who, li);
        if (li < ODMKV_NQ)
            ODMKV_CHECK_ARG(s->kcodes[li] && s->vcodes[li] && s->knorm[li] && s->vnorm[li],
                            "%s: missing buffers for level %d", who, li);
        else
            ODMKV_CHECK_ARG(s->kexact && s->vexact, "%s: missing exact buffers", who);
    }
    return 0;
}

extern "C" size_t odmkv_pack_workspace_bytes(int B, int Hkv, int T) {
    (void)T;
    return align_up((size_t)5 * B * Hkv * sizeof(int32_t), 256);
}

template <int DT>
static int launch_quant(const QuantArgs& qa, int li, int n_tiles, hipStream_t st) {
    dim3 grid(n_tiles, 2), block(64);
    switch (li) {
        case 0: hipLaunchKernelGGL((quant_pack_kernel<2, DT>), grid, block, 0, st, qa); break;
        case 1: hipLaunchKernelGGL((quant_pack_kernel<3, DT>), grid, block, 0, st, qa); break;
        case 2: hipLaunchKernelGGL((quant_pack_kernel<4, DT>), grid, block, 0, st, qa); break;
        default: hipLaunchKernelGGL((quant_pack_kernel<8, DT>), grid, block, 0, st, qa); break;
    }
    ODMKV_CHECK_LAUNCH("quant_pack_kernel");
    return 0;
}

template <int DT>
static int launch_exact(const ExactArgs& ea, int out_dt, int n_tiles, hipStream_t st) {
    if (out_dt == ODMKV_F16)
        hipLaunchKernelGGL((exact_gather_kernel<DT, ODMKV_F16>), dim3(n_tiles), dim3(64), 0, st, ea);
    else
        hipLaunchKernelGGL((exact_gather_kernel<DT, ODMKV_BF16>), dim3(n_tiles), dim3(64), 0, st, ea);
    ODMKV_CHECK_LAUNCH("exact_gather_kernel");
    return 0;
}

extern "C" int odmkv_quant_pack(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                                int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                const int32_t* bits, int pos_offset,
                                const float* pi_k, const float* pi_v, const float* codebooks,
                                const odmkv_packed_t* store, void* workspace, size_t workspace_bytes,
                                void* stream) {
    ODMKV_CHECK_ARG(K && V && bits && pi_k && pi_v && codebooks && workspace, "quant_pack: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "quant_pack: bad dtype %d", dtype);
    ODMKV_CHECK_ARG(B > 0 && Hkv > 0 && T > 0, "quant_pack: bad shape B=%d Hkv=%d T=%d", B, Hkv, T);
    if (int rc = check_store(store, "quant_pack")) return rc;
    ODMKV_CHECK_ARG(store->B == B && store->Hkv == Hkv, "quant_pack: store is (B=%d,Hkv=%d), tensors are (B=%d,Hkv=%d)",
                    store->B, store->Hkv, B, Hkv);
    const int align = dtype == ODMKV_F32 ? 4 : 8;
    ODMKV_CHECK_ARG(stride_b % align == 0 && stride_h % align == 0 && stride_t % align == 0 && stride_t >= HD,
                    "quant_pack: strides must keep rows 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)V & 15) == 0, "quant_pack: K/V must be 16-byte aligned");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_pack_workspace_bytes(B, Hkv, T), "quant_pack: workspace too small");
    hipStream_t st = (hipStream_t)stream;
    const int nseg = B * Hkv;
    int32_t* old_count = (int32_t*)workspace;

    CompactArgs ca;
    ca.bits = bits; ca.T = T; ca.pos_offset = pos_offset; ca.nseg = nseg; ca.old_count = old_count;
    for (int li = 0; li < 5; ++li) { ca.pos[li] = store->pos[li]; ca.seg_tile[li] = store->seg_tile[li]; ca.seg_count[li] = store->seg_count[li]; }
    hipLaunchKernelGGL(compact_kernel, dim3(nseg), dim3(256), 0, st, ca);
    ODMKV_CHECK_LAUNCH("compact_kernel");

    for (int li = 0; li < ODMKV_NQ; ++li) {
        if (store->n_tiles[li] == 0) continue;
        QuantArgs qa;
        qa.K = K; qa.V = V; qa.sB = stride_b; qa.sH = stride_h; qa.sT = stride_t;
        qa.Hkv = Hkv; qa.nseg = nseg; qa.pos_offset = pos_offset;
        qa.pi_k = pi_k; qa.pi_v = pi_v; qa.cb = codebooks + codebook_offset(li);
        qa.pos = store->pos[li]; qa.seg_tile = store->seg_tile[li]; qa.seg_count = store->seg_count[li];
        qa.old_count = old_count + (size_t)li * nseg;
        qa.kcodes = store->kcodes[li]; qa.vcodes = store->vcodes[li];
        qa.knorm = store->knorm[li]; qa.vnorm = store->vnorm[li];
        int rc = dtype == ODMKV_F16 ? launch_quant<ODMKV_F16>(qa, li, store->n_tiles[li], st)
               : dtype == ODMKV_BF16 ? launch_quant<ODMKV_BF16>(qa, li, store->n_tiles[li], st)
                                     : launch_quant<ODMKV_F32>(qa, li, store->n_tiles[li], st);
        if (rc) return rc;
    }
    if (store->n_tiles[4] > 0) {
        ExactArgs ea;
        ea.K = K; ea.V = V; ea.sB = stride_b; ea.sH = stride_h; ea.sT = stride_t;
        ea.Hkv = Hkv; ea.nseg = nseg; ea.pos_offset = pos_offset;
        ea.pos = store->pos[4]; ea.seg_tile = store->seg_tile[4]; ea.seg_count = store->seg_count[4];
        ea.old_count = old_count + (size_t)4 * nseg;
        ea.kexact = store->kexact; ea.vexact = store->vexact;
        int rc = dtype == ODMKV_F16 ? launch_exact<ODMKV_F16>(ea, store->exact_dtype, store->n_tiles[4], st)
               : dtype == ODMKV_BF16 ? launch_exact<ODMKV_BF16>(ea, store->exact_dtype, store->n_tiles[4], st)
                                     : launch_exact<ODMKV_F32>(ea, store->exact_dtype, store->n_tiles[4], st);
        if (rc) return rc;
    }
    return 0;
}

// ------------------------------------------------------------------------------------------------
// dequantise to dense tensors
// ------------------------------------------------------------------------------------------------
struct DequantArgs {
    void* K;
    void* V;
    int64_t sB, sH, sT;
    int Hkv, nseg, T;
    const float* pi_k;
    const float* pi_v;
    const float* cb;
    const int32_t* pos;
    const int32_t* seg_tile;
    const int32_t* seg_count;
    const uint8_t* kcodes;
    const uint8_t* vcodes;
    const float* knorm;
    const float* vnorm;
};

template <int W, int DT>
__global__ __launch_bounds__(64) void dequant_kernel(DequantArgs a) {
    __shared__ __align__(16) uint8_t codes[TILE * CODE_ROW];
    __shared__ float cb[1 << W];
    const int lane = threadIdx.x, tile = blockIdx.x;
    const bool is_v = blockIdx.y != 0;
    const int bh = find_segment(a.seg_tile, a.nseg, tile);
    const int ts = (tile - a.seg_tile[bh]) * TILE;
    const int hi = min(a.seg_count[bh] - ts, TILE);
    if (hi <= 0) return;
    for (int i = lane; i < (1 << W); i += WAVE) cb[i] = a.cb[i];
    const size_t slot = (size_t)tile * TILE + lane;
    const bool valid = lane < hi;

    float y[HD];
    if (!is_v) {
        uint32_t words[4 * W];
        const uint8_t* src = a.kcodes + (size_t)tile * (TILE * 16 * W);
#pragma unroll
        for (int c = 0; c < W; ++c) {
            const uint4 v = *reinterpret_cast<const uint4*>(src + ((size_t)c * TILE + lane) * 16);
            words[4 * c] = v.x; words[4 * c + 1] = v.y; words[4 * c + 2] = v.z; words[4 * c + 3] = v.w;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < HD; ++i) y[i] = cb[get_code<W>(words, i)];
    } else {
        const uint8_t* src = a.vcodes + (size_t)tile * (HD * 8 * W);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int j = lane + 64 * half;
            uint32_t words[2 * W];
#pragma unroll
            for (int k = 0; k < 2 * W; ++k) words[k] = *reinterpret_cast<const uint32_t*>(src + v_word_offset<W>(k, j));
#pragma unroll
            for (int t = 0; t < TILE; ++t) codes[t * CODE_ROW + j] = (uint8_t)get_code<W>(words, t);
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint4 v = *reinterpret_cast<const uint4*>(&codes[lane * CODE_ROW + 16 * c]);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 16; ++e) y[16 * c + e] = cb[(w[e >> 2] >> (8 * (e & 3))) & 0xffu];
        }
    }
    const float norm = valid ? (is_v ? a.vnorm[slot] : a.knorm[slot]) : 0.0f;
    const int t = valid ? a.pos[slot] : -1;
    const bool write = valid && t >= 0 && t < a.T;
    const size_t off = write ? (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT : 0;
    void* out = is_v ? a.V : a.K;
    const float* __restrict__ pi = is_v ? a.pi_v : a.pi_k;
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
        if (write) store8<DT>(out, off + j0, acc);
    }
}

template <int DT>
__global__ __launch_bounds__(64) void exact_scatter_kernel(odmkv_packed_t s, void* K, void* V, int64_t sB,
                                                           int64_t sH, int64_t sT, int T, int src_bf16) {
    const int lane = threadIdx.x, tile = blockIdx.x;
    const int nseg = s.B * s.Hkv;
    const int bh = find_segment(s.seg_tile[4], nseg, tile);
    const int ts = (tile - s.seg_tile[4][bh]) * TILE;
    if (lane >= s.seg_count[4][bh] - ts) return;
    const int t = s.pos[4][(size_t)tile * TILE + lane];
    if (t < 0 || t >= T) return;
    const size_t off = (size_t)(bh / s.Hkv) * sB + (size_t)(bh % s.Hkv) * sH + (size_t)t * sT;
    const uint16_t* ks = s.kexact + (size_t)tile * TILE * HD;
    const uint16_t* vs = s.vexact + (size_t)tile * TILE * HD;
    typename Elem<DT>::raw* kd = reinterpret_cast<typename Elem<DT>::raw*>(K) + off;
    typename Elem<DT>::raw* vd = reinterpret_cast<typename Elem<DT>::raw*>(V) + off;
    for (int j = 0; j < HD; ++j) {
        const uint16_t kr = ks[((size_t)(j >> 3) * TILE + lane) * 8 + (j & 7)];
        const uint16_t vr = vs[((size_t)(lane >> 2) * HD + j) * 4 + (lane & 3)];
        const float kf = src_bf16 ? Elem<ODMKV_BF16>::to_f32(kr) : Elem<ODMKV_F16>::to_f32(kr);
        const float vf = src_bf16 ? Elem<ODMKV_BF16>::to_f32(vr) : Elem<ODMKV_F16>::to_f32(vr);
        kd[j] = Elem<DT>::from_f32(kf);
        vd[j] = Elem<DT>::from_f32(vf);
    }
}

template <int DT>
static int launch_dequant(const DequantArgs& da, int li, int n_tiles, hipStream_t st) {
    dim3 grid(n_tiles, 2), block(64);
    switch (li) {
        case 0: hipLaunchKernelGGL((dequant_kernel<2, DT>), grid, block, 0, st, da); break;
        case 1: hipLaunchKernelGGL((dequant_kernel<3, DT>), grid, block, 0, st, da); break;
        case 2: hipLaunchKernelGGL((dequant_kernel<4, DT>), grid, block, 0, st, da); break;
        default: hipLaunchKernelGGL((dequant_kernel<8, DT>), grid, block, 0, st, da); break;
    }
    ODMKV_CHECK_LAUNCH("dequant_kernel");
    return 0;
}

extern "C" int odmkv_dequant(const odmkv_packed_t* store, void* K, void* V, int dtype, int T,
                             int64_t stride_b, int64_t stride_h, int64_t stride_t,
                             const float* pi_k, const float* pi_v, const float* codebooks,
                             int include_exact, void* stream) {
    ODMKV_CHECK_ARG(K && V && pi_k && pi_v && codebooks, "dequant: null pointer");
    ODMKV_CHECK_ARG(dtype == ODMKV_F16 || dtype == ODMKV_BF16 || dtype == ODMKV_F32, "dequant: bad dtype %d", dtype);
    if (int rc = check_store(store, "dequant")) return rc;
    const int align = dtype == ODMKV_F32 ? 4 : 8;
    ODMKV_CHECK_ARG(stride_b % align == 0 && stride_h % align == 0 && stride_t % align == 0 && stride_t >= HD,
                    "dequant: strides must keep rows 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)K & 15) == 0 && ((uintptr_t)V & 15) == 0, "dequant: K/V must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const int nseg = store->B * store->Hkv;
    for (int li = 0; li < ODMKV_NQ; ++li) {
        if (store->n_tiles[li] == 0) continue;
        DequantArgs da;
        da.K = K; da.V = V; da.sB = stride_b; da.sH = stride_h; da.sT = stride_t;
        da.Hkv = store->Hkv; da.nseg = nseg; da.T = T;
        da.pi_k = pi_k; da.pi_v = pi_v; da.cb = codebooks + codebook_offset(li);
        da.pos = store->pos[li]; da.seg_tile = store->seg_tile[li]; da.seg_count = store->seg_count[li];
        da.kcodes = store->kcodes[li]; da.vcodes = store->vcodes[li];
        da.knorm = store->knorm[li]; da.vnorm = store->vnorm[li];
        int rc = dtype == ODMKV_F16 ? launch_dequant<ODMKV_F16>(da, li, store->n_tiles[li], st)
               : dtype == ODMKV_BF16 ? launch_dequant<ODMKV_BF16>(da, li, store->n_tiles[li], st)
                                     : launch_dequant<ODMKV_F32>(da, li, store->n_tiles[li], st);
        if (rc) return rc;
    }
    if (include_exact && store->n_tiles[4] > 0) {
        const int bf = store->exact_dtype == ODMKV_BF16;
        dim3 grid(store->n_tiles[4]), block(64);
        if (dtype == ODMKV_F16)
            hipLaunchKernelGGL((exact_scatter_kernel<ODMKV_F16>), grid, block, 0, st, *store, K, V, stride_b, stride_h, stride_t, T, bf);
        else if (dtype == ODMKV_BF16)
            hipLaunchKernelGGL((exact_scatter_kernel<ODMKV_BF16>), grid, block, 0, st, *store, K, V, stride_b, stride_h, stride_t, T, bf);
        else
            hipLaunchKernelGGL((exact_scatter_kernel<ODMKV_F32>), grid, block, 0, st, *store, K, V, stride_b, stride_h, stride_t, T, bf);
        ODMKV_CHECK_LAUNCH("exact_scatter_kernel");
    }
    return 0;
}
