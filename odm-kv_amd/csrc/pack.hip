// Packed mixed-width KV store: level counts, position compaction, TurboQuant-MSE quantise + pack,
// exact-row gather, decode-time append, and dequantise-to-dense.
//
// One wavefront owns one 64-token tile.  The quantiser and the dequantiser run the rotation on the
// fp32 matrix cores one k at a time, a token per lane, and keep the sequential fp32 summation order of
// the definition; the tile's own layout (what the decode kernel's matrix operands want, quant.h) is
// produced and consumed by a re-layout through LDS.
#include <algorithm>
#include "quant.h"

// ------------------------------------------------------------------------------------------------
// level counts
// ------------------------------------------------------------------------------------------------
#define LC_THREADS 256
#define LC_CHUNK 4096           // tokens per workgroup

__device__ static inline int wave_sum_i32(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// 6-bit counters of the six levels in one 64-bit word; a value that is no level adds nothing.
// nibble b of the table = level index + 1 of bit width b (0: none); 16 is handled apart.
__device__ static inline unsigned long long level_increment(int bits) {
    const unsigned long long table = 0x0000000500043201ull;      // widths 0, 2, 3, 4, 8 -> 1, 2, 3, 4, 5
    const unsigned int ub = (unsigned int)bits;
    const unsigned int code = ub == 16u ? 6u : ub < 16u ? (unsigned int)(table >> (4 * ub)) & 15u : 0u;
    return code ? 1ull << (6 * (code - 1)) : 0ull;
}

// grid (chunks, rows): every workgroup adds its chunk's counts to the row's six counters (cleared by the
// launch before this one)
__global__ __launch_bounds__(LC_THREADS) void level_counts_kernel(const int32_t* __restrict__ bits, int T,
                                                                  int32_t* __restrict__ counts) {
    __shared__ int c[6];
    const int bh = blockIdx.y, tid = threadIdx.x;
    if (tid < 6) c[tid] = 0;
    __syncthreads();
    const int32_t* row = bits + (size_t)bh * T;
    const int t0 = blockIdx.x * LC_CHUNK;
    const int n = min(T - t0, LC_CHUNK);
    unsigned long long acc = 0ull;                       // at most 16 per thread and field
    const bool vec = ((reinterpret_cast<uintptr_t>(row + t0) & 15) == 0);
    if (vec) {
        const int4* p = reinterpret_cast<const int4*>(row + t0);
        int4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int q = u * LC_THREADS + tid;
            v[u] = 4 * q + 3 < n ? p[q] : make_int4(-1, -1, -1, -1);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            acc += level_increment(v[u].x) + level_increment(v[u].y) + level_increment(v[u].z) + level_increment(v[u].w);
        for (int t = (n & ~3) + tid; t < n; t += LC_THREADS) acc += level_increment(row[t0 + t]);
    } else {
        for (int t = tid; t < n; t += LC_THREADS) acc += level_increment(row[t0 + t]);
    }
#pragma unroll
    for (int k = 0; k < 6; ++k) {
        const int w = wave_sum_i32((int)((acc >> (6 * k)) & 63ull));
        if ((tid & 63) == 0 && w) atomicAdd(&c[k], w);
    }
    __syncthreads();
    if (tid < 6 && c[tid]) atomicAdd(&counts[bh * 6 + tid], c[tid]);
}

__global__ void level_counts_clear_kernel(int32_t* __restrict__ counts, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counts[i] = 0;
}

extern "C" int odmkv_level_counts(const int32_t* bits, int B, int Hkv, int T, int32_t* counts,
                                  void* stream) {
    ODMKV_CHECK_ARG(bits && counts, "level_counts: null pointer");
    ODMKV_CHECK_ARG(B > 0 && Hkv > 0 && T >= 0, "level_counts: bad shape B=%d Hkv=%d T=%d", B, Hkv, T);
    ODMKV_CHECK_ARG(B * Hkv <= 65535, "level_counts: at most 65535 (sequence, head) pairs per call");
    // a fill kernel, not a memset: callers may capture this call in a graph
    hipLaunchKernelGGL(level_counts_clear_kernel, dim3((B * Hkv * 6 + 255) / 256), dim3(256), 0, (hipStream_t)stream, counts, B * Hkv * 6);
    ODMKV_CHECK_LAUNCH("level_counts_clear_kernel");
    if (T == 0) return 0;
    hipLaunchKernelGGL(level_counts_kernel, dim3((T + LC_CHUNK - 1) / LC_CHUNK, B * Hkv), dim3(LC_THREADS), 0, (hipStream_t)stream,
                       bits, T, counts);
    ODMKV_CHECK_LAUNCH("level_counts_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// where a store's buffers lie inside one allocation (host arithmetic only), and the descriptor over them.
// Order of the 33 buffers: seg_tile[5], seg_count[5], (knorm, vnorm)[4], kexact, vexact, pos[5], (kcodes, vcodes)[4];
// every buffer starts on a multiple of 256 bytes.  What is cleared lies between marks[0] and marks[2], the
// positions end at marks[3].
// ------------------------------------------------------------------------------------------------
#define SL_BUFFERS 33

extern "C" int odmkv_store_layout(const int32_t* seg_tile, int nseg, uint64_t* offsets, uint64_t* sizes, uint64_t* marks) {
    ODMKV_CHECK_ARG(seg_tile && offsets && sizes && marks && nseg > 0, "store_layout: bad arguments");
    uint64_t nt[5];
    for (int li = 0; li < 5; ++li) {
        const int32_t last = seg_tile[(size_t)li * (nseg + 1) + nseg];
        ODMKV_CHECK_ARG(last >= 0, "store_layout: negative tile count");
        nt[li] = last > 0 ? (uint64_t)last : 1;                 // an unused level keeps one tile of room: no null pointers
    }
    uint64_t off = 0;
    int n = 0;
    auto take = [&](uint64_t bytes) { offsets[n] = off; sizes[n] = bytes; ++n; off += align_up(bytes, 256); };
    for (int li = 0; li < 5; ++li) take((uint64_t)(nseg + 1) * 4);
    marks[0] = off;                                              // end of the tables
    for (int li = 0; li < 5; ++li) take((uint64_t)nseg * 4);
    marks[1] = off;                                              // end of the segment counts
    for (int li = 0; li < 4; ++li) { take(nt[li] * TILE * 4); take(nt[li] * TILE * 4); }
    take(nt[4] * TILE * HD * 2);
    take(nt[4] * TILE * HD * 2);
    marks[2] = off;                                              // end of what is cleared
    for (int li = 0; li < 5; ++li) take(nt[li] * TILE * 4);
    marks[3] = off;                                              // end of the positions
    for (int li = 0; li < 4; ++li) { take(nt[li] * TILE * 16 * width_of(li)); take(nt[li] * TILE * 16 * width_of(li)); }
    marks[4] = off;                                              // bytes in all
    return 0;
}

extern "C" int odmkv_store_bind(void* arena, const uint64_t* offsets, const int32_t* seg_tile, int nseg, int B, int Hkv,
                                int exact_dtype, odmkv_packed_t* out) {
    ODMKV_CHECK_ARG(arena && offsets && seg_tile && out && nseg == B * Hkv && nseg > 0, "store_bind: bad arguments");
    ODMKV_CHECK_ARG(exact_dtype == ODMKV_F16 || exact_dtype == ODMKV_BF16, "store_bind: exact dtype must be fp16 or bf16");
    uint8_t* base = (uint8_t*)arena;
    out->B = B; out->Hkv = Hkv; out->exact_dtype = exact_dtype;
    for (int li = 0; li < 5; ++li) {
        out->n_tiles[li] = seg_tile[(size_t)li * (nseg + 1) + nseg];
        out->seg_tile[li] = (int32_t*)(base + offsets[li]);
        out->seg_count[li] = (int32_t*)(base + offsets[5 + li]);
        out->pos[li] = (int32_t*)(base + offsets[20 + li]);
        if (li < 4) {
            out->knorm[li] = (float*)(base + offsets[10 + 2 * li]);
            out->vnorm[li] = (float*)(base + offsets[11 + 2 * li]);
            out->kcodes[li] = base + offsets[25 + 2 * li];
            out->vcodes[li] = base + offsets[26 + 2 * li];
        }
    }
    out->kexact = (uint16_t*)(base + offsets[18]);
    out->vexact = (uint16_t*)(base + offsets[19]);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// a store's buffers before their first use: segment tables written, counters / norms / exact rows
// cleared, positions set to -1: one launch
// ------------------------------------------------------------------------------------------------
#define SI_MAX_TABLE 640                 // int32 words of tables that travel as kernel arguments

struct StoreInitArgs {
    uint8_t* arena;
    unsigned long long zero_begin, zero_end, fill_end;      // [zero_begin, zero_end) = 0, [zero_end, fill_end) = 0xff
    int n_words;                                            // words of `table`
    unsigned int table_off[5];                              // byte offset of each level's table in the arena
    int words_per_table;
    int32_t table[SI_MAX_TABLE];
};

__global__ __launch_bounds__(256) void store_init_kernel(StoreInitArgs a) {
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, nthreads = (size_t)gridDim.x * 256;
    if (tid < (size_t)a.n_words) {
        const int li = (int)tid / a.words_per_table, e = (int)tid % a.words_per_table;
        reinterpret_cast<int32_t*>(a.arena + a.table_off[li])[e] = a.table[tid];
    }
    // both regions start and end on multiples of 16 bytes
    uint4* p = reinterpret_cast<uint4*>(a.arena);
    const size_t z0 = a.zero_begin / 16, z1 = a.zero_end / 16, f1 = a.fill_end / 16;
    for (size_t i = z0 + tid; i < z1; i += nthreads) p[i] = make_uint4(0u, 0u, 0u, 0u);
    for (size_t i = z1 + tid; i < f1; i += nthreads) p[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
}

extern "C" int odmkv_store_init(void* arena, const int32_t* tables_host, int n_tables, int words_per_table,
                                const uint64_t* table_offsets, uint64_t zero_begin, uint64_t zero_end, uint64_t fill_end,
                                void* stream) {
    ODMKV_CHECK_ARG(arena && tables_host && table_offsets, "store_init: null pointer");
    ODMKV_CHECK_ARG(n_tables == 5 && words_per_table > 0, "store_init: five tables expected");
    ODMKV_CHECK_ARG(((uintptr_t)arena & 15) == 0 && zero_begin % 16 == 0 && zero_end % 16 == 0 && fill_end % 16 == 0 &&
                    zero_begin <= zero_end && zero_end <= fill_end, "store_init: regions must be ordered and 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    StoreInitArgs a;
    a.arena = (uint8_t*)arena; a.zero_begin = zero_begin; a.zero_end = zero_end; a.fill_end = fill_end;
    a.words_per_table = words_per_table;
    for (int li = 0; li < 5; ++li) {
        ODMKV_CHECK_ARG(table_offsets[li] < (1ull << 32), "store_init: the tables must lie in the first 4 GiB of the allocation");
        a.table_off[li] = (unsigned int)table_offsets[li];
    }
    const int n_words = 5 * words_per_table;
    if (n_words <= SI_MAX_TABLE) {
        a.n_words = n_words;
        for (int i = 0; i < n_words; ++i) a.table[i] = tables_host[i];
    } else {
        a.n_words = 0;                   // too many segments for the argument block: plain copies
        for (int li = 0; li < 5; ++li)
            ODMKV_CHECK_HIP(hipMemcpyAsync((uint8_t*)arena + table_offsets[li], tables_host + (size_t)li * words_per_table,
                                           (size_t)words_per_table * sizeof(int32_t), hipMemcpyHostToDevice, st));
    }
    const size_t chunks = (fill_end - zero_begin) / 16;
    const int grid = (int)std::min<size_t>(std::max<size_t>((chunks + 255) / 256, 1), 2048);
    hipLaunchKernelGGL(store_init_kernel, dim3(grid), dim3(256), 0, st, a);
    ODMKV_CHECK_LAUNCH("store_init_kernel");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// compaction: ascending token positions per (bh, level), appended behind what is stored.
// Two launches over chunks of 2048 tokens: count per (bh, chunk, level), then every chunk places
// its tokens behind the chunks before it.
// ------------------------------------------------------------------------------------------------
#define CP_THREADS 256
#define CP_TPT 8
#define CP_TOKENS (CP_THREADS * CP_TPT)

struct CompactArgs {
    const int32_t* bits;
    int T, pos_offset, nseg, n_chunks;
    int32_t* pos[5];
    const int32_t* seg_tile[5];
    int32_t* seg_count[5];
    int32_t* old_count;     // [5][nseg]
    int32_t* chunk_count;   // [nseg][n_chunks][5]
    int32_t* redo;          // two counters the quantise kernels use, cleared here (may be null)
    int32_t* totals;        // [nseg][n_chunks][6] tokens per chunk that are evicted / at each of the five levels, or null
};

// levels (1..5, 0 = evicted, -1 = past the end) of the 8 consecutive tokens this thread owns
__device__ static inline void load_slots(const CompactArgs& a, int bh, int t0, int* sl) {
    const int32_t* row = a.bits + (size_t)bh * a.T;
    if (t0 + CP_TPT <= a.T && ((reinterpret_cast<uintptr_t>(row + t0) & 15) == 0)) {
        const int4 v0 = *reinterpret_cast<const int4*>(row + t0);
        const int4 v1 = *reinterpret_cast<const int4*>(row + t0 + 4);
        const int b[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int e = 0; e < CP_TPT; ++e) sl[e] = level_slot(b[e]);
    } else {
#pragma unroll
        for (int e = 0; e < CP_TPT; ++e) sl[e] = (t0 + e < a.T) ? level_slot(row[t0 + e]) : -1;
    }
}

__global__ __launch_bounds__(CP_THREADS) void chunk_count_kernel(CompactArgs a) {
    __shared__ int c[5];
    __shared__ int c_evicted;
    const int bh = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    if (tid < 5) c[tid] = 0;
    if (tid == 5) c_evicted = 0;
    if (chunk == 0 && tid < 5) a.old_count[tid * a.nseg + bh] = a.seg_count[tid][bh];
    if (a.redo && chunk == 0 && bh == 0 && tid < 2) a.redo[tid] = 0;
    __syncthreads();
    int sl[CP_TPT];
    load_slots(a, bh, chunk * CP_TOKENS + tid * CP_TPT, sl);
#pragma unroll
    for (int L = 0; L < 5; ++L) {
        int n = 0;
#pragma unroll
        for (int e = 0; e < CP_TPT; ++e) n += (sl[e] == L + 1);
        n = wave_sum_i32(n);
        if ((tid & 63) == 0 && n) atomicAdd(&c[L], n);
    }
    if (a.totals) {                                       // wave-uniform
        int n = 0;
#pragma unroll
        for (int e = 0; e < CP_TPT; ++e) n += (sl[e] == 0);
        n = wave_sum_i32(n);
        if ((tid & 63) == 0 && n) atomicAdd(&c_evicted, n);
    }
    __syncthreads();
    if (tid < 5) a.chunk_count[((size_t)bh * a.n_chunks + chunk) * 5 + tid] = c[tid];
    if (a.totals && tid < 6) a.totals[((size_t)bh * a.n_chunks + chunk) * 6 + tid] = tid == 0 ? c_evicted : c[tid - 1];
}

__global__ __launch_bounds__(CP_THREADS) void compact_kernel(CompactArgs a) {
    __shared__ int base[5];
    __shared__ int cap[5];
    __shared__ int wave_tot[5][CP_THREADS / 64];
    const int bh = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < 5) {
        const int32_t* cc = a.chunk_count + (size_t)bh * a.n_chunks * 5 + tid;
        int before = 0, total = 0;
        for (int c = 0; c < a.n_chunks; ++c) {
            const int v = cc[(size_t)c * 5];
            total += v;
            before += (c < chunk) ? v : 0;
        }
        const int old = a.old_count[tid * a.nseg + bh];
        const int room = (a.seg_tile[tid][bh + 1] - a.seg_tile[tid][bh]) * TILE;
        base[tid] = old + before;
        cap[tid] = room;
        if (chunk == 0) a.seg_count[tid][bh] = min(old + total, room);
    }
    int sl[CP_TPT];
    const int t0 = chunk * CP_TOKENS + tid * CP_TPT;
    load_slots(a, bh, t0, sl);
    int mine[5], incl[5];
#pragma unroll
    for (int L = 0; L < 5; ++L) {
        int n = 0;
#pragma unroll
        for (int e = 0; e < CP_TPT; ++e) n += (sl[e] == L + 1);
        mine[L] = n;
        int x = n;                                         // inclusive scan over the wave
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int y = __shfl_up(x, o, WAVE);
            x += (lane >= o) ? y : 0;
        }
        incl[L] = x;
        if (lane == 63) wave_tot[L][wave] = x;
    }
    __syncthreads();
#pragma unroll
    for (int L = 0; L < 5; ++L) {
        int off = base[L] + incl[L] - mine[L];
        for (int w = 0; w < wave; ++w) off += wave_tot[L][w];
        if (mine[L]) {
            int32_t* dst = a.pos[L] + (size_t)a.seg_tile[L][bh] * TILE;
#pragma unroll
            for (int e = 0; e < CP_TPT; ++e) {
                if (sl[e] == L + 1) {
                    if (off < cap[L]) dst[off] = t0 + e + a.pos_offset;
                    ++off;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// quantise + pack
//
// The 128x128 rotation runs on the fp32 matrix cores with K = 1 per instruction
// (v_mfma_f32_32x32x1_2b_f32): one instruction adds u[token][j] * Pi[out][j] to a 64-token x
// 32-output block, so chaining j = 0..127 reproduces the sequential fp32 fma order of the scalar
// definition bit for bit, at twice the rate of the vector ALU and with the vector ALU free for
// the division, the centroid search and the packing.  Lane = token for the A operand; the B
// operand (Pi^T[j][4c..4c+3] for lane c of either half) is one ds_read_b128 from LDS.
//
// Workgroups are persistent: even ones take keys, odd ones values; each keeps its rotation in LDS
// and its waves walk the tiles of all quantised levels.
// ------------------------------------------------------------------------------------------------
struct QuantArgs {
    const void* K;
    const void* V;
    int64_t sB, sH, sT;
    int Hkv, nseg, pos_offset;
    const float* pi_k;
    const float* pi_v;
    const float* cb;             // centroids of widths 2, 3, 4, 8 back to back
    const int32_t* old_count;    // [5][nseg]
    int tile_base[ODMKV_NQ + 1]; // running sum of the levels' tile counts
    // Tiles handed from the fp16 kernel to this one: redo[0] / redo[1] = number of key / value tiles,
    // then redo_cap key tile numbers and redo_cap value tile numbers.  The fp16 kernel appends; with
    // from_list set the exact kernel walks the lists instead of all tiles.
    int32_t* redo;
    int redo_cap, from_list;
    odmkv_packed_t s;
};

typedef float f32x32 __attribute__((ext_vector_type(32)));

#define CODE_ROW 144      // K staging: LDS bytes per token row of codes (128 + padding, multiple of 16)
#define CODE_ROW_T 72     // V staging: LDS bytes per dim row of 64 token codes (64 + padding, multiple of 8)
#define QP_STAGE (TILE * CODE_ROW)
#define QP_PI_BYTES (HD * HD * 4)

// which segment owns `tile`: the largest bh with seg_tile[bh] <= tile
__device__ static inline int find_segment(const int32_t* seg_tile, int nseg, int tile) {
    int lo = 0, hi = nseg;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (seg_tile[mid] <= tile) lo = mid; else hi = mid;
    }
    return lo;
}

// token (0..63) that accumulator register vv of lane `lane` belongs to
__device__ static inline int mfma_token(int vv, int lane) {
    return (vv >> 4) * 32 + ((vv & 15) >> 2) * 8 + (lane >> 5) * 4 + (vv & 3);
}

// ---- nearest centroid through decision thresholds -------------------------------------------------
// The rule (quant.h: nearest_code) compares the distances to the two centroids that bracket y.  Both
// rounded distances are monotone in y between two neighbouring centroids, so for every boundary k
// there is one smallest float thr[k] from which on centroid k+1 wins, and
// code(y) = #{k : y >= thr[k]} reproduces the rule bit for bit.  The thresholds are found once per
// workgroup by bisection over the float bit patterns with the rule's own comparison.
__device__ static inline int float_key(float f) {            // monotone map float -> int
    const int b = __float_as_int(f);
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ static inline float key_float(int k) { return __int_as_float(k ^ ((k >> 31) & 0x7fffffff)); }

__device__ static inline float decision_threshold(float c_lo, float c_hi) {
    int lo = float_key(c_lo), hi = float_key(c_hi);          // rule false at c_lo, true at c_hi
    while (hi - lo > 1) {
        const int mid = lo + ((hi - lo) >> 1);
        const float y = key_float(mid);
        if (fabsf(y - c_hi) < fabsf(y - c_lo)) hi = mid; else lo = mid;
    }
    return key_float(hi);
}

// thresholds of width index li start at thr_offset(li): 3 + 7 + 15 + 255 floats
__device__ static inline int thr_offset(int li) { return li == 0 ? 0 : li == 1 ? 3 : li == 2 ? 10 : 25; }
#define QP_THR_FLOATS 280
#define QP_GROUP 32           // rotation steps whose matrix instructions are issued back to back

template <int W> struct Coder {
    static constexpr int K = 1 << W;
    float t[(W <= 3) ? K - 1 : 1];
    const float* thr;
    __device__ inline Coder(const float* thr_li) : thr(thr_li) {
        if constexpr (W <= 3) {
#pragma unroll
            for (int k = 0; k < K - 1; ++k) t[k] = thr_li[k];
        }
    }
    // r * 2^W + code(y): the code's bits are decided top down (each comparison picks the threshold of
    // the next one) and shifted into r one at a time, which the hardware does as r + r + carry
    __device__ __forceinline__ uint32_t push(uint32_t r, float y) const {
        if constexpr (W == 2) {
            const bool b1 = y >= t[1];
            r = r + r + (b1 ? 1u : 0u);
            const bool b0 = y >= (b1 ? t[2] : t[0]);
            return r + r + (b0 ? 1u : 0u);
        } else if constexpr (W == 3) {
            const bool b2 = y >= t[3];
            r = r + r + (b2 ? 1u : 0u);
            const bool b1 = y >= (b2 ? t[5] : t[1]);
            r = r + r + (b1 ? 1u : 0u);
            const float lo_pair = b1 ? t[2] : t[0], hi_pair = b1 ? t[6] : t[4];
            const bool b0 = y >= (b2 ? hi_pair : lo_pair);
            return r + r + (b0 ? 1u : 0u);
        } else {
            int pos = 0;                                     // #thresholds <= y, by binary search
#pragma unroll
            for (int s = K / 2; s >= 1; s >>= 1)
                if (y >= thr[pos + s - 1]) pos += s;
            return (r << W) | (uint32_t)pos;
        }
    }
    __device__ __forceinline__ uint32_t operator()(float y) const { return push(0u, y); }
};

template <int W>
__device__ static __forceinline__ void stage_codes_k(const f32x32& a0, const f32x32& a1, const f32x32& a2, const f32x32& a3,
                                            const float* thr, uint8_t* stage, int lane) {
    const Coder<W> code(thr);
    const int c = lane & 31;
#pragma unroll
    for (int vv = 0; vv < 32; ++vv) {
        const uint32_t w = code(a0[vv]) | (code(a1[vv]) << 8) | (code(a2[vv]) << 16) | (code(a3[vv]) << 24);
        *reinterpret_cast<uint32_t*>(stage + mfma_token(vv, lane) * CODE_ROW + 4 * c) = w;
    }
}

template <int W>
__device__ static __forceinline__ void stage_codes_v(const f32x32& acc, int g, const float* thr, uint8_t* stage, int lane) {
    const Coder<W> code(thr);
    const int c = lane & 31;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const uint32_t w = code(acc[4 * q]) | (code(acc[4 * q + 1]) << 8) | (code(acc[4 * q + 2]) << 16) |
                           (code(acc[4 * q + 3]) << 24);
        *reinterpret_cast<uint32_t*>(stage + (g * 32 + c) * CODE_ROW_T + mfma_token(4 * q, lane)) = w;
    }
}

// ---- direct packing (widths 2, 4, 8; tiles that start empty) -----------------------------------------
// The four outputs a lane holds for a token are neighbours in the token's code stream, and the four
// tokens it holds for a value dim are neighbours in the dim's stream: 4*W bits that go to the staging
// area already in their final bit order.  The second pass then only moves 16-byte pieces.
template <int W> struct Direct {
    static constexpr int GROUP_BYTES = W / 2;            // 4 codes
    static constexpr int ROW_K = 16 * W + 16;            // staging bytes per token (multiple of 16)
    static constexpr int ROW_V = 8 * W + 8;              // staging bytes per dim (multiple of 8)
};

template <int W>
__device__ static __forceinline__ void put_group(uint8_t* p, uint32_t bits) {
    if constexpr (W == 2) *p = (uint8_t)bits;
    else if constexpr (W == 4) *reinterpret_cast<uint16_t*>(p) = (uint16_t)bits;
    else *reinterpret_cast<uint32_t*>(p) = bits;
}

template <int W>
__device__ static __forceinline__ void stage_direct_k(const f32x32& a0, const f32x32& a1, const f32x32& a2, const f32x32& a3,
                                                      const float* thr, uint8_t* stage, int lane) {
    const Coder<W> code(thr);
    const int c = lane & 31;
#pragma unroll
    for (int vv = 0; vv < 32; ++vv) {
        const uint32_t bits = code.push(code.push(code.push(code.push(0u, a3[vv]), a2[vv]), a1[vv]), a0[vv]);
        put_group<W>(stage + mfma_token(vv, lane) * Direct<W>::ROW_K + c * Direct<W>::GROUP_BYTES, bits);
    }
}

// lane (n, j) gathers dims 32j..32j+31 of its four slots key_slot(n, 0..3) from the staged token streams
template <int W>
__device__ static __forceinline__ void store_direct_k(const uint8_t* stage, uint8_t* kcodes, int tile, int lane) {
    const int n = lane & 15, j = lane >> 4;
    uint32_t words[4 * W];
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int i = 0; i < W; ++i)
            words[b * W + i] = *reinterpret_cast<const uint32_t*>(stage + key_slot(n, b) * Direct<W>::ROW_K + 4 * W * j + 4 * i);
    uint8_t* dst = kcodes + (size_t)tile * (TILE * 16 * W);
#pragma unroll
    for (int ch = 0; ch < W; ++ch)
        *reinterpret_cast<uint4*>(dst + ((size_t)ch * TILE + lane) * 16) =
            make_uint4(words[4 * ch], words[4 * ch + 1], words[4 * ch + 2], words[4 * ch + 3]);
}

template <int W>
__device__ static __forceinline__ void stage_direct_v(const f32x32& acc, int g, const float* thr, uint8_t* stage, int lane) {
    const Coder<W> code(thr);
    const int c = lane & 31;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const uint32_t bits = code.push(code.push(code.push(code.push(0u, acc[4 * q + 3]), acc[4 * q + 2]), acc[4 * q + 1]), acc[4 * q]);
        put_group<W>(stage + (g * 32 + c) * Direct<W>::ROW_V + (mfma_token(4 * q, lane) >> 2) * Direct<W>::GROUP_BYTES, bits);
    }
}

// lane (n, j) gathers slots 32k+8j..+7 (k = 0, 1) of dims 16m+n (m = 0..7) from the staged dim streams:
// W bytes per (k, m)
template <int W>
__device__ static __forceinline__ void store_direct_v(const uint8_t* stage, uint8_t* vcodes, int tile, int lane) {
    const int n = lane & 15, j = lane >> 4;
    uint32_t words[4 * W];
#pragma unroll
    for (int i = 0; i < 4 * W; ++i) words[i] = 0u;
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const uint8_t* src = stage + (16 * m + n) * Direct<W>::ROW_V + (4 * k + j) * W;
            const int g = 8 * k + m;                                       // group of 8 codes = W bytes of the lane's stream
            if constexpr (W == 2) words[g >> 1] |= (uint32_t)(*reinterpret_cast<const uint16_t*>(src)) << (16 * (g & 1));
            else if constexpr (W == 4) words[g] = *reinterpret_cast<const uint32_t*>(src);
            else { const uint2 v = *reinterpret_cast<const uint2*>(src); words[2 * g] = v.x; words[2 * g + 1] = v.y; }
        }
    uint8_t* dst = vcodes + (size_t)tile * (TILE * 16 * W);
#pragma unroll
    for (int ch = 0; ch < W; ++ch)
        *reinterpret_cast<uint4*>(dst + ((size_t)ch * TILE + lane) * 16) =
            make_uint4(words[4 * ch], words[4 * ch + 1], words[4 * ch + 2], words[4 * ch + 3]);
}

// Generic stores (any width; tiles that already hold `lo` tokens keep them: KEEP).  Slots at and behind
// `hi` receive the codes of zero rows; they are not counted by anybody until a later call fills them.
template <int W, bool KEEP>
__device__ static __forceinline__ void pack_store_k(const uint8_t* stage, uint8_t* kcodes, int tile, int lane, int lo) {
    const int n = lane & 15, j = lane >> 4;
    uint8_t* dst = kcodes + (size_t)tile * (TILE * 16 * W);
    uint32_t words[4 * W];
#pragma unroll
    for (int k = 0; k < 4 * W; ++k) words[k] = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint4 v0 = *reinterpret_cast<const uint4*>(stage + key_slot(n, b) * CODE_ROW + 32 * j);
        const uint4 v1 = *reinterpret_cast<const uint4*>(stage + key_slot(n, b) * CODE_ROW + 32 * j + 16);
        const uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int e = 0; e < 32; ++e) put_code<W>(words, 32 * b + e, (w[e >> 2] >> (8 * (e & 3))) & 0xffu);
    }
    if constexpr (KEEP) {
        // a slot's codes are W whole words of the lane's stream
#pragma unroll
        for (int c = 0; c < W; ++c) {
            const uint4 old = *reinterpret_cast<const uint4*>(dst + ((size_t)c * TILE + lane) * 16);
            const uint32_t o[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int b = (4 * c + i) / W;
                if (key_slot(n, b) < lo) words[4 * c + i] = o[i];
            }
        }
    }
#pragma unroll
    for (int c = 0; c < W; ++c)
        *reinterpret_cast<uint4*>(dst + ((size_t)c * TILE + lane) * 16) =
            make_uint4(words[4 * c], words[4 * c + 1], words[4 * c + 2], words[4 * c + 3]);
}

template <int W, bool KEEP>
__device__ static __forceinline__ void pack_store_v(const uint8_t* stage, uint8_t* vcodes, int tile, int lane, int lo) {
    const int n = lane & 15, j = lane >> 4;
    uint8_t* dst = vcodes + (size_t)tile * (TILE * 16 * W);
    uint32_t old[4 * W];
    if constexpr (KEEP) {
#pragma unroll
        for (int c = 0; c < W; ++c) {
            const uint4 o = *reinterpret_cast<const uint4*>(dst + ((size_t)c * TILE + lane) * 16);
            old[4 * c] = o.x; old[4 * c + 1] = o.y; old[4 * c + 2] = o.z; old[4 * c + 3] = o.w;
        }
    }
    uint32_t words[4 * W];
#pragma unroll
    for (int k = 0; k < 4 * W; ++k) words[k] = 0;
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const uint2 v = *reinterpret_cast<const uint2*>(stage + (16 * m + n) * CODE_ROW_T + 32 * k + 8 * j);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ci = 64 * k + 8 * m + e;
                uint32_t c = ((e < 4 ? v.x : v.y) >> (8 * (e & 3))) & 0xffu;
                if constexpr (KEEP) c = (32 * k + 8 * j + e < lo) ? get_code<W>(old, ci) : c;     // stored earlier: keep
                put_code<W>(words, ci, c);
            }
        }
#pragma unroll
    for (int c = 0; c < W; ++c)
        *reinterpret_cast<uint4*>(dst + ((size_t)c * TILE + lane) * 16) =
            make_uint4(words[4 * c], words[4 * c + 1], words[4 * c + 2], words[4 * c + 3]);
}

// LDS writes of this wave visible to its own later reads (no other wave touches its staging area)
__device__ static inline void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// a row of 128 elements kept as loaded: fp32 as 128 floats, 16-bit types as 64 packed words
template <int DT> struct RowRegs {
    static constexpr int N = (DT == ODMKV_F32) ? HD : HD / 2;
    uint32_t w[N];
    __device__ inline void zero() {
#pragma unroll
        for (int i = 0; i < N; ++i) w[i] = 0;
    }
    __device__ inline void load(const void* base, size_t elem_off) {
        if constexpr (DT == ODMKV_F32) {
            const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(base) + elem_off);
#pragma unroll
            for (int c = 0; c < 32; ++c) { const uint4 v = p[c]; w[4 * c] = v.x; w[4 * c + 1] = v.y; w[4 * c + 2] = v.z; w[4 * c + 3] = v.w; }
        } else {
            const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + elem_off);
#pragma unroll
            for (int c = 0; c < 16; ++c) { const uint4 v = p[c]; w[4 * c] = v.x; w[4 * c + 1] = v.y; w[4 * c + 2] = v.z; w[4 * c + 3] = v.w; }
        }
    }
    __device__ inline float get(int j) const {
        if constexpr (DT == ODMKV_F32) return __uint_as_float(w[j]);
        else {
            // the conversion is one instruction; converting all 128 elements ahead of time and keeping
            // them (what the optimiser would do) costs 64 more registers than the packed words
            uint32_t word = w[j >> 1];
            asm volatile("" : "+v"(word));
            return Elem<DT>::to_f32((uint16_t)((j & 1) ? (word >> 16) : (word & 0xffffu)));
        }
    }
};

template <int DT, int NW>
__global__ __launch_bounds__(NW * 64) void quant_pack_kernel(QuantArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    float* piT = reinterpret_cast<float*>(smem);                                   // [j][slot]
    float* thrs = reinterpret_cast<float*>(smem + QP_PI_BYTES + NW * QP_STAGE);    // all widths
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);          // wave-uniform: keep it in a scalar register
    uint8_t* stage = smem + QP_PI_BYTES + wave * QP_STAGE;
    const bool is_v = (blockIdx.x & 1) != 0;
    const int32_t* tile_list = a.from_list ? a.redo + 2 + (is_v ? a.redo_cap : 0) : nullptr;
    const int n_work = a.from_list ? min(a.redo[is_v ? 1 : 0], a.redo_cap) : a.tile_base[ODMKV_NQ];
    if (n_work == 0) return;                                            // nothing handed over: the usual case

    // rotation -> LDS, transposed.  Keys: slot = output index.  Values: slot 4c+g holds output
    // g*32+c, so that a lane's four accumulators are 32 outputs apart and its registers hold four
    // consecutive tokens of one output (the dim-major order the V codes are stored in).
    {
        const float* __restrict__ pi = is_v ? a.pi_v : a.pi_k;
        for (int idx = tid; idx < HD * HD; idx += NW * 64) {
            const int i = idx >> 7, j = idx & 127;
            const int slot = is_v ? ((i & 31) * 4 + (i >> 5)) : i;
            piT[j * HD + slot] = pi[idx];
        }
        for (int i = tid; i < QP_THR_FLOATS; i += NW * 64) {
            const int li = i < 3 ? 0 : i < 10 ? 1 : i < 25 ? 2 : 3;
            const int k = i - thr_offset(li);
            thrs[i] = decision_threshold(a.cb[codebook_offset(li) + k], a.cb[codebook_offset(li) + k + 1]);
        }
    }
    __syncthreads();

    const int wg = blockIdx.x >> 1, n_wg = gridDim.x >> 1;
    for (int wi = wg * NW + wave; wi < n_work; wi += n_wg * NW) {
        const int gt = tile_list ? tile_list[wi] : wi;
        int li = 0;
#pragma unroll
        for (int k = 1; k < ODMKV_NQ; ++k) li += (gt >= a.tile_base[k]);
        const int tile = gt - a.tile_base[li];
        const int32_t* seg_tile = a.s.seg_tile[li];
        const int bh = find_segment(seg_tile, a.nseg, tile);
        const int ts = (tile - seg_tile[bh]) * TILE;
        const int lo = max(a.old_count[li * a.nseg + bh] - ts, 0);
        const int hi = min(a.s.seg_count[li][bh] - ts, TILE);
        if (lo >= hi) continue;                                 // nothing new in this tile (wave-uniform)

        const bool valid = lane >= lo && lane < hi;
        const size_t slot = (size_t)tile * TILE + lane;
        RowRegs<DT> x;
        if (valid) {
            const int t = a.s.pos[li][slot] - a.pos_offset;
            const size_t off = (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT;
            x.load(is_v ? a.V : a.K, off);
        } else {
            x.zero();
        }
        float ss = 0.0f, amin = INFINITY;                      // amin: smallest non-zero magnitude of the row
#pragma unroll
        for (int j = 0; j < HD; ++j) {
            const float xj = x.get(j);
            ss = __fmaf_rn(xj, xj, ss);
            if constexpr (DT != ODMKV_F16) {                   // fp16 inputs cannot get that small against their norm
                const float ax = fabsf(xj);
                amin = fminf(amin, ax == 0.0f ? INFINITY : ax);
            }
        }
        const float norm = sqrtf(ss);
        const float den = norm + 1e-10f;

        f32x32 acc0, acc1, acc2, acc3;
#pragma unroll
        for (int i = 0; i < 32; ++i) { acc0[i] = 0.0f; acc1[i] = 0.0f; acc2[i] = 0.0f; acc3[i] = 0.0f; }
        __builtin_amdgcn_s_setprio(0);
        const float4* __restrict__ brow = reinterpret_cast<const float4*>(piT) + (lane & 31);
        // u_j = x_j / den, correctly rounded.  With den in [2^-40, 2^60] and every non-zero |x_j| at
        // least den * 2^-60 the hardware division sequence never rescales its operands, so the part
        // of it that depends on den alone (reciprocal estimate and its refinement) is computed once
        // per row and five multiply-adds per element remain; the results are the same bits.  Rows
        // outside that range (any lane of the wave) take the plain division.
        const bool row_plain = !(den >= 9.094947017729282e-13f && den <= 1.152921504606847e18f &&
                                 amin >= den * 8.673617379884035e-19f);
        if (!__any(row_plain)) {
            const float r0 = __builtin_amdgcn_rcpf(den);
            const float rr = __fmaf_rn(__fmaf_rn(-den, r0, 1.0f), r0, r0);
            const float nden = -den;
            // Issue order is pinned.  A vector instruction between two matrix instructions of one
            // wave costs the matrix pipe about 13 idle clocks (a later one 4 more each) and never
            // runs in its shadow, while an LDS read costs about one; so the quotients of QP_GROUP
            // steps are computed in one block, and the matrix instructions of those steps then go
            // back to back with only the LDS reads of the rotation between them.
            const auto quotient = [&](int j) {
                const float n = x.get(j);
                const float q0 = __fmul_rn(n, rr);
                const float q1 = __fmaf_rn(__fmaf_rn(nden, q0, n), rr, q0);
                return __fmaf_rn(__fmaf_rn(nden, q1, n), rr, q1);
            };
            float4 b = brow[0];
#pragma unroll
            for (int j0 = 0; j0 < HD; j0 += QP_GROUP) {
                float u[QP_GROUP];
#pragma unroll
                for (int g = 0; g < QP_GROUP; ++g) u[g] = quotient(j0 + g);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int g = 0; g < QP_GROUP; ++g) {
                    const int jn = j0 + g + 1 < HD ? j0 + g + 1 : j0 + g;
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(u[g], b.x, acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(u[g], b.y, acc1, 0, 0, 0);
                    acc2 = __builtin_amdgcn_mfma_f32_32x32x1f32(u[g], b.z, acc2, 0, 0, 0);
                    acc3 = __builtin_amdgcn_mfma_f32_32x32x1f32(u[g], b.w, acc3, 0, 0, 0);
                    b = brow[jn * (HD / 4)];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < HD; ++j) {
                const float u = x.get(j) / den;
                const float4 b = brow[j * (HD / 4)];
                acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(u, b.x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(u, b.y, acc1, 0, 0, 0);
                acc2 = __builtin_amdgcn_mfma_f32_32x32x1f32(u, b.z, acc2, 0, 0, 0);
                acc3 = __builtin_amdgcn_mfma_f32_32x32x1f32(u, b.w, acc3, 0, 0, 0);
            }
        }

        const float* cb = thrs + thr_offset(li);
        // the lane index as the coding phase sees it: opaque to the compiler, so that the staging and
        // store addresses are computed here and not carried (spilled) across the rotation loop
        int ln = lane;
        asm volatile("" : "+v"(ln));
        // while one wave of a SIMD streams matrix instructions (it needs one issue slot in 64 clocks),
        // the other's vector and memory instructions are the ones that must not wait
        __builtin_amdgcn_s_setprio(3);
        // widths 2, 4, 8; keys into a tile that starts empty, values into a tile this call fills whole
        const bool direct = li != 1 && lo == 0 && (!is_v || hi == TILE);
        if (!is_v) {
            if (direct) {
                switch (li) {
                    case 0: stage_direct_k<2>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                    case 2: stage_direct_k<4>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                    default: stage_direct_k<8>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                }
            } else {
                switch (li) {
                    case 0: stage_codes_k<2>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                    case 1: stage_codes_k<3>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                    case 2: stage_codes_k<4>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                    default: stage_codes_k<8>(acc0, acc1, acc2, acc3, cb, stage, ln); break;
                }
            }
            wave_lds_fence();
            if (direct) {
                switch (li) {
                    case 0: store_direct_k<2>(stage, a.s.kcodes[0], tile, ln); break;
                    case 2: store_direct_k<4>(stage, a.s.kcodes[2], tile, ln); break;
                    default: store_direct_k<8>(stage, a.s.kcodes[3], tile, ln); break;
                }
            } else if (lo > 0) {
                switch (li) {
                    case 0: pack_store_k<2, true>(stage, a.s.kcodes[0], tile, ln, lo); break;
                    case 1: pack_store_k<3, true>(stage, a.s.kcodes[1], tile, ln, lo); break;
                    case 2: pack_store_k<4, true>(stage, a.s.kcodes[2], tile, ln, lo); break;
                    default: pack_store_k<8, true>(stage, a.s.kcodes[3], tile, ln, lo); break;
                }
            } else {
                switch (li) {
                    case 0: pack_store_k<2, false>(stage, a.s.kcodes[0], tile, ln, 0); break;
                    case 1: pack_store_k<3, false>(stage, a.s.kcodes[1], tile, ln, 0); break;
                    case 2: pack_store_k<4, false>(stage, a.s.kcodes[2], tile, ln, 0); break;
                    default: pack_store_k<8, false>(stage, a.s.kcodes[3], tile, ln, 0); break;
                }
            }
            if (valid) a.s.knorm[li][slot] = norm;
        } else {
            if (direct) {
                switch (li) {
                    case 0: stage_direct_v<2>(acc0, 0, cb, stage, ln); stage_direct_v<2>(acc1, 1, cb, stage, ln);
                            stage_direct_v<2>(acc2, 2, cb, stage, ln); stage_direct_v<2>(acc3, 3, cb, stage, ln); break;
                    case 2: stage_direct_v<4>(acc0, 0, cb, stage, ln); stage_direct_v<4>(acc1, 1, cb, stage, ln);
                            stage_direct_v<4>(acc2, 2, cb, stage, ln); stage_direct_v<4>(acc3, 3, cb, stage, ln); break;
                    default: stage_direct_v<8>(acc0, 0, cb, stage, ln); stage_direct_v<8>(acc1, 1, cb, stage, ln);
                             stage_direct_v<8>(acc2, 2, cb, stage, ln); stage_direct_v<8>(acc3, 3, cb, stage, ln); break;
                }
                wave_lds_fence();
                switch (li) {
                    case 0: store_direct_v<2>(stage, a.s.vcodes[0], tile, ln); break;
                    case 2: store_direct_v<4>(stage, a.s.vcodes[2], tile, ln); break;
                    default: store_direct_v<8>(stage, a.s.vcodes[3], tile, ln); break;
                }
            } else {
                switch (li) {
                    case 0: stage_codes_v<2>(acc0, 0, cb, stage, ln); stage_codes_v<2>(acc1, 1, cb, stage, ln);
                            stage_codes_v<2>(acc2, 2, cb, stage, ln); stage_codes_v<2>(acc3, 3, cb, stage, ln); break;
                    case 1: stage_codes_v<3>(acc0, 0, cb, stage, ln); stage_codes_v<3>(acc1, 1, cb, stage, ln);
                            stage_codes_v<3>(acc2, 2, cb, stage, ln); stage_codes_v<3>(acc3, 3, cb, stage, ln); break;
                    case 2: stage_codes_v<4>(acc0, 0, cb, stage, ln); stage_codes_v<4>(acc1, 1, cb, stage, ln);
                            stage_codes_v<4>(acc2, 2, cb, stage, ln); stage_codes_v<4>(acc3, 3, cb, stage, ln); break;
                    default: stage_codes_v<8>(acc0, 0, cb, stage, ln); stage_codes_v<8>(acc1, 1, cb, stage, ln);
                             stage_codes_v<8>(acc2, 2, cb, stage, ln); stage_codes_v<8>(acc3, 3, cb, stage, ln); break;
                }
                wave_lds_fence();
                if (lo > 0) {
                    switch (li) {
                        case 0: pack_store_v<2, true>(stage, a.s.vcodes[0], tile, ln, lo); break;
                        case 1: pack_store_v<3, true>(stage, a.s.vcodes[1], tile, ln, lo); break;
                        case 2: pack_store_v<4, true>(stage, a.s.vcodes[2], tile, ln, lo); break;
                        default: pack_store_v<8, true>(stage, a.s.vcodes[3], tile, ln, lo); break;
                    }
                } else {
                    switch (li) {
                        case 0: pack_store_v<2, false>(stage, a.s.vcodes[0], tile, ln, 0); break;
                        case 1: pack_store_v<3, false>(stage, a.s.vcodes[1], tile, ln, 0); break;
                        case 2: pack_store_v<4, false>(stage, a.s.vcodes[2], tile, ln, 0); break;
                        default: pack_store_v<8, false>(stage, a.s.vcodes[3], tile, ln, 0); break;
                    }
                }
            }
            if (valid) a.s.vnorm[li][slot] = norm;
        }
        wave_lds_fence();                                       // staging area free for the next tile
    }
}

// ------------------------------------------------------------------------------------------------
// quantise + pack, fp16 and bf16 inputs: rotation on the 16-bit matrix cores, exact codes through a guard band
//
// A code is the number of decision thresholds at or below y = sum_j u_j Pi[i][j] (summed in the
// sequential fp32 order of the definition).  The chain of 128 dependent fp32 steps is what the exact
// kernel above spends its time on, yet the chain's last bits matter only when y lies next to a
// threshold.  So y is first computed fast: the fp16 row as it is, against Pi split into two fp16
// terms (hi + lo, 22 bits), on v_mfma_f32_16x16x32_f16, then scaled by 1 / (|x| + 1e-10).  That
// estimate differs from the chain's result by rounding alone: at most about 2.5e-5 on the scale
// |y| <= 1 under the most pessimistic model of the matrix unit's adder (every one of the 128 terms
// truncated at the scale of the largest partial sum); measured, a band of 1e-7 already leaves no code
// different over 1e8 values.  Values farther than QF_BAND (twice that bound) from every threshold therefore have the chain's code already; the few within the band
// (two to eight in a thousand) are listed, and whenever a wave has 64 of them it recomputes them by
// the chain itself, one lane per value, and replaces their codes in the packed tiles it has already
// written.  Rows of zeros are exact either way.
// Tiles the scheme does not cover go to the exact kernel through a list: 8-bit tiles (a tenth of
// their values lie inside the band), tiles with a row whose squared norm is not finite, and tiles
// with more listed values than the list has room for.
//
// Operands: for keys D = Pi (rows) x tokens (columns), so a lane ends with four consecutive outputs
// of one token; for values the same registers with the operands swapped give D = tokens x outputs
// and four consecutive tokens of one output: in both cases the 4*W bits that are neighbours in the
// packed stream, as the staging formats of the exact kernel expect them.
// ------------------------------------------------------------------------------------------------
typedef _Float16 qf_h8 __attribute__((ext_vector_type(8)));
typedef __bf16 qf_b8 __attribute__((ext_vector_type(8)));
typedef float qf_f4 __attribute__((ext_vector_type(4)));

#ifndef QF_BAND
#define QF_BAND 5.0e-5f
#endif
// bf16 rows meet Pi as two bf16 terms (16 bits: up to 7.6e-6 more on the estimate, by Cauchy-Schwarz over the row)
#define QF_BAND_BF16 7.0e-5f

// D += A x B on the matrix cores of the rows' own 16-bit type (operands as they sit in four 32-bit registers)
template <int DT>
__device__ static __forceinline__ qf_f4 qf_mfma(const uint4& a, const uint4& b, const qf_f4& c) {
    if constexpr (DT == ODMKV_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qf_h8, a), __builtin_bit_cast(qf_h8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(qf_b8, a), __builtin_bit_cast(qf_b8, b), c, 0, 0, 0);
}
#define QF_LIST 256                     // listed values a wave can hold (it works them off 64 at a time)
#define QF_GT_BITS 19                   // tile numbers in a list entry
#define QF_NW 8
#define QF_PI_BYTES (2 * HD * HD * 2)   // Pi as fp16 hi and lo, in matrix-operand order
#define QF_THR_BYTES 1152               // QP_THR_FLOATS floats, padded to a multiple of 16

struct QfWave {                          // per-wave scratch in LDS
    unsigned long long off[TILE];        // element offset of the token's row (~0: no row, zeros)
    float den[TILE], rinv[TILE], band[TILE];
    uint32_t list[QF_LIST];              // slot in the tile | output << 6 | tile number << 13
    int count, pad[3];
};

template <int W> struct GuardCoder {
    static constexpr int K = 1 << W;
    float t[(W <= 3) ? K - 1 : 1];
    const float* thr;
    __device__ inline GuardCoder(const float* thr_li) : thr(thr_li) {
        if constexpr (W <= 3) {
#pragma unroll
            for (int k = 0; k < K - 1; ++k) t[k] = thr_li[k];
        }
    }
    // r * 2^W + code(y), and m = distance from y to the nearest threshold: the binary search meets
    // both neighbours of y on its way, so the minimum over the thresholds it compares with is exact
    __device__ __forceinline__ uint32_t push(uint32_t r, float y, float& m) const {
        if constexpr (W == 2) {
            const bool b1 = y >= t[1];
            r = r + r + (b1 ? 1u : 0u);
            const float ts = b1 ? t[2] : t[0];
            const bool b0 = y >= ts;
            m = fminf(fabsf(y - t[1]), fabsf(y - ts));
            return r + r + (b0 ? 1u : 0u);
        } else if constexpr (W == 3) {
            const bool b2 = y >= t[3];
            r = r + r + (b2 ? 1u : 0u);
            const float ta = b2 ? t[5] : t[1];
            const bool b1 = y >= ta;
            r = r + r + (b1 ? 1u : 0u);
            const float lo_pair = b1 ? t[2] : t[0], hi_pair = b1 ? t[6] : t[4];
            const float tb = b2 ? hi_pair : lo_pair;
            const bool b0 = y >= tb;
            m = fminf(fminf(fabsf(y - t[3]), fabsf(y - ta)), fabsf(y - tb));
            return r + r + (b0 ? 1u : 0u);
        } else {
            int pos = 0;
            m = INFINITY;
#pragma unroll
            for (int s = K / 2; s >= 1; s >>= 1) {
                const float tv = thr[pos + s - 1];
                m = fminf(m, fabsf(y - tv));
                if (y >= tv) pos += s;
            }
            return (r << W) | (uint32_t)pos;
        }
    }
};

// rotation estimate -> codes into the staging area; values inside the band -> the wave's list
template <int DT, int W, bool IS_V, bool DIRECT>
__device__ static __forceinline__ void qf_code_tile(const void* base, const uint4* piA, const float* thr, QfWave& w,
                                                    uint8_t* stage, int lane, int gt) {
    const int r16 = lane & 15, q = lane >> 4;
    const GuardCoder<W> code(thr);
    constexpr int NT = IS_V ? 16 : 4;
    float rinv[NT], band[NT];
    uint4 xb[4][4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
        if constexpr (IS_V) {
            const float4 ri = *reinterpret_cast<const float4*>(&w.rinv[16 * tb + 4 * q]);
            const float4 bd = *reinterpret_cast<const float4*>(&w.band[16 * tb + 4 * q]);
            rinv[4 * tb] = ri.x; rinv[4 * tb + 1] = ri.y; rinv[4 * tb + 2] = ri.z; rinv[4 * tb + 3] = ri.w;
            band[4 * tb] = bd.x; band[4 * tb + 1] = bd.y; band[4 * tb + 2] = bd.z; band[4 * tb + 3] = bd.w;
        } else {
            rinv[tb] = w.rinv[16 * tb + r16];
            band[tb] = w.band[16 * tb + r16];
        }
        const unsigned long long o = w.off[16 * tb + r16];
        const uint4* row = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + (o == ~0ull ? 0ull : o)) + q;
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) xb[tb][ch] = (o == ~0ull) ? make_uint4(0u, 0u, 0u, 0u) : row[4 * ch];
    }
#pragma unroll 1
    for (int k = 0; k < 4; ++k) {
        uint32_t f = 0u;                                        // band flags of this pair of output blocks, first value on top
#pragma unroll
        for (int o2 = 0; o2 < 2; ++o2) {
            const int ob = 2 * k + o2;
            qf_f4 acc[4];
#pragma unroll
            for (int tb = 0; tb < 4; ++tb) acc[tb] = (qf_f4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) {
                const uint4 ah = piA[(ob * 4 + ch) * 64 + lane];
                const uint4 al = piA[HD * HD / 8 + (ob * 4 + ch) * 64 + lane];
#pragma unroll
                for (int tb = 0; tb < 4; ++tb) {
                    if constexpr (IS_V) {
                        acc[tb] = qf_mfma<DT>(xb[tb][ch], ah, acc[tb]);
                        acc[tb] = qf_mfma<DT>(xb[tb][ch], al, acc[tb]);
                    } else {
                        acc[tb] = qf_mfma<DT>(ah, xb[tb][ch], acc[tb]);
                        acc[tb] = qf_mfma<DT>(al, xb[tb][ch], acc[tb]);
                    }
                }
            }
#pragma unroll
            for (int tb = 0; tb < 4; ++tb) {
                uint32_t g = 0u;
#pragma unroll
                for (int r = 3; r >= 0; --r) {
                    const float y = acc[tb][r] * (IS_V ? rinv[4 * tb + r] : rinv[tb]);
                    float m;
                    if constexpr (DIRECT) g = code.push(g, y, m);
                    else g = (g << 8) | code.push(0u, y, m);
                    const bool near = m < (IS_V ? band[4 * tb + r] : band[tb]);
                    f = f + f + (near ? 1u : 0u);
                }
                if constexpr (!IS_V) {
                    const int token = 16 * tb + r16, grp = 4 * ob + q;
                    if constexpr (DIRECT) put_group<W>(stage + token * Direct<W>::ROW_K + grp * Direct<W>::GROUP_BYTES, g);
                    else *reinterpret_cast<uint32_t*>(stage + token * CODE_ROW + 4 * grp) = g;
                } else {
                    const int dim = 16 * ob + r16, tg = 4 * tb + q;
                    if constexpr (DIRECT) put_group<W>(stage + dim * Direct<W>::ROW_V + tg * Direct<W>::GROUP_BYTES, g);
                    else *reinterpret_cast<uint32_t*>(stage + dim * CODE_ROW_T + 4 * tg) = g;
                }
            }
        }
        while (f) {                                             // rare: a few values per lane and tile
            const int b = 31 - __clz(f);
            f &= ~(1u << b);
            const int v = 31 - b;                               // v = o2*16 + tb*4 + (3 - r)
            const int ob = 2 * k + (v >> 4), tb = (v >> 2) & 3, r = 3 - (v & 3);
            const int token = IS_V ? 16 * tb + 4 * q + r : 16 * tb + r16;
            const int out = IS_V ? 16 * ob + r16 : 16 * ob + 4 * q + r;
            const int idx = atomicAdd(&w.count, 1);
            if (idx < QF_LIST) w.list[idx] = (uint32_t)token | ((uint32_t)out << 6) | ((uint32_t)gt << 13);
        }
    }
}

// Entries first .. first + n - 1 of the wave's list (n <= 64), a lane each: the value by the definition's
// own chain, its code, and that code in place of the estimate's in the packed tile.  The tile's codes,
// positions and norms were written by this wave: the caller has waited for those stores.
template <int DT, bool IS_V>
__device__ static void qf_fix_listed(const QuantArgs& a, const float* thrs, const QfWave& w, int lane, int first, int n) {
    const bool on = lane < n;
    const uint32_t e = w.list[first + (on ? lane : 0)];
    const int token = e & 63, out = (e >> 6) & 127, gt = (int)(e >> 13);
    int li = 0;
#pragma unroll
    for (int k = 1; k < ODMKV_NQ; ++k) li += (gt >= a.tile_base[k]);
    const int tile = gt - a.tile_base[li];
    const int bh = find_segment(a.s.seg_tile[li], a.nseg, tile);
    const size_t slot = (size_t)tile * TILE + token;
    const size_t off = (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH +
                       (size_t)(a.s.pos[li][slot] - a.pos_offset) * a.sT;
    // written by this wave a moment ago: read past the vector cache
    const float den = __hip_atomic_load((IS_V ? a.s.vnorm[li] : a.s.knorm[li]) + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1e-10f;
    RowRegs<DT> x;
    x.load(IS_V ? a.V : a.K, off);
    const float4* __restrict__ prow = reinterpret_cast<const float4*>((IS_V ? a.pi_v : a.pi_k) + out * HD);
    float y = 0.0f;
    bool row_plain = !(den >= 9.094947017729282e-13f && den <= 1.152921504606847e18f);
    if constexpr (DT != ODMKV_F16) {                            // fp16 elements cannot get that small against their norm
        float amin = INFINITY;
#pragma unroll
        for (int j = 0; j < HD; ++j) {
            const float ax = fabsf(x.get(j));
            amin = fminf(amin, ax == 0.0f ? INFINITY : ax);
        }
        row_plain = row_plain || !(amin >= den * 8.673617379884035e-19f);
    }
    if (!__any(row_plain)) {                                    // same quotient sequence as the exact kernel
        const float r0 = __builtin_amdgcn_rcpf(den);
        const float rr = __fmaf_rn(__fmaf_rn(-den, r0, 1.0f), r0, r0);
        const float nden = -den;
#pragma unroll
        for (int c = 0; c < HD / 4; ++c) {
            const float4 p = prow[c];
            const float pv[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const float nv = x.get(4 * c + e4);
                const float q0 = __fmul_rn(nv, rr);
                const float q1 = __fmaf_rn(__fmaf_rn(nden, q0, nv), rr, q0);
                const float u = __fmaf_rn(__fmaf_rn(nden, q1, nv), rr, q1);
                y = __fmaf_rn(u, pv[e4], y);
            }
        }
    } else {
#pragma unroll
        for (int c = 0; c < HD / 4; ++c) {
            const float4 p = prow[c];
            const float pv[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) y = __fmaf_rn(x.get(4 * c + e4) / den, pv[e4], y);
        }
    }
    // code = number of thresholds at or below y; the entries of a pass may be of different widths
    const int W = width_of(li);
    const float* thr = thrs + thr_offset(li);
    int code = 0;
#pragma unroll
    for (int st = 8; st >= 1; st >>= 1)
        if (st < (1 << W) && y >= thr[code + st - 1]) code += st;
    if (!on) return;
    // where the code lives (quant.h: tile layouts): lane l of the tile, code number ci of its stream
    int l, ci;
    if constexpr (!IS_V) {
        const int b = 2 * (token >> 5) + (token & 1), nn = 4 * ((token >> 3) & 3) + ((token >> 1) & 3);   // token = key_slot(nn, b)
        l = 16 * (out >> 5) + nn;
        ci = 32 * b + (out & 31);
    } else {
        l = 16 * ((token >> 3) & 3) + (out & 15);
        ci = 64 * (token >> 5) + 8 * (out >> 4) + (token & 7);
    }
    uint8_t* tile_codes = (IS_V ? a.s.vcodes[li] : a.s.kcodes[li]) + (size_t)tile * (TILE * 16 * W);
    const int bit = ci * W, k = bit >> 5, sh = bit & 31;
    uint32_t* word = reinterpret_cast<uint32_t*>(tile_codes + ((size_t)(k >> 2) * TILE + l) * 16) + (k & 3);
    const uint32_t mask = (1u << W) - 1u;
    uint32_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> sh;
    uint32_t* word2 = nullptr;
    if (sh + W > 32) {                                          // a 3-bit code across two words of the stream
        const int k2 = k + 1;
        word2 = reinterpret_cast<uint32_t*>(tile_codes + ((size_t)(k2 >> 2) * TILE + l) * 16) + (k2 & 3);
        old |= __hip_atomic_load(word2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) << (32 - sh);
    }
    const uint32_t diff = (old & mask) ^ (uint32_t)code;
    if (diff) {
        atomicXor(word, diff << sh);                            // other lanes may change other codes of the same word
        if (word2) atomicXor(word2, diff >> (32 - sh));
    }
}

// the staged codes packed into the store
template <int W, bool IS_V, bool DIRECT>
__device__ static __forceinline__ void qf_store_tile(const QuantArgs& a, const uint8_t* stage, int lane, int li, int tile, int lo) {
    uint8_t* codes = IS_V ? a.s.vcodes[li] : a.s.kcodes[li];
    if constexpr (!IS_V) {
        if constexpr (DIRECT) store_direct_k<W>(stage, codes, tile, lane);
        else if (lo > 0) pack_store_k<W, true>(stage, codes, tile, lane, lo);
        else pack_store_k<W, false>(stage, codes, tile, lane, 0);
    } else {
        if constexpr (DIRECT) store_direct_v<W>(stage, codes, tile, lane);
        else if (lo > 0) pack_store_v<W, true>(stage, codes, tile, lane, lo);
        else pack_store_v<W, false>(stage, codes, tile, lane, 0);
    }
}

struct QfTile { int wi, gt, li, tile, bh, lo, hi; };
#define QF_MAX_RUNS 1024                // (level, segment) pairs whose tile counts fit the walk table

// Per wave: the next tile and the positions of its tokens are looked up while the current tile's rows are on
// their way.  (Requesting the next tile's rows a whole tile ahead was measured: no faster, and its 64 registers
// per lane are the ones the kernel does not have.)
template <int DT, bool IS_V>
__device__ static void qf_walk(const QuantArgs& a, const uint4* piA, const float* thrs, QfWave& w, uint8_t* stage,
                               int lane, int wave, const int* wbase) {
    // wbase (LDS, or null): running count, over the (level, segment) pairs, of the tiles that receive tokens in this
    // call.  The waves then share out those tiles alone; a store laid out for the worst case, or one that already
    // holds a long context, has many times more tiles than that.  Without the table every tile is looked at.
    const int n_runs = ODMKV_NQ * a.nseg;
    const int total_tiles = wbase ? wbase[n_runs] : a.tile_base[ODMKV_NQ];
    const int stride = (gridDim.x >> 1) * QF_NW;
    int32_t* redo_count = a.redo + (IS_V ? 1 : 0);
    int32_t* redo_list = a.redo + 2 + (IS_V ? a.redo_cap : 0);
    const void* base = IS_V ? a.V : a.K;
    const auto hand_over = [&](int gt) {
        if (lane == 0) {
            const int k = atomicAdd(redo_count, 1);
            if (k < a.redo_cap) redo_list[k] = gt;
        }
    };
    // the next tile at or behind gt with new tokens of widths 2, 3, 4; 8-bit tiles on the way are handed over
    const auto next_tile = [&](int wi, QfTile& d) -> bool {
        for (; wi < total_tiles; wi += stride) {
            int li, bh, tile, lo, hi;
            if (wbase) {
                int e = 0;                                       // the largest pair with wbase[e] <= wi
                for (int step = QF_MAX_RUNS / 2; step >= 1; step >>= 1)
                    if (e + step < n_runs && wbase[e + step] <= wi) e += step;
                li = e / a.nseg; bh = e - li * a.nseg;
                const int old = a.old_count[e];
                const int local = old / TILE + (wi - wbase[e]);
                tile = a.s.seg_tile[li][bh] + local;
                lo = max(old - local * TILE, 0);
                hi = min(a.s.seg_count[li][bh] - local * TILE, TILE);
            } else {
                li = 0;
#pragma unroll
                for (int k = 1; k < ODMKV_NQ; ++k) li += (wi >= a.tile_base[k]);
                tile = wi - a.tile_base[li];
                const int32_t* seg_tile = a.s.seg_tile[li];
                bh = find_segment(seg_tile, a.nseg, tile);
                const int ts = (tile - seg_tile[bh]) * TILE;
                lo = max(a.old_count[li * a.nseg + bh] - ts, 0);
                hi = min(a.s.seg_count[li][bh] - ts, TILE);
                if (lo >= hi) continue;                         // nothing new in this tile (wave-uniform)
            }
            const int gt = a.tile_base[li] + tile;
            if (li == 3) { hand_over(gt); continue; }
            d.wi = wi; d.gt = gt; d.li = li; d.tile = tile; d.bh = bh; d.lo = lo; d.hi = hi;
            return true;
        }
        return false;
    };
    const auto row_offset = [&](const QfTile& d, int pos) {
        return (size_t)(d.bh / a.Hkv) * a.sB + (size_t)(d.bh % a.Hkv) * a.sH + (size_t)(pos - a.pos_offset) * a.sT;
    };

    QfTile cur;
    bool more = next_tile((blockIdx.x >> 1) * QF_NW + wave, cur);
    if (!more) return;
    int n_listed = 0;                                           // == w.count between tiles
    if (lane == 0) w.count = 0;
    int pos = 0;
    if (lane >= cur.lo && lane < cur.hi) pos = a.s.pos[cur.li][(size_t)cur.tile * TILE + lane];
    while (true) {
        const bool valid = lane >= cur.lo && lane < cur.hi;
        size_t off = 0;
        RowRegs<DT> x;
        if (valid) {
            off = row_offset(cur, pos);
            x.load(base, off);
        } else {
            x.zero();
        }
        // the next tile and its positions are found while this tile's rows are on their way
        QfTile nxt;
        more = next_tile(cur.wi + stride, nxt);
        if (more && lane >= nxt.lo && lane < nxt.hi) pos = a.s.pos[nxt.li][(size_t)nxt.tile * TILE + lane];

        // a token per lane: the norm in the definition's order, and what the matrix layout needs per token
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < HD; ++j) {
            const float xj = x.get(j);
            ss = __fmaf_rn(xj, xj, ss);
        }
        const float norm = sqrtf(ss);
        bool odd = !(ss <= 3.4028234663852886e38f);              // a row with an infinite or NaN norm: exact kernel
        if constexpr (DT != ODMKV_F16) {
            // bf16 reaches down to 1e-38: a row whose squares vanish or nearly do (but which is not all zeros) also goes there
            uint32_t any = 0u;
#pragma unroll
            for (int i = 0; i < RowRegs<DT>::N; ++i) any |= x.w[i];
            odd = odd || ((any & 0x7fff7fffu) != 0u && ss < 1e-30f);
        }
        const bool ok = !__any(odd);
        const float* thr = thrs + thr_offset(cur.li);
        const bool direct = cur.li != 1 && cur.lo == 0 && (!IS_V || cur.hi == TILE);
        const int variant = cur.li == 0 ? (direct ? 0 : 1) : cur.li == 1 ? 2 : (direct ? 3 : 4);
        const int n_before = n_listed;
        int n = 0;
        if (ok) {
            const float den = norm + 1e-10f;
            w.off[lane] = valid ? (unsigned long long)off : ~0ull;
            w.den[lane] = den;
            w.rinv[lane] = 1.0f / den;
            w.band[lane] = (valid && ss > 0.0f) ? (DT == ODMKV_F16 ? QF_BAND : QF_BAND_BF16) : -1.0f;  // rows of zeros: the estimate is the exact 0
            wave_lds_fence();
            switch (variant) {
                case 0: qf_code_tile<DT, 2, IS_V, true>(base, piA, thr, w, stage, lane, cur.gt); break;
                case 1: qf_code_tile<DT, 2, IS_V, false>(base, piA, thr, w, stage, lane, cur.gt); break;
                case 2: qf_code_tile<DT, 3, IS_V, false>(base, piA, thr, w, stage, lane, cur.gt); break;
                case 3: qf_code_tile<DT, 4, IS_V, true>(base, piA, thr, w, stage, lane, cur.gt); break;
                default: qf_code_tile<DT, 4, IS_V, false>(base, piA, thr, w, stage, lane, cur.gt); break;
            }
            wave_lds_fence();
            n = w.count;
        }
        if (ok && n <= QF_LIST) {
            switch (variant) {
                case 0: qf_store_tile<2, IS_V, true>(a, stage, lane, cur.li, cur.tile, cur.lo); break;
                case 1: qf_store_tile<2, IS_V, false>(a, stage, lane, cur.li, cur.tile, cur.lo); break;
                case 2: qf_store_tile<3, IS_V, false>(a, stage, lane, cur.li, cur.tile, cur.lo); break;
                case 3: qf_store_tile<4, IS_V, true>(a, stage, lane, cur.li, cur.tile, cur.lo); break;
                default: qf_store_tile<4, IS_V, false>(a, stage, lane, cur.li, cur.tile, cur.lo); break;
            }
            if (valid) (IS_V ? a.s.vnorm[cur.li] : a.s.knorm[cur.li])[(size_t)cur.tile * TILE + lane] = norm;
            n_listed = n;
        } else {
            // a row the estimate does not cover, or more listed values than there was room for: the exact
            // kernel does the whole tile (what the list got of it is dropped)
            hand_over(cur.gt);
            n_listed = n_before;
            if (ok && lane == 0) w.count = n_before;
        }
        wave_lds_fence();                                       // staging area and scratch free for the next tile
        if (n_listed >= WAVE || (!more && n_listed > 0)) {
            __builtin_amdgcn_s_waitcnt(0);                      // this wave's codes, positions and norms are in memory
            while (n_listed >= WAVE) {
                n_listed -= WAVE;
                qf_fix_listed<DT, IS_V>(a, thrs, w, lane, n_listed, WAVE);
            }
            if (!more && n_listed > 0) { qf_fix_listed<DT, IS_V>(a, thrs, w, lane, 0, n_listed); n_listed = 0; }
            if (lane == 0) w.count = n_listed;
            wave_lds_fence();
        }
        if (!more) break;
        cur = nxt;
    }
}

template <int DT>
__global__ __launch_bounds__(QF_NW * 64) void quant_pack_f16_kernel(QuantArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    uint16_t* pih = reinterpret_cast<uint16_t*>(smem);
    float* thrs = reinterpret_cast<float*>(smem + QF_PI_BYTES + QF_NW * QP_STAGE);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t* stage = smem + QF_PI_BYTES + wave * QP_STAGE;
    QfWave& w = reinterpret_cast<QfWave*>(smem + QF_PI_BYTES + QF_NW * QP_STAGE + QF_THR_BYTES)[wave];
    int* wbase = reinterpret_cast<int*>(smem + QF_PI_BYTES + QF_NW * QP_STAGE + QF_THR_BYTES + QF_NW * sizeof(QfWave));
    const bool is_v = (blockIdx.x & 1) != 0;
    const int n_runs = ODMKV_NQ * a.nseg;
    const bool walk_table = n_runs <= QF_MAX_RUNS;
    if (walk_table) {
        // tiles of every (level, segment) pair that receive tokens: behind the tiles filled before, up to the new count
        for (int e = tid; e < QF_MAX_RUNS; e += QF_NW * 64) {
            int n = 0;
            if (e < n_runs) {
                const int old = a.old_count[e], cnt = a.s.seg_count[e / a.nseg][e % a.nseg];
                n = cnt > old ? (cnt + TILE - 1) / TILE - old / TILE : 0;
            }
            wbase[e + 1] = n;
        }
    }
    {
        // Pi -> hi + lo in the rows' 16-bit type, in the order the matrix instruction reads a 16-output x 32-step block:
        // lane 16q + r of block (ob, ch) holds Pi[16 ob + r][32 ch + 8 q .. + 7]
        // (all of a thread's reads are asked for at once: eight round trips to memory would cost more
        // than the tiles of a short call)
        const float4* __restrict__ pi4 = reinterpret_cast<const float4*>(is_v ? a.pi_v : a.pi_k);
        constexpr int PER_THREAD = HD * HD / 4 / (QF_NW * 64);
        float4 p[PER_THREAD];
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) p[k] = pi4[tid + k * (QF_NW * 64)];
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) {
            const int c = tid + k * (QF_NW * 64);               // four consecutive j of row i
            const int i = c >> 5, j = (c & 31) * 4;
            const int ob = i >> 4, r = i & 15, ch = j >> 5, q = (j >> 3) & 3, e = j & 7;
            const int dst = (((ob * 4 + ch) * 64) + 16 * q + r) * 8 + e;
            const float pv[4] = {p[k].x, p[k].y, p[k].z, p[k].w};
            uint16_t h[4], l[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                h[t] = Elem<DT>::from_f32(pv[t]);
                l[t] = Elem<DT>::from_f32(pv[t] - Elem<DT>::to_f32(h[t]));
            }
            *reinterpret_cast<uint2*>(pih + dst) = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
            *reinterpret_cast<uint2*>(pih + HD * HD + dst) = make_uint2(l[0] | ((uint32_t)l[1] << 16), l[2] | ((uint32_t)l[3] << 16));
        }
        for (int i = tid; i < QP_THR_FLOATS; i += QF_NW * 64) {
            const int li = i < 3 ? 0 : i < 10 ? 1 : i < 25 ? 2 : 3;
            const int k = i - thr_offset(li);
            thrs[i] = decision_threshold(a.cb[codebook_offset(li) + k], a.cb[codebook_offset(li) + k + 1]);
        }
    }
    __syncthreads();
    if (walk_table && wave == 0) {
        // running sum by one wave: 16 entries per lane, a scan over the lanes' totals, the entries again
        int mine[QF_MAX_RUNS / 64], tot = 0;
#pragma unroll
        for (int i = 0; i < QF_MAX_RUNS / 64; ++i) { mine[i] = wbase[lane * (QF_MAX_RUNS / 64) + i + 1]; tot += mine[i]; }
        int incl = tot;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, WAVE);
            if (lane >= o) incl += up;
        }
        int run = incl - tot;
#pragma unroll
        for (int i = 0; i < QF_MAX_RUNS / 64; ++i) { run += mine[i]; wbase[lane * (QF_MAX_RUNS / 64) + i + 1] = run; }
        if (lane == 0) wbase[0] = 0;
    }
    __syncthreads();
    const uint4* piA = reinterpret_cast<const uint4*>(smem);
    if (is_v) qf_walk<DT, true>(a, piA, thrs, w, stage, lane, wave, walk_table ? wbase : nullptr);
    else qf_walk<DT, false>(a, piA, thrs, w, stage, lane, wave, walk_table ? wbase : nullptr);
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
    // grid (slices, segments): the workgroups of a segment share out its tiles that receive tokens (a store laid
    // out for the worst case has thousands of tiles and a handful of them in use)
    const int lane = threadIdx.x, bh = blockIdx.y;
    const int old = a.old_count[bh], cnt = a.seg_count[bh], first = a.seg_tile[bh];
    for (int local = old / TILE + blockIdx.x; local * TILE < cnt; local += gridDim.x) {
    const int tile = first + local;
    const int ts = local * TILE;
    const int lo = max(old - ts, 0);
    const int hi = min(cnt - ts, TILE);
    if (lane < lo || lane >= hi) continue;
    const size_t slot = (size_t)tile * TILE + lane;
    const int t = a.pos[slot] - a.pos_offset;
    const size_t off = (size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT;
    uint16_t* kd = a.kexact + (size_t)tile * TILE * HD;
    uint16_t* vd = a.vexact + (size_t)tile * TILE * HD;
    float x[HD];
    load_row<DT>(a.K, off, x);
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        uint4 pk;
        pk.x = Elem<ODT>::from_f32(x[8 * c]) | ((uint32_t)Elem<ODT>::from_f32(x[8 * c + 1]) << 16);
        pk.y = Elem<ODT>::from_f32(x[8 * c + 2]) | ((uint32_t)Elem<ODT>::from_f32(x[8 * c + 3]) << 16);
        pk.z = Elem<ODT>::from_f32(x[8 * c + 4]) | ((uint32_t)Elem<ODT>::from_f32(x[8 * c + 5]) << 16);
        pk.w = Elem<ODT>::from_f32(x[8 * c + 6]) | ((uint32_t)Elem<ODT>::from_f32(x[8 * c + 7]) << 16);
        *reinterpret_cast<uint4*>(kd + exact_k_index(lane, 8 * c)) = pk;
    }
    load_row<DT>(a.V, off, x);
#pragma unroll
    for (int j = 0; j < HD; ++j) vd[exact_v_index(lane, j)] = Elem<ODT>::from_f32(x[j]);
    }
}

// one new token per (b, h) behind the stored exact tokens
__global__ __launch_bounds__(128) void append_exact_kernel(odmkv_packed_t s, const uint16_t* __restrict__ k,
                                                           const uint16_t* __restrict__ v, int64_t stride_b,
                                                           int64_t stride_h, int pos) {
    const int bh = blockIdx.x, j = threadIdx.x;
    const size_t src = (size_t)(bh / s.Hkv) * stride_b + (size_t)(bh % s.Hkv) * stride_h + j;
    const int cnt = s.seg_count[4][bh];
    const int cap = (s.seg_tile[4][bh + 1] - s.seg_tile[4][bh]) * TILE;
    if (cnt >= cap) return;                                  // full: the host sized it too small
    const int tile = s.seg_tile[4][bh] + cnt / TILE;
    const int l = cnt % TILE;
    uint16_t* kd = s.kexact + (size_t)tile * TILE * HD;
    uint16_t* vd = s.vexact + (size_t)tile * TILE * HD;
    kd[exact_k_index(l, j)] = k[src];
    vd[exact_v_index(l, j)] = v[src];
    __syncthreads();
    if (j == 0) {
        s.pos[4][(size_t)tile * TILE + l] = pos;
        s.seg_count[4][bh] = cnt + 1;
    }
}

extern "C" int odmkv_append_exact(const odmkv_packed_t* store, const void* k, const void* v, int64_t stride_b,
                                  int64_t stride_h, int pos, void* stream) {
    ODMKV_CHECK_ARG(store && k && v, "append_exact: null pointer");
    ODMKV_CHECK_ARG(stride_b >= 0 && stride_h >= 0, "append_exact: negative strides (%lld, %lld)", (long long)stride_b,
                    (long long)stride_h);
    ODMKV_CHECK_ARG(store->kexact && store->vexact && store->seg_tile[4] && store->seg_count[4] && store->pos[4],
                    "append_exact: store has no exact segments");
    hipLaunchKernelGGL(append_exact_kernel, dim3(store->B * store->Hkv), dim3(128), 0, (hipStream_t)stream,
                       *store, (const uint16_t*)k, (const uint16_t*)v, stride_b, stride_h, pos);
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

static inline int compact_chunks(int T) { return (T + CP_TOKENS - 1) / CP_TOKENS; }
// tiles one call can touch, per tensor: a level that receives n tokens of a segment touches at most
// n / 64 + 2 tiles, and the four quantised levels share the segment's T tokens
static inline int redo_capacity(int nseg, int T) { return nseg * (T / TILE + 2 * ODMKV_NQ); }

// byte offset, inside the pack workspace, of the hand-over list (two counters, then the tile numbers)
size_t pack_redo_offset(int nseg, int T) {
    return align_up((size_t)5 * nseg * sizeof(int32_t), 256) +
           align_up((size_t)5 * nseg * compact_chunks(T) * sizeof(int32_t), 256);
}

extern "C" size_t odmkv_pack_workspace_bytes(int B, int Hkv, int T) {
    if (B <= 0 || Hkv <= 0 || T <= 0) return 0;
    return pack_redo_offset(B * Hkv, T) + align_up((size_t)(2 + 2 * redo_capacity(B * Hkv, T)) * sizeof(int32_t), 256);
}

template <int DT>
static int launch_quant_f16(const QuantArgs& qa, hipStream_t st) {
    const size_t lds = QF_PI_BYTES + (size_t)QF_NW * QP_STAGE + QF_THR_BYTES + QF_NW * sizeof(QfWave) + (QF_MAX_RUNS + 1) * sizeof(int);
    static bool attr_set = false;
    if (!attr_set) {
        ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&quant_pack_f16_kernel<DT>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    const int total = qa.tile_base[ODMKV_NQ];
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    const int per_tensor = std::max(1, std::min((total + QF_NW - 1) / QF_NW, std::max(cus / 2, 1)));
    hipLaunchKernelGGL(quant_pack_f16_kernel<DT>, dim3(2 * per_tensor), dim3(QF_NW * 64), lds, st, qa);
    ODMKV_CHECK_LAUNCH("quant_pack_f16_kernel");
    return 0;
}

template <int DT>
static int launch_quant(const QuantArgs& qa, hipStream_t st) {
    // fp32 rows take 128 registers on top of the 128 accumulators: one wave per SIMD then
    constexpr int NW = (DT == ODMKV_F32) ? 4 : 8;
    const size_t lds = QP_PI_BYTES + (size_t)NW * QP_STAGE + QP_THR_FLOATS * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&quant_pack_kernel<DT, NW>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    const int total = qa.tile_base[ODMKV_NQ];
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    const int per_tensor = std::max(1, std::min((total + NW - 1) / NW, std::max(cus / 2, 1)));
    hipLaunchKernelGGL((quant_pack_kernel<DT, NW>), dim3(2 * per_tensor), dim3(NW * 64), lds, st, qa);
    ODMKV_CHECK_LAUNCH("quant_pack_kernel");
    return 0;
}

template <int DT>
static int launch_exact(const ExactArgs& ea, int out_dt, int n_tiles, hipStream_t st) {
    const dim3 grid(std::max(1, std::min(64, n_tiles / std::max(ea.nseg, 1))), ea.nseg);
    if (out_dt == ODMKV_F16)
        hipLaunchKernelGGL((exact_gather_kernel<DT, ODMKV_F16>), grid, dim3(64), 0, st, ea);
    else
        hipLaunchKernelGGL((exact_gather_kernel<DT, ODMKV_BF16>), grid, dim3(64), 0, st, ea);
    ODMKV_CHECK_LAUNCH("exact_gather_kernel");
    return 0;
}

// totals_dev / totals_host / totals_event: null, or where the per-chunk level counts go as soon as they are known
// (device buffer, page-locked host copy, event recorded behind the copy)
static int quant_pack_impl(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                           int64_t stride_b, int64_t stride_h, int64_t stride_t,
                           const int32_t* bits, int pos_offset,
                           const float* pi_k, const float* pi_v, const float* codebooks,
                           const odmkv_packed_t* store, void* workspace, size_t workspace_bytes,
                           void* stream, int32_t* totals_dev, int32_t* totals_host, void* totals_event) {
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
    ca.n_chunks = compact_chunks(T);
    ca.chunk_count = (int32_t*)((char*)workspace + align_up((size_t)5 * nseg * sizeof(int32_t), 256));
    // fp16 rows take the matrix-core estimate first; what it leaves over reaches the exact kernel through this list
    int32_t* redo = (int32_t*)((char*)workspace + pack_redo_offset(nseg, T));
    ca.redo = redo;
    ca.totals = totals_dev;
    for (int li = 0; li < 5; ++li) { ca.pos[li] = store->pos[li]; ca.seg_tile[li] = store->seg_tile[li]; ca.seg_count[li] = store->seg_count[li]; }
    ODMKV_CHECK_ARG(nseg <= 65535, "quant_pack: at most 65535 (sequence, head) pairs per call");
    hipLaunchKernelGGL(chunk_count_kernel, dim3(ca.n_chunks, nseg), dim3(CP_THREADS), 0, st, ca);
    ODMKV_CHECK_LAUNCH("chunk_count_kernel");
    if (totals_dev) {
        ODMKV_CHECK_HIP(hipMemcpyAsync(totals_host, totals_dev, (size_t)nseg * ca.n_chunks * 6 * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        ODMKV_CHECK_HIP(hipEventRecord((hipEvent_t)totals_event, st));
    }
    hipLaunchKernelGGL(compact_kernel, dim3(ca.n_chunks, nseg), dim3(CP_THREADS), 0, st, ca);
    ODMKV_CHECK_LAUNCH("compact_kernel");

    {
        QuantArgs qa;
        qa.K = K; qa.V = V; qa.sB = stride_b; qa.sH = stride_h; qa.sT = stride_t;
        qa.Hkv = Hkv; qa.nseg = nseg; qa.pos_offset = pos_offset;
        qa.pi_k = pi_k; qa.pi_v = pi_v; qa.cb = codebooks; qa.old_count = old_count;
        qa.s = *store;
        qa.tile_base[0] = 0;
        for (int li = 0; li < ODMKV_NQ; ++li) qa.tile_base[li + 1] = qa.tile_base[li] + store->n_tiles[li];
        qa.redo = redo; qa.redo_cap = redo_capacity(nseg, T); qa.from_list = 0;
        if (qa.tile_base[ODMKV_NQ] > 0) {
            int rc;
            if (dtype != ODMKV_F32 && qa.tile_base[ODMKV_NQ] < (1 << QF_GT_BITS)) {
                rc = dtype == ODMKV_F16 ? launch_quant_f16<ODMKV_F16>(qa, st) : launch_quant_f16<ODMKV_BF16>(qa, st);
                qa.from_list = 1;
                if (!rc) rc = dtype == ODMKV_F16 ? launch_quant<ODMKV_F16>(qa, st) : launch_quant<ODMKV_BF16>(qa, st);
            } else {
                // (16-bit stores of 2^19 tiles and more: the list entries of the matrix-core kernel have no room for their numbers)
                rc = dtype == ODMKV_F16 ? launch_quant<ODMKV_F16>(qa, st)
                   : dtype == ODMKV_BF16 ? launch_quant<ODMKV_BF16>(qa, st) : launch_quant<ODMKV_F32>(qa, st);
            }
            if (rc) return rc;
        }
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

extern "C" int odmkv_quant_pack(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                                int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                const int32_t* bits, int pos_offset,
                                const float* pi_k, const float* pi_v, const float* codebooks,
                                const odmkv_packed_t* store, void* workspace, size_t workspace_bytes,
                                void* stream) {
    return quant_pack_impl(K, V, dtype, B, Hkv, T, stride_b, stride_h, stride_t, bits, pos_offset, pi_k, pi_v, codebooks,
                           store, workspace, workspace_bytes, stream, nullptr, nullptr, nullptr);
}

extern "C" int odmkv_pack_count_chunks(int T) { return T > 0 ? compact_chunks(T) : 0; }

// The first fill of a store, everything that does not depend on the level counts in one call: empty the staging store,
// count the levels chunk by chunk (the compaction needs those counts anyway), send the counts to the host (page-locked
// memory, an event behind the copy) and quantise into the staging store.
extern "C" int odmkv_quant_pack_staged(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                                       int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                       const int32_t* bits, int pos_offset,
                                       const float* pi_k, const float* pi_v, const float* codebooks,
                                       const odmkv_packed_t* staging, void* staging_arena, const int32_t* staging_tables_host,
                                       const uint64_t* staging_offsets, uint64_t tables_end, uint64_t counts_end,
                                       int32_t* counts_dev, int32_t* counts_host, void* counts_event,
                                       void* workspace, size_t workspace_bytes, void* stream) {
    ODMKV_CHECK_ARG(staging && staging_arena && staging_tables_host && staging_offsets && counts_dev && counts_host && counts_event,
                    "quant_pack_staged: null pointer");
    ODMKV_CHECK_ARG(B > 0 && Hkv > 0 && T > 0, "quant_pack_staged: bad shape B=%d Hkv=%d T=%d", B, Hkv, T);
    if (int rc = odmkv_store_init(staging_arena, staging_tables_host, 5, B * Hkv + 1, staging_offsets, tables_end, counts_end, counts_end, stream))
        return rc;
    return quant_pack_impl(K, V, dtype, B, Hkv, T, stride_b, stride_h, stride_t, bits, pos_offset, pi_k, pi_v, codebooks,
                           staging, workspace, workspace_bytes, stream, counts_dev, counts_host, counts_event);
}

// ------------------------------------------------------------------------------------------------
// the tiles of a staging store (every segment laid out for the worst case, so that it can be filled
// before anybody knows the level counts) moved into a store laid out for the counts
// ------------------------------------------------------------------------------------------------
struct GatherArgs {
    odmkv_packed_t src, dst;
    int nseg;
    int slice_begin[ODMKV_NQ + 2];      // workgroups along x: level li owns slice_begin[li] .. slice_begin[li + 1] - 1
};

__global__ __launch_bounds__(256) void store_gather_kernel(GatherArgs a) {
    // grid (slices of all levels, segments): the wavefronts of a (level, segment)'s workgroups share out its tiles that
    // hold tokens, a tile per wavefront at a time.  A level gets slices for the tiles the destination has of it (a level
    // nobody uses: one, which copies the zero counts), so that the launch is not mostly workgroups with nothing to do.
    const int tid = threadIdx.x & 63, wave = threadIdx.x >> 6, bh = blockIdx.y;
    int li = 0;
#pragma unroll
    for (int k = 1; k <= ODMKV_NQ; ++k) li += ((int)blockIdx.x >= a.slice_begin[k]);
    const int slice = blockIdx.x - a.slice_begin[li], nslice = a.slice_begin[li + 1] - a.slice_begin[li];
    const int count = a.src.seg_count[li][bh];
    if (slice == 0 && threadIdx.x == 0) a.dst.seg_count[li][bh] = count;
    const int src0 = a.src.seg_tile[li][bh], dst0 = a.dst.seg_tile[li][bh];
    for (int local = slice * 4 + wave; local * TILE < count; local += nslice * 4) {
    const int tile = dst0 + local;
    const int hi = min(count - local * TILE, TILE);
    const size_t st = (size_t)src0 + local;                      // the tile in the staging store
    // lanes behind the count keep what the destination was prepared with (position -1, norm 0, zero rows)
    if (tid < hi) a.dst.pos[li][(size_t)tile * TILE + tid] = a.src.pos[li][st * TILE + tid];
    if (li < ODMKV_NQ) {
        const int W = width_of(li);
        if (tid < hi) {
            a.dst.knorm[li][(size_t)tile * TILE + tid] = a.src.knorm[li][st * TILE + tid];
            a.dst.vnorm[li][(size_t)tile * TILE + tid] = a.src.vnorm[li][st * TILE + tid];
        }
        const int n16 = TILE * W;                                // 16-byte pieces per tensor and tile
        const uint4* sk = reinterpret_cast<const uint4*>(a.src.kcodes[li]) + st * n16;
        const uint4* sv = reinterpret_cast<const uint4*>(a.src.vcodes[li]) + st * n16;
        uint4* dk = reinterpret_cast<uint4*>(a.dst.kcodes[li]) + (size_t)tile * n16;
        uint4* dv = reinterpret_cast<uint4*>(a.dst.vcodes[li]) + (size_t)tile * n16;
        for (int i = tid; i < n16; i += 64) { dk[i] = sk[i]; dv[i] = sv[i]; }
    } else {
        // exact rows (quant.h: tile layouts): key piece 4b + k of lane (n, j) belongs to slot key_slot(n, b); value
        // piece 8k + m of the lane holds slots 32k + 8j .. + 7 of one dim.  Rows behind the count are not copied.
        constexpr int n16 = TILE * HD * 2 / 16;
        const uint4* sk = reinterpret_cast<const uint4*>(a.src.kexact) + st * n16;
        const uint4* sv = reinterpret_cast<const uint4*>(a.src.vexact) + st * n16;
        uint4* dk = reinterpret_cast<uint4*>(a.dst.kexact) + (size_t)tile * n16;
        uint4* dv = reinterpret_cast<uint4*>(a.dst.vexact) + (size_t)tile * n16;
        for (int i = tid; i < n16; i += 64) {
            const int c = i >> 6, l = i & 63, n = l & 15, j = l >> 4;
            if (key_slot(n, c >> 2) < hi) dk[i] = sk[i];
            const int s0 = 32 * (c >> 3) + 8 * j;                // first of the piece's eight slots
            if (s0 < hi) {
                uint4 v = sv[i];
                const int keep = hi - s0;                        // slots s0 .. s0 + keep - 1 are stored
                if (keep < 8) {
                    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (e >= keep) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
                    v = make_uint4(w[0], w[1], w[2], w[3]);
                }
                dv[i] = v;
            }
        }
    }
    }
}

extern "C" int odmkv_store_gather(const odmkv_packed_t* staging, const odmkv_packed_t* store, void* stream) {
    if (int rc = check_store(staging, "store_gather")) return rc;
    if (int rc = check_store(store, "store_gather")) return rc;
    ODMKV_CHECK_ARG(staging->B == store->B && staging->Hkv == store->Hkv && staging->exact_dtype == store->exact_dtype,
                    "store_gather: the two stores differ in shape or exact dtype");
    GatherArgs a;
    a.src = *staging; a.dst = *store; a.nseg = store->B * store->Hkv;
    ODMKV_CHECK_ARG(a.nseg <= 65535, "store_gather: at most 65535 (sequence, head) pairs");
    a.slice_begin[0] = 0;
    for (int li = 0; li <= ODMKV_NQ; ++li)        // four tiles (one per wavefront) per workgroup and trip
        a.slice_begin[li + 1] = a.slice_begin[li] + std::max(1, std::min(128, (store->n_tiles[li] / a.nseg + 4) / 4));
    const dim3 grid(a.slice_begin[ODMKV_NQ + 1], a.nseg);
    hipLaunchKernelGGL(store_gather_kernel, grid, dim3(256), 0, (hipStream_t)stream, a);
    ODMKV_CHECK_LAUNCH("store_gather_kernel");
    return 0;
}

// The second half of a staged first fill, in one call, for the moment the level counts have arrived: add up the chunks,
// size every segment (a tile per 64 tokens; the exact segments with `exact_slack` tokens of room to grow; with
// `quant_headroom` every quantised segment a sixteenth more tiles, two at least, for the tokens later flushes add), lay the store
// out in `arena`, prepare it (odmkv_store_init), fill the descriptor and move the staging store's tiles over
// (odmkv_store_gather).  What the host does between the arrival of the counts and the launch of the gather decides
// whether the GPU runs dry behind the quantiser; here that is a few microseconds of arithmetic and two launches.
extern "C" int odmkv_store_finish_staged(const int32_t* chunk_counts, int n_chunks, int B, int Hkv, int T,
                                         int exact_slack, int quant_headroom, int exact_dtype, void* arena,
                                         uint64_t arena_bytes,
                                         const odmkv_packed_t* staging, int32_t* counts, int32_t* seg_tile,
                                         uint64_t* offsets, uint64_t* sizes, uint64_t* marks,
                                         odmkv_packed_t* store, uint64_t* need_bytes, void* stream) {
    ODMKV_CHECK_ARG(chunk_counts && staging && counts && seg_tile && offsets && sizes && marks && store && need_bytes,
                    "store_finish_staged: null pointer");
    ODMKV_CHECK_ARG(B > 0 && Hkv > 0 && T > 0 && n_chunks > 0 && exact_slack >= 0, "store_finish_staged: bad shape");
    const int nseg = B * Hkv;
    long long all = 0;
    for (int s = 0; s < nseg; ++s)
        for (int k = 0; k < 6; ++k) {
            long long v = 0;
            for (int c = 0; c < n_chunks; ++c) v += chunk_counts[((size_t)s * n_chunks + c) * 6 + k];
            counts[s * 6 + k] = (int32_t)v;
            all += v;
        }
    ODMKV_CHECK_ARG(all == (long long)nseg * T, "store_finish_staged: bits must take values in (0, 2, 3, 4, 8, 16)");
    for (int li = 0; li < 5; ++li) {
        int32_t* row = seg_tile + (size_t)li * (nseg + 1);
        row[0] = 0;
        for (int s = 0; s < nseg; ++s) {
            const long long n = (long long)counts[s * 6 + li + 1] + (li == 4 ? exact_slack : 0);
            long long tiles = (n + TILE - 1) / TILE;
            if (li < 4 && quant_headroom) tiles += std::max(tiles / 16, 2LL);
            row[s + 1] = row[s] + (int32_t)tiles;
        }
    }
    if (int rc = odmkv_store_layout(seg_tile, nseg, offsets, sizes, marks)) return rc;
    *need_bytes = marks[4];
    if (arena == nullptr || arena_bytes < marks[4]) {
        odmkv_set_error("store_finish_staged: the store needs %llu bytes, the allocation has %llu",
                        (unsigned long long)marks[4], (unsigned long long)arena_bytes);
        return ODMKV_ENOSPACE;
    }
    if (int rc = odmkv_store_init(arena, seg_tile, 5, nseg + 1, offsets, marks[0], marks[2], marks[3], stream)) return rc;
    if (int rc = odmkv_store_bind(arena, offsets, seg_tile, nseg, B, Hkv, exact_dtype, store)) return rc;
    return odmkv_store_gather(staging, store, stream);
}

// ------------------------------------------------------------------------------------------------
// dequantise to dense tensors
// ------------------------------------------------------------------------------------------------
struct DequantArgs {
    void* K;
    void* V;
    int64_t sB, sH, sT;
    int Hkv, nseg, T, t_min;           // positions t_min <= t < T are written
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

// x_hat[token][j] = |x| * sum_i c[code_i] * Pi[i][j] on the fp16 matrix cores (v_mfma_f32_16x16x32_f16): operand
// A = Pi^T (rows = outputs j, steps = i), B = the centroids of 16 tokens' codes, both as fp16 high + low terms
// (three products: hi*hi, lo*hi, hi*lo; the fourth is below 2^-22), accumulated in fp32.  The result differs from
// the fp32 sum by about 1e-6 of the row's norm: less than the rounding of a 16-bit cache by two orders of magnitude.
// Persistent workgroups of DQ_NW waves keep Pi^T in LDS in operand order (even workgroups keys, odd ones values) and
// walk the level's tiles, a wave per tile.  A lane ends up with four consecutive outputs of one token: 8 (16) bytes
// of a row per store.
#define DQ_NW 8
template <int W, int DT>
__global__ __launch_bounds__(DQ_NW * 64) void dequant_kernel(DequantArgs a, int n_tiles) {
    extern __shared__ __align__(16) uint8_t smem[];
    uint16_t* pih = reinterpret_cast<uint16_t*>(smem);                             // Pi^T hi, then lo, in operand order
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint8_t* codes = smem + QP_PI_BYTES + wave * QP_STAGE;                         // this wave's [token][dim] codes (values)
    uint32_t* cb = reinterpret_cast<uint32_t*>(smem + QP_PI_BYTES + DQ_NW * QP_STAGE);   // [256] centroids: fp16 hi | lo << 16
    float* norms = reinterpret_cast<float*>(cb + 256) + wave * TILE;              // [DQ_NW][64] norm of the wave's tokens
    long long* offs = reinterpret_cast<long long*>(cb + 256 + DQ_NW * TILE) + wave * TILE;   // element offset of the row, -1: none
    const bool is_v = (blockIdx.x & 1) != 0;
    {
        // lane 16q + r of block (jb, ch) holds Pi[32 ch + 8 q .. + 7][16 jb + r]
        const float4* __restrict__ src = reinterpret_cast<const float4*>(is_v ? a.pi_v : a.pi_k);
        constexpr int PER_THREAD = HD * HD / 4 / (DQ_NW * 64);
        float4 p[PER_THREAD];
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) p[k] = src[tid + k * (DQ_NW * 64)];
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) {
            const int c = tid + k * (DQ_NW * 64);                // four consecutive j of row i
            const int i = c >> 5, j0 = (c & 31) * 4;
            const int ch = i >> 5, q = (i >> 3) & 3, e = i & 7;
            const float pv[4] = {p[k].x, p[k].y, p[k].z, p[k].w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int j = j0 + t, jb = j >> 4, r = j & 15;
                const int dst = (((jb * 4 + ch) * 64) + 16 * q + r) * 8 + e;
                const uint16_t h = Elem<ODMKV_F16>::from_f32(pv[t]);
                pih[dst] = h;
                pih[HD * HD + dst] = Elem<ODMKV_F16>::from_f32(pv[t] - Elem<ODMKV_F16>::to_f32(h));
            }
        }
        for (int i = tid; i < (1 << W); i += DQ_NW * 64) {
            const float c = a.cb[i];
            const uint16_t h = Elem<ODMKV_F16>::from_f32(c);
            cb[i] = (uint32_t)h | ((uint32_t)Elem<ODMKV_F16>::from_f32(c - Elem<ODMKV_F16>::to_f32(h)) << 16);
        }
    }
    __syncthreads();
    const uint4* piA = reinterpret_cast<const uint4*>(smem);
    void* out = is_v ? a.V : a.K;
    const int wg = blockIdx.x >> 1, n_wg = gridDim.x >> 1;
    const int r16 = lane & 15, q = lane >> 4;
    for (int tile = wg * DQ_NW + wave; tile < n_tiles; tile += n_wg * DQ_NW) {
        const int bh = find_segment(a.seg_tile, a.nseg, tile);
        const int ts = (tile - a.seg_tile[bh]) * TILE;
        const int hi = min(a.seg_count[bh] - ts, TILE);
        if (hi <= 0) continue;                                       // wave-uniform
        // positions ascend inside a segment: a tile whose last token lies before t_min has nothing to write
        if (a.t_min > 0 && a.pos[(size_t)tile * TILE + hi - 1] < a.t_min) continue;
        const size_t slot = (size_t)tile * TILE + lane;
        const bool valid = lane < hi;
        {
            const int t = valid ? a.pos[slot] : -1;
            const bool write = valid && t >= a.t_min && t < a.T;
            offs[lane] = write ? (long long)((size_t)(bh / a.Hkv) * a.sB + (size_t)(bh % a.Hkv) * a.sH + (size_t)t * a.sT) : -1ll;
            norms[lane] = valid ? (is_v ? a.vnorm[slot] : a.knorm[slot]) : 0.0f;
        }
        // the lane's 128 codes -> one byte each in LDS, [token][dim]: the matrix operand below wants eight consecutive
        // dims of a token per lane, the tile keeps (4 tokens x 32 dims) of keys or (16 tokens x 8 dims) of values per lane
        {
            const int n = lane & 15, j = lane >> 4;
            const uint8_t* src = (is_v ? a.vcodes : a.kcodes) + (size_t)tile * (TILE * 16 * W);
            uint32_t words[4 * W];
#pragma unroll
            for (int c = 0; c < W; ++c) {
                const uint4 v = *reinterpret_cast<const uint4*>(src + ((size_t)c * TILE + lane) * 16);
                words[4 * c] = v.x; words[4 * c + 1] = v.y; words[4 * c + 2] = v.z; words[4 * c + 3] = v.w;
            }
            if (!is_v) {
#pragma unroll
                for (int b = 0; b < 4; ++b)
#pragma unroll
                    for (int i = 0; i < 32; i += 4) {
                        const uint32_t w4 = get_code<W>(words, 32 * b + i) | (get_code<W>(words, 32 * b + i + 1) << 8) |
                                            (get_code<W>(words, 32 * b + i + 2) << 16) | (get_code<W>(words, 32 * b + i + 3) << 24);
                        *reinterpret_cast<uint32_t*>(&codes[key_slot(n, b) * CODE_ROW + 32 * j + i]) = w4;
                    }
            } else {
#pragma unroll
                for (int k = 0; k < 2; ++k)
#pragma unroll
                    for (int m = 0; m < 8; ++m)
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            codes[(32 * k + 8 * j + e) * CODE_ROW + 16 * m + n] = (uint8_t)get_code<W>(words, 64 * k + 8 * m + e);
            }
        }
        wave_lds_fence();
#pragma unroll 1
        for (int tb = 0; tb < 4; ++tb) {
            // (the lane index is made opaque per round: Pi^T's 64 operand reads do not depend on the round, and hoisted
            // out of it they would take every register there is)
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int token = 16 * tb + r16;
            const long long off = offs[token];
            const float nrm = norms[token];
            // operand B: the centroids of the token's codes 32 ch + 8 q .. + 7, high and low halves
            uint4 bh4[4], bl4[4];
#pragma unroll
            for (int ch = 0; ch < 4; ++ch) {
                const uint2 cw = *reinterpret_cast<const uint2*>(&codes[token * CODE_ROW + 32 * ch + 8 * q]);
                const uint32_t w2[2] = {cw.x, cw.y};
                uint32_t t[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) t[e] = cb[(w2[e >> 2] >> (8 * (e & 3))) & 0xffu];
                bh4[ch] = make_uint4(__builtin_amdgcn_perm(t[1], t[0], 0x05040100u), __builtin_amdgcn_perm(t[3], t[2], 0x05040100u),
                                     __builtin_amdgcn_perm(t[5], t[4], 0x05040100u), __builtin_amdgcn_perm(t[7], t[6], 0x05040100u));
                bl4[ch] = make_uint4(__builtin_amdgcn_perm(t[1], t[0], 0x07060302u), __builtin_amdgcn_perm(t[3], t[2], 0x07060302u),
                                     __builtin_amdgcn_perm(t[5], t[4], 0x07060302u), __builtin_amdgcn_perm(t[7], t[6], 0x07060302u));
            }
#pragma unroll
            for (int jb = 0; jb < 8; ++jb) {
                qf_f4 acc = (qf_f4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int ch = 0; ch < 4; ++ch) {
                    const uint4 ah = piA[(jb * 4 + ch) * 64 + ln];
                    const uint4 al = piA[HD * HD / 8 + (jb * 4 + ch) * 64 + ln];
                    acc = qf_mfma<ODMKV_F16>(ah, bh4[ch], acc);
                    acc = qf_mfma<ODMKV_F16>(al, bh4[ch], acc);
                    acc = qf_mfma<ODMKV_F16>(ah, bl4[ch], acc);
                }
                if (off >= 0) {                                     // outputs 16 jb + 4 q .. + 3 of the token
                    const float r[4] = {acc[0] * nrm, acc[1] * nrm, acc[2] * nrm, acc[3] * nrm};
                    const int c4 = 16 * jb + 4 * q;
                    if constexpr (DT == ODMKV_F32) {
                        *reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + off + c4) = make_float4(r[0], r[1], r[2], r[3]);
                    } else {
                        const uint32_t lo = (uint32_t)Elem<DT>::from_f32(r[0]) | ((uint32_t)Elem<DT>::from_f32(r[1]) << 16);
                        const uint32_t hi2 = (uint32_t)Elem<DT>::from_f32(r[2]) | ((uint32_t)Elem<DT>::from_f32(r[3]) << 16);
                        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(out) + off + c4) = make_uint2(lo, hi2);
                    }
                }
            }
        }
        wave_lds_fence();                                            // offs / norms / codes free for the next tile
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
        const uint16_t kr = ks[exact_k_index(lane, j)];
        const uint16_t vr = vs[exact_v_index(lane, j)];
        const float kf = src_bf16 ? Elem<ODMKV_BF16>::to_f32(kr) : Elem<ODMKV_F16>::to_f32(kr);
        const float vf = src_bf16 ? Elem<ODMKV_BF16>::to_f32(vr) : Elem<ODMKV_F16>::to_f32(vr);
        kd[j] = Elem<DT>::from_f32(kf);
        vd[j] = Elem<DT>::from_f32(vf);
    }
}

template <int W, int DT>
static int launch_dequant_w(const DequantArgs& da, int n_tiles, hipStream_t st) {
    const size_t lds = QP_PI_BYTES + (size_t)DQ_NW * QP_STAGE + 256 * sizeof(float) + DQ_NW * TILE * (sizeof(float) + sizeof(long long));
    static bool attr_set = false;
    if (!attr_set) {
        ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dequant_kernel<W, DT>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    int dev = 0, cus = 256;
    ODMKV_CHECK_HIP(hipGetDevice(&dev));
    ODMKV_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    // one persistent workgroup per compute unit, keys on the even and values on the odd ones; never
    // more workgroups than there are tiles for their waves
    int pairs = cus / 2;
    const int need = (n_tiles + DQ_NW - 1) / DQ_NW;
    if (pairs > need) pairs = need;
    if (pairs < 1) pairs = 1;
    hipLaunchKernelGGL((dequant_kernel<W, DT>), dim3(2 * pairs), dim3(DQ_NW * 64), lds, st, da, n_tiles);
    ODMKV_CHECK_LAUNCH("dequant_kernel");
    return 0;
}

template <int DT>
static int launch_dequant(const DequantArgs& da, int li, int n_tiles, hipStream_t st) {
    switch (li) {
        case 0: return launch_dequant_w<2, DT>(da, n_tiles, st);
        case 1: return launch_dequant_w<3, DT>(da, n_tiles, st);
        case 2: return launch_dequant_w<4, DT>(da, n_tiles, st);
        default: return launch_dequant_w<8, DT>(da, n_tiles, st);
    }
}

extern "C" int odmkv_dequant(const odmkv_packed_t* store, void* K, void* V, int dtype, int T,
                             int64_t stride_b, int64_t stride_h, int64_t stride_t,
                             const float* pi_k, const float* pi_v, const float* codebooks,
                             int include_exact, void* stream) {
    return odmkv_dequant_from(store, K, V, dtype, 0, T, stride_b, stride_h, stride_t, pi_k, pi_v, codebooks, include_exact, stream);
}

extern "C" int odmkv_dequant_from(const odmkv_packed_t* store, void* K, void* V, int dtype, int t_min, int T,
                                  int64_t stride_b, int64_t stride_h, int64_t stride_t,
                                  const float* pi_k, const float* pi_v, const float* codebooks,
                                  int include_exact, void* stream) {
    ODMKV_CHECK_ARG(K && V && pi_k && pi_v && codebooks, "dequant: null pointer");
    ODMKV_CHECK_ARG(t_min >= 0 && !(t_min > 0 && include_exact), "dequant: t_min=%d (>= 0; quantised tokens only when > 0)", t_min);
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
        da.Hkv = store->Hkv; da.nseg = nseg; da.T = T; da.t_min = t_min;
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
