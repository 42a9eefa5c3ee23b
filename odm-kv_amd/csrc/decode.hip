// Fused LUT decode attention over the packed mixed-width KV store (one query token per sequence).
//
// Three launches per call:
//   1. prep:   q16 = the query rounded to fp16 (what a model in fp16/bf16 hands over anyway);
//              q' = Pi_k q16 in fp32 (queries in the rotated basis of the quantised keys)
//   2. main:   one workgroup per work item = a run of 64-token tiles of one (sequence, kv-head,
//              level).  The packed bytes are read once from HBM; nothing else is.
//   3. merge:  log-sum-exp merge of a kv-head's items per query head, rotation of the quantised
//              part back to the model basis (acc . Pi_v), addition of the exact part, normalise.
//
// Main kernel, per wavefront and tile (MFMA 4x4x4 f16, 16 blocks of 4 lanes):
//   keys    lane = token.  Four consecutive codes of the token index an LDS table that returns
//           their four centroids as fp16; that is operand A (row = token of the quad) of
//             D[i][j] = sum_k A[lane 4b+i][k] * B[lane 4b+j][k]
//           and operand B is the query of head j = lane % 4.  After 32 steps over the 128 dims,
//           lane (quad b, j) holds the logits of tokens 4b..4b+3 for head j.
//   softmax one head per lane: scale by |k|, running max over the 16 lanes that share the head,
//           p = exp2(logit - m), times |v|, rounded to fp16: already laid out as operand A
//           (row = head, k = token of the quad) of the value product.
//   values  lane = dim.  Values are stored dim-major, so four consecutive codes are four tokens
//           of this lane's dim: the same LDS table gives operand B, and the A operand of step s
//           is broadcast from quad s (cbsz/abid).  16 steps accumulate sum_t p_t |v_t| c[code]
//           for four heads x 128 dims in the rotated basis.
// The LDS table is replicated over 32 slots (slot = lane % 32) so that lanes never share a bank.
// All softmax state is kept in base-2 logarithms.
#include "quant.h"
#include <hip/hip_ext.h>

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

#define PSTRIDE 132          // floats per (item, head) partial: 128 acc + m + l + 2 pad
#ifndef NWAVES
#define NWAVES 8        // wavefronts of a workgroup of the main kernel: two per SIMD, one workgroup per CU
#endif
#define LUT_BYTES 65536
#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

// optional per-workgroup timestamps for tuning (compiled out of the shipped library)
#ifdef ODMKV_TRACE
__device__ unsigned long long g_trace[8192 * 8];
#define TRACE(k) if (tid == 0 && blockIdx.x < 8192) g_trace[blockIdx.x * 8 + (k)] = wall_clock64();
extern "C" int odmkv_debug_read_trace(unsigned long long* host, int n) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_trace), sizeof(unsigned long long) * n);
}
#else
#define TRACE(k)
#endif

struct DecodeArgs {
    odmkv_packed_t s;
    const void* q;
    int q_dt, out_dt;   // element types of q and out (ODMKV_F16 / BF16 / F32)
    int Hq, G, B;
    float scaling;
    const int32_t* items;
    const int32_t* item_range;
    const int32_t* order;      // order[k] = item that workgroup k takes (long items first), or null: item k
    const float* pi_k_t;   // Pi_k transposed
    const float* pi_v;
    const float* cb;
    uint4* qrot;      // [B*Hq, 32] per 4-dim step: fp16 high halves (8 bytes) and low halves (8 bytes) of Pi_k q16
    uint4* qs;        // [B*Hq, 32] the same for q16 itself (low halves are zero)
    float inv_s[4];   // 1 / table scale per width
    float cbs[28];    // scaled centroids of widths 2, 3, 4 (kept in scalar registers; 8-bit ones stay in memory)
    int gp;           // head slots per item in `partial`: 4 or 8
    float* partial;   // [n_items, gp, PSTRIDE]
    void* out;
    float* lse;
};

// ------------------------------------------------------------------------------------------------
// prep: rotate and scale the queries
// ------------------------------------------------------------------------------------------------
__device__ static inline uint32_t half_bits(float f) { return (uint32_t)__half_as_ushort(__float2half_rn(f)); }

#ifndef PREP_SPLIT
#define PREP_SPLIT 4                       // workgroups per query head, each producing HD / PREP_SPLIT rotated dims
#endif
#define PREP_THREADS 512
__global__ __launch_bounds__(PREP_THREADS) void decode_prep_kernel(DecodeArgs a) {
    constexpr int QD = HD / PREP_SPLIT;     // rotated dims of this workgroup
    constexpr int JS = PREP_THREADS / QD;   // slices of the sum over j
    constexpr int JN = HD / JS;             // terms per slice
    __shared__ float qsh[HD];
    __shared__ float part[JS][QD];
    const int bq = blockIdx.x / PREP_SPLIT, quarter = blockIdx.x % PREP_SPLIT, tid = threadIdx.x;
    const int ii = tid % QD, js = tid / QD, i = quarter * QD + ii;
    // this thread's JN elements of column i of Pi_k (rows of the transposed matrix): all requested at once.
    // No workgroup pulls the whole 64 KB matrix through one compute unit.
    float pk[JN];
#pragma unroll
    for (int jj = 0; jj < JN; ++jj) pk[jj] = a.pi_k_t[(size_t)(js * JN + jj) * HD + i];
    if (tid < HD) {
        // the query is consumed at fp16 precision, like the attention it replaces (model dtype)
        const size_t qi = (size_t)bq * HD + tid;
        const float qf = a.q_dt == ODMKV_F32 ? reinterpret_cast<const float*>(a.q)[qi]
                       : a.q_dt == ODMKV_F16 ? Elem<ODMKV_F16>::to_f32(reinterpret_cast<const uint16_t*>(a.q)[qi])
                                             : Elem<ODMKV_BF16>::to_f32(reinterpret_cast<const uint16_t*>(a.q)[qi]);
        const __half q16 = __float2half_rn(qf);
        qsh[tid] = __half2float(q16);
        if (tid / QD == quarter) {           // the un-rotated copy (for exact tiles): every workgroup writes its own dims
            uint16_t* qs16 = reinterpret_cast<uint16_t*>(a.qs + (size_t)bq * 32);
            qs16[(tid >> 2) * 8 + (tid & 3)] = __half_as_ushort(q16);
            qs16[(tid >> 2) * 8 + 4 + (tid & 3)] = 0;
        }
    }
    __syncthreads();
    // q'_i = sum_j Pi_k[i][j] q_j: every slice sums its share of j in order, the slices are added in order
    float acc = 0.0f;
#pragma unroll
    for (int jj = 0; jj < JN; ++jj) acc = __fmaf_rn(pk[jj], qsh[js * JN + jj], acc);
    part[js][ii] = acc;
    __syncthreads();
    if (tid < QD) {
        float tot = part[0][tid];
#pragma unroll
        for (int sl = 1; sl < JS; ++sl) tot += part[sl][tid];
        uint16_t* qr16 = reinterpret_cast<uint16_t*>(a.qrot + (size_t)bq * 32);
        const __half hi = __float2half_rn(tot);
        qr16[(i >> 2) * 8 + (i & 3)] = __half_as_ushort(hi);
        qr16[(i >> 2) * 8 + 4 + (i & 3)] = (uint16_t)half_bits(tot - __half2float(hi));
    }
}

// ------------------------------------------------------------------------------------------------
// small helpers
// ------------------------------------------------------------------------------------------------
__device__ static inline h4 as_h4(uint32_t lo, uint32_t hi) {
    union { uint32_t u[2]; h4 h; } x;
    x.u[0] = lo; x.u[1] = hi;
    return x.h;
}

// two bf16 in a dword -> two fp16 in a dword
__device__ static inline uint32_t bf16x2_to_f16x2(uint32_t w) {
    const float lo = __uint_as_float(w << 16), hi = __uint_as_float(w & 0xffff0000u);
    return half_bits(lo) | (half_bits(hi) << 16);
}

template <int CTRL>
__device__ static inline float dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
#define DPP_ROR4 0x124
#define DPP_ROR8 0x128
#define DPP_QUAD(i) ((i) | ((i) << 2) | ((i) << 4) | ((i) << 6))

// reduce over the 16 lanes that share lane % 4
__device__ static inline float head_max(float v) {
    v = fmaxf(v, dpp<DPP_ROR4>(v));
    v = fmaxf(v, dpp<DPP_ROR8>(v));
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    v = fmaxf(v, __shfl_xor(v, 32, WAVE));
    return v;
}
__device__ static inline float head_sum(float v) {
    v += dpp<DPP_ROR4>(v);
    v += dpp<DPP_ROR8>(v);
    v += __shfl_xor(v, 16, WAVE);
    v += __shfl_xor(v, 32, WAVE);
    return v;
}

// workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight
// (__syncthreads would first wait for every outstanding load of the wavefront)
__device__ static inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_4x4x4f16((a), (b), (c), 0, 0, 0)
#define MFMA_BCAST(a, b, c, s) __builtin_amdgcn_mfma_f32_4x4x4f16((a), (b), (c), 4, (s), 0)

// ------------------------------------------------------------------------------------------------
// LDS tables: code group -> fp16 centroids, replicated over 32 slots
//   W = 2: index = byte (4 codes) -> 4 halfs (8 bytes),  row = 256 bytes
//   W = 3: index = 6 bits (2 codes) -> 2 halfs (4 bytes), row = 128 bytes
//   W = 4: index = byte (2 codes) -> 2 halfs,             row = 128 bytes
//   W = 8: index = byte (1 code)  -> the half in both halves of a dword, row = 128 bytes
// ------------------------------------------------------------------------------------------------
// pick table[idx] from a table that lives in scalar registers (no memory access: every workgroup
// of a launch would otherwise hammer the same cache line)
template <int N>
__device__ static inline float pick(const float* t, uint32_t idx) {
    float v = t[0];
#pragma unroll
    for (int k = 1; k < N; ++k) v = idx == (uint32_t)k ? t[k] : v;
    return v;
}

// Thread tid computes table entry tid; the entry is then replicated over its row.  A thread writing
// its own row would put all lanes of a wavefront on the same banks (rows are 256 or 128 bytes
// apart), so the wavefront writes row after row instead: the lanes of one store instruction cover
// consecutive 16-byte pieces of four (eight) rows, and fetch the row's entry from its owner by a
// cross-lane read.
template <int W>
__device__ static inline void build_lut(uint8_t* lut, const DecodeArgs& a, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    if constexpr (W == 2) {
        // row = code byte: its lowest code is lane >> 4 and the other three are the same for the whole
        // wavefront, so the row's eight bytes are put together from the four centroids without any
        // cross-lane traffic; the lanes of one store cover consecutive 16-byte pieces of four rows
        uint32_t h[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) h[k] = half_bits(a.cbs[k]);
        const auto sel = [&](int k) { return k == 0 ? h[0] : k == 1 ? h[1] : k == 2 ? h[2] : h[3]; };
        const uint32_t own = sel(lane >> 4);
        constexpr int ROWS = 256 / NWAVES;                   // rows of this wavefront
#pragma unroll
        for (int i = 0; i < ROWS / 4; ++i) {
            const int base = wave * ROWS + i * 4;            // wave-uniform; the row is base + (lane >> 4)
            const uint32_t x = own | (sel((base >> 2) & 3) << 16), y = sel((base >> 4) & 3) | (sel(base >> 6) << 16);
            *reinterpret_cast<uint4*>(lut + (base + (lane >> 4)) * 256 + (lane & 15) * 16) = make_uint4(x, y, x, y);
        }
    } else {
        uint32_t v;
        if constexpr (W == 3) { v = half_bits(pick<8>(a.cbs + 4, tid & 7)) | (half_bits(pick<8>(a.cbs + 4, (tid >> 3) & 7)) << 16); }
        else if constexpr (W == 4) { v = half_bits(pick<16>(a.cbs + 12, tid & 15)) | (half_bits(pick<16>(a.cbs + 12, (tid >> 4) & 15)) << 16); }
        else { v = half_bits(a.cb[codebook_offset(3) + (tid & 255)]) * 0x10001u; }
        const bool on = wave < 4 && (W != 3 || wave == 0);  // 256 entries (64 for the 3-bit table): four wavefronts' worth
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int src = i * 8 + (lane >> 3);
            const uint32_t x = __shfl(v, src, WAVE);
            if (on) *reinterpret_cast<uint4*>(lut + (wave * 64 + src) * 128 + (lane & 7) * 16) = make_uint4(x, x, x, x);
        }
    }
}

// centroids of code group s (codes 4s..4s+3 of the stream held in w), as four halfs
template <int W>
__device__ static inline h4 lut4(const uint32_t* w, int s, const uint8_t* lut, uint32_t slot4) {
    if constexpr (W == 2) {
        // address = (byte s of the stream) * 256 + slot * 8, formed by one byte permute:
        // byte 0 <- slot * 8 (< 256), byte 1 <- the code byte, bytes 2, 3 <- 0
        const uint32_t sel = 0x0c0c0000u | ((4u + (uint32_t)(s & 3)) << 8);
        const uint32_t addr = __builtin_amdgcn_perm(w[s >> 2], 2 * slot4, sel);
        const uint2 v = *reinterpret_cast<const uint2*>(lut + addr);
        return as_h4(v.x, v.y);
    } else if constexpr (W == 4) {
        const int bit = 16 * s;
        const uint32_t x = w[bit >> 5] >> (bit & 31);
        const uint32_t lo = *reinterpret_cast<const uint32_t*>(lut + ((x & 0xffu) << 7) + slot4);
        const uint32_t hi = *reinterpret_cast<const uint32_t*>(lut + (((x >> 8) & 0xffu) << 7) + slot4);
        return as_h4(lo, hi);
    } else if constexpr (W == 8) {
        const uint32_t x = w[s];
        const uint32_t t0 = *reinterpret_cast<const uint32_t*>(lut + ((x & 0xffu) << 7) + slot4);
        const uint32_t t1 = *reinterpret_cast<const uint32_t*>(lut + (((x >> 8) & 0xffu) << 7) + slot4);
        const uint32_t t2 = *reinterpret_cast<const uint32_t*>(lut + (((x >> 16) & 0xffu) << 7) + slot4);
        const uint32_t t3 = *reinterpret_cast<const uint32_t*>(lut + ((x >> 24) << 7) + slot4);
        return as_h4((t0 & 0xffffu) | (t1 & 0xffff0000u), (t2 & 0xffffu) | (t3 & 0xffff0000u));
    } else {
        const int bit = 12 * s, k = bit >> 5, sh = bit & 31;
        uint32_t x = w[k] >> sh;
        if (sh + 12 > 32) x |= w[k + 1] << (32 - sh);
        const uint32_t lo = *reinterpret_cast<const uint32_t*>(lut + ((x & 63u) << 7) + slot4);
        const uint32_t hi = *reinterpret_cast<const uint32_t*>(lut + (((x >> 6) & 63u) << 7) + slot4);
        return as_h4(lo, hi);
    }
}

// ------------------------------------------------------------------------------------------------
// per-wavefront running state: one softmax head per lane and pass, four heads x two dims per lane
// ------------------------------------------------------------------------------------------------
template <int NP>
struct WaveState {
    float m[NP], l[NP];
    f4 acc[NP][2];
};

// logits of this lane's head for the quad's four tokens -> p (fp16, times |v|), state update
template <int NP>
__device__ static inline h4 softmax_step(WaveState<NP>& st, int p, const f4& logit, const f4& vn) {
    float mx = fmaxf(fmaxf(logit[0], logit[1]), fmaxf(logit[2], logit[3]));
    mx = head_max(mx);
    const float mn = fmaxf(st.m[p], mx);
    const float alpha = __builtin_amdgcn_exp2f(st.m[p] - mn);     // first tile: exp2(-inf) = 0
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) pr[i] = __builtin_amdgcn_exp2f(logit[i] - mn);   // padded tokens: -inf -> 0
    st.l[p] = __fmaf_rn(st.l[p], alpha, (pr[0] + pr[1]) + (pr[2] + pr[3]));
    st.m[p] = mn;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {         // the maximum moved for some head
        const float a0 = dpp<DPP_QUAD(0)>(alpha), a1 = dpp<DPP_QUAD(1)>(alpha);
        const float a2 = dpp<DPP_QUAD(2)>(alpha), a3 = dpp<DPP_QUAD(3)>(alpha);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            st.acc[p][h][0] *= a0; st.acc[p][h][1] *= a1; st.acc[p][h][2] *= a2; st.acc[p][h][3] *= a3;
        }
    }
    h4 pa;
#pragma unroll
    for (int i = 0; i < 4; ++i) pa[i] = (_Float16)(pr[i] * vn[i]);
    return pa;
}

// ---- quantised tiles -----------------------------------------------------------------------------
template <int W>
struct TileData {
    uint32_t kw[4 * W];
    uint32_t vw[2][2 * W];
    f4 kn, vn;
};

// the packed codes are read once per call and never again before the whole cache has streamed by:
// loaded with the non-temporal hint, so that they do not push the small per-layer operands (rotations,
// work lists, tables) out of the caches
__device__ static inline uint4 stream_load(const uint4* p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ static inline uint2 stream_load(const uint2* p) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return make_uint2(v.x, v.y);
}

template <int W>
__device__ static inline void load_tile(TileData<W>& t, const DecodeArgs& a, int li, int tile, int lane) {
    const uint8_t* ksrc = a.s.kcodes[li] + (size_t)tile * (TILE * 16 * W);
#pragma unroll
    for (int c = 0; c < W; ++c) {
        const uint4 v = stream_load(reinterpret_cast<const uint4*>(ksrc + ((size_t)c * TILE + lane) * 16));
        t.kw[4 * c] = v.x; t.kw[4 * c + 1] = v.y; t.kw[4 * c + 2] = v.z; t.kw[4 * c + 3] = v.w;
    }
    const uint8_t* vsrc = a.s.vcodes[li] + (size_t)tile * (HD * 8 * W);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int j = lane + 64 * h;
        if constexpr (W == 3) {
#pragma unroll
            for (int u = 0; u < 3; ++u) {
                const uint2 v = stream_load(reinterpret_cast<const uint2*>(vsrc + ((size_t)u * HD + j) * 8));
                t.vw[h][2 * u] = v.x; t.vw[h][2 * u + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int u = 0; u < W / 2; ++u) {
                const uint4 v = stream_load(reinterpret_cast<const uint4*>(vsrc + ((size_t)u * HD + j) * 16));
                t.vw[h][4 * u] = v.x; t.vw[h][4 * u + 1] = v.y; t.vw[h][4 * u + 2] = v.z; t.vw[h][4 * u + 3] = v.w;
            }
        }
    }
    const size_t quad = (size_t)tile * TILE + (lane & ~3);
    t.kn = __builtin_nontemporal_load(reinterpret_cast<const f4*>(a.s.knorm[li] + quad));
    t.vn = __builtin_nontemporal_load(reinterpret_cast<const f4*>(a.s.vnorm[li] + quad));
}

#define PV_STEP(s)                                                                              \
    {                                                                                           \
        const h4 b0 = lut4<W>(t.vw[0], (s), lut, slot4), b1 = lut4<W>(t.vw[1], (s), lut, slot4); \
        _Pragma("unroll") for (int p = 0; p < NP; ++p) {                                        \
            st.acc[p][0] = MFMA_BCAST(pa[p], b0, st.acc[p][0], (s));                            \
            st.acc[p][1] = MFMA_BCAST(pa[p], b1, st.acc[p][1], (s));                            \
        }                                                                                       \
    }

template <int W, int NP>
__device__ static inline void compute_tile(const TileData<W>& t, int nvalid, int lane, const uint8_t* lut,
                                           uint32_t slot4, const h4* qr, const h4* ql, float ksc, float vsc,
                                           WaveState<NP>& st) {
    // ---- keys ----
    f4 dk[NP][4];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) dk[p][c] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 32; ++s) {
        const h4 kv = lut4<W>(t.kw, s, lut, slot4);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            dk[p][s & 3] = MFMA(kv, qr[p * 32 + s], dk[p][s & 3]);
            dk[p][(s + 2) & 3] = MFMA(kv, ql[p * 32 + s], dk[p][(s + 2) & 3]);    // low half of the query
        }
    }
    const int tok0 = lane & ~3;
    h4 pa[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const f4 d = (dk[p][0] + dk[p][1]) + (dk[p][2] + dk[p][3]);
        f4 logit;
#pragma unroll
        for (int i = 0; i < 4; ++i) logit[i] = tok0 + i < nvalid ? d[i] * (t.kn[i] * ksc) : -INFINITY;
        f4 vn;
#pragma unroll
        for (int i = 0; i < 4; ++i) vn[i] = tok0 + i < nvalid ? t.vn[i] * vsc : 0.0f;
        pa[p] = softmax_step<NP>(st, p, logit, vn);
    }
    // ---- values ----
    PV_STEP(0) PV_STEP(1) PV_STEP(2) PV_STEP(3) PV_STEP(4) PV_STEP(5) PV_STEP(6) PV_STEP(7)
    PV_STEP(8) PV_STEP(9) PV_STEP(10) PV_STEP(11) PV_STEP(12) PV_STEP(13) PV_STEP(14) PV_STEP(15)
}

// LDS row of one head's query halves: 32 steps of 16 bytes plus one of padding, so that the four heads a
// wavefront reads in one instruction (lane % 4) sit on different banks
#define QS 33
// stage the group's queries (fp16 high/low halves per 4-dim step) in LDS; heads beyond the group are 0
// nq: query heads staged by the workgroup (4, or 8 when its two wave groups serve four heads each)
__device__ static inline uint4 load_query_slice(const uint4* src, int tid, int nq, int nheads) {
    return (tid < nq * 32 && (tid >> 5) < nheads) ? src[tid] : make_uint4(0u, 0u, 0u, 0u);
}
__device__ static inline void stage_queries(uint4 v, uint4* qsh, int tid, int nq) {
    if (tid < nq * 32) qsh[(tid >> 5) * QS + (tid & 31)] = v;
}
// hbase: first of the four heads this wavefront serves
__device__ static inline void fetch_queries(const uint4* qsh, int lane, int hbase, h4* qr, h4* ql) {
#pragma unroll
    for (int s = 0; s < 32; ++s) {
        const uint4 v = qsh[(hbase + (lane & 3)) * QS + s];
        qr[s] = as_h4(v.x, v.y);
        ql[s] = as_h4(v.z, v.w);
    }
}

// One work item of a quantised level.  TW wavefronts walk the item's tiles for the same four heads (all
// eight, or four per head group when the workgroup serves eight heads); wq is this wavefront's place among them.
template <int W, int NP, int TW>
__device__ static inline void run_quant_level(const DecodeArgs& a, int li, int bq_first, int nq, int nheads_all, int hbase,
                                              int tile0, int ntiles, int ntok,
                                              int tid, uint8_t* lut, uint4* qsh, WaveState<NP>& st) {
    const int wave = tid >> 6, lane = tid & 63, wq = wave % TW;
    const uint32_t slot4 = (lane & 31) * 4;
    const float vsc = a.inv_s[li], ksc = a.inv_s[li] * a.scaling * LOG2E;
    // The table needs nothing from memory and is built before the tiles are requested: behind a
    // wavefront's tile requests its LDS traffic would wait for the memory pipeline to accept them
    // (every wavefront of the chip asks for its tiles at the same moment).  Loads return in issue
    // order: the (small) query slice goes first so that staging it does not have to wait for the tile.
    const uint4 qslice = load_query_slice(a.qrot + (size_t)bq_first * 32, tid, nq, nheads_all);   // one request: lands while the table is built
    build_lut<W>(lut, a, tid);
    TileData<W> cur;
    int tt = wq;
    int nvalid = tt < ntiles ? min(ntok - tt * TILE, TILE) : 0;
    if (nvalid > 0) load_tile<W>(cur, a, li, tile0 + tt, lane);
    stage_queries(qslice, qsh, tid, nq);
    lds_barrier();
    TRACE(1)
    // second buffer (not for the widest rows: the registers go to the query there), requested before
    // the queries are fetched into registers
    TileData<W> nxt;
    int nv1 = 0;
    if constexpr (W != 8) {
        nv1 = tt + TW < ntiles ? min(ntok - (tt + TW) * TILE, TILE) : 0;
        if (nv1 > 0) load_tile<W>(nxt, a, li, tile0 + tt + TW, lane);
    }
    h4 qr[NP * 32], ql[NP * 32];
    fetch_queries(qsh, lane, hbase, qr, ql);
    if (nvalid <= 0) return;
    TRACE(2)
    if constexpr (W == 8) {
        while (true) {
            compute_tile<W, NP>(cur, nvalid, lane, lut, slot4, qr, ql, ksc, vsc, st);
            tt += TW;
            nvalid = tt < ntiles ? min(ntok - tt * TILE, TILE) : 0;
            if (nvalid <= 0) break;
            load_tile<W>(cur, a, li, tile0 + tt, lane);
        }
    } else {
        while (true) {
            compute_tile<W, NP>(cur, nvalid, lane, lut, slot4, qr, ql, ksc, vsc, st);
            if (nv1 <= 0) break;
            tt += 2 * TW;
            nvalid = tt < ntiles ? min(ntok - tt * TILE, TILE) : 0;
            if (nvalid > 0) load_tile<W>(cur, a, li, tile0 + tt, lane);
            compute_tile<W, NP>(nxt, nv1, lane, lut, slot4, qr, ql, ksc, vsc, st);
            if (nvalid <= 0) break;
            nv1 = tt + TW < ntiles ? min(ntok - (tt + TW) * TILE, TILE) : 0;
            if (nv1 > 0) load_tile<W>(nxt, a, li, tile0 + tt + TW, lane);
        }
    }
}

// ---- exact (fp16 / bf16) tiles ---------------------------------------------------------------------
// One exact tile in registers: 64 tokens x 128 dims of keys (token-major chunks) and of values
// (dim-major groups of four tokens).  Everything is requested at once; the products then run
// without touching memory again.
struct ExactTile {
    uint4 k[16];
    uint2 v[16][2];
};

__device__ static inline void load_exact_tile(ExactTile& t, const DecodeArgs& a, int tile, int lane) {
    const uint16_t* ksrc = a.s.kexact + (size_t)tile * TILE * HD;
    const uint16_t* vsrc = a.s.vexact + (size_t)tile * TILE * HD;
#pragma unroll
    for (int c = 0; c < 16; ++c) t.k[c] = stream_load(reinterpret_cast<const uint4*>(ksrc + ((size_t)c * TILE + lane) * 8));
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        t.v[s][0] = stream_load(reinterpret_cast<const uint2*>(vsrc + ((size_t)s * HD + lane) * 4));
        t.v[s][1] = stream_load(reinterpret_cast<const uint2*>(vsrc + ((size_t)s * HD + lane + 64) * 4));
    }
}

template <int NP>
__device__ static inline void compute_exact_tile(const ExactTile& t, bool bf, int nvalid, int lane, float esc,
                                                 const h4* qr, WaveState<NP>& st) {
    f4 dk[NP][4];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) dk[p][c] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        uint4 v = t.k[c];
        if (bf) { v.x = bf16x2_to_f16x2(v.x); v.y = bf16x2_to_f16x2(v.y); v.z = bf16x2_to_f16x2(v.z); v.w = bf16x2_to_f16x2(v.w); }
        const h4 k0 = as_h4(v.x, v.y), k1 = as_h4(v.z, v.w);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            dk[p][(2 * c) & 3] = MFMA(k0, qr[p * 32 + 2 * c], dk[p][(2 * c) & 3]);
            dk[p][(2 * c + 1) & 3] = MFMA(k1, qr[p * 32 + 2 * c + 1], dk[p][(2 * c + 1) & 3]);
        }
    }
    const int tok0 = lane & ~3;
    h4 pa[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const f4 d = (dk[p][0] + dk[p][1]) + (dk[p][2] + dk[p][3]);
        f4 logit, vn;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            logit[i] = tok0 + i < nvalid ? d[i] * esc : -INFINITY;
            vn[i] = tok0 + i < nvalid ? 1.0f : 0.0f;
        }
        pa[p] = softmax_step<NP>(st, p, logit, vn);
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        uint2 r0 = t.v[s][0], r1 = t.v[s][1];
        if (bf) { r0.x = bf16x2_to_f16x2(r0.x); r0.y = bf16x2_to_f16x2(r0.y);
                  r1.x = bf16x2_to_f16x2(r1.x); r1.y = bf16x2_to_f16x2(r1.y); }
        const h4 b0 = as_h4(r0.x, r0.y), b1 = as_h4(r1.x, r1.y);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            // the A operand of step s comes from quad s; the broadcast selector must be a constant
            switch (s) {
#define ODMKV_CASE(S) case S: st.acc[p][0] = MFMA_BCAST(pa[p], b0, st.acc[p][0], S); st.acc[p][1] = MFMA_BCAST(pa[p], b1, st.acc[p][1], S); break;
                ODMKV_CASE(0) ODMKV_CASE(1) ODMKV_CASE(2) ODMKV_CASE(3) ODMKV_CASE(4) ODMKV_CASE(5) ODMKV_CASE(6) ODMKV_CASE(7)
                ODMKV_CASE(8) ODMKV_CASE(9) ODMKV_CASE(10) ODMKV_CASE(11) ODMKV_CASE(12) ODMKV_CASE(13) ODMKV_CASE(14) ODMKV_CASE(15)
#undef ODMKV_CASE
            }
        }
    }
}

// Exact (16-bit) tokens: the query is the fp16-rounded one itself (its low halves are zero), so only
// the high halves are fetched.  The first tile's loads are issued before anything is waited for.
template <int NP, int TW>
__device__ static inline void run_exact_level(const DecodeArgs& a, int bh, int bq_first, int nq, int nheads_all, int hbase,
                                              int tile0, int ntiles, int seg_first,
                                              int tid, uint4* qsh, WaveState<NP>& st) {
    const int wave = tid >> 6, lane = tid & 63, wq = wave % TW;
    const bool bf = a.s.exact_dtype == ODMKV_BF16;
    const float esc = a.scaling * LOG2E;
    const uint4 qslice = load_query_slice(a.qs + (size_t)bq_first * 32, tid, nq, nheads_all);
    const int count = a.s.seg_count[4][bh];          // exact segments grow between work-list rebuilds
    ExactTile cur;
    int tt = wq;
    int nvalid = tt < ntiles ? min(count - (tile0 + tt - seg_first) * TILE, TILE) : 0;
    if (nvalid > 0) load_exact_tile(cur, a, tile0 + tt, lane);
    stage_queries(qslice, qsh, tid, nq);
    lds_barrier();
    h4 qr[NP * 32];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            const uint2 v = *reinterpret_cast<const uint2*>(&qsh[(hbase + 4 * p + (lane & 3)) * QS + s]);
            qr[p * 32 + s] = as_h4(v.x, v.y);
        }
    while (nvalid > 0) {
        compute_exact_tile<NP>(cur, bf, nvalid, lane, esc, qr, st);
        tt += TW;
        nvalid = tt < ntiles ? min(count - (tile0 + tt - seg_first) * TILE, TILE) : 0;
        if (nvalid > 0) load_exact_tile(cur, a, tile0 + tt, lane);
    }
}

// ------------------------------------------------------------------------------------------------
// main kernel: four query heads per workgroup; a larger GQA group (SPLIT) is served by the two halves of
// the workgroup, wavefronts 0-3 the first four heads and wavefronts 4-7 the rest, over the same tiles
// (the second read of a tile hits the compute unit's own cache): one set-up and one launch wave per item
// ------------------------------------------------------------------------------------------------
template <int NP, bool SPLIT, bool ORDERED>
__global__ __launch_bounds__(NWAVES * 64, 2) void decode_main_kernel(DecodeArgs a) {
    constexpr int NQ = SPLIT ? 8 : 4;                     // query heads of the workgroup
    constexpr int TW = SPLIT ? NWAVES / 2 : NWAVES;       // wavefronts that share the item's tiles for the same heads
    __shared__ __align__(16) uint8_t lut[LUT_BYTES];     // centroid table; reused to combine the wavefronts
    __shared__ float wm[NWAVES][4], wl[NWAVES][4];
    __shared__ uint4 qsh[NQ * QS];

    const int item = ORDERED ? a.order[blockIdx.x] : (int)blockIdx.x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int hbase = SPLIT ? 4 * (wave / TW) : 0;       // first head (within the group) this wavefront serves
    TRACE(0)
    const int4 d0 = reinterpret_cast<const int4*>(a.items)[2 * item];       // bh, level, first tile, tiles
    const int4 d1 = reinterpret_cast<const int4*>(a.items)[2 * item + 1];   // tokens, first tile of the segment
    const int bh = d0.x, li = d0.y, tile0 = d0.z, ntiles = d0.w;
    const int bq_first = (bh / a.s.Hkv) * a.Hq + (bh % a.s.Hkv) * a.G;      // first query head of the group

    WaveState<NP> st;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        st.m[p] = -INFINITY; st.l[p] = 0.0f;
        st.acc[p][0] = (f4){0.f, 0.f, 0.f, 0.f}; st.acc[p][1] = (f4){0.f, 0.f, 0.f, 0.f};
    }
    switch (li) {
        case 0: run_quant_level<2, NP, TW>(a, 0, bq_first, NQ, a.G, hbase, tile0, ntiles, d1.x, tid, lut, qsh, st); break;
        case 1: run_quant_level<3, NP, TW>(a, 1, bq_first, NQ, a.G, hbase, tile0, ntiles, d1.x, tid, lut, qsh, st); break;
        case 2: run_quant_level<4, NP, TW>(a, 2, bq_first, NQ, a.G, hbase, tile0, ntiles, d1.x, tid, lut, qsh, st); break;
        case 3: run_quant_level<8, NP, TW>(a, 3, bq_first, NQ, a.G, hbase, tile0, ntiles, d1.x, tid, lut, qsh, st); break;
        default: run_exact_level<NP, TW>(a, bh, bq_first, NQ, a.G, hbase, tile0, ntiles, d1.y, tid, qsh, st); break;
    }

    // ---- combine the wavefronts that served the same heads (the table is no longer needed) ----
    TRACE(3)
    __syncthreads();
    TRACE(4)
    float* wacc = reinterpret_cast<float*>(lut);          // [NWAVES][4][128]
    {
        const float ls = head_sum(st.l[0]);
        if (lane < 4) { wm[wave][lane] = st.m[0]; wl[wave][lane] = ls; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wacc[(wave * 4 + i) * HD + lane] = st.acc[0][0][i];
            wacc[(wave * 4 + i) * HD + lane + 64] = st.acc[0][1][i];
        }
    }
    __syncthreads();
    float* dst = a.partial + (size_t)item * NQ * PSTRIDE;
    for (int e = tid; e < NQ * HD; e += NWAVES * 64) {
        const int g = e / HD, j = e % HD, gl = g & 3, w0 = SPLIT ? (g >> 2) * TW : 0;
        float M = wm[w0][gl];
#pragma unroll
        for (int w = 1; w < TW; ++w) M = fmaxf(M, wm[w0 + w][gl]);
        float s = 0.0f, L = 0.0f;
        if (M > -INFINITY) {
#pragma unroll
            for (int w = 0; w < TW; ++w) {
                const float f = __builtin_amdgcn_exp2f(wm[w0 + w][gl] - M);
                s = __fmaf_rn(wacc[((w0 + w) * 4 + gl) * HD + j], f, s);
                L = __fmaf_rn(wl[w0 + w][gl], f, L);
            }
        }
        dst[g * PSTRIDE + j] = s;
        if (j == 0) { dst[g * PSTRIDE + HD] = M; dst[g * PSTRIDE + HD + 1] = L; }
    }
    TRACE(5)
}

// ------------------------------------------------------------------------------------------------
// merge: one workgroup per query head
// ------------------------------------------------------------------------------------------------
#define MERGE_THREADS 512
#define MERGE_SLICES (MERGE_THREADS / HD)
#ifndef MERGE_SPLIT
#define MERGE_SPLIT 4
#endif
#define MERGE_MAX_ITEMS ODMKV_MAX_ITEMS_PER_SEGMENT

template <int GP>
__global__ __launch_bounds__(MERGE_THREADS) void decode_merge_kernel(DecodeArgs a) {
    __shared__ float wts[MERGE_MAX_ITEMS];           // exp2(m_item - M); the sign bit marks exact items
    __shared__ float red[MERGE_THREADS / 64];
    __shared__ float part[2][MERGE_SLICES][HD];      // [rotated | exact][slice][dim]
    __shared__ float rot[HD];
    __shared__ float Lsh;
    // MERGE_SPLIT workgroups per query head: each merges the head's partial results in full (they are small and
    // shared through the caches) and rotates back a quarter of the output dims, so that no workgroup has to pull
    // the whole 64 KB rotation through one compute unit
    const int bq = blockIdx.x / MERGE_SPLIT, quarter = blockIdx.x % MERGE_SPLIT;
    const int tid = threadIdx.x, j = tid & (HD - 1), slice = tid >> 7;
    const int b = bq / a.Hq, hq = bq % a.Hq;
    const int bh = b * a.s.Hkv + hq / a.G, g = hq % a.G;
    const int i0 = a.item_range[bh], n = min(a.item_range[bh + 1] - i0, MERGE_MAX_ITEMS);
    // Everything that does not depend on the weights is requested now, in one round trip: this thread's
    // share of the value rotation, the first MERGE_PRE accumulator values of its slice, its item's (m, l, level)
    constexpr int QD = HD / MERGE_SPLIT;                 // output dims of this workgroup
    constexpr int RS = MERGE_THREADS / QD;                // row slices of the rotation
    constexpr int IN = HD / RS;                           // rows per slice
    const int jj = tid % QD, rs = tid / QD;
    float pv[IN];
#pragma unroll
    for (int ii = 0; ii < IN; ++ii) pv[ii] = a.pi_v[(size_t)(rs * IN + ii) * HD + quarter * QD + jj];
    constexpr int MERGE_PRE = 16;
    float pre[MERGE_PRE];
#pragma unroll
    for (int k = 0; k < MERGE_PRE; ++k) {
        const int it = slice + k * MERGE_SLICES;
        pre[k] = it < n ? a.partial[((size_t)(i0 + it) * GP + g) * PSTRIDE + j] : 0.0f;
    }
    float my_m = -INFINITY, my_l = 0.0f;
    int my_level = 0;
    if (tid < n) {
        const float* p = a.partial + ((size_t)(i0 + tid) * GP + g) * PSTRIDE;
        my_m = p[HD]; my_l = p[HD + 1];
        my_level = a.items[8 * (i0 + tid) + 1];
    }
    // maximum over the items
    float mx = my_m;
    for (int it = tid + MERGE_THREADS; it < n; it += MERGE_THREADS)
        mx = fmaxf(mx, a.partial[((size_t)(i0 + it) * GP + g) * PSTRIDE + HD]);
    mx = wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    float M = red[0];
#pragma unroll
    for (int w = 1; w < MERGE_THREADS / 64; ++w) M = fmaxf(M, red[w]);
    __syncthreads();
    // weights and the normaliser
    float lpart = 0.0f;
    if (tid < n) {
        const float f = M > -INFINITY ? __builtin_amdgcn_exp2f(my_m - M) : 0.0f;
        lpart = my_l * f;
        wts[tid] = my_level == 4 ? -f : f;
    }
    for (int it = tid + MERGE_THREADS; it < n; it += MERGE_THREADS) {
        const float* p = a.partial + ((size_t)(i0 + it) * GP + g) * PSTRIDE;
        const float f = M > -INFINITY ? __builtin_amdgcn_exp2f(p[HD] - M) : 0.0f;
        lpart = __fmaf_rn(p[HD + 1], f, lpart);
        wts[it] = a.items[8 * (i0 + it) + 1] == 4 ? -f : f;
    }
    lpart = wave_sum(lpart);
    if ((tid & 63) == 0) red[tid >> 6] = lpart;
    __syncthreads();
    if (tid == 0) {
        float L = 0.0f;
        for (int w = 0; w < MERGE_THREADS / 64; ++w) L += red[w];
        Lsh = L;
    }
    float arot = 0.0f, aex = 0.0f;
    __syncthreads();                                   // weights written
#pragma unroll
    for (int k = 0; k < MERGE_PRE; ++k) {
        const int it = slice + k * MERGE_SLICES;
        if (it < n) {
            const float w = wts[it];
            if (__float_as_uint(w) >> 31) aex = __fmaf_rn(pre[k], -w, aex);
            else arot = __fmaf_rn(pre[k], w, arot);
        }
    }
#pragma unroll 4
    for (int it = slice + MERGE_PRE * MERGE_SLICES; it < n; it += MERGE_SLICES) {
        const float w = wts[it];
        const float v = a.partial[((size_t)(i0 + it) * GP + g) * PSTRIDE + j];
        if (__float_as_uint(w) >> 31) aex = __fmaf_rn(v, -w, aex);
        else arot = __fmaf_rn(v, w, arot);
    }
    part[0][slice][j] = arot;
    part[1][slice][j] = aex;
    __syncthreads();
    if (tid < HD) {
        float r = 0.0f;
#pragma unroll
        for (int s = 0; s < MERGE_SLICES; ++s) r += part[0][s][tid];
        rot[tid] = r;
    }
    __syncthreads();
    // rotate the quantised part back: out_j = sum_i rot_i Pi_v[i][j] for this workgroup's dims; the slices split the i range
    float o = 0.0f;
#pragma unroll
    for (int ii = 0; ii < IN; ++ii) o = __fmaf_rn(rot[rs * IN + ii], pv[ii], o);
    __syncthreads();
    float* part2 = &part[0][0][0];                        // [RS][QD], the first half of `part` is free again
    part2[rs * QD + jj] = o;
    __syncthreads();
    if (tid < QD) {
        const int dim = quarter * QD + tid;
        float tot = 0.0f;
#pragma unroll
        for (int r = 0; r < RS; ++r) tot += part2[r * QD + tid];
#pragma unroll
        for (int s = 0; s < MERGE_SLICES; ++s) tot += part[1][s][dim];
        const float L = Lsh;
        const float o32 = L > 0.0f ? tot / L : 0.0f;
        const size_t oi = (size_t)bq * HD + dim;
        if (a.out_dt == ODMKV_F32) reinterpret_cast<float*>(a.out)[oi] = o32;
        else if (a.out_dt == ODMKV_F16) reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_F16>::from_f32(o32);
        else reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_BF16>::from_f32(o32);
        if (a.lse && tid == 0 && quarter == 0) a.lse[bq] = L > 0.0f ? (M + __log2f(L)) * LN2 : -INFINITY;
    }
}

// ---- measurement hooks: event pairs around the main kernel ----
#include <vector>
static std::vector<hipEvent_t> g_prof_events;   // 2 per record
static int g_prof_used = 0;
static bool g_prof_on = false;

extern "C" int odmkv_profile_disable(void) {
    for (auto& e : g_prof_events) (void)hipEventDestroy(e);
    g_prof_events.clear();
    g_prof_used = 0;
    g_prof_on = false;
    return 0;
}

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

// plain streaming read of a buffer (grid-stride 16-byte loads folded into one word per thread):
// the yardstick for what a single launch of a given size can reach on the machine
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, size_t n16, unsigned int* sink) {
    unsigned int acc = 0u;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
        const uint4 v = p[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;       // practically never taken: keeps the loads alive
}

extern "C" int odmkv_probe_read(const void* buf, size_t bytes, int grid, void* sink, void* stream) {
    ODMKV_CHECK_ARG(buf && sink && grid > 0 && ((uintptr_t)buf & 15) == 0, "probe_read: bad arguments");
    hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint4*>(buf), bytes / 16, reinterpret_cast<unsigned int*>(sink));
    ODMKV_CHECK_LAUNCH("probe_read_kernel");
    return 0;
}

static int g_stage_mask = 7;
extern "C" int odmkv_decode_stage_mask(int mask) {
    const int old = g_stage_mask;
    g_stage_mask = mask & 7;
    return old;
}

static inline int group_pad(int G) { return G <= 4 ? 4 : 8; }

extern "C" size_t odmkv_decode_workspace_bytes(int B, int Hq, int n_items) {
    size_t q = align_up((size_t)B * Hq * 32 * sizeof(uint4), 256);
    return 2 * q + align_up((size_t)n_items * ODMKV_MAX_GROUP * PSTRIDE * sizeof(float), 256);
}

static int decode_launch(const void* q, int q_dtype, int B, int Hq, float scaling,
                         const odmkv_packed_t* store,
                         const int32_t* items, int n_items, const int32_t* item_range,
                         const int32_t* dispatch_order,
                         const float* pi_k_t, const float* pi_v, const float* codebooks,
                         const float* codebooks_host, const float* inv_scales,
                         void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                         void* stream) {
    ODMKV_CHECK_ARG(q_dtype == ODMKV_F16 || q_dtype == ODMKV_BF16 || q_dtype == ODMKV_F32, "decode_attn: bad query dtype %d", q_dtype);
    ODMKV_CHECK_ARG(out_dtype == ODMKV_F16 || out_dtype == ODMKV_BF16 || out_dtype == ODMKV_F32, "decode_attn: bad output dtype %d", out_dtype);
    ODMKV_CHECK_ARG(codebooks_host != nullptr, "decode_attn: null host copy of the centroid tables");
    ODMKV_CHECK_ARG(inv_scales != nullptr, "decode_attn: null table scales");
    ODMKV_CHECK_ARG(q && store && item_range && pi_k_t && pi_v && codebooks && out && workspace, "decode_attn: null pointer");
    ODMKV_CHECK_ARG(n_items == 0 || items, "decode_attn: null work list");
    ODMKV_CHECK_ARG(B > 0 && Hq > 0 && store->B == B && store->Hkv > 0 && Hq % store->Hkv == 0,
                    "decode_attn: bad head counts B=%d Hq=%d store(B=%d,Hkv=%d)", B, Hq, store->B, store->Hkv);
    const int G = Hq / store->Hkv;
    ODMKV_CHECK_ARG(G <= ODMKV_MAX_GROUP, "decode_attn: GQA group %d exceeds %d", G, ODMKV_MAX_GROUP);
    ODMKV_CHECK_ARG(n_items >= 0, "decode_attn: negative item count");
    ODMKV_CHECK_ARG((long)n_items <= (long)ODMKV_MAX_ITEMS_PER_SEGMENT * B * store->Hkv,
                    "decode_attn: %d items exceed %d per (sequence, kv-head)", n_items, ODMKV_MAX_ITEMS_PER_SEGMENT);
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_decode_workspace_bytes(B, Hq, n_items), "decode_attn: workspace too small");
    hipStream_t st = (hipStream_t)stream;
    DecodeArgs a;
    a.s = *store; a.q = q; a.q_dt = q_dtype; a.out_dt = out_dtype; a.Hq = Hq; a.G = G; a.B = B; a.scaling = scaling;
    a.items = items; a.item_range = item_range; a.order = dispatch_order;
    a.pi_k_t = pi_k_t; a.pi_v = pi_v; a.cb = codebooks;
    for (int w = 0; w < 4; ++w) a.inv_s[w] = inv_scales[w];
    for (int k = 0; k < 28; ++k) a.cbs[k] = codebooks_host[k];
    const size_t qbytes = align_up((size_t)B * Hq * 32 * sizeof(uint4), 256);
    a.qrot = (uint4*)workspace;
    a.qs = (uint4*)((char*)workspace + qbytes);
    a.partial = (float*)((char*)workspace + 2 * qbytes);
    a.out = out; a.lse = lse;
    if (g_stage_mask & 1) {
        hipLaunchKernelGGL(decode_prep_kernel, dim3(B * Hq * PREP_SPLIT), dim3(PREP_THREADS), 0, st, a);
        ODMKV_CHECK_LAUNCH("decode_prep_kernel");
    }
    const int GP = group_pad(G);
    a.gp = GP;
    if (n_items > 0 && (g_stage_mask & 2)) {
        const bool rec = g_prof_on && (size_t)(2 * g_prof_used + 1) < g_prof_events.size();
        // when measuring, the events are attached to the dispatch itself: they carry the kernel's own
        // start and end timestamps, not those of separate marker packets
        hipEvent_t e0 = rec ? g_prof_events[2 * g_prof_used] : nullptr;
        hipEvent_t e1 = rec ? g_prof_events[2 * g_prof_used + 1] : nullptr;
        // (the plain case keeps its own instantiation: a branch on either option at the kernel's start costs it 0.25 us)
        if (GP == 4 && !a.order) hipExtLaunchKernelGGL((decode_main_kernel<1, false, false>), dim3(n_items), dim3(NWAVES * 64), 0, st, e0, e1, 0, a);
        else if (GP == 4) hipExtLaunchKernelGGL((decode_main_kernel<1, false, true>), dim3(n_items), dim3(NWAVES * 64), 0, st, e0, e1, 0, a);
        else if (!a.order) hipExtLaunchKernelGGL((decode_main_kernel<1, true, false>), dim3(n_items), dim3(NWAVES * 64), 0, st, e0, e1, 0, a);
        else hipExtLaunchKernelGGL((decode_main_kernel<1, true, true>), dim3(n_items), dim3(NWAVES * 64), 0, st, e0, e1, 0, a);
        ODMKV_CHECK_LAUNCH("decode_main_kernel");
        if (rec) ++g_prof_used;
    }
    if (g_stage_mask & 4) {
        if (GP == 4) hipLaunchKernelGGL((decode_merge_kernel<4>), dim3(B * Hq * MERGE_SPLIT), dim3(MERGE_THREADS), 0, st, a);
        else hipLaunchKernelGGL((decode_merge_kernel<8>), dim3(B * Hq * MERGE_SPLIT), dim3(MERGE_THREADS), 0, st, a);
        ODMKV_CHECK_LAUNCH("decode_merge_kernel");
    }
    return 0;
}

extern "C" int odmkv_decode_attn(const void* q, int q_dtype, int B, int Hq, float scaling,
                                 const odmkv_packed_t* store,
                                 const int32_t* items, int n_items, const int32_t* item_range,
                                 const int32_t* dispatch_order,
                                 const float* pi_k_t, const float* pi_v, const float* codebooks,
                                 const float* codebooks_host, const float* inv_scales,
                                 void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    return decode_launch(q, q_dtype, B, Hq, scaling, store, items, n_items, item_range, dispatch_order, pi_k_t, pi_v,
                         codebooks, codebooks_host, inv_scales, out, out_dtype, lse, workspace, workspace_bytes, stream);
}

// ------------------------------------------------------------------------------------------------
// The same call for callers that cannot allocate and have no workspace to hand over: the partial
// results and the prepared queries live in a fixed array of the library's own device image.
// ------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[ODMKV_STATIC_SCRATCH_BYTES];

#include <mutex>
#define ODMKV_MAX_DEVICES 64
static void* g_scratch_ptr[ODMKV_MAX_DEVICES];      // device address of `scratch` per device, looked up once
static std::mutex g_scratch_mutex;

// the address of this device's copy of `scratch` (every device that loads the library holds its own)
static int static_scratch(void** ptr) {
    int dev = -1;
    ODMKV_CHECK_HIP(hipGetDevice(&dev));
    ODMKV_CHECK_ARG(dev >= 0 && dev < ODMKV_MAX_DEVICES, "decode_attn_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        ODMKV_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" int odmkv_decode_attn_static(const void* q, int q_dtype, int B, int Hq, float scaling,
                                        const odmkv_packed_t* store,
                                        const int32_t* items, int n_items, const int32_t* item_range,
                                        const int32_t* dispatch_order,
                                        const float* pi_k_t, const float* pi_v, const float* codebooks,
                                        const float* codebooks_host, const float* inv_scales,
                                        void* out, int out_dtype, float* lse, void* stream) {
    ODMKV_CHECK_ARG(B > 0 && Hq > 0 && n_items >= 0, "decode_attn_static: bad shape B=%d Hq=%d items=%d", B, Hq, n_items);
    const size_t need = odmkv_decode_workspace_bytes(B, Hq, n_items);
    if (need > (size_t)ODMKV_STATIC_SCRATCH_BYTES) {
        odmkv_set_error("decode_attn_static: B=%d Hq=%d items=%d need %zu bytes of scratch, the fixed array holds %zu; "
                        "use odmkv_decode_attn with a workspace", B, Hq, n_items, need, (size_t)ODMKV_STATIC_SCRATCH_BYTES);
        return ODMKV_ENOSPACE;
    }
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return decode_launch(q, q_dtype, B, Hq, scaling, store, items, n_items, item_range, dispatch_order, pi_k_t, pi_v,
                         codebooks, codebooks_host, inv_scales, out, out_dtype, lse, ws, (size_t)ODMKV_STATIC_SCRATCH_BYTES, stream);
}
