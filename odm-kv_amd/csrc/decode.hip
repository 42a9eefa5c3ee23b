// Fused LUT decode attention over the packed mixed-width KV store (one query token per sequence; a block of query
// tokens is handed over as further heads of their kv-head).
//
// Two launches per call:
//   1. main:  one workgroup (8, 12 or 16 wavefronts) per work item = a run of 64-token tiles of one (sequence,
//             kv-head, level).  It rounds the group's queries to fp16 (what a model in fp16/bf16 hands over
//             anyway), rotates them into the basis of the quantised keys on the matrix cores (q' = Pi_k q16 from a
//             precomputed fp16 high + low operand table, kept as fp16 high + low rows), and streams the item's packed
//             bytes once from HBM; nothing else is read from there.  A workgroup may take several consecutive items
//             (the quantised levels of one (sequence, kv-head): a chain) with one rotation and one result.  For lists
//             with more items than compute units there is a build of the eight-wavefront workgroup that two of share
//             a compute unit (128 registers a wavefront, half the LDS): one streams while the other starts or ends.
//   2. merge: log-sum-exp merge of a kv-head's items per query head, rotation of the quantised
//             part back to the model basis (acc . Pi_v), addition of the exact part, normalise (one to four workgroups
//             per query head; from 512 heads on one workgroup per (sequence, kv-head) for all heads of the group).
// (Merging inside the main kernel, by the workgroup that finishes last among a kv-head's items, was built
// and measured twice: the count and the other workgroups' results have to cross the device at agent scope, two
// to three dependent trips to memory of 2-3 us each under the streaming load, against one launch of 4-5 us.
// A separate query-preparation launch was measured too: the same time per call, one launch more.)
//
// Two forms of the quantised levels: the general one (compute_unit: up to 8 heads of a group in one pass), and one for
// groups of up to four heads at four wavefronts per SIMD (sixteen wavefronts, or two workgroups of eight;
// compute_unit_g4: the lanes are shared out between a unit's two token blocks, the softmax step runs once per unit).
//
// Main kernel, per wavefront and unit of 32 tokens (half a tile), on v_mfma_f32_16x16x32_f16 (D[16x16] += A[16x32]
// B[32x16]; lane l supplies A[l%16][8(l/16)+e] and B[8(l/16)+e][l%16], e = 0..7, and holds D[4(l/16)+r][l%16]):
//   keys    A = the queries: row 2h = high half of head h, row 2h+1 = low half (up to 8 heads of the
//           GQA group, 16 bytes per lane and step, read from LDS once per work item).  B = the centroids of
//           16 tokens x 32 dims, fetched from an LDS table by the code bytes; the packed layout puts
//           the codes of (2 tokens x 32 dims) per unit into each lane's bytes.  2 token blocks x 4 dim
//           blocks = 8 matrix instructions; lane (n, j) then holds the logits of its two slots
//           (one per block) for heads 2j and 2j+1.
//   softmax two heads per lane, base-2 exponentials, running (m, l) per head, m a reference point that moves
//           (DPP row reduction, rescale of the accumulators) only when a logit exceeds it by more than a slack;
//           p |v| is rounded to fp16 and handed to the value product through a per-wave LDS buffer (the product
//           needs tokens along the contraction).
//   values  A = p |v| (row = head), B = the centroids of 32 tokens x 16 dims; 8 matrix instructions accumulate
//           sum_t p_t |v_t| c[code] for 8 heads x 128 dims in the rotated basis.
// The LDS table is replicated over 32 slots (slot = lane % 32) so that lanes never share a bank.
// All softmax state is kept in base-2 logarithms.
#include "decode.h"
#include <stdlib.h>

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

#define LUT_BYTES 65536
#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f
#define UNIT 32             // tokens of a unit of work: half a tile
#define PROW 96             // bytes per head row of a wave's p buffer: 32 x 16 bit + padding (bank spread)
#define PBUF (8 * PROW)     // one p buffer: 8 head rows

// LDS of the main kernel: [table, later the combine area] [rotated query rows]
// [p buffers] [per-wave scalars].  NW = wavefronts of the workgroup: 8 (short items: less set-up and a lighter combine),
// 16 (long items: four wavefronts per SIMD keep its issue slots full) or 12 (three units in flight per wavefront).
// One p buffer per wavefront (bf16 exact rows need a second one for the weights' low pieces: it lies in the table's
// space, which an exact item does not use), so that eight wavefronts stay under half a compute unit's 160 KB.
#define QROW_LDS 272                             // bytes of a query row in LDS: 128 x 16 bit + 16 (bank spread)
#define LDS_QROWS LUT_BYTES
#define LDS_PBUFS (LDS_QROWS + 16 * QROW_LDS)
template <int NW>
struct Lds {
    static constexpr int SCALARS = LDS_PBUFS + NW * PBUF;
    static constexpr int TOTAL = SCALARS + NW * 4 * 8 * 4 + 8 * 4;
    static_assert(NW * ODMKV_MAX_GROUP * HD * 4 <= LUT_BYTES, "combine area must fit the table's space");
    static_assert(NW >= 8 && NW <= 16, "wave count (the first eight rotate the queries)");
    static_assert(TOTAL <= 160 * 1024, "LDS of one workgroup");
};

__device__ static inline uint32_t half_bits(float f) { return (uint32_t)__half_as_ushort(__float2half_rn(f)); }

// ------------------------------------------------------------------------------------------------
// small helpers
// ------------------------------------------------------------------------------------------------
__device__ static inline h4 as_h4(uint32_t lo, uint32_t hi) {
    union { uint32_t u[2]; h4 h; } x;
    x.u[0] = lo; x.u[1] = hi;
    return x.h;
}
__device__ static inline h8 as_h8(const uint4& v) {
    union { uint4 u; h8 h; } x;
    x.u = v;
    return x.h;
}
__device__ static inline bf8 as_bf8(const uint4& v) {
    union { uint4 u; bf8 h; } x;
    x.u = v;
    return x.h;
}
__device__ static inline h8 join(const h4& lo, const h4& hi) { return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }

template <int CTRL>
__device__ static inline float dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
#define DPP_ROR(n) (0x120 + (n))

// reduce over the 16 lanes of a row (lanes that share lane / 16); every lane ends with the result
__device__ static inline float row_max(float v) {
    v = fmaxf(v, dpp<DPP_ROR(8)>(v));
    v = fmaxf(v, dpp<DPP_ROR(4)>(v));
    v = fmaxf(v, dpp<DPP_ROR(2)>(v));
    v = fmaxf(v, dpp<DPP_ROR(1)>(v));
    return v;
}
// the same for two values at once, as fused DPP instructions (the two chains fill each other's wait states)
__device__ static inline void row_max2(float& a, float& b) {
    asm volatile(
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "+v"(b));
}
__device__ static inline float row_sum(float v) {
    v += dpp<DPP_ROR(8)>(v);
    v += dpp<DPP_ROR(4)>(v);
    v += dpp<DPP_ROR(2)>(v);
    v += dpp<DPP_ROR(1)>(v);
    return v;
}

// workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight
// (__syncthreads would first wait for every outstanding load of the wavefront)
__device__ static inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// LDS writes of this wave visible to its own later reads (no other wave touches its p buffer)
__device__ static inline void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

#define MFMA_F16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_f16((a), (b), (c), 0, 0, 0)
#define MFMA_BF16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16((a), (b), (c), 0, 0, 0)

// ------------------------------------------------------------------------------------------------
// LDS tables: code group -> fp16 centroids, replicated over 32 slots
//   W = 2: index = byte (4 codes) -> 4 halfs (8 bytes),  row = 256 bytes
//   W = 3: index = 6 bits (2 codes) -> 2 halfs (4 bytes), row = 128 bytes
//   W = 4: index = byte (2 codes) -> 2 halfs,             row = 128 bytes
//   W = 8: index = byte (1 code)  -> the centroid's fp16 high half (low word) and low half (high word), row = 128 bytes
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
template <int W, int NW>
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
        // groups of four rows go round the wavefronts
#pragma unroll
        for (int i = 0; i < (64 + NW - 1) / NW; ++i) {
            const int base = (i * NW + wave) * 4;            // wave-uniform; the row is base + (lane >> 4)
            if (base >= 256) break;
            const uint32_t x = own | (sel((base >> 2) & 3) << 16), y = sel((base >> 4) & 3) | (sel(base >> 6) << 16);
            *reinterpret_cast<uint4*>(lut + (base + (lane >> 4)) * 256 + (lane & 15) * 16) = make_uint4(x, y, x, y);
        }
    } else {
        uint32_t v;
        if constexpr (W == 3) { v = half_bits(pick<8>(a.cbs + 4, tid & 7)) | (half_bits(pick<8>(a.cbs + 4, (tid >> 3) & 7)) << 16); }
        else if constexpr (W == 4) { v = half_bits(pick<16>(a.cbs + 12, tid & 15)) | (half_bits(pick<16>(a.cbs + 12, (tid >> 4) & 15)) << 16); }
        else {
            // the 256-entry table does not round well to fp16 as a whole (no common scale suits 128 magnitudes): an
            // entry keeps the centroid's high half and, in its upper 16 bits, the low half
            const float c = a.cb[codebook_offset(3) + (tid & 255)];
            const __half hi = __float2half_rn(c);
            v = (uint32_t)__half_as_ushort(hi) | (half_bits(c - __half2float(hi)) << 16);
        }
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
        return as_h4(__builtin_amdgcn_perm(t1, t0, 0x05040100u), __builtin_amdgcn_perm(t3, t2, 0x05040100u));     // the high halves
    } else {
        const int bit = 12 * s, k = bit >> 5, sh = bit & 31;
        uint32_t x = w[k] >> sh;
        if (sh + 12 > 32) x |= w[k + 1] << (32 - sh);
        const uint32_t lo = *reinterpret_cast<const uint32_t*>(lut + ((x & 63u) << 7) + slot4);
        const uint32_t hi = *reinterpret_cast<const uint32_t*>(lut + (((x >> 6) & 63u) << 7) + slot4);
        return as_h4(lo, hi);
    }
}
// 8-bit codes 8g..8g+7: the high halves and the low halves of the centroids, two matrix operands
__device__ static inline void lut8_split(const uint32_t* w, int g, const uint8_t* lut, uint32_t slot4, h8& hi, h8& lo) {
    uint32_t t[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t x = w[2 * g + (e >> 2)] >> (8 * (e & 3));
        t[e] = *reinterpret_cast<const uint32_t*>(lut + ((x & 0xffu) << 7) + slot4);
    }
    uint32_t h[4], l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        h[e] = __builtin_amdgcn_perm(t[2 * e + 1], t[2 * e], 0x05040100u);       // low words of the two entries
        l[e] = __builtin_amdgcn_perm(t[2 * e + 1], t[2 * e], 0x07060302u);       // high words
    }
    hi = join(as_h4(h[0], h[1]), as_h4(h[2], h[3]));
    lo = join(as_h4(l[0], l[1]), as_h4(l[2], l[3]));
}
// centroids of codes 8g..8g+7 of the stream: one matrix operand
template <int W>
__device__ static inline h8 lut8(const uint32_t* w, int g, const uint8_t* lut, uint32_t slot4) {
    return join(lut4<W>(w, 2 * g, lut, slot4), lut4<W>(w, 2 * g + 1, lut, slot4));
}

// ------------------------------------------------------------------------------------------------
// per-wavefront running state.  Softmax: lane (n = lane % 16, j = lane / 16) keeps heads 2j and 2j+1
// (m: running maximum, l: this lane's share of the running sum).  Output: lane (n, j) keeps
// acc[nb][r] = head 4j+r (heads 8..15 repeat 0..7), dim 16nb+n, in the rotated (or model) basis.
// ------------------------------------------------------------------------------------------------
struct WaveState {
    float mA, mB, lA, lB;
    f4 acc[8];
};

// the packed codes are read once per call and never again before the whole cache has streamed by:
// loaded with the non-temporal hint, so that they do not push the small per-layer operands (rotations,
// work lists, queries) out of the caches
__device__ static inline uint4 stream_load(const uint4* p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// eight consecutive elements of the query: the request (one or two 16-byte loads) and, apart from it, the
// conversion to floats rounded to fp16 (the precision at which the attention this call replaces consumes its
// query).  Keeping them apart lets other requests be issued before the first value is needed.
struct RawQ8 { uint4 x, y; };
__device__ static inline RawQ8 request_q8(const void* q, int dt, size_t elem) {
    RawQ8 r;
    if (dt == ODMKV_F32) {
        r.x = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(q) + elem);
        r.y = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(q) + elem + 4);
    } else {
        r.x = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(q) + elem);
        r.y = make_uint4(0u, 0u, 0u, 0u);
    }
    return r;
}
// (fp32 and bf16 queries beyond fp16's range saturate at +-65504 instead of becoming infinite)
__device__ static inline float to_q16(float x) { return __half2float(__float2half_rn(fminf(fmaxf(x, -65504.0f), 65504.0f))); }
__device__ static inline void convert_q8(const RawQ8& r, int dt, float* out) {
    const uint32_t w[8] = {r.x.x, r.x.y, r.x.z, r.x.w, r.y.x, r.y.y, r.y.z, r.y.w};
    if (dt == ODMKV_F32) {
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = to_q16(__uint_as_float(w[e]));
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint16_t bits = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            out[e] = dt == ODMKV_F16 ? Elem<ODMKV_F16>::to_f32(bits) : to_q16(Elem<ODMKV_BF16>::to_f32(bits));
        }
    }
}
__device__ static inline void load_q8(const void* q, int dt, size_t elem, float* out) { convert_q8(request_q8(q, dt, elem), dt, out); }

__device__ static inline uint32_t bf16_pair(float a, float b) {
    return (uint32_t)Elem<ODMKV_BF16>::from_f32(a) | ((uint32_t)Elem<ODMKV_BF16>::from_f32(b) << 16);
}
__device__ static inline float bf16_rest(float a) { return a - Elem<ODMKV_BF16>::to_f32(Elem<ODMKV_BF16>::from_f32(a)); }

__device__ static inline uint32_t pack_h2(float a, float b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    union { h2 h; uint32_t u; } x;
    x.h = (h2){(_Float16)a, (_Float16)b};
    return x.u;
}

// Softmax step of one unit (32 tokens) for this lane's two heads.  tA/tB: base-2 logits of the lane's two
// slots (padding: -inf).  Returns the weights p = exp2(t - m) and updates (m, l).  m is a reference point, not
// the exact running maximum: it moves (and the accumulators are rescaled) only when a logit exceeds it by more
// than SOFTMAX_SLACK, so p stays below 2^SOFTMAX_SLACK and most units need neither a cross-lane reduction nor a
// pass over the accumulators.  Any reference point gives the same quotient sum(p v) / sum(p).
// The weights are kept 2^P_SHIFT times larger than that: they reach the matrix instructions as fp16, whose normal
// range ends at 6e-5, and in a long context next to a dominant token most weights lie far below (rounded to a few bits,
// or to zero, as they would otherwise be).  The normaliser carries the same factor, so the quotient does not; the
// merge takes it out of the log-sum-exp.
#define SOFTMAX_SLACK 3.0f
#define P_SHIFT 8.0f
#define FP16_MAX 65504.0f
__device__ static inline void softmax_unit(WaveState& st, const float* tA, const float* tB, int lane,
                                           float* alpha_sh, float* pA, float* pB) {
    const int n = lane & 15, j = lane >> 4;
    float mxA = fmaxf(tA[0], tA[1]);
    float mxB = fmaxf(tB[0], tB[1]);
    if (__builtin_amdgcn_ballot_w64(mxA > st.mA + SOFTMAX_SLACK || mxB > st.mB + SOFTMAX_SLACK) != 0) {      // wave-uniform
        row_max2(mxA, mxB);
        const float mnA = fmaxf(st.mA, mxA), mnB = fmaxf(st.mB, mxB);
        if (__builtin_amdgcn_ballot_w64(st.mA > -INFINITY || st.mB > -INFINITY) != 0) {     // not the wave's first unit
            const float aA = __builtin_amdgcn_exp2f(st.mA - mnA), aB = __builtin_amdgcn_exp2f(st.mB - mnB);
            st.lA *= aA; st.lB *= aB;
            if (n == 0) { alpha_sh[2 * j] = aA; alpha_sh[2 * j + 1] = aB; }
            wave_lds_fence();
            const f4 al = *reinterpret_cast<const f4*>(alpha_sh + 4 * (j & 1));      // heads 4j..4j+3 of the output rows
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) st.acc[nb] *= al;
        }
        st.mA = mnA; st.mB = mnB;
    }
    const float mnA = st.mA - P_SHIFT, mnB = st.mB - P_SHIFT;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        pA[b] = __builtin_amdgcn_exp2f(tA[b] - mnA);      // padded slots: -inf -> 0
        pB[b] = __builtin_amdgcn_exp2f(tB[b] - mnB);
    }
    st.lA += pA[0] + pA[1];
    st.lB += pB[0] + pB[1];
}

// this lane's two slots inside a unit are 2 * pair_slot(n) and the next one (see key_slot)
__device__ static inline int pair_slot(int n) { return 8 * (n >> 2) + 2 * (n & 3); }

// ---- quantised units -----------------------------------------------------------------------------
// Unit h of a tile = slots 32h .. 32h+31 = the h-th half of every lane's code bytes:
//   keys:   the lane's 64 codes of the unit are  code 32b + i = dim 32j + i of slot 32h + pair_slot(n) + b
//   values: the lane's 64 codes of the unit are  code 8m + e  = slot 32h + 8j + e of dim 16m + n
template <int W>
struct Unit {
    uint32_t kw[2 * W];
    uint32_t vw[2 * W];
    f2 kn, vn;
};

// the h-th half (8 * W bytes) of a lane's 16 * W bytes of a tile buffer
template <int W>
__device__ static inline void load_half_stream(uint32_t* w, const uint8_t* tile_base, int h, int lane) {
    if constexpr (W == 3) {
        // 24 bytes: chunk 0 and half of chunk 1, or the other half of chunk 1 and chunk 2
        const uint8_t* mid = tile_base + ((size_t)TILE + lane) * 16;
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        if (h == 0) {
            const uint4 x = stream_load(reinterpret_cast<const uint4*>(tile_base + (size_t)lane * 16));
            const u32x2 y = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(mid));
            w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w; w[4] = y.x; w[5] = y.y;
        } else {
            const u32x2 y = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(mid + 8));
            const uint4 x = stream_load(reinterpret_cast<const uint4*>(tile_base + ((size_t)2 * TILE + lane) * 16));
            w[0] = y.x; w[1] = y.y; w[2] = x.x; w[3] = x.y; w[4] = x.z; w[5] = x.w;
        }
    } else {
        constexpr int C = W / 2;                            // whole 16-byte chunks per half
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const uint4 v = stream_load(reinterpret_cast<const uint4*>(tile_base + ((size_t)(C * h + c) * TILE + lane) * 16));
            w[4 * c] = v.x; w[4 * c + 1] = v.y; w[4 * c + 2] = v.z; w[4 * c + 3] = v.w;
        }
    }
}

template <int W>
__device__ static inline void load_unit(Unit<W>& t, const DecodeArgs& a, int li, int unit, int lane) {
    const int tile = unit >> 1, h = unit & 1;               // wave-uniform
    load_half_stream<W>(t.kw, a.s.kcodes[li] + (size_t)tile * (TILE * 16 * W), h, lane);
    load_half_stream<W>(t.vw, a.s.vcodes[li] + (size_t)tile * (TILE * 16 * W), h, lane);
    const size_t pair = (size_t)unit * UNIT + pair_slot(lane & 15);
    t.kn = __builtin_nontemporal_load(reinterpret_cast<const f2*>(a.s.knorm[li] + pair));
    t.vn = __builtin_nontemporal_load(reinterpret_cast<const f2*>(a.s.vnorm[li] + pair));
}

template <int W>
__device__ static inline void compute_unit(const Unit<W>& t, int nvalid, int lane, const uint8_t* lut,
                                           uint32_t slot4, const h8* qa, float ksc, float vsc,
                                           uint8_t* pbuf, float* alpha_sh, WaveState& st) {
    const int n = lane & 15, j = lane >> 4;
    // ---- keys: D[q row][token], two token blocks x four dim blocks ----
    f4 dk[2];
    dk[0] = (f4){0.f, 0.f, 0.f, 0.f};
    dk[1] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if constexpr (W == 8) {
                h8 chi, clo;
                lut8_split(t.kw, 4 * b + kb, lut, slot4, chi, clo);
                dk[b] = MFMA_F16(qa[kb], chi, dk[b]);
                dk[b] = MFMA_F16(qa[kb], clo, dk[b]);
            } else {
                dk[b] = MFMA_F16(qa[kb], lut8<W>(t.kw, 4 * b + kb, lut, slot4), dk[b]);
            }
        }
    float tA[2], tB[2];
    {
        const float kn0 = t.kn.x * ksc, kn1 = t.kn.y * ksc;
        tA[0] = (dk[0][0] + dk[0][1]) * kn0; tB[0] = (dk[0][2] + dk[0][3]) * kn0;
        tA[1] = (dk[1][0] + dk[1][1]) * kn1; tB[1] = (dk[1][2] + dk[1][3]) * kn1;
    }
    if (nvalid < UNIT) {                                   // the last unit of a run (wave-uniform)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const bool ok = pair_slot(n) + b < nvalid;
            tA[b] = ok ? tA[b] : -INFINITY;
            tB[b] = ok ? tB[b] : -INFINITY;
        }
    }
    float pA[2], pB[2];
    softmax_unit(st, tA, tB, lane, alpha_sh, pA, pB);
    {
        // p |v| as fp16 into the lane's two slots (bytes 2 * pair_slot(n) = 4n .. 4n+3) of rows 2j and 2j+1
        const float vn0 = t.vn.x * vsc, vn1 = t.vn.y * vsc;
        // (the clamp only matters for value norms thousands of times the table's scale: no infinities)
        *reinterpret_cast<uint32_t*>(pbuf + (2 * j) * PROW + 4 * n) = pack_h2(fminf(pA[0] * vn0, FP16_MAX), fminf(pA[1] * vn1, FP16_MAX));
        *reinterpret_cast<uint32_t*>(pbuf + (2 * j + 1) * PROW + 4 * n) = pack_h2(fminf(pB[0] * vn0, FP16_MAX), fminf(pB[1] * vn1, FP16_MAX));
    }
    wave_lds_fence();
    // ---- values: D[head][dim], eight dim blocks ----
    const h8 pa = as_h8(*reinterpret_cast<const uint4*>(pbuf + (n & 7) * PROW + 16 * j));
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        if constexpr (W == 8) {
            h8 chi, clo;
            lut8_split(t.vw, m, lut, slot4, chi, clo);
            st.acc[m] = MFMA_F16(pa, chi, st.acc[m]);
            st.acc[m] = MFMA_F16(pa, clo, st.acc[m]);
        } else {
            st.acc[m] = MFMA_F16(pa, lut8<W>(t.vw, m, lut, slot4), st.acc[m]);
        }
    }
    wave_lds_fence();                                      // the p buffer is free for the next unit
}

// ---- groups of up to four query heads on sixteen wavefronts (decode_main_kernel<4, ., 16, true>) ------------------
// Four heads need 8 of the 16 matrix rows.  The general form leaves rows 8..15 empty and every lane of wave rows 2, 3
// (lanes 32..63) then runs the softmax step on heads that do not exist.  Here rows 8..15 repeat rows 0..7
// (load_queries_g4) and the two token blocks of a unit share the lanes out between them: after the key products lane
// (n, j) of rows j < 2 keeps block 0's logits of slot pair_slot(n) for heads 2j, 2j+1, and a lane of rows j >= 2 keeps
// block 1's logits of slot pair_slot(n) + 1 for heads 2(j-2), 2(j-2)+1: one slot and two heads per lane, every lane with
// work of its own, half the softmax instructions.  The value product reads p of head (n & 3) for every row n, so all
// four row groups accumulate the same 4 heads x 128 dims (acc[m][r] = head r, dim 16m + n).
// While a work item runs, st.mA / st.mB hold the reference points minus P_SHIFT (the form the loop subtracts) and
// st.lA / st.lB this lane's own share of the normalisers; g4_finish puts them into the form the combine expects.
#define G4_PROW 80          // bytes per head row of the p buffer: 32 x 16 bit + 16 (rows on different banks)
template <int W>
struct Unit4 {
    uint32_t kw[2 * W];
    uint32_t vw[2 * W];
    float kn, vn;           // of the lane's one slot
};
template <int W>
__device__ static inline void load_unit4(Unit4<W>& t, const DecodeArgs& a, int li, int unit, int lane) {
    const int tile = unit >> 1, h = unit & 1;               // wave-uniform
    load_half_stream<W>(t.kw, a.s.kcodes[li] + (size_t)tile * (TILE * 16 * W), h, lane);
    load_half_stream<W>(t.vw, a.s.vcodes[li] + (size_t)tile * (TILE * 16 * W), h, lane);
    const size_t slot = (size_t)unit * UNIT + pair_slot(lane & 15) + (lane >> 5);
    t.kn = __builtin_nontemporal_load(a.s.knorm[li] + slot);
    t.vn = __builtin_nontemporal_load(a.s.vnorm[li] + slot);
}
template <int W>
__device__ static inline void compute_unit_g4(const Unit4<W>& t, int nvalid, int lane, const uint8_t* lut,
                                              uint32_t slot4, const h8* qa, float ksc, float vsc,
                                              uint8_t* pbuf, WaveState& st) {
    const int n = lane & 15, j = lane >> 4;
    f4 dk[2];
    dk[0] = (f4){0.f, 0.f, 0.f, 0.f};
    dk[1] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if constexpr (W == 8) {
                h8 chi, clo;
                lut8_split(t.kw, 4 * b + kb, lut, slot4, chi, clo);
                dk[b] = MFMA_F16(qa[kb], chi, dk[b]);
                dk[b] = MFMA_F16(qa[kb], clo, dk[b]);
            } else {
                dk[b] = MFMA_F16(qa[kb], lut8<W>(t.kw, 4 * b + kb, lut, slot4), dk[b]);
            }
        }
    // high + low row sums; rows 2, 3 of the wave take block 1's (a DPP move that writes those rows only)
    const float kn = t.kn * ksc;
    float tA = dk[0][0] + dk[0][1], tB = dk[0][2] + dk[0][3];
    {
        const float uA = dk[1][0] + dk[1][1], uB = dk[1][2] + dk[1][3];
        tA = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(tA), __float_as_int(uA), 0xe4, 0xc, 0xf, false));
        tB = __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(tB), __float_as_int(uB), 0xe4, 0xc, 0xf, false));
    }
    tA *= kn; tB *= kn;
    const int slot = pair_slot(n) + (j >> 1);
    if (nvalid < UNIT) {                                   // the last unit of a run (wave-uniform)
        const bool ok = slot < nvalid;
        tA = ok ? tA : -INFINITY;
        tB = ok ? tB : -INFINITY;
    }
    float xA = tA - st.mA, xB = tB - st.mB;
    if (__builtin_amdgcn_ballot_w64(fmaxf(xA, xB) > SOFTMAX_SLACK + P_SHIFT) != 0) {      // wave-uniform; always on the first unit
        float mxA = tA, mxB = tB;
        row_max2(mxA, mxB);
        mxA = fmaxf(mxA, __shfl_xor(mxA, 32, WAVE));       // the same heads live in rows j and j ^ 2
        mxB = fmaxf(mxB, __shfl_xor(mxB, 32, WAVE));
        const float nA = fmaxf(st.mA, mxA - P_SHIFT), nB = fmaxf(st.mB, mxB - P_SHIFT);
        if (__builtin_amdgcn_ballot_w64(st.mA > -INFINITY || st.mB > -INFINITY) != 0) {     // not the wave's first unit
            const float aA = st.mA > -INFINITY ? __builtin_amdgcn_exp2f(st.mA - nA) : 0.0f;
            const float aB = st.mB > -INFINITY ? __builtin_amdgcn_exp2f(st.mB - nB) : 0.0f;
            st.lA *= aA; st.lB *= aB;
            f4 al;                                          // heads 0, 1 sit in row 0 of the wave, heads 2, 3 in row 1
            al[0] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aA), 0));
            al[1] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aB), 0));
            al[2] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aA), 16));
            al[3] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(aB), 16));
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) st.acc[nb] *= al;
        }
        st.mA = nA; st.mB = nB;
        xA = tA - nA; xB = tB - nB;
    }
    const float pA = __builtin_amdgcn_exp2f(xA), pB = __builtin_amdgcn_exp2f(xB);      // padded slots: -inf -> 0
    st.lA += pA; st.lB += pB;
    {
        // p |v| as fp16 into this lane's slot of head rows 2(j & 1) and 2(j & 1) + 1
        // (the clamp only matters for value norms thousands of times the table's scale: no infinities)
        const float vn = t.vn * vsc;
        const uint32_t pk = pack_h2(fminf(pA * vn, FP16_MAX), fminf(pB * vn, FP16_MAX));
        uint8_t* dst = pbuf + (2 * (j & 1)) * G4_PROW + 2 * slot;
        *reinterpret_cast<uint16_t*>(dst) = (uint16_t)pk;
        *reinterpret_cast<uint16_t*>(dst + G4_PROW) = (uint16_t)(pk >> 16);
    }
    wave_lds_fence();
    const h8 pa = as_h8(*reinterpret_cast<const uint4*>(pbuf + (n & 3) * G4_PROW + 16 * j));
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        if constexpr (W == 8) {
            h8 chi, clo;
            lut8_split(t.vw, m, lut, slot4, chi, clo);
            st.acc[m] = MFMA_F16(pa, chi, st.acc[m]);
            st.acc[m] = MFMA_F16(pa, clo, st.acc[m]);
        } else {
            st.acc[m] = MFMA_F16(pa, lut8<W>(t.vw, m, lut, slot4), st.acc[m]);
        }
    }
    wave_lds_fence();                                      // the p buffer is free for the next unit
}
// the state of compute_unit_g4 in the form of the general one: reference points without the shift, and rows 0, 1 of the
// wave (the lanes whose heads the combine reads) with the whole wave's normaliser shares once summed over their 16 lanes
__device__ static inline void g4_finish(WaveState& st) {
    st.mA += P_SHIFT; st.mB += P_SHIFT;                     // (-inf stays -inf)
    st.lA += __shfl_xor(st.lA, 32, WAVE);
    st.lB += __shfl_xor(st.lB, 32, WAVE);
}
// rows 8..15 of the A operand repeat rows 0..7
__device__ static inline void load_queries_g4(const uint8_t* qrows, int lane, h8* qa) {
    const int n = lane & 7, j = lane >> 4;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
        qa[kb] = as_h8(*reinterpret_cast<const uint4*>(qrows + n * QROW_LDS + (32 * j + 8 * kb) * 2));
}

// the A operand of the key products: rows 2h, 2h+1 = high, low half of head h; row `n` of this lane,
// dims 32j + 8kb .. + 7 for step kb, from the query rows in LDS.  Rows behind the group's slots are zero.
__device__ static inline void load_queries(const uint8_t* qrows, int lane, int nrows, h8* qa) {
    const int n = lane & 15, j = lane >> 4;
    const bool on = n < nrows;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
        qa[kb] = as_h8(on ? *reinterpret_cast<const uint4*>(qrows + n * QROW_LDS + (32 * j + 8 * kb) * 2) : make_uint4(0u, 0u, 0u, 0u));
}

// The queries in the rotated basis of the quantised keys, q' = Pi_k q16, as fp16 high + low halves, on the matrix cores.
// Pi_k arrives as a table of A operands (odmkv_rotation_operands): block (rb, kk, part) = rows 16 rb .. + 15 of Pi_k, columns
// 32 kk .. + 31, part 0 = the entries rounded to fp16, part 1 = 2^12 times what the rounding left (fp16 again): 64 lanes x
// 16 bytes in operand order, 64 KB in all.  Wavefront w < 8 requests the eight blocks of its 16 rows (8 KB, out of the L2
// for all but the first workgroup to ask) together with the queries, ahead of its first unit, and forms output dims
// 16 w .. + 15 of all heads of the group: D[dim][head] = sum over 4 column blocks of A . B, B = the group's queries rounded
// to fp16 (columns = heads), products exact, sums fp32, the two parts in accumulators of their own.  Lane (n, j) ends with
// dims 16 w + 4j .. + 3 of head n and writes their fp16 high and low halves into rows 2n, 2n + 1 of the A operand of
// the key products: one barrier, no LDS staging.  (Copying the table into LDS with LDS-direct loads when the kernel
// starts, before the item is known, measured the same; the vector-ALU rotation it replaces cost 0.9 us more per item on
// 28-head stores and long items, and the same on the 32-head 32k-token store.)
// the rotation's operands of a rotating wavefront: a[2 kk + part] = its block (kk, part) of the table; r[kk] = the group's
// queries as B operands, lane (n, j) = elements 32 kk + 8j .. + 7 of head n (head 0 for the columns behind the group,
// zeroed later).  fp32 queries (no model hands them over) would take twice the registers: they are fetched when the
// rotation runs.
struct RotQuery { uint4 r[4]; uint4 a[8]; };
__device__ static inline void request_rot_query(RotQuery& rq, const DecodeArgs& a, int bq_first, int tid) {
    const int lane = tid & 63, n = lane & 15, j = lane >> 4;
    const size_t elem = (size_t)(bq_first + (n < a.G ? n : 0)) * HD + 8 * j;
    if ((tid >> 6) >= 8) return;                         // wave-uniform
    {
#pragma unroll
        for (int i = 0; i < 8; ++i) rq.a[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.pi_k_ops) + (size_t)(((tid >> 6) * 8 + i) * 64 + lane) * 16);
    }
    if (a.q_dt != ODMKV_F32) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) rq.r[kk] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.q) + elem + 32 * kk);
    }
}
// The low part of the table is kept 2^12 times larger (odmkv_rotation_operands): as it is it would lie in fp16's subnormal
// range, which the matrix instruction does not read; its products are summed apart and scaled back.
#define ROT_LOW_SCALE 4096.0f
template <int GP>
__device__ static inline void rotate_queries(const DecodeArgs& a, uint8_t* smem, int tid, int bq_first, const RotQuery& rq) {
    const int wave = tid >> 6, lane = tid & 63, n = lane & 15, j = lane >> 4;
    if (wave >= 8) return;                               // wave-uniform
    f4 dh = (f4){0.f, 0.f, 0.f, 0.f}, dl = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        uint4 b;
        if (a.q_dt == ODMKV_F16) {
            b = rq.r[kk];
        } else {
            float qv[8];
            if (a.q_dt == ODMKV_F32) {
                load_q8(a.q, ODMKV_F32, (size_t)(bq_first + (n < a.G ? n : 0)) * HD + 32 * kk + 8 * j, qv);
            } else {
                RawQ8 raw;
                raw.x = rq.r[kk]; raw.y = make_uint4(0u, 0u, 0u, 0u);
                convert_q8(raw, ODMKV_BF16, qv);
            }
            b = make_uint4(pack_h2(qv[0], qv[1]), pack_h2(qv[2], qv[3]), pack_h2(qv[4], qv[5]), pack_h2(qv[6], qv[7]));
        }
        if (n >= a.G) b = make_uint4(0u, 0u, 0u, 0u);
        dh = MFMA_F16(as_h8(rq.a[2 * kk]), as_h8(b), dh);
        dl = MFMA_F16(as_h8(rq.a[2 * kk + 1]), as_h8(b), dl);
    }
    if (n < GP) {
        uint32_t hi[2], lo[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float x0 = __fmaf_rn(dl[2 * e], 1.0f / ROT_LOW_SCALE, dh[2 * e]), x1 = __fmaf_rn(dl[2 * e + 1], 1.0f / ROT_LOW_SCALE, dh[2 * e + 1]);
            const __half h0 = __float2half_rn(x0), h1 = __float2half_rn(x1);
            hi[e] = (uint32_t)__half_as_ushort(h0) | ((uint32_t)__half_as_ushort(h1) << 16);
            lo[e] = half_bits(x0 - __half2float(h0)) | (half_bits(x1 - __half2float(h1)) << 16);
        }
        uint8_t* row = smem + LDS_QROWS + (2 * n) * QROW_LDS + (16 * wave + 4 * j) * 2;
        *reinterpret_cast<uint2*>(row) = make_uint2(hi[0], hi[1]);
        *reinterpret_cast<uint2*>(row + QROW_LDS) = make_uint2(lo[0], lo[1]);
    }
}

// One work item of a quantised level: the workgroup's wavefronts walk the item's units.
// first: the workgroup's first item (the queries are rotated now); a further item of a chain (another level of the same
// (sequence, kv-head), same queries, same accumulators) only waits until every wavefront has left the previous table.
template <int W, int GP, int NW>
__device__ static inline void run_quant_level(const DecodeArgs& a, int li, int bq_first, int tile0, int ntiles, int ntok,
                                              int tid, uint8_t* smem, uint8_t* pbuf, float* alpha_sh, WaveState& st, bool first) {
    uint8_t* lut = smem;
    const int wave = tid >> 6, lane = tid & 63;
    const uint32_t slot4 = (lane & 31) * 4;
    const float vsc = a.inv_s[li], ksc = a.inv_s[li] * a.scaling * LOG2E;
    const int unit0 = 2 * tile0;
    const auto tokens_of = [&](int u) { return min(ntok - u * UNIT, UNIT); };    // <= 0 behind the item's last token
    // Each wavefront requests the queries and its first unit, builds its share of the centroid table while memory answers,
    // and the first eight rotate the queries; the second unit is requested after that (LDS stores behind a long queue of
    // requests wait until the memory pipeline has accepted them: with both units requested first the table was ready a
    // microsecond later).  Loads return in issue order: the (small) query goes first.
    RotQuery rq;
    if (first) request_rot_query(rq, a, bq_first, tid);
    // DEPTH units of this wavefront are under way at any time: two (one for the widest rows: registers); twelve
    // wavefronts have the registers for a third 2-bit unit.  (Six units in flight with eight wavefronts were measured:
    // no gain, the eight are bound by their arithmetic.)
    constexpr int DEPTH = W == 8 ? 1 : (NW == 12 && W == 2) ? 3 : 2;
    if constexpr (DEPTH <= 2) {
        // two buffers, written out: the compiler schedules this form a microsecond per item better than the ring.
        Unit<W> cur;
        int u = wave;
        int nvalid = tokens_of(u);
        if (nvalid > 0) load_unit<W>(cur, a, li, unit0 + u, lane);
        if (!first) __syncthreads();                       // (the level's first bytes are on their way while the others finish)
        build_lut<W, NW>(lut, a, tid);
        if (first) rotate_queries<GP>(a, smem, tid, bq_first, rq);
        lds_barrier();
        // second buffer (not for the widest rows), requested before the first unit is used (requested before the
        // rotation instead, it delays the table's LDS stores behind its queue of requests: 0.9 us per item slower)
        Unit<W> nxt;
        int nv1 = 0;
        if constexpr (W != 8) {
            nv1 = tokens_of(u + NW);
            if (nv1 > 0) load_unit<W>(nxt, a, li, unit0 + u + NW, lane);
        }
        if (nvalid <= 0) return;
        h8 qa[4];
        load_queries(smem + LDS_QROWS, lane, 2 * GP, qa);
        if constexpr (W == 8) {
            while (true) {
                compute_unit<W>(cur, nvalid, lane, lut, slot4, qa, ksc, vsc, pbuf, alpha_sh, st);
                u += NW;
                nvalid = tokens_of(u);
                if (nvalid <= 0) break;
                load_unit<W>(cur, a, li, unit0 + u, lane);
            }
        } else {
            while (true) {
                compute_unit<W>(cur, nvalid, lane, lut, slot4, qa, ksc, vsc, pbuf, alpha_sh, st);
                if (nv1 <= 0) break;
                u += 2 * NW;
                nvalid = tokens_of(u);
                if (nvalid > 0) load_unit<W>(cur, a, li, unit0 + u, lane);
                compute_unit<W>(nxt, nv1, lane, lut, slot4, qa, ksc, vsc, pbuf, alpha_sh, st);
                if (nvalid <= 0) break;
                nv1 = tokens_of(u + NW);
                if (nv1 > 0) load_unit<W>(nxt, a, li, unit0 + u + NW, lane);
            }
        }
    } else {
        Unit<W> buf[DEPTH];
        int nv[DEPTH];
        nv[0] = tokens_of(wave);
        if (nv[0] > 0) load_unit<W>(buf[0], a, li, unit0 + wave, lane);
        if (!first) __syncthreads();
        build_lut<W, NW>(lut, a, tid);
        if (first) rotate_queries<GP>(a, smem, tid, bq_first, rq);
        lds_barrier();
        // the rest of the ring, requested before the first unit is used
    #pragma unroll
        for (int d = 1; d < DEPTH; ++d) {
            nv[d] = tokens_of(wave + d * NW);
            if (nv[d] > 0) load_unit<W>(buf[d], a, li, unit0 + wave + d * NW, lane);
        }
        if (nv[0] <= 0) return;
        h8 qa[4];
        load_queries(smem + LDS_QROWS, lane, 2 * GP, qa);
        // units wave, wave + NW, ...: a unit's buffer is requested again as soon as it has been used
        for (int u = wave;; u += DEPTH * NW) {
    #pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (nv[d] <= 0) return;                         // the units of a wavefront run out in order
                compute_unit<W>(buf[d], nv[d], lane, lut, slot4, qa, ksc, vsc, pbuf, alpha_sh, st);
                const int nu = u + (d + DEPTH) * NW;
                nv[d] = tokens_of(nu);
                if (nv[d] > 0) load_unit<W>(buf[d], a, li, unit0 + nu, lane);
            }
        }
    }
}

// The same walk for groups of up to four heads with compute_unit_g4 (sixteen wavefronts, two unit buffers; an
// eight-wavefront ring of five buffers, every unit of a short item requested at once, measured no faster).
template <int W, int NW>
__device__ static inline void run_quant_level_g4(const DecodeArgs& a, int li, int bq_first, int tile0, int ntiles, int ntok,
                                              int tid, uint8_t* smem, uint8_t* pbuf, float* alpha_sh, WaveState& st, bool first) {
    uint8_t* lut = smem;
    const int wave = tid >> 6, lane = tid & 63;
    const uint32_t slot4 = (lane & 31) * 4;
    const float vsc = a.inv_s[li], ksc = a.inv_s[li] * a.scaling * LOG2E;
    const int unit0 = 2 * tile0;
    const auto tokens_of = [&](int u) { return min(ntok - u * UNIT, UNIT); };    // <= 0 behind the item's last token
    // (the order of the requests, the table and the rotation is run_quant_level's)
    RotQuery rq;
    if (first) request_rot_query(rq, a, bq_first, tid);
    Unit4<W> cur;
    int u = wave;
    int nvalid = tokens_of(u);
    if (nvalid > 0) load_unit4<W>(cur, a, li, unit0 + u, lane);
    if (!first) __syncthreads();                           // (the level's first bytes are on their way while the others finish)
    build_lut<W, NW>(lut, a, tid);
    if (first) rotate_queries<4>(a, smem, tid, bq_first, rq);
    lds_barrier();
    // second buffer (not for the widest rows)
    Unit4<W> nxt;
    int nv1 = 0;
    if constexpr (W != 8) {
        nv1 = tokens_of(u + NW);
        if (nv1 > 0) load_unit4<W>(nxt, a, li, unit0 + u + NW, lane);
    }
    if (nvalid <= 0) return;
    h8 qa[4];
    load_queries_g4(smem + LDS_QROWS, lane, qa);
    if constexpr (W == 8) {
        while (true) {
            compute_unit_g4<W>(cur, nvalid, lane, lut, slot4, qa, ksc, vsc, pbuf, st);
            u += NW;
            nvalid = tokens_of(u);
            if (nvalid <= 0) break;
            load_unit4<W>(cur, a, li, unit0 + u, lane);
        }
    } else {
        while (true) {
            compute_unit_g4<W>(cur, nvalid, lane, lut, slot4, qa, ksc, vsc, pbuf, st);
            if (nv1 <= 0) break;
            u += 2 * NW;
            nvalid = tokens_of(u);
            if (nvalid > 0) load_unit4<W>(cur, a, li, unit0 + u, lane);
            compute_unit_g4<W>(nxt, nv1, lane, lut, slot4, qa, ksc, vsc, pbuf, st);
            if (nvalid <= 0) break;
            nv1 = tokens_of(u + NW);
            if (nv1 > 0) load_unit4<W>(nxt, a, li, unit0 + u + NW, lane);
        }
    }
}

// ---- exact (fp16 / bf16) units ---------------------------------------------------------------------
// Unit h of a tile is chunks 8h .. 8h+7 of every lane.  Keys: chunk 8h + 4b + kb of lane (n, j) = dims
// 32j+8kb..+7 of slot 32h + pair_slot(n) + b.  Values: chunk 8h + m = slots 32h+8j..+7 of dim 16m+n.
// Chunk c of lane l sits at byte (c*64 + l)*16 of the tile.
struct ExactUnit { uint4 c[8]; };

__device__ static inline void load_exact_unit(ExactUnit& t, const uint16_t* base, int unit, int lane) {
    const uint8_t* src = reinterpret_cast<const uint8_t*>(base) + (size_t)(unit >> 1) * (TILE * HD * 2) + (size_t)(unit & 1) * (8 * TILE * 16);
#pragma unroll
    for (int c = 0; c < 8; ++c) t.c[c] = stream_load(reinterpret_cast<const uint4*>(src + ((size_t)c * TILE + lane) * 16));
}

// BF: the store keeps bf16 rows; they meet the query (bf16 high + low piece of q16, exact) and the
// softmax weights (bf16 high + low piece) on the bf16 matrix instructions, products exact, sums fp32.
template <bool BF, int NW>
__device__ static inline void run_exact_level(const DecodeArgs& a, int bh, int bq_first, int tile0, int ntiles, int seg_first,
                                              int tid, uint8_t* pbuf, uint8_t* pbuf_lo, float* alpha_sh, WaveState& st) {
    const int wave = tid >> 6, lane = tid & 63, n = lane & 15, j = lane >> 4;
    const float esc = a.scaling * LOG2E;
    // the query itself (no rotation): row 2h = q16 of head h, row 2h+1 = zero for fp16 rows; for bf16 rows the two
    // bf16 pieces of q16 (11 significant bits in two pieces of 8: exact)
    uint4 qraw[4];
    {
        const int h = n >> 1, lo = n & 1;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if (h < a.G && (BF || !lo)) {
                float qv[8];
                load_q8(a.q, a.q_dt, (size_t)(bq_first + h) * HD + 32 * j + 8 * kb, qv);
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    if constexpr (BF) w[e >> 1] = lo ? bf16_pair(bf16_rest(qv[e]), bf16_rest(qv[e + 1])) : bf16_pair(qv[e], qv[e + 1]);
                    else w[e >> 1] = pack_h2(qv[e], qv[e + 1]);
                }
            }
            qraw[kb] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    const int count = a.s.seg_count[4][bh] - (tile0 - seg_first) * TILE;     // exact segments grow between work-list rebuilds
    for (int u = wave; u < 2 * ntiles; u += NW) {
        const int nvalid = min(count - u * UNIT, UNIT);
        if (nvalid <= 0) break;
        ExactUnit k;
        load_exact_unit(k, a.s.kexact, 2 * tile0 + u, lane);
        f4 dk[2];
        dk[0] = (f4){0.f, 0.f, 0.f, 0.f};
        dk[1] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                if constexpr (BF) dk[b] = MFMA_BF16(as_bf8(qraw[kb]), as_bf8(k.c[4 * b + kb]), dk[b]);
                else dk[b] = MFMA_F16(as_h8(qraw[kb]), as_h8(k.c[4 * b + kb]), dk[b]);
            }
        ExactUnit v;
        load_exact_unit(v, a.s.vexact, 2 * tile0 + u, lane);
        float tA[2], tB[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const bool ok = pair_slot(n) + b < nvalid;
            tA[b] = ok ? (dk[b][0] + dk[b][1]) * esc : -INFINITY;
            tB[b] = ok ? (dk[b][2] + dk[b][3]) * esc : -INFINITY;
        }
        float pA[2], pB[2];
        softmax_unit(st, tA, tB, lane, alpha_sh, pA, pB);
        if constexpr (BF) {
            // p = hi + lo in bf16: two p buffers (the second in the table's space, which an exact item does not use), two products
            *reinterpret_cast<uint32_t*>(pbuf + (2 * j) * PROW + 4 * n) = bf16_pair(pA[0], pA[1]);
            *reinterpret_cast<uint32_t*>(pbuf + (2 * j + 1) * PROW + 4 * n) = bf16_pair(pB[0], pB[1]);
            *reinterpret_cast<uint32_t*>(pbuf_lo + (2 * j) * PROW + 4 * n) = bf16_pair(bf16_rest(pA[0]), bf16_rest(pA[1]));
            *reinterpret_cast<uint32_t*>(pbuf_lo + (2 * j + 1) * PROW + 4 * n) = bf16_pair(bf16_rest(pB[0]), bf16_rest(pB[1]));
        } else {
            *reinterpret_cast<uint32_t*>(pbuf + (2 * j) * PROW + 4 * n) = pack_h2(pA[0], pA[1]);
            *reinterpret_cast<uint32_t*>(pbuf + (2 * j + 1) * PROW + 4 * n) = pack_h2(pB[0], pB[1]);
        }
        wave_lds_fence();
        const uint4 phi = *reinterpret_cast<const uint4*>(pbuf + (n & 7) * PROW + 16 * j);
        if constexpr (BF) {
            const uint4 plo = *reinterpret_cast<const uint4*>(pbuf_lo + (n & 7) * PROW + 16 * j);
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                st.acc[m] = MFMA_BF16(as_bf8(phi), as_bf8(v.c[m]), st.acc[m]);
                st.acc[m] = MFMA_BF16(as_bf8(plo), as_bf8(v.c[m]), st.acc[m]);
            }
        } else {
#pragma unroll
            for (int m = 0; m < 8; ++m) st.acc[m] = MFMA_F16(as_h8(phi), as_h8(v.c[m]), st.acc[m]);
        }
        wave_lds_fence();
    }
}

// ------------------------------------------------------------------------------------------------
// main kernel
// ------------------------------------------------------------------------------------------------
// G4: the quantised levels run compute_unit_g4 (GP = 4 and sixteen wavefronts only)
// CHAIN: a workgroup may take several consecutive items, the quantised levels of one (sequence, kv-head) one after the
// other (item word 6 = how many follow): the queries are rotated once, the accumulators run through, the table is rebuilt
// between the levels, one result is written at the first item's place and empty results at the others'.
// PAIR: eight wavefronts held to 128 registers each (four wavefronts per SIMD) and half a compute unit's LDS, so that two
// workgroups share a compute unit: while one sets up or combines, the other streams.  For lists with more items than
// compute units, whose workgroups would otherwise run one after the other, each paying its start and its end alone.
template <int GP, bool ORDERED, int NW, bool G4 = false, bool CHAIN = false, bool PAIR = false>
__global__ __launch_bounds__(NW * 64, PAIR ? 4 : 1) void decode_main_kernel(DecodeArgs a) {
    static_assert(!G4 || (GP == 4 && (NW == 16 || PAIR)), "the shared-lane form is built for four heads and four wavefronts per SIMD");
    static_assert(!PAIR || (NW == 8 && 2 * Lds<NW>::TOTAL <= 160 * 1024), "two workgroups of eight wavefronts share a compute unit");
    static_assert(!CHAIN || ORDERED, "chains come with a dispatch order (fewer workgroups than items)");
    // one static LDS block: the table sits at LDS address 0 and that is known when the kernel is compiled, so a
    // lookup address needs no base added
    __shared__ __align__(16) uint8_t smem[Lds<NW>::TOTAL];
    uint8_t* lut = smem;                                               // centroid table; reused to combine the wavefronts
    float* alphas = reinterpret_cast<float*>(smem + Lds<NW>::SCALARS);      // [NWAVES][8]
    float* wm = alphas + NW * 8;                            // [NWAVES][8]
    float* wl = wm + NW * 8;                                // [NWAVES][8]
    float* wf = wl + NW * 8;                                // [NWAVES][8]
    float* wM = wf + NW * 8;                                // [8]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int item = ORDERED ? a.order[blockIdx.x] : (int)blockIdx.x;
    const int4 d0 = reinterpret_cast<const int4*>(a.items)[2 * item];       // bh, level, first tile, tiles
    const int4 d1 = reinterpret_cast<const int4*>(a.items)[2 * item + 1];   // tokens, first tile of the segment
    // the rotation's operand table on its way into LDS right behind the request for the work item (loads return in the
    // order of their requests: asked for first, the table would hold the item back; it does not depend on the item)
    const int bh = d0.x;
    int li = d0.y, tile0 = d0.z, ntiles = d0.w, ntok = d1.x;
    const int bq_first = (bh / a.s.Hkv) * a.Hq + (bh % a.s.Hkv) * a.G;      // first query head of the group

    float* dst = a.partial + (size_t)item * GP * PSTRIDE;      // where this item's result goes

    WaveState st;
    st.mA = -INFINITY; st.mB = -INFINITY; st.lA = 0.0f; st.lB = 0.0f;
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) st.acc[nb] = (f4){0.f, 0.f, 0.f, 0.f};
    uint8_t* pbuf = smem + LDS_PBUFS + wave * PBUF;
    uint8_t* pbuf_lo = smem + wave * PBUF;                 // bf16 exact rows: the weights' low pieces (the table's space)
    float* alpha_sh = alphas + wave * 8;
#define ODMKV_RUN_LEVEL(W, L, FIRST) \
    do { if constexpr (G4) run_quant_level_g4<W, NW>(a, L, bq_first, tile0, ntiles, ntok, tid, smem, pbuf, alpha_sh, st, FIRST); \
         else run_quant_level<W, GP, NW>(a, L, bq_first, tile0, ntiles, ntok, tid, smem, pbuf, alpha_sh, st, FIRST); } while (0)
    if constexpr (!CHAIN) {
        switch (li) {
            case 0: ODMKV_RUN_LEVEL(2, 0, true); break;
            case 1: ODMKV_RUN_LEVEL(3, 1, true); break;
            case 2: ODMKV_RUN_LEVEL(4, 2, true); break;
            case 3: ODMKV_RUN_LEVEL(8, 3, true); break;
            default:
                if (a.s.exact_dtype == ODMKV_BF16) run_exact_level<true, NW>(a, bh, bq_first, tile0, ntiles, d1.y, tid, pbuf, pbuf_lo, alpha_sh, st);
                else run_exact_level<false, NW>(a, bh, bq_first, tile0, ntiles, d1.y, tid, pbuf, pbuf_lo, alpha_sh, st);
                break;
        }
    } else if (li == 4) {
        if (a.s.exact_dtype == ODMKV_BF16) run_exact_level<true, NW>(a, bh, bq_first, tile0, ntiles, d1.y, tid, pbuf, pbuf_lo, alpha_sh, st);
        else run_exact_level<false, NW>(a, bh, bq_first, tile0, ntiles, d1.y, tid, pbuf, pbuf_lo, alpha_sh, st);
    } else {
        // The levels of a chain ascend: the four walkers stand one behind the other, each taken if the chain has an item of
        // its level.  A 2-bit item is always a chain's first: its walker rotates the queries as an unchained one does (beside
        // its first requests); chains that start higher rotate them up front.
        if (li != 0) {
            RotQuery rq;
            request_rot_query(rq, a, bq_first, tid);
            rotate_queries<GP>(a, smem, tid, bq_first, rq);
        }
        // the (up to three) items behind the first one, asked for together (the list is padded: reading past a chain's
        // end reads other items, which are then not used)
        const int follow = d1.z;
        int4 r0[3], r1[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int idx = min(item + 1 + k, a.n_items - 1);
            r0[k] = reinterpret_cast<const int4*>(a.items)[2 * idx];
            r1[k] = reinterpret_cast<const int4*>(a.items)[2 * idx + 1];
        }
        // the places of the items this workgroup takes along get an empty result (no visible token), now, while the first
        // bytes are on their way: the merge reads them like any other item's
        for (int e = tid; e < follow * GP * PSTRIDE; e += NW * 64) dst[GP * PSTRIDE + e] = (e % PSTRIDE) == HD ? -INFINITY : 0.0f;
        const int first_li = li, first_tile0 = tile0, first_ntiles = ntiles, first_ntok = ntok;
#define ODMKV_PICK_LEVEL(L) \
        bool has = first_li == L; \
        tile0 = first_tile0; ntiles = first_ntiles; ntok = first_ntok; \
        _Pragma("unroll") for (int k = 0; k < 3; ++k) \
            if (k < follow && r0[k].y == L) { has = true; tile0 = r0[k].z; ntiles = r0[k].w; ntok = r1[k].x; }
        { ODMKV_PICK_LEVEL(0) if (has) ODMKV_RUN_LEVEL(2, 0, true); }
        { ODMKV_PICK_LEVEL(1) if (has) ODMKV_RUN_LEVEL(3, 1, false); }
        { ODMKV_PICK_LEVEL(2) if (has) ODMKV_RUN_LEVEL(4, 2, false); }
        { ODMKV_PICK_LEVEL(3) if (has) ODMKV_RUN_LEVEL(8, 3, false); }
#undef ODMKV_PICK_LEVEL
        li = 0;                                                // (a quantised item: the shared-lane state is finished below)
    }
#undef ODMKV_RUN_LEVEL
    if constexpr (G4) {
        if (li < 4) g4_finish(st);                             // (wave-uniform; exact items keep the general form)
    }

    // ---- combine the wavefronts (the table is no longer needed) ----
    // Every wavefront publishes its maxima; after the barrier it takes the maximum over all wavefronts (lane n of a
    // row reads wavefront n's value), derives its own factor exp2(m - M) and publishes the factor, its scaled share of
    // the normaliser and its accumulators as they are.  After a second barrier one thread per (head, dim) forms the
    // weighted sum over the wavefronts.
    const int n = lane & 15, j = lane >> 4;
    const float lsA = row_sum(st.lA), lsB = row_sum(st.lB);
    if (n == 0) { wm[wave * 8 + 2 * j] = st.mA; wm[wave * 8 + 2 * j + 1] = st.mB; }
    __syncthreads();
    float* wacc = reinterpret_cast<float*>(lut);          // [NWAVES][128 dims][GP heads]
    {
        float MA = n < NW ? wm[n * 8 + 2 * j] : -INFINITY, MB = n < NW ? wm[n * 8 + 2 * j + 1] : -INFINITY;
        row_max2(MA, MB);
        const float fA = st.mA > -INFINITY ? __builtin_amdgcn_exp2f(st.mA - MA) : 0.0f;
        const float fB = st.mB > -INFINITY ? __builtin_amdgcn_exp2f(st.mB - MB) : 0.0f;
        if (n == 0 && 2 * j < GP) {
            wf[wave * 8 + 2 * j] = fA; wf[wave * 8 + 2 * j + 1] = fB;
            wl[wave * 8 + 2 * j] = lsA * fA; wl[wave * 8 + 2 * j + 1] = lsB * fB;
            if (wave == 0) { wM[2 * j] = MA; wM[2 * j + 1] = MB; }
        }
        if (4 * j < GP) {
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) *reinterpret_cast<f4*>(&wacc[((wave * HD) + 16 * nb + n) * GP + 4 * j]) = st.acc[nb];
        }
    }
    __syncthreads();
    for (int e = tid; e < GP * HD; e += NW * 64) {
        const int g = e % GP, dim = e / GP;               // consecutive threads walk consecutive LDS words
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s = __fmaf_rn(wacc[w * HD * GP + e], wf[w * 8 + g], s);
        dst[g * PSTRIDE + dim] = s;
    }
    if (tid >= NW * 64 - GP) {                 // the last wavefront has the least to do above
        const int g = tid - (NW * 64 - GP);
        float L = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) L += wl[w * 8 + g];
        dst[g * PSTRIDE + HD] = wM[g];
        dst[g * PSTRIDE + HD + 1] = L;
    }
}

// ------------------------------------------------------------------------------------------------
// merge: MERGE_SPLIT workgroups per query head
// ------------------------------------------------------------------------------------------------
#define MERGE_THREADS 512
#define MERGE_SLICES (MERGE_THREADS / HD)
#define MERGE_CHUNK 64            // items merged per round: one per lane of a wavefront

// MERGE_SPLIT: workgroups per query head (4 when there are few heads, so that the launch still covers the device;
// 1 for large batches, where every further workgroup only repeats the reading)
template <int GP, int MERGE_SPLIT>
__global__ __launch_bounds__(MERGE_THREADS) void decode_merge_kernel(DecodeArgs a) {
    __shared__ float part[2][MERGE_SLICES][HD];      // [rotated | exact][slice][dim]
    constexpr int QD = HD / MERGE_SPLIT;                 // output dims of this workgroup
    constexpr int RS = MERGE_THREADS / QD;                // row slices of the rotation
    constexpr int IN = HD / RS;                           // rows per slice
    __shared__ float part2[RS * QD];
    // MERGE_SPLIT workgroups per query head: each merges the head's partial results in full (they are small and
    // shared through the caches) and rotates back its share of the output dims, so that no workgroup has to pull
    // the whole 64 KB rotation through one compute unit
    const int bq = blockIdx.x / MERGE_SPLIT, quarter = blockIdx.x % MERGE_SPLIT;
    const int tid = threadIdx.x, lane = tid & 63, j = tid & (HD - 1);
    const int slice = __builtin_amdgcn_readfirstlane(tid >> 7);
    const int b = bq / a.Hq, hq = bq % a.Hq;
    const int bh = b * a.s.Hkv + hq / a.G, g = hq % a.G;
    const int i0 = a.item_range[bh], n = a.item_range[bh + 1] - i0;
    // this thread's share of the value rotation: requested first, it does not depend on the items
    const int jj = tid % QD, rs = tid / QD;
    float pv[IN];
#pragma unroll
    for (int ii = 0; ii < IN; ++ii) pv[ii] = a.pi_v[(size_t)(rs * IN + ii) * HD + quarter * QD + jj];
    // The items are merged MERGE_CHUNK at a time with a running maximum, like an online softmax.  Inside a round
    // nothing crosses wavefronts: lane i of every wavefront holds item i's (m, l, level), the maximum and the
    // normaliser come from wave reductions, and the weight of the item a wavefront is adding (the same item for the
    // whole wavefront) is read from its lane.  Every wavefront thus repeats the few scalars and no barrier is needed.
    float M = -INFINITY, L = 0.0f, arot = 0.0f, aex = 0.0f;
    for (int c0 = 0; c0 < n; c0 += MERGE_CHUNK) {
        const int nc = min(n - c0, MERGE_CHUNK);
        float m_i = -INFINITY, l_i = 0.0f;
        int level = 0;
        if (lane < nc) {
            const float* p = a.partial + ((size_t)(i0 + c0 + lane) * GP + g) * PSTRIDE;
            m_i = p[HD]; l_i = p[HD + 1];
            level = a.items[8 * (i0 + c0 + lane) + 1];
        }
        float vals[MERGE_CHUNK / MERGE_SLICES];
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK / MERGE_SLICES; ++k) {
            const int it = slice + k * MERGE_SLICES;
            vals[k] = it < nc ? a.partial[((size_t)(i0 + c0 + it) * GP + g) * PSTRIDE + j] : 0.0f;
        }
        const float Mc = fmaxf(M, wave_max(m_i));
        const float f_old = M > -INFINITY ? __builtin_amdgcn_exp2f(M - Mc) : 0.0f;
        const float w = m_i > -INFINITY ? __builtin_amdgcn_exp2f(m_i - Mc) : 0.0f;
        L = __fmaf_rn(L, f_old, wave_sum(l_i * w));
        arot *= f_old; aex *= f_old;
        const int wsgn = __float_as_int(level == 4 ? -w : w);          // the sign bit marks exact items
#pragma unroll
        for (int k = 0; k < MERGE_CHUNK / MERGE_SLICES; ++k) {
            const int it = slice + k * MERGE_SLICES;                     // wave-uniform
            if (it < nc) {
                const float ww = __int_as_float(__builtin_amdgcn_readlane(wsgn, it));
                if (__float_as_uint(ww) >> 31) aex = __fmaf_rn(vals[k], -ww, aex);
                else arot = __fmaf_rn(vals[k], ww, arot);
            }
        }
        M = Mc;
    }
    part[0][slice][j] = arot;
    part[1][slice][j] = aex;
    __syncthreads();
    // rotate the quantised part back: out_j = sum_i rot_i Pi_v[i][j] for this workgroup's dims; the slices split the i range
    float o = 0.0f;
#pragma unroll
    for (int ii = 0; ii < IN; ++ii) {
        const int i = rs * IN + ii;
        float r = part[0][0][i];
#pragma unroll
        for (int sl = 1; sl < MERGE_SLICES; ++sl) r += part[0][sl][i];
        o = __fmaf_rn(r, pv[ii], o);
    }
    part2[rs * QD + jj] = o;
    __syncthreads();
    if (tid < QD) {
        const int dim = quarter * QD + tid;
        float tot = 0.0f;
#pragma unroll
        for (int r = 0; r < RS; ++r) tot += part2[r * QD + tid];
#pragma unroll
        for (int sl = 0; sl < MERGE_SLICES; ++sl) tot += part[1][sl][dim];
        const float o32 = L > 0.0f ? tot / L : 0.0f;
        const size_t oi = (size_t)bq * HD + dim;
        if (a.out_dt == ODMKV_F32) reinterpret_cast<float*>(a.out)[oi] = o32;
        else if (a.out_dt == ODMKV_F16) reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_F16>::from_f32(o32);
        else reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_BF16>::from_f32(o32);
        if (a.lse && tid == 0 && quarter == 0) a.lse[bq] = L > 0.0f ? (M + __log2f(L) - P_SHIFT) * LN2 : -INFINITY;
    }
}

// The merge for large batches: one workgroup per (sequence, kv-head) merges and rotates back all heads of the group, so
// the 64 KB of Pi_v are pulled into a compute unit once per group, not once per query head (2048 heads: 134 MB of reads
// out of the L2s for 1 MB of results).  The four 128-thread slices take a head each (two each for groups of five to
// eight); a slice walks its head's items in rounds of MERGE_CHUNK with a running maximum, as above.
template <int GP>
__global__ __launch_bounds__(MERGE_THREADS) void decode_merge_group_kernel(DecodeArgs a) {
    constexpr int HPS = GP / MERGE_SLICES;                // heads per slice
    static_assert(HPS >= 1, "a slice takes whole heads");
    constexpr int RS = MERGE_THREADS / HD;                // row slices of the rotation
    constexpr int IN = HD / RS;                           // rows per slice
    __shared__ __align__(16) float part[2][GP][HD];       // [rotated | exact][head][dim]
    __shared__ float part2[GP][RS][HD];
    __shared__ float headL[GP], headM[GP];
    const int bh = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, j = tid & (HD - 1);
    const int slice = __builtin_amdgcn_readfirstlane(tid >> 7);
    const int b = bh / a.s.Hkv, hq0 = (bh % a.s.Hkv) * a.G;
    const int i0 = a.item_range[bh], n = a.item_range[bh + 1] - i0;
    float pv[IN];
#pragma unroll
    for (int ii = 0; ii < IN; ++ii) pv[ii] = a.pi_v[(size_t)(slice * IN + ii) * HD + j];
#pragma unroll
    for (int h = 0; h < HPS; ++h) {
        const int g = slice * HPS + h;                    // wave-uniform
        float M = -INFINITY, L = 0.0f, arot = 0.0f, aex = 0.0f;
        if (g < a.G) {
            for (int c0 = 0; c0 < n; c0 += MERGE_CHUNK) {
                const int nc = min(n - c0, MERGE_CHUNK);
                float m_i = -INFINITY, l_i = 0.0f;
                int level = 0;
                if (lane < nc) {
                    const float* p = a.partial + ((size_t)(i0 + c0 + lane) * GP + g) * PSTRIDE;
                    m_i = p[HD]; l_i = p[HD + 1];
                    level = a.items[8 * (i0 + c0 + lane) + 1];
                }
                const float Mc = fmaxf(M, wave_max(m_i));
                const float f_old = M > -INFINITY ? __builtin_amdgcn_exp2f(M - Mc) : 0.0f;
                const float w = m_i > -INFINITY ? __builtin_amdgcn_exp2f(m_i - Mc) : 0.0f;
                L = __fmaf_rn(L, f_old, wave_sum(l_i * w));
                arot *= f_old; aex *= f_old;
                const int wsgn = __float_as_int(level == 4 ? -w : w);      // the sign bit marks exact items
                for (int it0 = 0; it0 < nc; it0 += 4) {                    // four items' values under way at a time
                    float vals[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        vals[k] = it0 + k < nc ? a.partial[((size_t)(i0 + c0 + it0 + k) * GP + g) * PSTRIDE + j] : 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (it0 + k < nc) {
                            const float ww = __int_as_float(__builtin_amdgcn_readlane(wsgn, it0 + k));
                            if (__float_as_uint(ww) >> 31) aex = __fmaf_rn(vals[k], -ww, aex);
                            else arot = __fmaf_rn(vals[k], ww, arot);
                        }
                    }
                }
                M = Mc;
            }
        }
        part[0][g][j] = arot;
        part[1][g][j] = aex;
        if (j == 0) { headL[g] = L; headM[g] = M; }
    }
    __syncthreads();
    // rotate the quantised parts back: out_g[j] = sum_i rot_g[i] Pi_v[i][j]; the slices split the i range
    float o[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) o[g] = 0.0f;
#pragma unroll
    for (int ii = 0; ii < IN; ii += 4) {
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const f4 r = *reinterpret_cast<const f4*>(&part[0][g][slice * IN + ii]);   // (one address per slice: a broadcast)
            o[g] = __fmaf_rn(r[0], pv[ii], o[g]); o[g] = __fmaf_rn(r[1], pv[ii + 1], o[g]);
            o[g] = __fmaf_rn(r[2], pv[ii + 2], o[g]); o[g] = __fmaf_rn(r[3], pv[ii + 3], o[g]);
        }
    }
#pragma unroll
    for (int g = 0; g < GP; ++g) part2[g][slice][j] = o[g];
    __syncthreads();
#pragma unroll
    for (int h = 0; h < HPS; ++h) {
        const int g = slice * HPS + h;
        if (g >= a.G) continue;
        float tot = part[1][g][j];
#pragma unroll
        for (int r = 0; r < RS; ++r) tot += part2[g][r][j];
        const float L = headL[g];
        const float o32 = L > 0.0f ? tot / L : 0.0f;
        const size_t bq = (size_t)b * a.Hq + hq0 + g;
        const size_t oi = bq * HD + j;
        if (a.out_dt == ODMKV_F32) reinterpret_cast<float*>(a.out)[oi] = o32;
        else if (a.out_dt == ODMKV_F16) reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_F16>::from_f32(o32);
        else reinterpret_cast<uint16_t*>(a.out)[oi] = Elem<ODMKV_BF16>::from_f32(o32);
        if (a.lse && j == 0) a.lse[bq] = L > 0.0f ? (headM[g] + __log2f(L) - P_SHIFT) * LN2 : -INFINITY;
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
static inline int group_pad(int G) { return G <= 4 ? 4 : 8; }

// Pi_k -> the operand table of rotate_queries: thread t of block (rb, kk) writes lane t's eight values of both parts
__global__ __launch_bounds__(64) void rotation_operands_kernel(const float* __restrict__ pi_k, uint16_t* __restrict__ ops) {
    const int rb = blockIdx.x >> 2, kk = blockIdx.x & 3, lane = threadIdx.x, n = lane & 15, j = lane >> 4;
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        float x[2];
        uint32_t h[2], l[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            x[k] = pi_k[(size_t)(16 * rb + n) * HD + 32 * kk + 8 * j + e + k];
            const __half hv = __float2half_rn(x[k]);
            h[k] = (uint32_t)__half_as_ushort(hv);
            l[k] = half_bits((x[k] - __half2float(hv)) * ROT_LOW_SCALE);
        }
        hi[e >> 1] = h[0] | (h[1] << 16);
        lo[e >> 1] = l[0] | (l[1] << 16);
    }
    uint4* dst = reinterpret_cast<uint4*>(ops) + (size_t)(blockIdx.x * 2) * 64 + lane;
    dst[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    dst[64] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
}

extern "C" int odmkv_rotation_operands(const float* pi_k, uint16_t* ops, void* stream) {
    ODMKV_CHECK_ARG(pi_k && ops, "rotation_operands: null pointer");
    ODMKV_CHECK_ARG(((uintptr_t)ops & 15) == 0, "rotation_operands: the table must be 16-byte aligned");
    hipLaunchKernelGGL(rotation_operands_kernel, dim3(32), dim3(64), 0, (hipStream_t)stream, pi_k, ops);
    ODMKV_CHECK_LAUNCH("rotation_operands_kernel");
    return 0;
}

extern "C" size_t odmkv_decode_workspace_bytes(int B, int Hq, int n_items) {
    if (B <= 0 || Hq <= 0 || n_items < 0) return 0;
    return align_up((size_t)(n_items > 0 ? n_items : 1) * ODMKV_MAX_GROUP * PSTRIDE * sizeof(float), 256);
}

template <int GP, bool ORDERED, int NW, bool G4 = false, bool CHAIN = false, bool PAIR = false>
static int launch_main(const DecodeArgs& a, int grid, hipEvent_t e0, hipEvent_t e1, hipStream_t st) {
    hipExtLaunchKernelGGL((decode_main_kernel<GP, ORDERED, NW, G4, CHAIN, PAIR>), dim3(grid), dim3(NW * 64), 0, st, e0, e1, 0, a);
    ODMKV_CHECK_LAUNCH("decode_main_kernel");
    return 0;
}

int odmkv_decode_launch(const void* q, int q_dtype, int B, int Hq, float scaling,
                        const odmkv_packed_t* store, const odmkv_worklist_t* work,
                        const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                        const float* codebooks_host, const float* inv_scales,
                        void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                        void* stream, int stage_mask, void* ev_start, void* ev_stop) {
    ODMKV_CHECK_ARG(q_dtype == ODMKV_F16 || q_dtype == ODMKV_BF16 || q_dtype == ODMKV_F32, "decode_attn: bad query dtype %d", q_dtype);
    ODMKV_CHECK_ARG(out_dtype == ODMKV_F16 || out_dtype == ODMKV_BF16 || out_dtype == ODMKV_F32, "decode_attn: bad output dtype %d", out_dtype);
    ODMKV_CHECK_ARG(codebooks_host != nullptr, "decode_attn: null host copy of the centroid tables");
    ODMKV_CHECK_ARG(inv_scales != nullptr, "decode_attn: null table scales");
    ODMKV_CHECK_ARG(q && store && work && pi_k_ops && pi_v && codebooks && out && workspace, "decode_attn: null pointer");
    ODMKV_CHECK_ARG(((uintptr_t)q & 15) == 0, "decode_attn: the query must be 16-byte aligned");
    ODMKV_CHECK_ARG(((uintptr_t)pi_k_ops & 15) == 0, "decode_attn: the rotation's operand table must be 16-byte aligned");
    const int n_items = work->n_items;
    ODMKV_CHECK_ARG(n_items >= 0, "decode_attn: negative item count");
    ODMKV_CHECK_ARG(work->wavefronts == 0 || work->wavefronts == 8 || work->wavefronts == 12 || work->wavefronts == 16,
                    "decode_attn: %d wavefronts per work item (0, 8, 12 or 16)", work->wavefronts);
    ODMKV_CHECK_ARG(work->item_range, "decode_attn: null item ranges");
    ODMKV_CHECK_ARG(n_items == 0 || work->items, "decode_attn: null work list");
    ODMKV_CHECK_ARG(work->two_per_cu == 0 || ((work->wavefronts == 0 || work->wavefronts == 8) && work->dispatch_order),
                    "decode_attn: two workgroups per compute unit take eight wavefronts each and a dispatch order");
    ODMKV_CHECK_ARG(work->n_workgroups >= 0 && work->n_workgroups <= n_items, "decode_attn: %d workgroups for %d items", work->n_workgroups, n_items);
    ODMKV_CHECK_ARG(work->n_workgroups == 0 || work->n_workgroups == n_items || work->dispatch_order,
                    "decode_attn: workgroups that take several items need the dispatch order (their first items)");
    ODMKV_CHECK_ARG(B > 0 && Hq > 0 && store->B == B && store->Hkv > 0 && Hq % store->Hkv == 0,
                    "decode_attn: bad head counts B=%d Hq=%d store(B=%d,Hkv=%d)", B, Hq, store->B, store->Hkv);
    ODMKV_CHECK_ARG(store->exact_dtype == ODMKV_F16 || store->exact_dtype == ODMKV_BF16, "decode_attn: exact dtype must be fp16 or bf16");
    const int G = Hq / store->Hkv;
    ODMKV_CHECK_ARG(G <= ODMKV_MAX_GROUP, "decode_attn: GQA group %d exceeds %d", G, ODMKV_MAX_GROUP);
    if (workspace_bytes < odmkv_decode_workspace_bytes(B, Hq, n_items)) {
        odmkv_set_error("decode_attn: workspace of %zu bytes, %zu needed", workspace_bytes, odmkv_decode_workspace_bytes(B, Hq, n_items));
        return ODMKV_ENOSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    DecodeArgs a;
    a.s = *store; a.q = q; a.q_dt = q_dtype; a.out_dt = out_dtype; a.Hq = Hq; a.G = G; a.B = B; a.scaling = scaling;
    a.items = work->items; a.item_range = work->item_range; a.order = work->dispatch_order;
    a.n_items = n_items;
    a.pi_k_ops = pi_k_ops; a.pi_v = pi_v; a.cb = codebooks;
    for (int w = 0; w < 4; ++w) a.inv_s[w] = inv_scales[w];
    for (int k = 0; k < 28; ++k) a.cbs[k] = codebooks_host[k];
    a.partial = (float*)workspace;
    a.out = out; a.lse = lse;
    const int GP = group_pad(G);
    a.gp = GP;
    if (n_items > 0 && (stage_mask & 2)) {
        // when measuring, the events are attached to the dispatch itself: they carry the kernel's own
        // start and end timestamps, not those of separate marker packets
        hipEvent_t e0 = (hipEvent_t)ev_start, e1 = (hipEvent_t)ev_stop;
        const int nw = work->wavefronts == 0 ? 8 : work->wavefronts;
        int rc;
#define ODMKV_LAUNCH_MAIN(GPV, ORD, CH) \
        (nw == 16 ? launch_main<GPV, ORD, 16, false, CH>(a, grid, e0, e1, st) : nw == 12 ? launch_main<GPV, ORD, 12, false, CH>(a, grid, e0, e1, st) \
                                                                               : launch_main<GPV, ORD, 8, false, CH>(a, grid, e0, e1, st))
        // groups of up to four heads on sixteen wavefronts: the form that shares the lanes out between a unit's two token
        // blocks (its softmax step costs half the instructions); ODMKV_DECODE_G4=0 selects the general form, for measurements
        static const int g4_forced = [] { const char* e = getenv("ODMKV_DECODE_G4"); return e ? atoi(e) : -1; }();
        const bool g4 = GP == 4 && nw == 16 && g4_forced != 0;
        const bool chain = work->n_workgroups > 0 && work->n_workgroups != n_items;      // workgroups that take several items
        const int grid = chain ? work->n_workgroups : n_items;
        // two eight-wavefront workgroups per compute unit (always with a dispatch order: the list has more items than
        // compute units); groups of up to four heads in the shared-lane form
        const bool pair = work->two_per_cu != 0 && (GP == 8 || g4_forced != 0);
        if (pair && GP == 4) rc = chain ? launch_main<4, true, 8, true, true, true>(a, grid, e0, e1, st)
                                                          : launch_main<4, true, 8, true, false, true>(a, grid, e0, e1, st);
        else if (pair) rc = chain ? launch_main<8, true, 8, false, true, true>(a, grid, e0, e1, st)
                                  : launch_main<8, true, 8, false, false, true>(a, grid, e0, e1, st);
        else if (chain && g4) rc = launch_main<4, true, 16, true, true>(a, grid, e0, e1, st);
        else if (chain && GP == 4) rc = ODMKV_LAUNCH_MAIN(4, true, true);
        else if (chain) rc = ODMKV_LAUNCH_MAIN(8, true, true);
        else if (g4 && !a.order) rc = launch_main<4, false, 16, true>(a, grid, e0, e1, st);
        else if (g4) rc = launch_main<4, true, 16, true>(a, grid, e0, e1, st);
        else if (GP == 4 && !a.order) rc = ODMKV_LAUNCH_MAIN(4, false, false);
        else if (GP == 4) rc = ODMKV_LAUNCH_MAIN(4, true, false);
        else if (!a.order) rc = ODMKV_LAUNCH_MAIN(8, false, false);
        else rc = ODMKV_LAUNCH_MAIN(8, true, false);
#undef ODMKV_LAUNCH_MAIN
        if (rc) return rc;
    }
    if (stage_mask & 4) {
        const int heads = B * Hq;
        // from 512 query heads on, a workgroup per (sequence, kv-head) merges all heads of the group (64 x 2048 tokens, 2048
        // heads: the merge 10.8 -> 4.8 us; 512 heads: 3.5 -> 3.2 us); ODMKV_MERGE_GROUP_FROM moves the limit, for measurements
        static const int group_from = [] { const char* e = getenv("ODMKV_MERGE_GROUP_FROM"); return e ? atoi(e) : 512; }();
        if (heads >= group_from) {
            if (GP == 4) hipLaunchKernelGGL((decode_merge_group_kernel<4>), dim3(B * store->Hkv), dim3(MERGE_THREADS), 0, st, a);
            else hipLaunchKernelGGL((decode_merge_group_kernel<8>), dim3(B * store->Hkv), dim3(MERGE_THREADS), 0, st, a);
        } else if (heads >= 256) {
            if (GP == 4) hipLaunchKernelGGL((decode_merge_kernel<4, 1>), dim3(heads), dim3(MERGE_THREADS), 0, st, a);
            else hipLaunchKernelGGL((decode_merge_kernel<8, 1>), dim3(heads), dim3(MERGE_THREADS), 0, st, a);
        } else if (heads >= 128) {
            if (GP == 4) hipLaunchKernelGGL((decode_merge_kernel<4, 2>), dim3(heads * 2), dim3(MERGE_THREADS), 0, st, a);
            else hipLaunchKernelGGL((decode_merge_kernel<8, 2>), dim3(heads * 2), dim3(MERGE_THREADS), 0, st, a);
        } else {
            if (GP == 4) hipLaunchKernelGGL((decode_merge_kernel<4, 4>), dim3(heads * 4), dim3(MERGE_THREADS), 0, st, a);
            else hipLaunchKernelGGL((decode_merge_kernel<8, 4>), dim3(heads * 4), dim3(MERGE_THREADS), 0, st, a);
        }
        ODMKV_CHECK_LAUNCH("decode_merge_kernel");
    }
    return 0;
}

extern "C" int odmkv_decode_attn(const void* q, int q_dtype, int B, int Hq, float scaling,
                                 const odmkv_packed_t* store, const odmkv_worklist_t* work,
                                 const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                                 const float* codebooks_host, const float* inv_scales,
                                 void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    return odmkv_decode_launch(q, q_dtype, B, Hq, scaling, store, work, pi_k_ops, pi_v, codebooks, codebooks_host, inv_scales,
                               out, out_dtype, lse, workspace, workspace_bytes, stream, 7, nullptr, nullptr);
}

// One decode step of a layer in a single call: the new token of every (sequence, kv-head) goes behind the stored
// exact tokens, then the attention of the step's query runs over the store, the new token included.
extern "C" int odmkv_decode_step(const odmkv_step_t* step, const void* q, const void* k_new, const void* v_new,
                                 int64_t stride_b, int64_t stride_h, int pos, void* out, float* lse, void* stream) {
    ODMKV_CHECK_ARG(step != nullptr, "decode_step: null step block");
    if (k_new || v_new) {
        ODMKV_CHECK_ARG(step->store != nullptr, "decode_step: null store");
        if (int rc = odmkv_append_exact(step->store, k_new, v_new, stride_b, stride_h, pos, stream)) return rc;
    }
    return odmkv_decode_launch(q, step->q_dtype, step->B, step->Hq, step->scaling, step->store, step->work, step->pi_k_ops,
                               step->pi_v, step->codebooks, step->codebooks_host, step->inv_scales, out, step->out_dtype, lse,
                               step->workspace, step->workspace_bytes, stream, 7, nullptr, nullptr);
}

// ------------------------------------------------------------------------------------------------
// The same call for callers that cannot allocate and have no workspace to hand over: the prepared
// queries and the partial results live in a fixed array of the library's own device image.
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
                                        const odmkv_packed_t* store, const odmkv_worklist_t* work,
                                        const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                                        const float* codebooks_host, const float* inv_scales,
                                        void* out, int out_dtype, float* lse, void* stream) {
    ODMKV_CHECK_ARG(work != nullptr, "decode_attn_static: null work list");
    ODMKV_CHECK_ARG(B > 0 && Hq > 0 && work->n_items >= 0, "decode_attn_static: bad shape B=%d Hq=%d items=%d", B, Hq, work->n_items);
    const size_t need = odmkv_decode_workspace_bytes(B, Hq, work->n_items);
    if (need > (size_t)ODMKV_STATIC_SCRATCH_BYTES) {
        odmkv_set_error("decode_attn_static: B=%d Hq=%d items=%d need %zu bytes of scratch, the fixed array holds %zu; "
                        "use odmkv_decode_attn with a workspace", B, Hq, work->n_items, need, (size_t)ODMKV_STATIC_SCRATCH_BYTES);
        return ODMKV_ENOSPACE;
    }
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return odmkv_decode_launch(q, q_dtype, B, Hq, scaling, store, work, pi_k_ops, pi_v, codebooks, codebooks_host, inv_scales,
                               out, out_dtype, lse, ws, (size_t)ODMKV_STATIC_SCRATCH_BYTES, stream, 7, nullptr, nullptr);
}
