// Lagrangian bit allocation: for every non-sink token pick  argmin_k  s * eps_k + lambda * b_k,
// with lambda found by bisection so that the mean of the chosen widths meets the row's budget,
// then close the remaining gap by moving the lowest- (or highest-) scored tokens one level.
//
// The search is the fixed sequence the host formulation runs: lambda = 1, up to 8 widenings of the
// bracket (x10 each), 64 halvings, one final assignment.  It is evaluated in 18 launches:
//   launch 0      all nine widening candidates 1, 10, .. 1e8 at once;
//   launch 1..16  four halvings each: the 15 midpoints the next four steps can reach form a binary
//                 tree that is known in advance, so one pass over the scores evaluates them all;
//   launch 17     the final lambda, which also records the chosen level of every token.
// The costs use lambda rounded to fp32, so once the bracket's ends are neighbouring fp32 numbers
// (after about 32 halvings on typical scores) the rest of the search is decided by rounding alone:
// it is walked on the spot and the remaining halving launches return immediately.
// Every workgroup writes its partial bit sums with plain stores and is done.  The next launch begins,
// in every workgroup, by adding up the row's partial sums of the launch before (a few hundred
// numbers) and walking the bracket with them; the row's first workgroup also writes the new state
// down for the launch after.  Nothing waits on another workgroup, no atomics cross workgroups, and
// the host is never consulted.  All sums are integers, so the result does not depend on the order
// in which workgroups run.  Partial sums and states are double-buffered by launch parity: a workgroup
// that finishes early must not overwrite what a late one of the same launch still reads.
//
// Arithmetic is kept exactly as the host formulation it replaces: fp32 products rounded
// separately and then added (no fused multiply-add), lambda rounded to fp32 before use, the
// first (lowest-width) level wins a tie, avg = fp32(sum) / fp32(n), bracket and gap in fp64.
#include "common.h"

#define NLV ODMKV_MAX_LEVELS
#define STEPS 4                               // halvings per launch
#define NCAND ((1 << STEPS) - 1)              // 15 tree nodes, numbered 1..15
#define N_WIDEN 9
#define N_HALVE_LAUNCH (64 / STEPS)
#define N_LAUNCH (1 + N_HALVE_LAUNCH + 1)
#define L_FINAL (N_LAUNCH - 1)
#define SLOTS 16                              // partial sums per workgroup
#define EV_THREADS 512
#ifndef EV_TPT
#define EV_TPT 2                              // tokens per thread in an evaluation
#endif
#define EV_TOKENS (EV_THREADS * EV_TPT)
#define CAND_MAX 16                           // repair moves of at most this many tokens take the short path

struct RowState {
    double lo, hi, target, gap, lam;
    int n_active;
    unsigned int max_finite; // bit pattern
    int has_finite, has_nonfinite;
    int lo_moved, hi_within;       // the bracket ends' averages are known (lo: above budget, hi: within)
    int collapsed;                 // the remaining halvings were resolved without evaluations
    int final_hist[NLV];
};

struct AllocArgs {
    const float* scores;
    const uint8_t* sink_mask;
    int rows, n, period, n_sink, sink_bits, K, n_chunks;
    float eps[NLV];
    float bitsf[NLV];
    int nominal[NLV];
    const double* target;          // device, [rows]
    uint8_t* chosen;               // [rows, n]
    unsigned int* partial;         // [2][rows, n_chunks, SLOTS]: launch L writes half L & 1
    unsigned long long* cand;      // [rows, n_chunks, CAND_MAX]
    RowState* state;               // [3][rows]: launch L >= 1 leaves the state it starts from in third L & 1 (launch 0 starts
                                   // from third 0, which the set-up kernels fill); third 2 is the final one
    int32_t* bits_out;
    int32_t* level_counts;
    double* lambda_out;
};

__device__ static inline bool is_sink(const AllocArgs& a, int row, int i) {
    if (a.sink_mask) return a.sink_mask[(size_t)row * a.n + i] != 0;
    return a.n_sink > 0 && (i % a.period) < a.n_sink;
}

// torch's clamp(min=0) / non-finite patch / nan_to_num, in that order
__device__ static inline float clean_score(float v, bool patch, float top) {
    if (!(v != v)) v = fmaxf(v, 0.0f);                // clamp(min=0) keeps NaN
    if (patch && !isfinite(v)) v = top;
    if (v != v) v = 0.0f;
    else if (v == INFINITY) v = 3.4028234663852886e38f;
    return v;
}

struct Cleaner {
    bool patch;
    float top;
    __device__ inline Cleaner(const RowState& st) : patch(st.has_finite && st.has_nonfinite), top(__uint_as_float(st.max_finite)) {}
    __device__ inline float operator()(float v) const { return clean_score(v, patch, top); }
};

__device__ static inline int wave_sum_int(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// ---- clear counters, set up the bracket ----
__global__ void alloc_init_kernel(AllocArgs a) {
    const int row = blockIdx.x;
    if (a.level_counts && (int)threadIdx.x < a.K) a.level_counts[row * a.K + threadIdx.x] = 0;
    if (threadIdx.x == 0) {
        RowState& st = a.state[row];
        double t = a.target[row];                    // clamp the budget into the level range
        t = fmin(t, (double)a.nominal[a.K - 1]);
        t = fmax(t, (double)a.nominal[0]);
        st.lo = 0.0; st.hi = 1.0; st.target = t; st.gap = 0.0; st.lam = 1.0;
        st.n_active = 0; st.max_finite = 0u; st.has_finite = 0; st.has_nonfinite = 0;
        st.lo_moved = 0; st.hi_within = 0; st.collapsed = 0;
        for (int k = 0; k < NLV; ++k) st.final_hist[k] = 0;
    }
}

// ---- what the sanitiser needs to know about a row ----
#define SC_THREADS 512
#define SC_TPT 8
#define SC_TOKENS (SC_THREADS * SC_TPT)
__global__ __launch_bounds__(SC_THREADS) void alloc_scan_kernel(AllocArgs a) {
    __shared__ unsigned int smax;
    __shared__ int sfin, snon, sact;
    const int row = blockIdx.y;
    if (threadIdx.x == 0) { smax = 0u; sfin = 0; snon = 0; sact = 0; }
    __syncthreads();
    unsigned int mx = 0u;
    int fin = 0, non = 0, act = 0;
    const int base = blockIdx.x * SC_TOKENS;
    float raw[SC_TPT];
    bool on[SC_TPT];
#pragma unroll
    for (int e = 0; e < SC_TPT; ++e) {                       // all reads first: one round trip, not SC_TPT
        const int i = base + e * SC_THREADS + threadIdx.x;
        on[e] = i < a.n && !is_sink(a, row, i);
        raw[e] = on[e] ? a.scores[(size_t)row * a.n + i] : 0.0f;
    }
#pragma unroll
    for (int e = 0; e < SC_TPT; ++e) {
        if (on[e]) {
            ++act;
            float v = raw[e];
            if (!(v != v)) v = fmaxf(v, 0.0f);
            if (isfinite(v)) { fin = 1; mx = max(mx, __float_as_uint(v)); }
            else non = 1;
        }
    }
    // a wavefront first combines its own lanes: 512 threads updating the same four words one after the other took
    // longer than reading the scores
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        mx = max(mx, (unsigned int)__shfl_xor((int)mx, o, WAVE));
        act += __shfl_xor(act, o, WAVE);
    }
    fin = __any(fin);
    non = __any(non);
    if ((threadIdx.x & 63) == 0) {
        if (mx) atomicMax(&smax, mx);
        if (fin) atomicOr(&sfin, 1);
        if (non) atomicOr(&snon, 1);
        if (act) atomicAdd(&sact, act);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        RowState& st = a.state[row];
        if (smax) atomicMax(&st.max_finite, smax);
        if (sfin) atomicOr(&st.has_finite, 1);
        if (snon) atomicOr(&st.has_nonfinite, 1);
        if (sact) atomicAdd(&st.n_active, sact);
    }
}

// lambda candidates of the four halvings that follow bracket (lo, hi): node 1 is the midpoint;
// from node m the search moves to 2m when the average is within budget (hi = mid), else to 2m + 1
__device__ static inline float tree_candidate(double lo, double hi, int node) {
    int depth = 31 - __clz(node);
    for (int d = depth - 1; d >= 0; --d) {
        const double mid = (lo + hi) * 0.5;
        if ((node >> d) & 1) lo = mid; else hi = mid;
    }
    return (float)((lo + hi) * 0.5);
}

// sums[] holds the row's totals of launch L, st the state that launch started from: advance the search
__device__ static void advance(const AllocArgs& a, RowState& st, int L, const unsigned int* sums) {
    const float nf = (float)st.n_active;
    if (L == 0) {
        double hi = 1.0;
        int j = 0;
        double avg_hi = (double)((float)sums[0] / nf);
        while (avg_hi > st.target && hi < 1e8) {
            hi *= 10.0;
            ++j;
            avg_hi = (double)((float)sums[j] / nf);
        }
        st.lo = 0.0; st.hi = hi;
        st.hi_within = !(avg_hi > st.target);
    } else if (L < L_FINAL) {
        double lo = st.lo, hi = st.hi;
        int node = 1;
        for (int s = 0; s < STEPS; ++s) {
            const double mid = (lo + hi) * 0.5;
            const double avg = (double)((float)sums[node] / nf);
            if (avg > st.target) { lo = mid; node = 2 * node + 1; st.lo_moved = 1; } else { hi = mid; node = 2 * node; st.hi_within = 1; }
        }
        // The costs see lambda rounded to fp32.  Once fp32(lo) and fp32(hi) are neighbouring floats,
        // every later midpoint rounds to one of the two, whose averages are known (lo was evaluated
        // above the budget, hi within it): the remaining halvings need no pass over the scores and
        // are walked here; the launches that would have evaluated them return at once.
        const float fl = (float)lo, fh = (float)hi;
        if (st.lo_moved && st.hi_within && fl < fh && nextafterf(fl, INFINITY) == fh) {
            for (int s = L * STEPS; s < N_HALVE_LAUNCH * STEPS; ++s) {
                const double mid = (lo + hi) * 0.5;
                if ((float)mid == fl) lo = mid; else hi = mid;
            }
            st.collapsed = 1;
            st.lam = (lo + hi) * 0.5;
        }
        st.lo = lo; st.hi = hi;
    } else {
        unsigned long long S = 0ull;
        for (int k = 0; k < a.K; ++k) {
            S += (unsigned long long)sums[k] * (unsigned long long)a.nominal[k];
            st.final_hist[k] = (int)sums[k];
        }
        const double avg = (double)((float)S / nf);
        st.gap = (avg - st.target) * (double)st.n_active;
        return;
    }
    if (L + 1 == L_FINAL) st.lam = (st.lo + st.hi) * 0.5;
}

// the lambda that slot c of launch L evaluates (slots a launch does not use evaluate lambda = 0 and are ignored)
__device__ static inline float candidate(const RowState& st, int L, int c) {
    if (L == 0) {
        double h = 1.0;
        for (int j = 0; j < c; ++j) h *= 10.0;
        return c < N_WIDEN ? (float)h : 0.0f;
    }
    if (L == L_FINAL) return (float)((st.lo + st.hi) * 0.5);
    return c >= 1 ? tree_candidate(st.lo, st.hi, c) : 0.0f;
}

// did launch L pass over the scores, given the state it started from?
__device__ static inline bool launch_evaluates(int n_active, int collapsed, int L) {
    return n_active != 0 && !(L > 0 && L < L_FINAL && collapsed);
}
__device__ static inline bool launch_evaluates(const RowState& st, int L) { return launch_evaluates(st.n_active, st.collapsed, L); }

// Start of launch L >= 1 (the candidate kernel calls it as launch L_FINAL + 1): the state launch L - 1
// started from plus that launch's partial sums give the state this launch starts from, left in `cur`
// (shared memory) for the whole workgroup; the row's first workgroup writes it to `out` as well.
// Ends with a barrier.
__device__ static void carry_state(const AllocArgs& a, int row, int L, RowState* out, RowState* cur, unsigned int* tot) {
    const int tid = threadIdx.x;
    const RowState* in = a.state + (size_t)((L - 1) & 1) * a.rows + row;
    // Everything the launch needs of the last one is asked for here, at once: the two fields that say whether that
    // launch evaluated, a thread's first partial sum (discarded if it did not), and the whole state, which thread 0
    // copies into shared memory and advances there (a private copy lived in scratch memory, behind the barriers, and
    // every access to it was a round trip of its own).
    const int in_active = in->n_active, in_collapsed = in->collapsed;
    const unsigned int* p = a.partial + ((size_t)((L - 1) & 1) * a.rows + row) * a.n_chunks * SLOTS;
    const int n_part = a.n_chunks * SLOTS;
    const unsigned int v0 = tid < n_part ? p[tid] : 0u;
    if (tid == 0) *cur = *in;
    if (tid < SLOTS) tot[tid] = 0u;
    __syncthreads();
    const bool evaluated = launch_evaluates(in_active, in_collapsed, L - 1);
    if (evaluated) {
        // thread tid holds slot tid % SLOTS of chunk tid / SLOTS (the block size is a multiple of SLOTS, so every
        // further element of the thread is the same slot); the four chunks of a wavefront are added across its
        // 16-lane rows before one lane per slot updates the total
        static_assert(SLOTS == 16 && EV_THREADS % SLOTS == 0, "a slot per lane of a 16-lane row");
        unsigned int v = v0;
        for (int idx = tid + blockDim.x; idx < n_part; idx += blockDim.x) v += p[idx];
        v += (unsigned int)__shfl_xor((int)v, 16, WAVE);
        v += (unsigned int)__shfl_xor((int)v, 32, WAVE);
        if ((tid & 63) < SLOTS && v) atomicAdd(&tot[tid & (SLOTS - 1)], v);
    }
    __syncthreads();
    if (tid == 0) {
        if (evaluated) advance(a, *cur, L - 1, tot);
        if (blockIdx.x == 0) {
            *out = *cur;
            if (L - 1 == L_FINAL && evaluated && a.lambda_out) a.lambda_out[row] = cur->lam;
        }
    }
    __syncthreads();
}

// sums of 16-bit fields over the wave: on return, lanes with (lane & 7) == 0 hold packed pair
// number (lane >> 3) in v[0]
__device__ static inline void reduce_scatter8(unsigned int (&v)[8], int lane) {
#pragma unroll
    for (int half = 4; half >= 1; half >>= 1) {
        const int o = half * 8;                 // 32, 16, 8
        const bool upper = (lane & o) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const unsigned int send = upper ? v[i] : v[i + half];
            const unsigned int keep = upper ? v[i + half] : v[i];
            v[i] = keep + (unsigned int)__shfl_xor((int)send, o, WAVE);
        }
    }
#pragma unroll
    for (int o = 4; o > 0; o >>= 1) v[0] += (unsigned int)__shfl_xor((int)v[0], o, WAVE);
}

template <int K>
__global__ __launch_bounds__(EV_THREADS) void alloc_eval_kernel(AllocArgs a, int L) {
    __shared__ __align__(16) float lamb[SLOTS][NLV];     // fl32(lambda_c * b_k)
    __shared__ int lsum[SLOTS];
    __shared__ unsigned int tot[SLOTS];
    __shared__ RowState cur;
    const int row = blockIdx.y, tid = threadIdx.x;
    // the scores are asked for first: they do not depend on the state, which takes a round trip of its own
    const int base = blockIdx.x * EV_TOKENS;
    float raw[EV_TPT];
    bool active[EV_TPT];
#pragma unroll
    for (int e = 0; e < EV_TPT; ++e) {
        const int i = base + e * EV_THREADS + tid;
        active[e] = i < a.n && !is_sink(a, row, i);
        raw[e] = active[e] ? a.scores[(size_t)row * a.n + i] : 0.0f;
    }
    if (L == 0) {
        if (tid == 0) cur = a.state[row];
        __syncthreads();
    } else {
        carry_state(a, row, L, a.state + (size_t)(L & 1) * a.rows + row, &cur, tot);
    }
    const RowState& st = cur;
    if (!launch_evaluates(st, L)) return;                   // an empty row, or this launch's halvings are already decided
    if (tid < SLOTS * NLV) {
        const int c = tid / NLV, k = tid % NLV;
        lamb[c][k] = __fmul_rn(candidate(st, L, c), a.bitsf[k]);
    }
    if (tid < SLOTS) lsum[tid] = 0;
    __syncthreads();

    const Cleaner clean(st);
    float se[EV_TPT][K];
#pragma unroll
    for (int e = 0; e < EV_TPT; ++e) {
        const float s = active[e] ? clean(raw[e]) : 0.0f;
#pragma unroll
        for (int k = 0; k < K; ++k) se[e][k] = __fmul_rn(s, a.eps[k]);
    }

    if (L != L_FINAL) {
        unsigned int acc[8];
#pragma unroll
        for (int p = 0; p < 8; ++p) acc[p] = 0u;
#pragma unroll
        for (int c = 0; c < SLOTS; ++c) {
            const float4 l0 = *reinterpret_cast<const float4*>(&lamb[c][0]);
            const float4 l1 = *reinterpret_cast<const float4*>(&lamb[c][4]);
            const float lb[NLV] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
            unsigned int sum = 0u;
#pragma unroll
            for (int e = 0; e < EV_TPT; ++e) {
                float bc = __fadd_rn(se[e][0], lb[0]);
                int bn = a.nominal[0];
#pragma unroll
                for (int k = 1; k < K; ++k) {
                    const float cst = __fadd_rn(se[e][k], lb[k]);
                    if (cst < bc) { bc = cst; bn = a.nominal[k]; }
                }
                sum += active[e] ? (unsigned int)bn : 0u;
            }
            acc[c >> 1] += sum << (16 * (c & 1));           // at most 64 lanes * EV_TPT * 16 per field
        }
        reduce_scatter8(acc, tid & 63);
        if ((tid & 7) == 0) {
            const int p = (tid & 63) >> 3;
            if (acc[0] & 0xffffu) atomicAdd(&lsum[2 * p], (int)(acc[0] & 0xffffu));
            if (acc[0] >> 16) atomicAdd(&lsum[2 * p + 1], (int)(acc[0] >> 16));
        }
    } else {
        int cnt[NLV];
#pragma unroll
        for (int k = 0; k < NLV; ++k) cnt[k] = 0;
#pragma unroll
        for (int e = 0; e < EV_TPT; ++e) {
            float bc = __fadd_rn(se[e][0], lamb[0][0]);
            int best = 0;
#pragma unroll
            for (int k = 1; k < K; ++k) {
                const float cst = __fadd_rn(se[e][k], lamb[0][k]);
                if (cst < bc) { bc = cst; best = k; }
            }
            if (active[e]) {
                a.chosen[(size_t)row * a.n + base + e * EV_THREADS + tid] = (uint8_t)best;
#pragma unroll
                for (int k = 0; k < NLV; ++k) cnt[k] += (best == k);
            }
        }
#pragma unroll
        for (int k = 0; k < NLV; ++k) {
            const int s = wave_sum_int(cnt[k]);
            if ((tid & 63) == 0 && s) atomicAdd(&lsum[k], s);
        }
    }
    __syncthreads();
    unsigned int* mine = a.partial + (((size_t)(L & 1) * a.rows + row) * a.n_chunks + blockIdx.x) * SLOTS;
    if (tid < SLOTS) mine[tid] = (unsigned int)lsum[tid];
}

// ---- budget repair -------------------------------------------------------------------------------
// The host formulation sorts the row by score (stable) and, walking the level pairs, moves the
// n lowest-scored tokens of the upper level down (over budget) or the n highest-scored tokens of the
// lower level up (under budget).  Equivalent without a sort: among the tokens at level `from`,
// take the n smallest (largest) 64-bit keys (score bits, index).
struct Move { int from, to, want, i; bool lowest; double delta; };

// the first level pair, at or after pair index i in walking order, that moves tokens
__device__ static inline bool next_move(const AllocArgs& a, const int* hist, double gap_abs, bool over, int i, Move& m) {
    for (; over ? i < a.K - 1 : i >= 0; i += over ? 1 : -1) {
        const double delta = (double)a.bitsf[i + 1] - (double)a.bitsf[i];
        if (delta <= 0) continue;
        const int have = over ? hist[i + 1] : hist[i];
        const int n = min(have, (int)(gap_abs / delta + 0.5));
        if (n <= 0) continue;
        m.from = over ? i + 1 : i; m.to = over ? i : i + 1; m.want = n; m.i = i; m.lowest = over; m.delta = delta;
        return true;
    }
    return false;
}

__device__ static inline unsigned long long token_key(float s, int i, bool lowest) {
    // + 1 keeps both k and ~k away from the "no key" value
    const unsigned long long k = (((unsigned long long)__float_as_uint(s) << 32) | (unsigned int)i) + 1ull;
    return lowest ? k : ~k;            // always select minima
}
__device__ static inline unsigned int key_index(unsigned long long g, bool lowest) {
    return (unsigned int)(((lowest ? g : ~g) - 1ull) & 0xffffffffull);
}

__device__ static inline unsigned long long wave_min_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(v, o, WAVE);
        v = other < v ? other : v;
    }
    return v;
}

#define KEY_NONE 0xffffffffffffffffull

// `want` rounds of a workgroup-wide minimum over the keys held in registers; every selected key is
// handed to `emit(round, key)` by thread 0 and struck from its owner's registers
template <int NK, int NWAVES, typename F>
__device__ static inline void select_smallest(unsigned long long (&keys)[NK], int want, unsigned long long* wbest, F emit) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    for (int r = 0; r < want; ++r) {
        unsigned long long best = KEY_NONE;
#pragma unroll
        for (int e = 0; e < NK; ++e) best = keys[e] < best ? keys[e] : best;
        const unsigned long long wb = wave_min_u64(best);
        if (lane == 0) wbest[wave] = wb;
        __syncthreads();
        unsigned long long g = KEY_NONE;
        for (int w = 0; w < NWAVES; ++w) g = wbest[w] < g ? wbest[w] : g;
        if (g != KEY_NONE) {
#pragma unroll
            for (int e = 0; e < NK; ++e) keys[e] = keys[e] == g ? KEY_NONE : keys[e];
        }
        if (tid == 0) emit(r, g);
        __syncthreads();
    }
}

// per chunk: the candidates for the first move when it is small
__global__ __launch_bounds__(EV_THREADS) void alloc_cand_kernel(AllocArgs a) {
    __shared__ unsigned long long wbest[EV_THREADS / 64];
    __shared__ unsigned int tot[SLOTS];
    __shared__ RowState cur;
    const int row = blockIdx.y, tid = threadIdx.x;
    carry_state(a, row, L_FINAL + 1, a.state + (size_t)2 * a.rows + row, &cur, tot);     // the final state: gap, histogram, lambda
    const RowState& st = cur;
    if (st.n_active == 0 || fabs(st.gap) <= 0.5) return;
    const bool over = st.gap > 0;
    Move m;
    if (!next_move(a, st.final_hist, fabs(st.gap), over, over ? 0 : a.K - 2, m) || m.want > CAND_MAX) return;
    const Cleaner clean(st);
    unsigned long long keys[EV_TPT];
    const int base = blockIdx.x * EV_TOKENS;
#pragma unroll
    for (int e = 0; e < EV_TPT; ++e) {
        const int i = base + e * EV_THREADS + tid;
        keys[e] = KEY_NONE;
        if (i < a.n && !is_sink(a, row, i) && a.chosen[(size_t)row * a.n + i] == m.from)
            keys[e] = token_key(clean(a.scores[(size_t)row * a.n + i]), i, m.lowest);
    }
    unsigned long long* out = a.cand + ((size_t)row * a.n_chunks + blockIdx.x) * CAND_MAX;
    select_smallest<EV_TPT, EV_THREADS / 64>(keys, m.want, wbest, [&](int r, unsigned long long g) { out[r] = g; });
}

#define RB 1024

// Moves `want` tokens currently at level `from` to level `to`: those with the smallest
// (score, index) if lowest, else those with the largest.  Scores are non-negative and finite,
// so their bit patterns order like the values.
__device__ static void move_tokens(const AllocArgs& a, int row, const Cleaner& clean, int from, int to, int want,
                                   bool lowest, unsigned int* hist256, int* scratch) {
    const float* s = a.scores + (size_t)row * a.n;
    uint8_t* ch = a.chosen + (size_t)row * a.n;
    const int tid = threadIdx.x;
    // radix select, most significant byte first: find the key of the want-th token
    unsigned int prefix = 0u, pmask = 0u;
    int remaining = want;       // rank still to find inside the current prefix class
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int e = tid; e < 256; e += RB) hist256[e] = 0u;
        __syncthreads();
        for (int i = tid; i < a.n; i += RB) {
            if (ch[i] == from && !is_sink(a, row, i)) {
                const unsigned int key = __float_as_uint(clean(s[i]));
                if ((key & pmask) == prefix) atomicAdd(&hist256[(key >> shift) & 0xffu], 1u);
            }
        }
        __syncthreads();
        if (tid == 0) {
            int acc = 0, bin;
            if (lowest) {
                for (bin = 0; bin < 256; ++bin) { if (acc + (int)hist256[bin] >= remaining) break; acc += hist256[bin]; }
            } else {
                for (bin = 255; bin >= 0; --bin) { if (acc + (int)hist256[bin] >= remaining) break; acc += hist256[bin]; }
            }
            bin = bin < 0 ? 0 : (bin > 255 ? 255 : bin);
            scratch[0] = bin;
            scratch[1] = remaining - acc;
        }
        __syncthreads();
        prefix |= ((unsigned int)scratch[0]) << shift;
        pmask |= 0xffu << shift;
        remaining = scratch[1];
        __syncthreads();
    }
    // `prefix` is the threshold key; `remaining` of the tokens equal to it move, in index order
    // (the first ones if lowest, the last ones otherwise)
    if (tid == 0) scratch[2] = 0;      // ties seen so far
    if (!lowest) {
        // count the ties to know how many to skip
        if (tid == 0) scratch[3] = 0;
        __syncthreads();
        int local = 0;
        for (int i = tid; i < a.n; i += RB)
            if (ch[i] == from && !is_sink(a, row, i) && __float_as_uint(clean(s[i])) == prefix) ++local;
        if (local) atomicAdd(&scratch[3], local);
        __syncthreads();
    }
    __syncthreads();
    const int n_eq = lowest ? 0 : scratch[3];
    const int first_tie = lowest ? 0 : n_eq - remaining;          // ties with rank in [first_tie, first_tie + remaining) move
    const int wave = tid >> 6, lane = tid & 63;
    int* wave_cnt = scratch + 8;                                  // [16]
    for (int c = 0; c < a.n; c += RB) {
        const int i = c + tid;
        bool member = false, tie = false, strict = false;
        if (i < a.n && ch[i] == from && !is_sink(a, row, i)) {
            member = true;
            const unsigned int key = __float_as_uint(clean(s[i]));
            tie = key == prefix;
            strict = lowest ? key < prefix : key > prefix;
        }
        const unsigned long long m = __ballot(tie);
        if (lane == 0) wave_cnt[wave] = __popcll(m);
        __syncthreads();
        int rank = scratch[2] + __popcll(m & ((1ull << lane) - 1ull));
        for (int w = 0; w < wave; ++w) rank += wave_cnt[w];
        if (member && (strict || (tie && rank >= first_tie && rank < first_tie + remaining))) ch[i] = (uint8_t)to;
        __syncthreads();
        if (tid == 0) {
            int tot = 0;
            for (int w = 0; w < RB / 64; ++w) tot += wave_cnt[w];
            scratch[2] += tot;
        }
        __syncthreads();
    }
}

// one workgroup per row: apply the first move from the chunk candidates when it is small, any other
// move by a radix select over the row
__global__ __launch_bounds__(RB) void alloc_repair_kernel(AllocArgs a) {
    __shared__ unsigned int hist256[256];
    __shared__ int scratch[32];
    __shared__ unsigned long long wbest[RB / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    const RowState& st = a.state[(size_t)2 * a.rows + row];
    if (st.n_active == 0) return;
    double gap = st.gap;
    if (fabs(gap) <= 0.5) return;
    const bool over = gap > 0;
    gap = fabs(gap);
    const Cleaner clean(st);
    int i = over ? 0 : a.K - 2;
    Move m;
    bool first = true;
    while (next_move(a, st.final_hist, gap, over, i, m)) {
        if (first && m.want <= CAND_MAX) {
            uint8_t* ch = a.chosen + (size_t)row * a.n;
            const unsigned long long* cand = a.cand + (size_t)row * a.n_chunks * CAND_MAX;
            const int total = a.n_chunks * m.want;
            if (total <= 4 * RB) {
                unsigned long long keys[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int idx = e * RB + tid;
                    keys[e] = idx < total ? cand[(size_t)(idx / m.want) * CAND_MAX + idx % m.want] : KEY_NONE;
                }
                select_smallest<4, RB / 64>(keys, m.want, wbest, [&](int, unsigned long long g) {
                    if (g != KEY_NONE) ch[key_index(g, m.lowest)] = (uint8_t)m.to;
                });
            } else {
                move_tokens(a, row, clean, m.from, m.to, m.want, m.lowest, hist256, scratch);
            }
        } else {
            __syncthreads();
            move_tokens(a, row, clean, m.from, m.to, m.want, m.lowest, hist256, scratch);
        }
        first = false;
        gap -= m.want * m.delta;
        if (gap <= 0.5) break;
        i = m.i + (over ? 1 : -1);
    }
}

__global__ __launch_bounds__(EV_THREADS) void alloc_write_kernel(AllocArgs a, int single_level) {
    __shared__ int lh[NLV];
    const int row = blockIdx.y;
    if (threadIdx.x < NLV) lh[threadIdx.x] = 0;
    __syncthreads();
    const int base = blockIdx.x * EV_TOKENS;
    const bool count = a.level_counts != nullptr;          // the histogram is optional
    for (int e = 0; e < EV_TPT; ++e) {
        const int i = base + e * EV_THREADS + threadIdx.x;
        int k = -1;
        if (i < a.n) {
            int out;
            if (is_sink(a, row, i)) out = a.sink_bits;
            else {
                k = single_level ? 0 : a.chosen[(size_t)row * a.n + i];
                out = a.nominal[k];
            }
            a.bits_out[(size_t)row * a.n + i] = out;
        }
        if (count) {
            // a wavefront counts its lanes per level by ballot: a thousand threads adding 1 to the same word, one
            // after the other, took longer than writing the bits
            for (int lv = 0; lv < a.K; ++lv) {
                const int n = __popcll(__ballot(k == lv));
                if ((threadIdx.x & 63) == 0 && n) atomicAdd(&lh[lv], n);
            }
        }
    }
    __syncthreads();
    if (a.level_counts && (int)threadIdx.x < a.K && lh[threadIdx.x])
        atomicAdd(&a.level_counts[row * a.K + threadIdx.x], lh[threadIdx.x]);
}

struct AllocLayout { size_t chosen, partial, cand, state, total; };
static AllocLayout alloc_layout(int rows, int n) {
    AllocLayout L;
    const size_t chunks = ((size_t)n + EV_TOKENS - 1) / EV_TOKENS;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
    L.chosen = take((size_t)rows * n);
    L.partial = take((size_t)2 * rows * chunks * SLOTS * sizeof(unsigned int));
    L.cand = take((size_t)rows * chunks * CAND_MAX * sizeof(unsigned long long));
    L.state = take((size_t)3 * rows * sizeof(RowState));
    L.total = off;
    return L;
}

extern "C" size_t odmkv_allocate_workspace_bytes(int rows, int n) {
    if (rows <= 0 || n <= 0) return 0;
    return alloc_layout(rows, n).total;
}

extern "C" int odmkv_allocate(const float* scores, int rows, int n,
                              const uint8_t* sink_mask, int period, int n_sink, int sink_bits,
                              const int32_t* levels, int n_levels, const double* eps,
                              const double* target,
                              int32_t* bits_out, int32_t* level_counts, double* lambda_out,
                              void* workspace, size_t workspace_bytes, void* stream) {
    ODMKV_CHECK_ARG(scores && levels && eps && target && bits_out && workspace, "allocate: null pointer");
    ODMKV_CHECK_ARG(rows > 0 && n > 0, "allocate: bad shape rows=%d n=%d", rows, n);
    ODMKV_CHECK_ARG(n_levels >= 1 && n_levels <= NLV, "allocate: between 1 and %d levels, got %d", NLV, n_levels);
    for (int k = 0; k < n_levels; ++k) {
        ODMKV_CHECK_ARG(levels[k] >= 0 && levels[k] <= 16, "allocate: level %d out of range", levels[k]);
        ODMKV_CHECK_ARG(k == 0 || levels[k] > levels[k - 1], "allocate: levels must be strictly ascending");
    }
    ODMKV_CHECK_ARG(sink_mask || n_sink == 0 || (period > 0 && n % period == 0 && n_sink <= period),
                    "allocate: bad sink pattern period=%d n_sink=%d n=%d", period, n_sink, n);
    // bit sums up to 2^24 are exact in fp32, which the fp32 mean of the host formulation relies on
    ODMKV_CHECK_ARG((double)n * 16.0 <= 16777216.0, "allocate: rows longer than 1,048,576 tokens lose exactness of the fp32 mean");
    ODMKV_CHECK_ARG(rows <= 65535, "allocate: at most 65535 rows per call");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_allocate_workspace_bytes(rows, n), "allocate: workspace too small");
    hipStream_t st = (hipStream_t)stream;
    const AllocLayout L = alloc_layout(rows, n);
    char* ws = (char*)workspace;
    AllocArgs a;
    a.scores = scores; a.sink_mask = sink_mask; a.rows = rows; a.n = n;
    a.period = period > 0 ? period : n; a.n_sink = sink_mask ? 0 : n_sink; a.sink_bits = sink_bits; a.K = n_levels;
    a.n_chunks = (n + EV_TOKENS - 1) / EV_TOKENS;
    for (int k = 0; k < NLV; ++k) {
        a.eps[k] = k < n_levels ? (float)eps[k] : 0.0f;
        a.bitsf[k] = k < n_levels ? (float)levels[k] : 0.0f;
        a.nominal[k] = k < n_levels ? levels[k] : 0;
    }
    a.target = target;
    a.chosen = (uint8_t*)(ws + L.chosen);
    a.partial = (unsigned int*)(ws + L.partial);
    a.cand = (unsigned long long*)(ws + L.cand);
    a.state = (RowState*)(ws + L.state);
    a.bits_out = bits_out; a.level_counts = level_counts; a.lambda_out = lambda_out;
    const dim3 grid(a.n_chunks, rows), block(EV_THREADS);
    hipLaunchKernelGGL(alloc_init_kernel, dim3(rows), dim3(64), 0, st, a);
    ODMKV_CHECK_LAUNCH("alloc_init_kernel");
    if (n_levels > 1) {
        hipLaunchKernelGGL(alloc_scan_kernel, dim3((n + SC_TOKENS - 1) / SC_TOKENS, rows), dim3(SC_THREADS), 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_scan_kernel");
        for (int l = 0; l < N_LAUNCH; ++l) {
            switch (n_levels) {
                case 2: hipLaunchKernelGGL(alloc_eval_kernel<2>, grid, block, 0, st, a, l); break;
                case 3: hipLaunchKernelGGL(alloc_eval_kernel<3>, grid, block, 0, st, a, l); break;
                case 4: hipLaunchKernelGGL(alloc_eval_kernel<4>, grid, block, 0, st, a, l); break;
                case 5: hipLaunchKernelGGL(alloc_eval_kernel<5>, grid, block, 0, st, a, l); break;
                case 6: hipLaunchKernelGGL(alloc_eval_kernel<6>, grid, block, 0, st, a, l); break;
                case 7: hipLaunchKernelGGL(alloc_eval_kernel<7>, grid, block, 0, st, a, l); break;
                default: hipLaunchKernelGGL(alloc_eval_kernel<8>, grid, block, 0, st, a, l); break;
            }
            ODMKV_CHECK_LAUNCH("alloc_eval_kernel");
        }
        hipLaunchKernelGGL(alloc_cand_kernel, grid, block, 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_cand_kernel");
        hipLaunchKernelGGL(alloc_repair_kernel, dim3(rows), dim3(RB), 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_repair_kernel");
    }
    hipLaunchKernelGGL(alloc_write_kernel, grid, block, 0, st, a, n_levels == 1 ? 1 : 0);
    ODMKV_CHECK_LAUNCH("alloc_write_kernel");
    return 0;
}
