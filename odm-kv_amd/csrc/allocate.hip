// Lagrangian bit allocation: for every non-sink token pick  argmin_k  s * eps_k + lambda * b_k,
// with lambda found by bisection so that the mean of the chosen widths meets the row's budget,
// then close the remaining gap by moving the lowest- (or highest-) scored tokens one level.
//
// The search is a fixed sequence of 74 evaluations (1 at lambda = 1, up to 8 widenings of the
// bracket, 64 halvings, 1 final), each a launch that histograms the chosen levels of all rows.
// The workgroup that finishes an evaluation last turns the histogram into the average and
// advances that row's bracket for the next launch; nothing ever waits on another workgroup
// and the host is never consulted.  All counts are integers, so the result does not depend
// on the order in which workgroups run.
//
// Arithmetic is kept exactly as the host formulation it replaces: fp32 products rounded
// separately and then added (no fused multiply-add), lambda rounded to fp32 before use, the
// first (lowest-width) level wins a tie, avg = fp32(sum) / fp32(n), bracket and gap in fp64.
#include "common.h"

#define NLV ODMKV_MAX_LEVELS
#define ITERS 74
#define IT_FINAL 73
#define HIST_TPT 8                       // tokens per thread in an evaluation
#define HIST_TOKENS (256 * HIST_TPT)

struct RowState {
    double lo, hi, target, gap, lam;
    double avg_hi;
    float lam32;
    int skip_until;          // evaluations with index < skip_until do nothing
    int n_active;
    unsigned int max_finite; // bit pattern
    int has_finite, has_nonfinite;
    int final_hist[NLV];
};

struct AllocArgs {
    const float* scores;
    const uint8_t* sink_mask;
    int rows, n, period, n_sink, sink_bits, K;
    float eps[NLV];
    float bitsf[NLV];
    int nominal[NLV];
    const double* target;    // device, [rows]
    float* s_clean;          // [rows, n]
    uint8_t* chosen;         // [rows, n]
    unsigned int* hist;      // [rows, ITERS, NLV]
    unsigned int* tickets;   // [rows, ITERS]
    RowState* state;         // [rows]
    int32_t* bits_out;
    int32_t* level_counts;
    double* lambda_out;
};

__device__ static inline bool is_sink(const AllocArgs& a, int row, int i) {
    if (a.sink_mask) return a.sink_mask[(size_t)row * a.n + i] != 0;
    return a.n_sink > 0 && (i % a.period) < a.n_sink;
}

// ---- clear counters, set up the bracket ----
__global__ void alloc_init_kernel(AllocArgs a) {
    const int row = blockIdx.x;
    for (int e = threadIdx.x; e < ITERS * NLV; e += blockDim.x) a.hist[(size_t)row * ITERS * NLV + e] = 0u;
    for (int e = threadIdx.x; e < ITERS; e += blockDim.x) a.tickets[(size_t)row * ITERS + e] = 0u;
    if (a.level_counts && threadIdx.x < a.K) a.level_counts[row * a.K + threadIdx.x] = 0;
    if (threadIdx.x == 0) {
        RowState& st = a.state[row];
        double t = a.target[row];                    // clamp the budget into the level range
        t = fmin(t, (double)a.nominal[a.K - 1]);
        t = fmax(t, (double)a.nominal[0]);
        st.lo = 0.0; st.hi = 1.0; st.target = t; st.gap = 0.0; st.lam = 1.0; st.avg_hi = 0.0;
        st.lam32 = 1.0f; st.skip_until = 0; st.n_active = 0; st.max_finite = 0u;
        st.has_finite = 0; st.has_nonfinite = 0;
        for (int k = 0; k < NLV; ++k) st.final_hist[k] = 0;
    }
}

// ---- what the sanitiser needs to know about a row ----
__global__ __launch_bounds__(256) void alloc_scan_kernel(AllocArgs a) {
    __shared__ unsigned int smax;
    __shared__ int sfin, snon, sact;
    const int row = blockIdx.y;
    if (threadIdx.x == 0) { smax = 0u; sfin = 0; snon = 0; sact = 0; }
    __syncthreads();
    unsigned int mx = 0u;
    int fin = 0, non = 0, act = 0;
    const int base = blockIdx.x * HIST_TOKENS;
    for (int e = 0; e < HIST_TPT; ++e) {
        const int i = base + e * 256 + threadIdx.x;
        if (i < a.n && !is_sink(a, row, i)) {
            ++act;
            float v = a.scores[(size_t)row * a.n + i];
            if (!(v != v)) v = fmaxf(v, 0.0f);          // clamp(min=0) keeps NaN
            if (isfinite(v)) { fin = 1; mx = max(mx, __float_as_uint(v)); }
            else non = 1;
        }
    }
    if (mx) atomicMax(&smax, mx);
    if (fin) atomicOr(&sfin, 1);
    if (non) atomicOr(&snon, 1);
    if (act) atomicAdd(&sact, act);
    __syncthreads();
    if (threadIdx.x == 0) {
        RowState& st = a.state[row];
        if (smax) atomicMax(&st.max_finite, smax);
        if (sfin) atomicOr(&st.has_finite, 1);
        if (snon) atomicOr(&st.has_nonfinite, 1);
        if (sact) atomicAdd(&st.n_active, sact);
    }
}

__global__ __launch_bounds__(256) void alloc_clean_kernel(AllocArgs a) {
    const int row = blockIdx.y;
    const RowState& st = a.state[row];
    const bool patch = st.has_finite && st.has_nonfinite;
    const float top = __uint_as_float(st.max_finite);
    const int base = blockIdx.x * HIST_TOKENS;
    for (int e = 0; e < HIST_TPT; ++e) {
        const int i = base + e * 256 + threadIdx.x;
        if (i < a.n) {
            float v = a.scores[(size_t)row * a.n + i];
            if (!(v != v)) v = fmaxf(v, 0.0f);
            if (patch && !isfinite(v)) v = top;
            if (v != v) v = 0.0f;                         // nan_to_num
            else if (v == INFINITY) v = 3.4028234663852886e38f;
            a.s_clean[(size_t)row * a.n + i] = v;
        }
    }
}

__device__ static inline int pick_level(const AllocArgs& a, float s, float lam32) {
    int best = 0;
    float bc = __fadd_rn(__fmul_rn(s, a.eps[0]), __fmul_rn(lam32, a.bitsf[0]));
#pragma unroll
    for (int k = 1; k < NLV; ++k) {
        if (k < a.K) {
            const float c = __fadd_rn(__fmul_rn(s, a.eps[k]), __fmul_rn(lam32, a.bitsf[k]));
            if (c < bc) { bc = c; best = k; }
        }
    }
    return best;
}

// the last workgroup of evaluation `it` advances the row's search state
__device__ static void advance(const AllocArgs& a, int row, int it) {
    RowState& st = a.state[row];
    unsigned long long S = 0ull;
    unsigned int h[NLV];
    for (int k = 0; k < a.K; ++k) {
        h[k] = atomicAdd(&a.hist[((size_t)row * ITERS + it) * NLV + k], 0u);
        S += (unsigned long long)h[k] * (unsigned long long)a.nominal[k];
    }
    const float avg32 = (float)S / (float)st.n_active;
    const double avg = (double)avg32;
    if (it <= 8) {                      // bracket widening: lambda = hi
        st.avg_hi = avg;
        if (avg > st.target && st.hi < 1e8 && it < 8) {
            st.hi *= 10.0;
            st.lam = st.hi;
            st.lam32 = (float)st.hi;
            st.skip_until = it + 1;
        } else {
            st.lam = (st.lo + st.hi) * 0.5;
            st.lam32 = (float)st.lam;
            st.skip_until = 9;
        }
    } else if (it < IT_FINAL) {         // halving
        if (avg > st.target) st.lo = st.lam; else st.hi = st.lam;
        st.lam = (st.lo + st.hi) * 0.5;
        st.lam32 = (float)st.lam;
        st.skip_until = it + 1;
    } else {                            // final assignment done
        st.gap = (avg - st.target) * (double)st.n_active;
        for (int k = 0; k < a.K; ++k) st.final_hist[k] = (int)h[k];
        if (a.lambda_out) a.lambda_out[row] = st.lam;
    }
}

__global__ __launch_bounds__(256) void alloc_eval_kernel(AllocArgs a, int it) {
    __shared__ unsigned int lh[NLV];
    __shared__ int is_last;
    const int row = blockIdx.y;
    const RowState& st = a.state[row];
    if (it < st.skip_until || st.n_active == 0) return;
    if (threadIdx.x < NLV) lh[threadIdx.x] = 0u;
    __syncthreads();
    const float lam32 = st.lam32;
    unsigned int cnt[NLV];
#pragma unroll
    for (int k = 0; k < NLV; ++k) cnt[k] = 0u;
    const int base = blockIdx.x * HIST_TOKENS;
    for (int e = 0; e < HIST_TPT; ++e) {
        const int i = base + e * 256 + threadIdx.x;
        if (i < a.n && !is_sink(a, row, i)) {
            const int k = pick_level(a, a.s_clean[(size_t)row * a.n + i], lam32);
#pragma unroll
            for (int j = 0; j < NLV; ++j) cnt[j] += (k == j);
            if (it == IT_FINAL) a.chosen[(size_t)row * a.n + i] = (uint8_t)k;
        }
    }
#pragma unroll
    for (int k = 0; k < NLV; ++k)
        if (cnt[k]) atomicAdd(&lh[k], cnt[k]);
    __syncthreads();
    if (threadIdx.x < a.K && lh[threadIdx.x])
        atomicAdd(&a.hist[((size_t)row * ITERS + it) * NLV + threadIdx.x], lh[threadIdx.x]);
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int t = atomicAdd(&a.tickets[(size_t)row * ITERS + it], 1u);
        is_last = (t == gridDim.x - 1);
    }
    __syncthreads();
    if (is_last && threadIdx.x == 0) {
        __threadfence();
        advance(a, row, it);
    }
}

// ---- budget repair: one workgroup per row, ordered passes over the row ----
#define RB 1024

// Moves `want` tokens currently at level `from` to level `to`: those with the smallest
// (score, index) if lowest, else those with the largest.  Scores are non-negative and finite,
// so their bit patterns order like the values.
__device__ static void move_tokens(const AllocArgs& a, int row, int from, int to, int want, bool lowest,
                                   unsigned int* hist256, int* scratch) {
    const float* s = a.s_clean + (size_t)row * a.n;
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
                const unsigned int key = __float_as_uint(s[i]);
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
            if (ch[i] == from && !is_sink(a, row, i) && __float_as_uint(s[i]) == prefix) ++local;
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
            const unsigned int key = __float_as_uint(s[i]);
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

__global__ __launch_bounds__(RB) void alloc_repair_kernel(AllocArgs a) {
    __shared__ unsigned int hist256[256];
    __shared__ int scratch[32];
    const int row = blockIdx.x;
    const RowState& st = a.state[row];
    if (st.n_active == 0) return;
    double gap = st.gap;
    if (fabs(gap) <= 0.5) return;
    if (gap > 0) {
        for (int i = 0; i < a.K - 1; ++i) {
            const double delta = (double)a.bitsf[i + 1] - (double)a.bitsf[i];
            if (delta <= 0) continue;
            const int n_dem = min(st.final_hist[i + 1], (int)(gap / delta + 0.5));
            if (n_dem <= 0) continue;
            move_tokens(a, row, i + 1, i, n_dem, true, hist256, scratch);
            gap -= n_dem * delta;
            if (gap <= 0.5) break;
        }
    } else {
        gap = -gap;
        for (int i = a.K - 2; i >= 0; --i) {
            const double delta = (double)a.bitsf[i + 1] - (double)a.bitsf[i];
            if (delta <= 0) continue;
            const int n_pro = min(st.final_hist[i], (int)(gap / delta + 0.5));
            if (n_pro <= 0) continue;
            move_tokens(a, row, i, i + 1, n_pro, false, hist256, scratch);
            gap -= n_pro * delta;
            if (gap <= 0.5) break;
        }
    }
}

__global__ __launch_bounds__(256) void alloc_write_kernel(AllocArgs a, int single_level) {
    __shared__ int lh[NLV];
    const int row = blockIdx.y;
    if (threadIdx.x < NLV) lh[threadIdx.x] = 0;
    __syncthreads();
    const int base = blockIdx.x * HIST_TOKENS;
    for (int e = 0; e < HIST_TPT; ++e) {
        const int i = base + e * 256 + threadIdx.x;
        if (i < a.n) {
            int out;
            if (is_sink(a, row, i)) out = a.sink_bits;
            else {
                const int k = single_level ? 0 : a.chosen[(size_t)row * a.n + i];
                out = a.nominal[k];
                atomicAdd(&lh[k], 1);
            }
            a.bits_out[(size_t)row * a.n + i] = out;
        }
    }
    __syncthreads();
    if (a.level_counts && threadIdx.x < a.K && lh[threadIdx.x])
        atomicAdd(&a.level_counts[row * a.K + threadIdx.x], lh[threadIdx.x]);
}

struct AllocLayout { size_t s_clean, chosen, hist, tickets, state, total; };
static AllocLayout alloc_layout(int rows, int n) {
    AllocLayout L;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
    L.s_clean = take((size_t)rows * n * sizeof(float));
    L.chosen = take((size_t)rows * n);
    L.hist = take((size_t)rows * ITERS * NLV * sizeof(unsigned int));
    L.tickets = take((size_t)rows * ITERS * sizeof(unsigned int));
    L.state = take((size_t)rows * sizeof(RowState));
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
    ODMKV_CHECK_ARG((double)n * 16.0 < 16777216.0, "allocate: rows longer than 1,048,575 tokens lose exactness of the fp32 mean");
    ODMKV_CHECK_ARG(workspace_bytes >= odmkv_allocate_workspace_bytes(rows, n), "allocate: workspace too small");
    hipStream_t st = (hipStream_t)stream;
    const AllocLayout L = alloc_layout(rows, n);
    char* ws = (char*)workspace;
    AllocArgs a;
    a.scores = scores; a.sink_mask = sink_mask; a.rows = rows; a.n = n;
    a.period = period > 0 ? period : n; a.n_sink = sink_mask ? 0 : n_sink; a.sink_bits = sink_bits; a.K = n_levels;
    for (int k = 0; k < NLV; ++k) {
        a.eps[k] = k < n_levels ? (float)eps[k] : 0.0f;
        a.bitsf[k] = k < n_levels ? (float)levels[k] : 0.0f;
        a.nominal[k] = k < n_levels ? levels[k] : 0;
    }
    a.target = target;
    a.s_clean = (float*)(ws + L.s_clean); a.chosen = (uint8_t*)(ws + L.chosen);
    a.hist = (unsigned int*)(ws + L.hist); a.tickets = (unsigned int*)(ws + L.tickets);
    a.state = (RowState*)(ws + L.state);
    a.bits_out = bits_out; a.level_counts = level_counts; a.lambda_out = lambda_out;
    const dim3 grid((n + HIST_TOKENS - 1) / HIST_TOKENS, rows), block(256);
    hipLaunchKernelGGL(alloc_init_kernel, dim3(rows), dim3(256), 0, st, a);
    ODMKV_CHECK_LAUNCH("alloc_init_kernel");
    if (n_levels > 1) {
        hipLaunchKernelGGL(alloc_scan_kernel, grid, block, 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_scan_kernel");
        hipLaunchKernelGGL(alloc_clean_kernel, grid, block, 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_clean_kernel");
        for (int it = 0; it < ITERS; ++it) {
            hipLaunchKernelGGL(alloc_eval_kernel, grid, block, 0, st, a, it);
            ODMKV_CHECK_LAUNCH("alloc_eval_kernel");
        }
        hipLaunchKernelGGL(alloc_repair_kernel, dim3(rows), dim3(RB), 0, st, a);
        ODMKV_CHECK_LAUNCH("alloc_repair_kernel");
    }
    hipLaunchKernelGGL(alloc_write_kernel, grid, block, 0, st, a, n_levels == 1 ? 1 : 0);
    ODMKV_CHECK_LAUNCH("alloc_write_kernel");
    return 0;
}
