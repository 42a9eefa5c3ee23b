// Lloyd-Max codebook of the coordinate density of a randomly rotated unit vector, on the device.
//
// Follows the reference's offline routine (codebook.py:75-113, 36-72): a fixed grid of 10 000 points over
// [-x_range / sqrt(d), x_range / sqrt(d)], the density N(0, 1/d) at those points (d >= 100), centroids started
// evenly in [-3 / sqrt(d), 3 / sqrt(d)], and up to n_iter rounds of: walls = midpoints of neighbouring
// centroids; a cell's new centroid = sum(x w) * step / (sum(w) * step) over the grid points in [wall_i, wall_i+1);
// stop when no centroid moved by tol.  Everything in fp64, every expression rounded where numpy rounds it
// (the grid as start + j * step with the last point set to the end, the density as exp(-z*z/2)/sqrt(2 pi)/scale).
// Only the order inside a cell's two sums differs from numpy's (lanes stride over the cell, then a butterfly):
// the centroids agree with the host routine to about 1e-16 relative, far inside the rounding to the fp32 tables
// the kernels use.
//
// One workgroup: the density sits in LDS, a wavefront takes every sixteenth cell.  A table is a one-off per
// process; 500 rounds of the 256-level table take a couple of milliseconds.
#include "common.h"

#define LM_THREADS 1024
#define LM_GRID 10000
#define LM_MAXK 256

struct LloydArgs {
    int k, n_iter;
    double lo, hi, scale, tol, c_lo, c_hi;
    double* out;            // [k] centroids, ascending
    int* rounds;            // rounds run (or null)
};

__global__ __launch_bounds__(LM_THREADS) void lloyd_max_kernel(LloydArgs a) {
    extern __shared__ __align__(16) double w[];                       // [LM_GRID]
    __shared__ double cur[LM_MAXK], nxt[LM_MAXK], wall[LM_MAXK + 1];
    __shared__ double wdelta[LM_THREADS / WAVE];
    __shared__ int done;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int k = a.k;
    const double lin = (a.hi - a.lo) / (double)(LM_GRID - 1);
    const auto grid_at = [&](int j) { return j == LM_GRID - 1 ? a.hi : (double)j * lin + a.lo; };
    const double step = grid_at(1) - grid_at(0);
    for (int j = tid; j < LM_GRID; j += LM_THREADS) {
        const double z = (grid_at(j) - 0.0) / a.scale;
        w[j] = exp(-(z * z) / 2.0) / 2.5066282746310002 / a.scale;    // sqrt(2 pi)
    }
    if (tid < k) {
        const double cl = (a.c_hi - a.c_lo) / (double)(k - 1);
        cur[tid] = tid == k - 1 ? a.c_hi : (double)tid * cl + a.c_lo;
        nxt[tid] = cur[tid];
    }
    if (tid == 0) done = 0;
    __syncthreads();
    // first grid index whose point is >= v (the grid ascends)
    const auto first_at_or_above = [&](double v) {
        int lo = 0, hi = LM_GRID;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (grid_at(mid) < v) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    int it = 0;
    for (; it < a.n_iter; ++it) {
        if (tid <= k) wall[tid] = tid == 0 ? a.lo : tid == k ? a.hi : (cur[tid - 1] + cur[tid]) / 2.0;
        __syncthreads();
        for (int i = wave; i < k; i += LM_THREADS / WAVE) {
            const int first = first_at_or_above(wall[i]), last = first_at_or_above(wall[i + 1]);
            double s0 = 0.0, s1 = 0.0;
            for (int j = first + lane; j < last; j += WAVE) {
                const double wj = w[j];
                s0 += wj;
                s1 += grid_at(j) * wj;
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                s0 += __shfl_xor(s0, o, WAVE);
                s1 += __shfl_xor(s1, o, WAVE);
            }
            if (lane == 0) {
                const double mass = s0 * step;
                nxt[i] = mass > 0.0 ? s1 * step / mass : cur[i];
            }
        }
        __syncthreads();
        double moved = tid < k ? fabs(nxt[tid] - cur[tid]) : 0.0;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) moved = fmax(moved, __shfl_xor(moved, o, WAVE));
        if (lane == 0) wdelta[wave] = moved;
        __syncthreads();
        if (tid == 0) {
            double m = 0.0;
            for (int v = 0; v < LM_THREADS / WAVE; ++v) m = fmax(m, wdelta[v]);
            done = m < a.tol;
        }
        __syncthreads();
        if (done) { ++it; break; }                                     // the same for every thread
        if (tid < k) cur[tid] = nxt[tid];
        __syncthreads();
    }
    if (tid < k) a.out[tid] = nxt[tid];
    if (tid == 0 && a.rounds) *a.rounds = it;
}

extern "C" int odmkv_lloyd_max(int k, int d, int n_iter, double tol, double x_range, double* centroids,
                               int* rounds, void* stream) {
    ODMKV_CHECK_ARG(centroids != nullptr, "lloyd_max: null output");
    ODMKV_CHECK_ARG(k >= 2 && k <= LM_MAXK, "lloyd_max: %d levels (2 .. %d)", k, LM_MAXK);
    ODMKV_CHECK_ARG(d >= 100, "lloyd_max: dimension %d (the device routine covers the normal density of d >= 100)", d);
    ODMKV_CHECK_ARG(n_iter >= 1 && tol >= 0.0 && x_range > 0.0, "lloyd_max: bad iteration limits");
    LloydArgs a;
    a.k = k; a.n_iter = n_iter; a.tol = tol;
    a.scale = 1.0 / sqrt((double)d);
    a.lo = -x_range * a.scale; a.hi = x_range * a.scale;
    a.c_lo = -3 * a.scale; a.c_hi = 3 * a.scale;
    a.out = centroids; a.rounds = rounds;
    const int lds = LM_GRID * (int)sizeof(double);
    ODMKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&lloyd_max_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    hipLaunchKernelGGL(lloyd_max_kernel, dim3(1), dim3(LM_THREADS), lds, (hipStream_t)stream, a);
    ODMKV_CHECK_LAUNCH("lloyd_max_kernel");
    return 0;
}
