/* Oracle (test infrastructure): fixed-order fp32 restatement of the TurboQuant-MSE
 * quantiser, /root/reference/kvquant/tq_backend.py:185-197.
 *
 * The reference computes  norm = ||x||,  u = x / (norm + 1e-10),  y = u @ Pi^T  with
 * torch kernels whose fp32 summation order is not specified.  A code flips whenever
 * y lands within an ulp or two of a cell midpoint, so "bit-exact codes" needs one
 * agreed order.  This file fixes it, and the HIP kernel uses the same one:
 *
 *   ss   = fma(x[j], x[j], ss)           j = 0 .. d-1, starting from 0
 *   norm = sqrt(ss)                      (correctly rounded)
 *   u[j] = x[j] / (norm + 1e-10f)        (correctly rounded)
 *   y[i] = fma(u[j], Pi[i][j], y[i])     j = 0 .. d-1, starting from 0
 *   code = nearer of the two centroids bracketing y[i]; a tie keeps the lower index
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (fmaf is written out where a fused
 * operation is meant; nothing else may be contracted).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

/* First index i in [0, k) with c[i] >= y (torch.searchsorted, right=False), clamped to
 * [1, k-1]; then the nearer of c[i-1], c[i].  This is the op sequence the reference
 * comment describes (tq_backend.py:191-194): searchsorted, clamp, 2 subtract, 2 abs, where. */
static inline int nearest_centroid(float y, const float* c, int k) {
    int lo = 0, hi = k;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (c[mid] < y) lo = mid + 1; else hi = mid;
    }
    int pos = lo < 1 ? 1 : (lo > k - 1 ? k - 1 : lo);
    float dl = fabsf(y - c[pos - 1]);
    float dh = fabsf(y - c[pos]);
    return dh < dl ? pos : pos - 1;
}

void odmkv_canon_nearest(const float* y, size_t n, const float* c, int k, uint8_t* codes) {
    for (size_t i = 0; i < n; ++i) codes[i] = (uint8_t)nearest_centroid(y[i], c, k);
}

/* x: [n, d] fp32 (already widened from the cache dtype), pi: [d, d] row-major,
 * cb: [k] centroids.  Outputs: norms [n], codes [n, d] (one code per byte), and,
 * if y_out != NULL, the rotated unit vectors [n, d]. */
void odmkv_canon_quantize(const float* x, size_t n, int d, const float* pi,
                          const float* cb, int k, float* norms, uint8_t* codes,
                          float* y_out) {
    float u[1024];
    for (size_t r = 0; r < n; ++r) {
        const float* xr = x + r * (size_t)d;
        float ss = 0.0f;
        for (int j = 0; j < d; ++j) ss = fmaf(xr[j], xr[j], ss);
        float norm = sqrtf(ss);
        norms[r] = norm;
        float den = norm + 1e-10f;
        for (int j = 0; j < d; ++j) u[j] = xr[j] / den;
        /* eight outputs at a time: independent chains, each still summed in j order */
        for (int i0 = 0; i0 < d; i0 += 8) {
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            int nb = d - i0 < 8 ? d - i0 : 8;
            for (int j = 0; j < d; ++j)
                for (int b = 0; b < nb; ++b)
                    acc[b] = fmaf(u[j], pi[(size_t)(i0 + b) * d + j], acc[b]);
            for (int b = 0; b < nb; ++b) {
                if (y_out) y_out[r * (size_t)d + i0 + b] = acc[b];
                codes[r * (size_t)d + i0 + b] = (uint8_t)nearest_centroid(acc[b], cb, k);
            }
        }
    }
}
