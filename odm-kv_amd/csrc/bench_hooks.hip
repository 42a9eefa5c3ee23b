// Measurement entry points (libodmkv_bench.so only): per-call stage selection and kernel timing for
// the fused decode attention, and a plain streaming read as the roofline's yardstick.  No state
// outside the caller-owned timer.
#include "decode.h"
#include "../../include/odmkv_bench.h"
#include <vector>

struct BenchTimer {
    std::vector<hipEvent_t> events;   // 2 per record
    int used = 0;
};

extern "C" int odmkv_bench_timer_create(int max_records, void** timer) {
    ODMKV_CHECK_ARG(timer && max_records > 0 && max_records <= (1 << 20), "bench_timer_create: bad arguments");
    BenchTimer* t = new BenchTimer;
    t->events.resize((size_t)2 * max_records);
    for (auto& e : t->events) {
        if (hipEventCreate(&e) != hipSuccess) {
            odmkv_set_error("bench_timer_create: hipEventCreate failed");
            delete t;
            return ODMKV_EHIP;
        }
    }
    *timer = t;
    return 0;
}

extern "C" int odmkv_bench_timer_collect(void* timer, float* ms, int capacity, int* n_out) {
    ODMKV_CHECK_ARG(timer && ms && n_out && capacity >= 0, "bench_timer_collect: bad arguments");
    BenchTimer* t = (BenchTimer*)timer;
    int n = 0;
    for (int r = 0; r < t->used && n < capacity; ++r, ++n) {
        ODMKV_CHECK_HIP(hipEventSynchronize(t->events[2 * r + 1]));
        ODMKV_CHECK_HIP(hipEventElapsedTime(&ms[n], t->events[2 * r], t->events[2 * r + 1]));
    }
    *n_out = n;
    t->used = 0;
    return 0;
}

extern "C" int odmkv_bench_timer_destroy(void* timer) {
    ODMKV_CHECK_ARG(timer, "bench_timer_destroy: null timer");
    BenchTimer* t = (BenchTimer*)timer;
    for (auto& e : t->events) (void)hipEventDestroy(e);
    delete t;
    return 0;
}

extern "C" int odmkv_bench_decode_attn(const void* q, int q_dtype, int B, int Hq, float scaling,
                                       const odmkv_packed_t* store, const odmkv_worklist_t* work,
                                       const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                                       const float* codebooks_host, const float* inv_scales,
                                       void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                                       void* stream, int stage_mask, void* timer) {
    BenchTimer* t = (BenchTimer*)timer;
    const bool rec = t && work && (size_t)(2 * t->used + 1) < t->events.size() && work->n_items > 0 && (stage_mask & 2);
    hipEvent_t e0 = rec ? t->events[2 * t->used] : nullptr, e1 = rec ? t->events[2 * t->used + 1] : nullptr;
    const int rc = odmkv_decode_launch(q, q_dtype, B, Hq, scaling, store, work, pi_k_ops,
                                       pi_v, codebooks, codebooks_host, inv_scales, out, out_dtype, lse, workspace,
                                       workspace_bytes, stream, stage_mask & 7, e0, e1);
    if (rc == 0 && rec) ++t->used;
    return rc;
}

// plain streaming read of a buffer (grid-stride 16-byte loads folded into one word per thread)
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, size_t n16, unsigned int* sink) {
    unsigned int acc = 0u;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
        const uint4 v = p[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;       // practically never taken: keeps the loads alive
}

extern "C" int odmkv_bench_probe_read(const void* buf, size_t bytes, int grid, void* sink, void* stream) {
    ODMKV_CHECK_ARG(buf && sink && grid > 0 && ((uintptr_t)buf & 15) == 0, "probe_read: bad arguments");
    hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint4*>(buf), bytes / 16, reinterpret_cast<unsigned int*>(sink));
    ODMKV_CHECK_LAUNCH("probe_read_kernel");
    return 0;
}

extern "C" int odmkv_bench_pack_handed_over(const void* workspace, int B, int Hkv, int T, int32_t* counts, void* stream) {
    ODMKV_CHECK_ARG(workspace && counts && B > 0 && Hkv > 0 && T > 0, "bench_pack_handed_over: bad arguments");
    const char* p = (const char*)workspace + pack_redo_offset(B * Hkv, T);
    ODMKV_CHECK_HIP(hipMemcpyAsync(counts, p, 2 * sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream));
    ODMKV_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}
