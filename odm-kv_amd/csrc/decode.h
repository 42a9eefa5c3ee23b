// Internal interface of the fused decode attention: shared by the product entry points (decode.hip)
// and the measurement entry points (bench_hooks.hip, a library of its own).  Not part of the C ABI.
#pragma once
#include "quant.h"
#include <hip/hip_ext.h>

#define PSTRIDE 132          // floats per (item, head) partial result: 128 acc + m + l + 2 pad

struct DecodeArgs {
    odmkv_packed_t s;
    const void* q;
    int q_dt, out_dt;   // element types of q and out (ODMKV_F16 / BF16 / F32)
    int Hq, G, B;
    float scaling;
    const int32_t* items;
    int n_items;
    const int32_t* item_range;
    const int32_t* order;      // order[k] = item that workgroup k takes (long items first), or null: item k
    const uint16_t* pi_k_ops;   // Pi_k as the A operands of the query rotation (odmkv_rotation_operands)
    const float* pi_v;
    const float* cb;
    float inv_s[4];   // 1 / table scale per width
    float cbs[28];    // scaled centroids of widths 2, 3, 4 (kept in scalar registers; 8-bit ones stay in memory)
    int gp;           // head slots per item in `partial`: 4 or 8
    float* partial;   // [n_items, gp, PSTRIDE]
    void* out;
    float* lse;
};

// stage_mask: bit 1 the main kernel (query rotation included), bit 2 the merge (6 or 7 = the product
// call; bit 0 is unused).  ev_start / ev_stop: hipEvent_t attached to the main kernel's dispatch, or null.
int odmkv_decode_launch(const void* q, int q_dtype, int B, int Hq, float scaling,
                        const odmkv_packed_t* store, const odmkv_worklist_t* work,
                        const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                        const float* codebooks_host, const float* inv_scales,
                        void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                        void* stream, int stage_mask, void* ev_start, void* ev_stop);
