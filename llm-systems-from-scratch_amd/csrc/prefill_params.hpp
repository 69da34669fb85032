// Arguments of the prefill forward kernels (shared by the two kernel files).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

struct PrefillParams {
    const __bf16* q;
    const __bf16* k;
    const __bf16* v;
    __bf16* out;
    int64_t qs[3], ks[3], vs[3], os[3];   // batch, head, row strides (elements)
    const int32_t* cu_q;
    const int32_t* cu_k;
    const uint8_t* mask;
    int64_t ms[3];
    float* lse;                           // optional: natural-log sum of exp of the scaled scores, per query row
    int64_t ls[2];                        // its batch and head strides (elements); rows are contiguous
    int B, Hq, Hkv, Sq, Sk;
    float scale_log2;
    int mask_mode;
    int n_qtiles;
    int n_pairs;
};

// The 64-queries-per-wavefront kernel (head_dim 128, no mask or causal, no lse): prefill_fwd_w64.hip.
int launch_prefill_w64(const PrefillParams& p, hipStream_t stream);

}  // namespace mi355
