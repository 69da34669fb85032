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
    int n_pairs;                          // units per (batch, head) of the 8-wavefront kernel's grid: pairs of query tiles, or ...
    int single_tiles;                     // ... single query tiles when this is set (launches that would not fill the GPU)
    // paged keys and values (prefill of a chunk on top of cached context): k, v are cache pools
    // (num_blocks, Hkv, 16, D); sequence b owns blocks block_table[b * table_stride + j] and ctx_lens[b] keys
    const int32_t* block_table;
    const int32_t* ctx_lens;
    int64_t table_stride;
    int num_blocks;
    int max_blocks;                       // entries of a table row that may be read: a longer context is cut to 16 * max_blocks keys
    // split keys (n_split > 1): workgroup (.., split c) serves the c-th share of every query tile's K/V tiles and
    // writes, instead of `out`, a normalised fp32 partial result and its log-sum-exp per query row:
    //   part_o  (n_split, Hq, part_rows, D)    part_lse (n_split, Hq, part_rows)
    // row = packed row, or b * Sq + i in the dense layout; a second kernel merges the partials into `out`
    int n_split;
    float* part_o;
    float* part_lse;
    int64_t part_rows;
};

// The 64-queries-per-wavefront kernel (head_dim 128, no mask or causal): prefill_fwd_w64.hip.
// prefill_w64_takes: whether its 32-bit address arithmetic covers the strides of p.
bool prefill_w64_takes(const PrefillParams& p);
int launch_prefill_w64(const PrefillParams& p, hipStream_t stream);

}  // namespace mi355
