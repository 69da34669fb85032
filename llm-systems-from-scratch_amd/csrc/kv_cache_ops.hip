// Producers of the paged KV cache: interleaved-pair RoPE + scatter of new K/V rows into
// cache blocks, and per-(block, kv head) fp8-e4m3 quantisation of cache blocks.
// Both are plain streaming kernels (HBM-bound, a few bytes per element).
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"

namespace mi355 {

struct RopeCacheParams {
    const __bf16* q_in;
    const __bf16* k_in;
    const __bf16* v_in;
    __bf16* q_out;
    __bf16* k_cache;
    __bf16* v_cache;
    const float* freq;            // (2, context_length, D/2): cos plane then sin plane
    const int32_t* positions;     // (T)
    const int64_t* slots;         // (T): block * 16 + offset, negative = do not write the cache
    __bf16* k_out;                // optional: rotated keys, packed (T, Hkv, D), for a prefill over the same tokens
    int64_t q_tok, k_tok, v_tok, qo_tok, ko_tok;   // token strides (elements); heads are contiguous (stride D)
    int T, Hq, Hkv, D, ctx_len;
    int head_slots;                // head slots served per token: Hq query heads, then Hkv key heads, then Hkv value heads
    int64_t n_slots;               // num_blocks * 16: slots outside [0, n_slots) are not written
};

// One thread per (token, head slot, pair of adjacent elements).  Head slots: Hq query heads,
// then Hkv key heads, then Hkv value heads.  Rotation of the pair (x[2i], x[2i+1]) by the angle
// of (position, i), in fp32, rounded once to bf16.
__global__ __launch_bounds__(256) void rope_and_cache_kernel(RopeCacheParams p) {
    const int half = p.D / 2;
    const int slots_per_tok = p.head_slots;
    const int64_t total = (int64_t)p.T * slots_per_tok * half;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(idx % half);
        const int hs = (int)((idx / half) % slots_per_tok);
        const int t = (int)(idx / ((int64_t)half * slots_per_tok));
        const int pos = min(max(p.positions[t], 0), p.ctx_len - 1);     // a position outside the table is clamped into it
        int64_t slot = p.slots ? p.slots[t] : -1;
        if (slot >= p.n_slots) slot = -1;
        if (hs < p.Hq) {
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.q_in + t * p.q_tok + (int64_t)hs * p.D + 2 * i);
            const bf16x2 x = __builtin_bit_cast(bf16x2, raw);
            const float c = p.freq[(int64_t)pos * half + i];
            const float s = p.freq[((int64_t)p.ctx_len + pos) * half + i];
            const float x1 = (float)x[0], x2 = (float)x[1];
            *reinterpret_cast<uint32_t*>(p.q_out + t * p.qo_tok + (int64_t)hs * p.D + 2 * i) =
                pack_bf16(c * x1 - s * x2, s * x1 + c * x2);
        } else if (hs < p.Hq + p.Hkv) {
            if (slot < 0 && !p.k_out) continue;
            const int hk = hs - p.Hq;
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.k_in + t * p.k_tok + (int64_t)hk * p.D + 2 * i);
            const bf16x2 x = __builtin_bit_cast(bf16x2, raw);
            const float c = p.freq[(int64_t)pos * half + i];
            const float s = p.freq[((int64_t)p.ctx_len + pos) * half + i];
            const float x1 = (float)x[0], x2 = (float)x[1];
            const uint32_t rot = pack_bf16(c * x1 - s * x2, s * x1 + c * x2);
            if (slot >= 0)
                *reinterpret_cast<uint32_t*>(p.k_cache + (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D + 2 * i) = rot;
            if (p.k_out) *reinterpret_cast<uint32_t*>(p.k_out + t * p.ko_tok + (int64_t)hk * p.D + 2 * i) = rot;
        } else {
            if (slot < 0) continue;
            const int hk = hs - p.Hq - p.Hkv;
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.v_in + t * p.v_tok + (int64_t)hk * p.D + 2 * i);
            const int64_t dst = (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D + 2 * i;
            *reinterpret_cast<uint32_t*>(p.v_cache + dst) = raw;
        }
    }
}

// The same work with 16-byte accesses.  A thread owns one group of 4 pairs (8 elements, index c) of a token
// in kRopeHeads head slots, so the angles of (position, c) are fetched once for all of them: reading
// the table per head slot would put twice the payload's bytes through the vector memory pipeline and
// bound the kernel there instead of at HBM.  Consecutive threads own consecutive (head slot, c), so one
// wavefront instruction still covers 1 KiB of adjacent memory; the thread's head slots are
// hu, hu + n_hu, hu + 2 n_hu, ... with n_hu = ceil(head slots / kRopeHeads).
// Requires D % 8 == 0, token strides that are multiples of 8 elements and 16-byte aligned bases.
// The grid covers the work once (workgroups in dispatch order walk through memory as one window).
constexpr int kRopeHeads = 4;
// (block, n_blocks: this workgroup's index among the workgroups that share the work, and their number)
__device__ __forceinline__ void rope_and_cache_vec8_body(const RopeCacheParams& p, int n_hu, unsigned block, unsigned n_blocks) {
    const int groups = p.D / 8;
    const int half = p.D / 2;
    const int slots_per_tok = p.head_slots;
    const int64_t total = (int64_t)p.T * n_hu * groups;
    for (int64_t idx = block * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)n_blocks * blockDim.x) {
        const int c = (int)(idx % groups);
        const int hu = (int)((idx / groups) % n_hu);
        const int t = (int)(idx / ((int64_t)groups * n_hu));
        int64_t slot = p.slots ? p.slots[t] : -1;
        if (slot >= p.n_slots) slot = -1;
        const int pos = min(max(p.positions[t], 0), p.ctx_len - 1);     // a position outside the table is clamped into it
        u32x4 raw[kRopeHeads];
        __bf16 *dst[kRopeHeads], *dst2[kRopeHeads];        // dst2: a key's second home, the packed k_out
        bool rotate[kRopeHeads];
#pragma unroll
        for (int j = 0; j < kRopeHeads; ++j) {
            const int hs = hu + j * n_hu;
            const bool is_q = hs < p.Hq;
            dst[j] = dst2[j] = nullptr;
            rotate[j] = false;
            const bool is_v = hs >= p.Hq + p.Hkv;
            if (hs >= slots_per_tok || (!is_q && slot < 0 && (is_v || !p.k_out))) continue;
            const int hk = is_v ? hs - p.Hq - p.Hkv : hs - p.Hq;
            const __bf16* src = is_q ? p.q_in + t * p.q_tok + (int64_t)hs * p.D
                                     : (is_v ? p.v_in + t * p.v_tok : p.k_in + t * p.k_tok) + (int64_t)hk * p.D;
            raw[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + 8 * c));
            rotate[j] = !is_v;
            if (is_q) dst[j] = p.q_out + t * p.qo_tok + (int64_t)hs * p.D + 8 * c;
            else if (slot >= 0) dst[j] = (is_v ? p.v_cache : p.k_cache) + (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D + 8 * c;
            if (!is_q && !is_v && p.k_out) dst2[j] = p.k_out + t * p.ko_tok + (int64_t)hk * p.D + 8 * c;
        }
        const f32x4 cs = *reinterpret_cast<const f32x4*>(p.freq + (int64_t)pos * half + 4 * c);
        const f32x4 sn = *reinterpret_cast<const f32x4*>(p.freq + ((int64_t)p.ctx_len + pos) * half + 4 * c);
#pragma unroll
        for (int j = 0; j < kRopeHeads; ++j) {
            if (!dst[j] && !dst2[j]) continue;
            u32x4 w4 = raw[j];
            if (rotate[j]) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t w = raw[j][e];           // scalar copy first: a bit_cast of a vector element misreads it
                    const bf16x2 x = __builtin_bit_cast(bf16x2, w);
                    const float x1 = (float)x[0], x2 = (float)x[1];
                    w4[e] = pack_bf16(cs[e] * x1 - sn[e] * x2, sn[e] * x1 + cs[e] * x2);
                }
            }
            if (dst[j]) __builtin_nontemporal_store(w4, reinterpret_cast<u32x4*>(dst[j]));
            if (dst2[j]) __builtin_nontemporal_store(w4, reinterpret_cast<u32x4*>(dst2[j]));
        }
    }
}

__global__ __launch_bounds__(256) void rope_and_cache_vec8_kernel(RopeCacheParams p, int n_hu) {
    rope_and_cache_vec8_body(p, n_hu, blockIdx.x, gridDim.x);
}

// One wavefront per (block, kv head) slab of 16*D bf16: absmax -> scale = absmax/448 (1 for an
// all-zero slab) -> x/scale clamped to +-448 -> e4m3 (round to nearest even).
template <int D>
__global__ __launch_bounds__(256) void quantize_kv_fp8_kernel(const __bf16* __restrict__ src, unsigned char* __restrict__ dst,
                                                             float* __restrict__ scale, int64_t n_slabs) {
    constexpr int NV = 16 * D / 8 / 64;             // 16-byte loads per lane: load j covers elements [512 j, 512 j + 512)
    const int lane = threadIdx.x & 63;
    const int64_t wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    for (int64_t slab = wave; slab < n_slabs; slab += (int64_t)gridDim.x * 4) {
        const __bf16* s = src + slab * (16 * D) + lane * 8;
        u32x4 raw[NV];
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j) raw[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + 512 * j));
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const bf16x8 x = as_bf16x8(raw[j]);
#pragma unroll
            for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)x[e]));
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        const float sc = amax > 0.f ? amax / 448.0f : 1.0f;
        if (lane == 0) scale[slab] = sc;
        unsigned char* d = dst + slab * (16 * D) + lane * 8;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const bf16x8 x = as_bf16x8(raw[j]);
            float y[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = fminf(fmaxf((float)x[e] / sc, -448.0f), 448.0f);
            int w0 = 0, w1 = 0;
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
            w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
            w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
            u32x2 out;
            out[0] = (uint32_t)w0;
            out[1] = (uint32_t)w1;
            __builtin_nontemporal_store(out, reinterpret_cast<u32x2*>(d + 512 * j));
        }
    }
}


// ---- fused RoPE + write into an fp8 cache with per-(block, kv head) scales ------------------
struct RopeCacheFp8Params {
    const __bf16* k_in;
    const __bf16* v_in;
    unsigned char* k_cache;
    unsigned char* v_cache;
    float* k_scale;
    float* v_scale;
    const float* freq;
    const int32_t* positions;
    const int64_t* slots;
    int64_t k_tok, v_tok;
    int T, Hkv, ctx_len;
    int64_t n_slots;
};

__device__ __forceinline__ void quantize8(const float (&x)[8], float sc, unsigned char* dst) {
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = fminf(fmaxf(x[e] / sc, -448.0f), 448.0f);
    int w0 = 0, w1 = 0;
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    u32x2 out;
    out[0] = (uint32_t)w0;
    out[1] = (uint32_t)w1;
    *reinterpret_cast<u32x2*>(dst) = out;
}

// One wavefront per (window of `win` consecutive tokens, kv head, K or V).  A RUN is a stretch of
// consecutive tokens whose slots are consecutive inside one cache block; the wavefront writes every
// run that STARTS in its window, whole (at most 16 rows), so exactly one wavefront touches a
// (block, head) slab:
//   scale' = max(scale of the rows already in the block, absmax(new rows) / 448)
//   rows already in the block are re-expressed in scale' when it grew (fp8 -> fp32 -> fp8)
//   new rows (keys rotated and rounded to bf16 first, as the bf16 cache would hold them) -> e4m3
// The scale therefore always equals absmax/448 of the block's valid rows, as in quantize_kv_fp8_kernel.
// A lane owns 8 adjacent elements of one row: D/8 lanes per row, 512/D rows per pass.
// win = 16 for a packed prefill (one run per window when sequences start at block boundaries),
// win = 1 for a decode step (every token is its own run; all of them proceed in parallel).
template <int D>
__device__ __forceinline__ void rope_and_cache_fp8_body(const RopeCacheFp8Params& p, int win, int n_windows, unsigned block) {
    constexpr int LPR = D / 8, RPP = 64 / LPR, NP = 16 / RPP;
    const int lane = threadIdx.x & 63;
    const int64_t w = (int64_t)block * 4 + (threadIdx.x >> 6);
    if (w >= (int64_t)n_windows * 2 * p.Hkv) return;
    const int window = (int)(w / (2 * p.Hkv));
    const int rem = (int)(w % (2 * p.Hkv));
    const bool is_v = rem >= p.Hkv;
    const int hk = is_v ? rem - p.Hkv : rem;
    const int c = lane % LPR, rip = lane / LPR;
    const int half = D / 2;
    // Lane i holds the slot of token base - 1 + i: lane 0 the token before the window, lanes 1..win the
    // window, then 15 tokens of look-ahead (a run that starts in the window may end beyond it).
    const int base = window * win;
    const int64_t tok_i = (int64_t)base - 1 + lane;
    int64_t my_slot = -1;
    int my_pos = 0;                    // (fetched with the slot: a key row's angles then wait for one load, not two)
    if (lane < win + 16 && tok_i >= 0 && tok_i < p.T) {
        my_slot = p.slots[tok_i];
        if (!is_v) my_pos = p.positions[tok_i];
    }
    if (my_slot >= p.n_slots) my_slot = -1;
    const int64_t prev_slot = __shfl_up(my_slot, 1, 64);
    // a token continues the run of the token before it when both sit in the same block at consecutive offsets
    const bool cont = lane >= 1 && my_slot >= 0 && (my_slot & 15) != 0 && prev_slot == my_slot - 1;
    const uint64_t cont_mask = __builtin_amdgcn_ballot_w64(cont);
    uint64_t head_mask = __builtin_amdgcn_ballot_w64(lane >= 1 && lane <= win && my_slot >= 0 && !cont);
    while (head_mask != 0) {
        const int h = __builtin_ctzll(head_mask);
        head_mask &= head_mask - 1;
        const int t = base - 1 + h;
        const int64_t slot = __shfl(my_slot, h, 64);
        const int off0 = (int)(slot & 15);
        const int n = 1 + __builtin_ctzll(~(cont_mask >> (h + 1)));       // tokens of the run (at most 16 - off0)

        const int64_t slab = (slot >> 4) * p.Hkv + hk;
        unsigned char* cache = (is_v ? p.v_cache : p.k_cache) + slab * (16 * D);
        float* scale = (is_v ? p.v_scale : p.k_scale) + slab;

        float val[NP][8];
        float amax = 0.f;
#pragma unroll
        for (int pi = 0; pi < NP; ++pi) {
            const int j = pi * RPP + rip;                 // row of the block
#pragma unroll
            for (int e = 0; e < 8; ++e) val[pi][e] = 0.f;
            // (every lane takes part in the exchange: a lane outside the run reads some lane's value and drops it)
            const int pos_j = __shfl(my_pos, (h + j - off0) & 63, 64);
            if (j >= off0 && j < off0 + n) {
                const int tok = t + j - off0;
                const __bf16* src = (is_v ? p.v_in + tok * p.v_tok : p.k_in + tok * p.k_tok) + (int64_t)hk * D + 8 * c;
                u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src));
                if (!is_v) {
                    const int pos = min(max(pos_j, 0), p.ctx_len - 1);
                    const f32x4 cs = *reinterpret_cast<const f32x4*>(p.freq + (int64_t)pos * half + 4 * c);
                    const f32x4 sn = *reinterpret_cast<const f32x4*>(p.freq + ((int64_t)p.ctx_len + pos) * half + 4 * c);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t wd = raw[q];
                        const bf16x2 x = __builtin_bit_cast(bf16x2, wd);
                        const float x1 = (float)x[0], x2 = (float)x[1];
                        raw[q] = pack_bf16(cs[q] * x1 - sn[q] * x2, sn[q] * x1 + cs[q] * x2);
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t wd = raw[q];
                    const bf16x2 x = __builtin_bit_cast(bf16x2, wd);
                    val[pi][2 * q] = (float)x[0];
                    val[pi][2 * q + 1] = (float)x[1];
                    amax = fmaxf(amax, fmaxf(fabsf(val[pi][2 * q]), fabsf(val[pi][2 * q + 1])));
                }
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));

        float sc;
        if (off0 == 0) {
            sc = amax > 0.f ? amax / 448.0f : 1.0f;      // a fresh block: whatever the slab held is dead
        } else {
            const float old = *scale;
            sc = fmaxf(old, amax / 448.0f);
            if (sc != old) {
#pragma unroll
                for (int pi = 0; pi < NP; ++pi) {
                    const int j = pi * RPP + rip;
                    if (j < off0) {
                        unsigned char* row = cache + j * D + 8 * c;
                        const u32x2 raw = *reinterpret_cast<const u32x2*>(row);
                        const u32x2 lo = fp8x4_to_bf16x4(raw[0]), hi = fp8x4_to_bf16x4(raw[1]);
                        const uint32_t wd[4] = {lo[0], lo[1], hi[0], hi[1]};
                        float x[8];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const bf16x2 b = __builtin_bit_cast(bf16x2, wd[q]);
                            x[2 * q] = (float)b[0] * old;
                            x[2 * q + 1] = (float)b[1] * old;
                        }
                        quantize8(x, sc, row);
                    }
                }
            }
        }
        if (lane == 0) *scale = sc;
#pragma unroll
        for (int pi = 0; pi < NP; ++pi) {
            const int j = pi * RPP + rip;
            if (j >= off0 && j < off0 + n) quantize8(val[pi], sc, cache + j * D + 8 * c);
        }
    }
}

// Queries (rotation only, bf16) and keys/values (rotation, quantisation) of one call in ONE launch: the workgroups
// of the two kinds are dealt alternately (`ratio` query workgroups, then one key/value workgroup), so that the
// latency-bound key/value wavefronts -- slot ids, then rows, then scales, each a dependent load -- run in the shadow
// of the streaming query rows instead of after them.
template <int D>
__global__ __launch_bounds__(256) void rope_and_cache_fp8_fused_kernel(RopeCacheParams pq, int n_hu, unsigned q_blocks,
                                                                      RopeCacheFp8Params p, int win, int n_windows,
                                                                      unsigned kv_blocks, unsigned ratio) {
    const unsigned group = blockIdx.x / (ratio + 1), pos = blockIdx.x % (ratio + 1);
    if (pos < ratio) {
        const unsigned b = group * ratio + pos;
        if (b < q_blocks) rope_and_cache_vec8_body(pq, n_hu, b, q_blocks);
    } else if (group < kv_blocks) {
        rope_and_cache_fp8_body<D>(p, win, n_windows, group);
    }
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_rope_and_cache(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_cache,
                                    void* v_cache, const float* freq_cache, const int32_t* positions,
                                    const int64_t* slot_mapping, int64_t num_blocks, int T, int Hq, int Hkv, int D,
                                    int context_length,
                                    int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
                                    int64_t q_out_token_stride, void* k_out, int64_t k_out_token_stride, void* stream) {
    if (!q_in || !k_in || !v_in || !q_out || !freq_cache || !positions)
        return set_error(MI355_EINVAL, "rope_and_cache: null pointer argument");
    if (k_out && (k_out_token_stride & 1))
        return set_error(MI355_EINVAL, "rope_and_cache: token strides must be even (4-byte aligned pairs)");
    if (slot_mapping && (!k_cache || !v_cache))
        return set_error(MI355_EINVAL, "rope_and_cache: slot_mapping given without k_cache/v_cache");
    if (slot_mapping && num_blocks <= 0) return set_error(MI355_EINVAL, "rope_and_cache: num_blocks must be positive");
    if (T < 0 || Hq <= 0 || Hkv <= 0 || context_length <= 0)
        return set_error(MI355_EINVAL, "rope_and_cache: T, Hq, Hkv, context_length out of range");
    if (D <= 0 || (D & 1)) return set_error(MI355_EINVAL, "rope_and_cache: head_dim must be even");
    if ((q_token_stride | k_token_stride | v_token_stride | q_out_token_stride) & 1)
        return set_error(MI355_EINVAL, "rope_and_cache: token strides must be even (4-byte aligned pairs)");
    if (T == 0) return MI355_OK;
    RopeCacheParams p;
    p.q_in = (const __bf16*)q_in;
    p.k_in = (const __bf16*)k_in;
    p.v_in = (const __bf16*)v_in;
    p.q_out = (__bf16*)q_out;
    p.k_cache = (__bf16*)k_cache;
    p.v_cache = (__bf16*)v_cache;
    p.freq = freq_cache;
    p.positions = positions;
    p.slots = slot_mapping;
    p.q_tok = q_token_stride;
    p.k_tok = k_token_stride;
    p.v_tok = v_token_stride;
    p.qo_tok = q_out_token_stride;
    p.k_out = (__bf16*)k_out;
    p.ko_tok = k_out ? k_out_token_stride : 0;
    p.T = T;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.D = D;
    p.ctx_len = context_length;
    p.head_slots = slot_mapping ? Hq + 2 * Hkv : (k_out ? Hq + Hkv : Hq);     // nothing to do for values without a cache
    p.n_slots = slot_mapping ? num_blocks * 16 : 0;
    const auto aligned16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    const bool vec8 = D % 8 == 0 && ((q_token_stride | k_token_stride | v_token_stride | q_out_token_stride) & 7) == 0 &&
                      aligned16(q_in) && aligned16(k_in) && aligned16(v_in) && aligned16(q_out) && aligned16(k_cache) &&
                      aligned16(v_cache) && aligned16(freq_cache) && aligned16(k_out) && (p.ko_tok & 7) == 0;
    const int n_hu = (p.head_slots + kRopeHeads - 1) / kRopeHeads;
    const int64_t total = vec8 ? (int64_t)T * n_hu * (D / 8) : (int64_t)T * p.head_slots * (D / 2);
    const int64_t blocks = (total + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 0x7fffffffLL ? blocks : 0x7fffffffLL);
    if (vec8)
        hipLaunchKernelGGL(rope_and_cache_vec8_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, p, n_hu);
    else
        hipLaunchKernelGGL(rope_and_cache_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, p);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" int mi355_quantize_kv_fp8(const void* cache_bf16, void* cache_fp8, float* scale, int64_t num_blocks, int Hkv,
                                     int D, int block_size, void* stream) {
    if (!cache_bf16 || !cache_fp8 || !scale) return set_error(MI355_EINVAL, "quantize_kv_fp8: null pointer argument");
    if (block_size != 16) return set_error(MI355_EINVAL, "quantize_kv_fp8: block_size must be 16");
    if (num_blocks < 0 || Hkv <= 0) return set_error(MI355_EINVAL, "quantize_kv_fp8: num_blocks, Hkv out of range");
    if (!(D == 32 || D == 64 || D == 128)) return set_error(MI355_EINVAL, "quantize_kv_fp8: head_dim must be 32, 64 or 128");
    const int64_t n_slabs = num_blocks * Hkv;
    if (n_slabs == 0) return MI355_OK;
    const int64_t wgs = (n_slabs + 3) / 4;                  // four wavefronts (slabs) per workgroup
    const unsigned grid = (unsigned)(wgs < 0x7fffffffLL ? wgs : 0x7fffffffLL);
    hipStream_t s = (hipStream_t)stream;
    if (D == 128)
        hipLaunchKernelGGL(quantize_kv_fp8_kernel<128>, dim3(grid), dim3(256), 0, s, (const __bf16*)cache_bf16,
                           (unsigned char*)cache_fp8, scale, n_slabs);
    else if (D == 64)
        hipLaunchKernelGGL(quantize_kv_fp8_kernel<64>, dim3(grid), dim3(256), 0, s, (const __bf16*)cache_bf16,
                           (unsigned char*)cache_fp8, scale, n_slabs);
    else
        hipLaunchKernelGGL(quantize_kv_fp8_kernel<32>, dim3(grid), dim3(256), 0, s, (const __bf16*)cache_bf16,
                           (unsigned char*)cache_fp8, scale, n_slabs);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}


namespace mi355 {

// ---------------------------------------------------------------------------------------------
// Gather + dequantise: the keys and values of every sequence of a batch, read through the block tables out of an
// fp8 cache, written as packed bf16 rows (sequence b owns rows [cu_k[b], cu_k[b+1])) -- the K/V operands of a packed
// prefill (mi355_prefill_fwd with cu_seqlens), so that a chunk of a prompt can attend to an fp8 cache on the same
// kernels as to bf16 tensors.  One wavefront per (sequence, logical block, kv head): a K and a V slab of 16 x D bytes in,
// 16 rows of D bf16 out each; value = bf16(fp8 * scale), the scale of the slab.  Rows at or past the context length (the
// tail of a sequence's last block) and rows past `max_rows` are not written.
struct GatherFp8Params {
    const unsigned char* k_cache;
    const unsigned char* v_cache;
    const float* k_scale;
    const float* v_scale;
    const int32_t* tables;
    const int32_t* ctx_lens;
    const int32_t* cu_k;
    __bf16* k_out;
    __bf16* v_out;
    int64_t table_stride, out_tok, max_rows;
    int max_blocks, B, Hkv, num_blocks;
};

template <int D>
__global__ __launch_bounds__(256) void gather_kv_fp8_kernel(GatherFp8Params p) {
    const int lane = threadIdx.x & 63;
    const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)p.B * p.max_blocks * p.Hkv;
    if (w >= n_waves) return;
    const int hk = (int)(w % p.Hkv);
    const int64_t bj = w / p.Hkv;
    const int j = (int)(bj % p.max_blocks), b = (int)(bj / p.max_blocks);
    const int ctx = min(p.ctx_lens[b], 16 * p.max_blocks);          // a length beyond what the table addresses is truncated
    if (16 * j >= ctx) return;
    int phys = p.tables[(int64_t)b * p.table_stride + j];
    phys = min(max(phys, 0), p.num_blocks - 1);                     // a corrupt table cannot leave the pool
    const int64_t slab = (int64_t)phys * p.Hkv + hk;
    const int64_t row0 = (int64_t)p.cu_k[b] + 16 * j;
    constexpr int kPasses = (16 * D + 1023) / 1024;
    // all loads of the K and the V slab first (one dependent chain for both), then the conversions and the stores
    u32x4 raw[2][kPasses];
    float scale[2];
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const unsigned char* src = (which ? p.v_cache : p.k_cache) + slab * (16 * D);
        scale[which] = (which ? p.v_scale : p.k_scale)[slab];
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) {
            const int e = (pass * 64 + lane) * 16;                  // first of this lane's 16 elements of the slab
            raw[which][pass] = e < 16 * D ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + e)) : u32x4{0u, 0u, 0u, 0u};
        }
    }
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __bf16* out = which ? p.v_out : p.k_out;
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) {
            const int e = (pass * 64 + lane) * 16;
            if (e >= 16 * D) break;
            const int row = e / D, col = e % D;
            if (16 * j + row >= ctx || row0 + row >= p.max_rows) continue;
            uint32_t w16[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // (exact: e4m3 is a subset of bf16.  The upper two bytes are shifted down and converted with the same
                // selector: in this kernel the compiler merged the two conversions of one word that differ only in the
                // selector, and every second pair of elements came out as a copy of the pair before it.)
                const bf16x2 lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw[which][pass][i], 1.0f, false);
                const bf16x2 hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw[which][pass][i] >> 16, 1.0f, false);
                w16[2 * i] = pack_bf16((float)lo[0] * scale[which], (float)lo[1] * scale[which]);
                w16[2 * i + 1] = pack_bf16((float)hi[0] * scale[which], (float)hi[1] * scale[which]);
            }
            u32x4* dst = reinterpret_cast<u32x4*>(out + (row0 + row) * p.out_tok + (int64_t)hk * D + col);
            __builtin_nontemporal_store(u32x4{w16[0], w16[1], w16[2], w16[3]}, dst);
            __builtin_nontemporal_store(u32x4{w16[4], w16[5], w16[6], w16[7]}, dst + 1);
        }
    }
}

}  // namespace mi355

extern "C" int mi355_gather_kv_fp8(const void* k_cache_fp8, const void* v_cache_fp8, const float* k_scale,
                                   const float* v_scale, const int32_t* block_tables, int64_t table_stride,
                                   int64_t max_blocks, const int32_t* context_lens, const int32_t* cu_seqlens_k,
                                   void* k_out, void* v_out, int64_t out_token_stride, int64_t max_rows, int B, int Hkv,
                                   int D, int block_size, int64_t num_blocks, void* stream) {
    if (!k_cache_fp8 || !v_cache_fp8 || !k_scale || !v_scale || !block_tables || !context_lens || !cu_seqlens_k || !k_out || !v_out)
        return set_error(MI355_EINVAL, "gather_kv_fp8: null pointer argument");
    if (block_size != 16) return set_error(MI355_EINVAL, "gather_kv_fp8: block_size must be 16");
    if (B <= 0 || Hkv <= 0 || max_blocks <= 0 || max_blocks > 0x7ffffff || table_stride < max_blocks || max_rows < 0)
        return set_error(MI355_EINVAL, "gather_kv_fp8: B, Hkv, max_blocks, table_stride, max_rows out of range");
    if (num_blocks <= 0 || num_blocks > 0x7fffffffLL) return set_error(MI355_EINVAL, "gather_kv_fp8: num_blocks out of range");
    if (!(D == 32 || D == 64 || D == 128)) return set_error(MI355_EINVAL, "gather_kv_fp8: head_dim must be 32, 64 or 128");
    if ((out_token_stride & 7) != 0 || out_token_stride < (int64_t)Hkv * D)
        return set_error(MI355_EINVAL, "gather_kv_fp8: out_token_stride must be a multiple of 8 and at least Hkv * D");
    if (((uintptr_t)k_cache_fp8 | (uintptr_t)v_cache_fp8 | (uintptr_t)k_out | (uintptr_t)v_out) & 15)
        return set_error(MI355_EINVAL, "gather_kv_fp8: caches and outputs must be 16-byte aligned");
    GatherFp8Params p;
    p.k_cache = (const unsigned char*)k_cache_fp8;
    p.v_cache = (const unsigned char*)v_cache_fp8;
    p.k_scale = k_scale;
    p.v_scale = v_scale;
    p.tables = block_tables;
    p.ctx_lens = context_lens;
    p.cu_k = cu_seqlens_k;
    p.k_out = (__bf16*)k_out;
    p.v_out = (__bf16*)v_out;
    p.table_stride = table_stride;
    p.out_tok = out_token_stride;
    p.max_rows = max_rows;
    p.max_blocks = (int)max_blocks;
    p.B = B;
    p.Hkv = Hkv;
    p.num_blocks = (int)num_blocks;
    const int64_t n_waves = (int64_t)B * max_blocks * Hkv, wgs = (n_waves + 3) / 4;
    if (wgs > 0x7fffffffLL) return set_error(MI355_EINVAL, "gather_kv_fp8: too many blocks for one launch");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)wgs), block(256);
    if (D == 128) hipLaunchKernelGGL(gather_kv_fp8_kernel<128>, grid, block, 0, s, p);
    else if (D == 64) hipLaunchKernelGGL(gather_kv_fp8_kernel<64>, grid, block, 0, s, p);
    else hipLaunchKernelGGL(gather_kv_fp8_kernel<32>, grid, block, 0, s, p);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}


extern "C" int mi355_rope_and_cache_fp8(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                                        void* k_cache_fp8, void* v_cache_fp8, float* k_scale, float* v_scale,
                                        const float* freq_cache, const int32_t* positions, const int64_t* slot_mapping,
                                        int64_t num_blocks, int T, int Hq, int Hkv, int D, int context_length,
                                        int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
                                        int64_t q_out_token_stride, void* k_out, int64_t k_out_token_stride,
                                        void* stream) {
    if (!q_in || !k_in || !v_in || !q_out || !freq_cache || !positions || !slot_mapping || !k_cache_fp8 || !v_cache_fp8 ||
        !k_scale || !v_scale)
        return set_error(MI355_EINVAL, "rope_and_cache_fp8: null pointer argument");
    if (num_blocks <= 0) return set_error(MI355_EINVAL, "rope_and_cache_fp8: num_blocks must be positive");
    if (T < 0 || Hq <= 0 || Hkv <= 0 || context_length <= 0)
        return set_error(MI355_EINVAL, "rope_and_cache_fp8: T, Hq, Hkv, context_length out of range");
    if (!(D == 32 || D == 64 || D == 128)) return set_error(MI355_EINVAL, "rope_and_cache_fp8: head_dim must be 32, 64 or 128");
    const auto aligned16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    if (((q_token_stride | k_token_stride | v_token_stride | q_out_token_stride) & 7) != 0 || !aligned16(q_in) ||
        !aligned16(k_in) || !aligned16(v_in) || !aligned16(q_out) || !aligned16(k_cache_fp8) || !aligned16(v_cache_fp8) ||
        !aligned16(freq_cache) || !aligned16(k_out) || (k_out && (k_out_token_stride & 7) != 0))
        return set_error(MI355_EINVAL, "rope_and_cache_fp8: tensors must be 16-byte aligned with token strides that are multiples of 8");
    if (k_out && T > 0) {
        // The packed rotated keys are written by the query workgroups while the key/value workgroups of the same
        // launch read k_in, in no order: a k_out that shares memory with k_in would hand some of them rotated rows
        // to rotate again.  (mi355_rope_and_cache reads and writes a row in one thread, so it may alias.)
        const uintptr_t in_lo = reinterpret_cast<uintptr_t>(k_in), out_lo = reinterpret_cast<uintptr_t>(k_out);
        const uintptr_t in_hi = in_lo + ((uintptr_t)(T - 1) * (uintptr_t)k_token_stride + (uintptr_t)Hkv * D) * 2;
        const uintptr_t out_hi = out_lo + ((uintptr_t)(T - 1) * (uintptr_t)k_out_token_stride + (uintptr_t)Hkv * D) * 2;
        if (in_lo < out_hi && out_lo < in_hi)
            return set_error(MI355_EINVAL, "rope_and_cache_fp8: k_out must not overlap k_in (the keys are read again after k_out is written)");
    }
    if (T == 0) return MI355_OK;
    hipStream_t s = (hipStream_t)stream;
    // queries (and, when asked for, the packed rotated keys): the body of the bf16 kernel, without a cache
    RopeCacheParams pq{};
    pq.q_in = (const __bf16*)q_in;
    pq.k_in = (const __bf16*)k_in;
    pq.v_in = (const __bf16*)v_in;
    pq.q_out = (__bf16*)q_out;
    pq.freq = freq_cache;
    pq.positions = positions;
    pq.slots = nullptr;
    pq.q_tok = q_token_stride;
    pq.k_tok = k_token_stride;
    pq.v_tok = v_token_stride;
    pq.qo_tok = q_out_token_stride;
    pq.k_out = (__bf16*)k_out;
    pq.ko_tok = k_out ? k_out_token_stride : 0;
    pq.T = T;
    pq.Hq = Hq;
    pq.Hkv = Hkv;
    pq.D = D;
    pq.ctx_len = context_length;
    pq.head_slots = k_out ? Hq + Hkv : Hq;
    pq.n_slots = 0;
    RopeCacheFp8Params p;
    p.k_in = (const __bf16*)k_in;
    p.v_in = (const __bf16*)v_in;
    p.k_cache = (unsigned char*)k_cache_fp8;
    p.v_cache = (unsigned char*)v_cache_fp8;
    p.k_scale = k_scale;
    p.v_scale = v_scale;
    p.freq = freq_cache;
    p.positions = positions;
    p.slots = slot_mapping;
    p.k_tok = k_token_stride;
    p.v_tok = v_token_stride;
    p.T = T;
    p.Hkv = Hkv;
    p.ctx_len = context_length;
    p.n_slots = num_blocks * 16;
    // a decode step (few tokens, each its own run) spreads one token per wavefront; a packed prefill
    // gives every wavefront a window of 16 tokens, which holds one run when sequences start on block boundaries
    const int win = T >= 4096 ? 16 : 1;
    const int n_windows = (T + win - 1) / win;
    const int64_t kv_blocks = ((int64_t)n_windows * 2 * Hkv + 3) / 4;
    const int n_hu = (pq.head_slots + kRopeHeads - 1) / kRopeHeads;
    const int64_t q_blocks = ((int64_t)T * n_hu * (D / 8) + 255) / 256;
    // one launch: `ratio` query workgroups, then one key/value workgroup, and so on
    int64_t ratio = (q_blocks + kv_blocks - 1) / kv_blocks;
    if (ratio < 1) ratio = 1;
    const int64_t groups = std::max(kv_blocks, (q_blocks + ratio - 1) / ratio);
    const int64_t wgs = groups * (ratio + 1);
    if (wgs > 0x7fffffff) return set_error(MI355_EINVAL, "rope_and_cache_fp8: too many tokens for one launch");
    const dim3 grid((unsigned)wgs), block(256);
    if (D == 128)
        hipLaunchKernelGGL(rope_and_cache_fp8_fused_kernel<128>, grid, block, 0, s, pq, n_hu, (unsigned)q_blocks, p, win,
                           n_windows, (unsigned)kv_blocks, (unsigned)ratio);
    else if (D == 64)
        hipLaunchKernelGGL(rope_and_cache_fp8_fused_kernel<64>, grid, block, 0, s, pq, n_hu, (unsigned)q_blocks, p, win,
                           n_windows, (unsigned)kv_blocks, (unsigned)ratio);
    else
        hipLaunchKernelGGL(rope_and_cache_fp8_fused_kernel<32>, grid, block, 0, s, pq, n_hu, (unsigned)q_blocks, p, win,
                           n_windows, (unsigned)kv_blocks, (unsigned)ratio);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}
