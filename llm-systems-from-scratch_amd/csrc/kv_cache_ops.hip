// Producers of the paged KV cache: interleaved-pair RoPE + scatter of new K/V rows into
// cache blocks, and per-(block, kv head) fp8-e4m3 quantisation of cache blocks.
// Both are plain streaming kernels (HBM-bound, a few bytes per element).
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
    int64_t q_tok, k_tok, v_tok, qo_tok;   // token strides (elements); heads are contiguous (stride D)
    int T, Hq, Hkv, D, ctx_len;
    int64_t n_slots;               // num_blocks * 16: slots outside [0, n_slots) are not written
};

// One thread per (token, head slot, pair of adjacent elements).  Head slots: Hq query heads,
// then Hkv key heads, then Hkv value heads.  Rotation of the pair (x[2i], x[2i+1]) by the angle
// of (position, i), in fp32, rounded once to bf16.
__global__ __launch_bounds__(256) void rope_and_cache_kernel(RopeCacheParams p) {
    const int half = p.D / 2;
    const int slots_per_tok = p.Hq + 2 * p.Hkv;
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
            if (slot < 0) continue;
            const int hk = hs - p.Hq;
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.k_in + t * p.k_tok + (int64_t)hk * p.D + 2 * i);
            const bf16x2 x = __builtin_bit_cast(bf16x2, raw);
            const float c = p.freq[(int64_t)pos * half + i];
            const float s = p.freq[((int64_t)p.ctx_len + pos) * half + i];
            const float x1 = (float)x[0], x2 = (float)x[1];
            const int64_t dst = (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D + 2 * i;
            *reinterpret_cast<uint32_t*>(p.k_cache + dst) = pack_bf16(c * x1 - s * x2, s * x1 + c * x2);
        } else {
            if (slot < 0) continue;
            const int hk = hs - p.Hq - p.Hkv;
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.v_in + t * p.v_tok + (int64_t)hk * p.D + 2 * i);
            const int64_t dst = (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D + 2 * i;
            *reinterpret_cast<uint32_t*>(p.v_cache + dst) = raw;
        }
    }
}

// The same work with 16-byte accesses: one thread per (token, head slot, group of 4 pairs).
// Requires D % 8 == 0, token strides that are multiples of 8 elements and 16-byte aligned bases.
__global__ __launch_bounds__(256) void rope_and_cache_vec8_kernel(RopeCacheParams p) {
    const int groups = p.D / 8;
    const int half = p.D / 2;
    const int slots_per_tok = p.Hq + 2 * p.Hkv;
    const int64_t total = (int64_t)p.T * slots_per_tok * groups;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx % groups);
        const int hs = (int)((idx / groups) % slots_per_tok);
        const int t = (int)(idx / ((int64_t)groups * slots_per_tok));
        int64_t slot = p.slots ? p.slots[t] : -1;
        if (slot >= p.n_slots) slot = -1;
        const bool is_q = hs < p.Hq;
        if (!is_q && slot < 0) continue;
        const bool is_v = hs >= p.Hq + p.Hkv;
        const int hk = is_v ? hs - p.Hq - p.Hkv : hs - p.Hq;
        const __bf16* src = is_q ? p.q_in + t * p.q_tok + (int64_t)hs * p.D
                                 : (is_v ? p.v_in + t * p.v_tok : p.k_in + t * p.k_tok) + (int64_t)hk * p.D;
        u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + 8 * c));
        if (!is_v) {
            const int pos = min(max(p.positions[t], 0), p.ctx_len - 1);
            const f32x4 cs = *reinterpret_cast<const f32x4*>(p.freq + (int64_t)pos * half + 4 * c);
            const f32x4 sn = *reinterpret_cast<const f32x4*>(p.freq + ((int64_t)p.ctx_len + pos) * half + 4 * c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = raw[j];           // scalar copy first: a bit_cast of a vector element misreads it
                const bf16x2 x = __builtin_bit_cast(bf16x2, w);
                const float x1 = (float)x[0], x2 = (float)x[1];
                raw[j] = pack_bf16(cs[j] * x1 - sn[j] * x2, sn[j] * x1 + cs[j] * x2);
            }
        }
        __bf16* dst = is_q ? p.q_out + t * p.qo_tok + (int64_t)hs * p.D
                           : (is_v ? p.v_cache : p.k_cache) + (((slot >> 4) * p.Hkv + hk) * 16 + (slot & 15)) * p.D;
        *reinterpret_cast<u32x4*>(dst + 8 * c) = raw;
    }
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
            *reinterpret_cast<u32x2*>(d + 512 * j) = out;
        }
    }
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_rope_and_cache(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_cache,
                                    void* v_cache, const float* freq_cache, const int32_t* positions,
                                    const int64_t* slot_mapping, int64_t num_blocks, int T, int Hq, int Hkv, int D,
                                    int context_length,
                                    int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
                                    int64_t q_out_token_stride, void* stream) {
    if (!q_in || !k_in || !v_in || !q_out || !freq_cache || !positions)
        return set_error(MI355_EINVAL, "rope_and_cache: null pointer argument");
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
    p.T = T;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.D = D;
    p.ctx_len = context_length;
    p.n_slots = slot_mapping ? num_blocks * 16 : 0;
    const auto aligned16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    const bool vec8 = D % 8 == 0 && ((q_token_stride | k_token_stride | v_token_stride | q_out_token_stride) & 7) == 0 &&
                      aligned16(q_in) && aligned16(k_in) && aligned16(v_in) && aligned16(q_out) && aligned16(k_cache) &&
                      aligned16(v_cache) && aligned16(freq_cache);
    const int64_t total = (int64_t)T * (Hq + 2 * Hkv) * (vec8 ? D / 8 : D / 2);
    const int64_t blocks = (total + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 256 * 64 ? blocks : 256 * 64);
    if (vec8)
        hipLaunchKernelGGL(rope_and_cache_vec8_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, p);
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
    const unsigned grid = (unsigned)(wgs < 256 * 64 ? wgs : 256 * 64);
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
