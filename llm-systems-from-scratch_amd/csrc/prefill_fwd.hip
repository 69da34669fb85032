// FlashAttention-style prefill forward for gfx950 (bf16, MFMA 32x32x16).
//
// One workgroup = 4 wavefronts = one tile of 128 queries of one (batch, head);
// each wavefront owns 32 query rows.  K/V tiles of 64 keys are staged in LDS and
// shared by the four wavefronts.  Per wavefront and KV tile:
//
//   S^T (64 keys x 32 queries) = K . Q^T     K fragments: ds_read_b128 from LDS,
//                                            Q^T fragments live in registers
//   online softmax                           a lane owns ONE query column and 32
//                                            keys: row max/sum are in-lane plus
//                                            one exchange with lane^32
//   O^T (D x 32 queries)      += V^T . P^T   P^T is the S^T accumulator itself
//                                            (converted to bf16, no LDS trip);
//                                            V^T fragments: ds_read_b64_tr_b16
//
// Working on the transposed problem is what makes the S accumulator layout equal
// to the B-operand layout of the second MFMA (up to a key permutation that the
// V^T read mirrors).
#include "common.hpp"
#include "launch.hpp"

namespace mi355 {

constexpr int kPfWaves = 4;
constexpr int kBM = 128;   // queries per workgroup
constexpr int kBN = 64;    // keys per LDS tile

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
    int B, Hq, Hkv, Sq, Sk;
    float scale_log2;
    int mask_mode;
    int n_qtiles;
};

template <int D>
struct PrefillLds {
    static constexpr int kKRow = D * 2 + 16;      // bytes per K row: 16-lane b128 reads hit 16 distinct 16B bank groups
    static constexpr int kVRow = D * 2 + 64;      // bytes per V row: 4 rows x 64B of a transposed read cover all banks
    static constexpr int kKBytes = kBN * kKRow;
    static constexpr int kVBytes = kBN * kVRow;
};

template <int D>
__global__ __launch_bounds__(kPfWaves * 64, 2) void prefill_fwd_kernel(PrefillParams p) {
    constexpr int NS = D / 16;              // MFMA k-steps of K.Q^T
    constexpr int NDT = D / 32;             // 32-row tiles of O^T
    constexpr int kKRow = PrefillLds<D>::kKRow;
    constexpr int kVRow = PrefillLds<D>::kVRow;
    constexpr int CPR = D / 8;              // 16-byte chunks per row
    constexpr int NLD = kBN * CPR / (kPfWaves * 64);   // 16-byte staging loads per thread per tile

    __shared__ __attribute__((aligned(16))) unsigned char k_lds[PrefillLds<D>::kKBytes];
    __shared__ __attribute__((aligned(16))) unsigned char v_lds[PrefillLds<D>::kVBytes];

    // heavy (late) query tiles first: causal work grows with the tile index
    const int qtile = p.n_qtiles - 1 - (int)blockIdx.x;
    const int h = blockIdx.y;
    const int b = blockIdx.z;
    const int hk = h / (p.Hq / p.Hkv);

    int sq, sk;
    const __bf16 *qb, *kb, *vb;
    __bf16* ob;
    if (p.cu_q) {
        const int q_start = p.cu_q[b], k_start = p.cu_k[b];
        sq = p.cu_q[b + 1] - q_start;
        sk = p.cu_k[b + 1] - k_start;
        qb = p.q + (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
        kb = p.k + (int64_t)k_start * p.ks[2] + (int64_t)hk * p.ks[1];
        vb = p.v + (int64_t)k_start * p.vs[2] + (int64_t)hk * p.vs[1];
        ob = p.out + (int64_t)q_start * p.os[2] + (int64_t)h * p.os[1];
    } else {
        sq = p.Sq;
        sk = p.Sk;
        qb = p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[1];
        kb = p.k + (int64_t)b * p.ks[0] + (int64_t)hk * p.ks[1];
        vb = p.v + (int64_t)b * p.vs[0] + (int64_t)hk * p.vs[1];
        ob = p.out + (int64_t)b * p.os[0] + (int64_t)h * p.os[1];
    }
    const int q0 = qtile * kBM;
    if (q0 >= sq) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;          // query column of S^T / O^T, key row of K, d row of V^T
    const int kg = lane >> 5;         // 0..1

    const bool causal = p.mask_mode == MI355_MASK_CAUSAL;
    const bool boolmask = p.mask_mode == MI355_MASK_BOOL;
    const int coff = sk - sq;                          // bottom-right aligned causal diagonal
    const int qw0 = q0 + 32 * wave;                    // first query of this wavefront
    const int qi = qw0 + n;                            // this lane's query
    const bool q_ok = qi < sq;

    int kv_end = sk;
    if (causal) kv_end = max(0, min(sk, min(sq, q0 + kBM) + coff));
    const int n_tiles = (kv_end + kBN - 1) / kBN;

    // ---- Q^T fragments: step s covers d = 16s + 8kg + j ----------------------
    bf16x8 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        u32x4 t = {0u, 0u, 0u, 0u};
        if (q_ok) t = *reinterpret_cast<const u32x4*>(qb + (int64_t)qi * p.qs[2] + 16 * s + 8 * kg);
        qf[s] = as_bf16x8(t);
    }

    f32x16 o[NDT];
#pragma unroll
    for (int i = 0; i < NDT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) o[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const uint8_t* mrow = nullptr;
    if (boolmask) mrow = p.mask + (int64_t)b * p.ms[0] + (int64_t)h * p.ms[1] + (int64_t)qi * p.ms[2];

    // ---- staging registers ---------------------------------------------------
    u32x4 kst[NLD], vst[NLD];
    auto fetch = [&](int tile) {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int c = tid + j * (kPfWaves * 64);
            const int row = c / CPR, cc = c % CPR;
            const int key = tile * kBN + row;
            u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
            if (key < sk) {
                kk = *reinterpret_cast<const u32x4*>(kb + (int64_t)key * p.ks[2] + cc * 8);
                vv = *reinterpret_cast<const u32x4*>(vb + (int64_t)key * p.vs[2] + cc * 8);
            }
            kst[j] = kk;
            vst[j] = vv;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int c = tid + j * (kPfWaves * 64);
            const int row = c / CPR, cc = c % CPR;
            *reinterpret_cast<u32x4*>(k_lds + row * kKRow + cc * 16) = kst[j];
            *reinterpret_cast<u32x4*>(v_lds + row * kVRow + cc * 16) = vst[j];
        }
    };

    if (n_tiles > 0) fetch(0);

    for (int tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();                 // everyone is done reading the previous tile
        stash();
        __syncthreads();
        if (tile + 1 < n_tiles) fetch(tile + 1);

        const int k0 = tile * kBN;
        // wavefront-level skip: every key of the tile is above this wavefront's diagonal
        if (causal && k0 > qw0 + 31 + coff) continue;

        // ---- S^T = K . Q^T -----------------------------------------------------
        f32x16 s_acc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int j = 0; j < 16; ++j) s_acc[t][j] = 0.f;
            const unsigned char* kp = k_lds + (32 * t + n) * kKRow + kg * 16;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const u32x4 kf = *reinterpret_cast<const u32x4*>(kp + s * 32);
                s_acc[t] = mfma32(as_bf16x8(kf), qf[s], s_acc[t]);
            }
        }

        // ---- scale, mask, online softmax ----------------------------------------
        // element (t,i) of this lane: key k0 + 32t + 8(i/4) + 4kg + i%4, query qi
        const bool need_mask = (causal && k0 + kBN - 1 > qw0 + coff) || (k0 + kBN > sk) || boolmask;
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float x = s_acc[t][i] * p.scale_log2;
                if (need_mask) {
                    const int key = k0 + 32 * t + 8 * (i >> 2) + 4 * kg + (i & 3);
                    bool keep = key < sk;
                    if (causal) keep = keep && (key <= qi + coff);
                    if (boolmask) keep = keep && q_ok && (mrow[key < sk ? key : 0] != 0);
                    if (!keep) x = -INFINITY;
                }
                s_acc[t][i] = x;
                mx = fmaxf(mx, x);
            }
        }
        mx = xor32_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;    // row with no key yet: keep p = 0, not NaN
        const float alpha = fast_exp2(m_run - m_use);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = fast_exp2(s_acc[t][i] - m_use);
                s_acc[t][i] = e;
                psum += e;
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;

        // ---- O^T += V^T . P^T ------------------------------------------------------
        // 16-key slice u: P^T fragment = accumulator registers 8(u%2).. of tile u/2, i.e.
        // keys 16u + 4kg + (0..3) and 16u + 8 + 4kg + (0..3); the V^T read mirrors it.
        const int g16 = lane >> 4, s16 = lane & 15;
        const unsigned char* vp = v_lds + (4 * (g16 >> 1) + (s16 >> 2)) * kVRow + (16 * (g16 & 1) + 4 * (s16 & 3)) * 2;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = u >> 1, e0 = 8 * (u & 1);
            u32x4 pw;
            pw[0] = pack_bf16(s_acc[t][e0 + 0], s_acc[t][e0 + 1]);
            pw[1] = pack_bf16(s_acc[t][e0 + 2], s_acc[t][e0 + 3]);
            pw[2] = pack_bf16(s_acc[t][e0 + 4], s_acc[t][e0 + 5]);
            pw[3] = pack_bf16(s_acc[t][e0 + 6], s_acc[t][e0 + 7]);
            const bf16x8 pf = as_bf16x8(pw);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const unsigned char* a = vp + (16 * u) * kVRow + dt * 64;
                const i16x4 lo = lds_read_tr16(a);
                const i16x4 hi = lds_read_tr16(a + 8 * kVRow);
                o[dt] = mfma32(join_bf16x8(lo, hi), pf, o[dt]);
            }
        }
    }

    // ---- normalise and store: lane owns query qi, d = 32dt + 8(i/4) + 4kg + i%4 ---
    l_run = xor32_sum(l_run);
    const float inv = 1.0f / l_run;          // l == 0 (no key kept) -> NaN row, like the reference softmax
    if (q_ok) {
        __bf16* orow = ob + (int64_t)qi * p.os[2];
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w[0] = pack_bf16(o[dt][4 * g + 0] * inv, o[dt][4 * g + 1] * inv);
                w[1] = pack_bf16(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
                *reinterpret_cast<u32x2*>(orow + 32 * dt + 8 * g + 4 * kg) = w;
            }
    }
}

template <int D>
static int launch_prefill(const PrefillParams& p, hipStream_t stream) {
    dim3 grid(p.n_qtiles, p.Hq, p.B);
    hipLaunchKernelGGL((prefill_fwd_kernel<D>), grid, dim3(kPfWaves * 64), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_prefill_fwd(const void* q, const void* k, const void* v, void* out,
                                 const int64_t q_strides[3], const int64_t k_strides[3],
                                 const int64_t v_strides[3], const int64_t o_strides[3],
                                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                 const uint8_t* mask, const int64_t mask_strides[3], int B, int Hq, int Hkv,
                                 int Sq_max, int Sk_max, int D, float softmax_scale, int mask_mode, int dtype,
                                 void* stream) {
    if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !o_strides)
        return set_error(MI355_EINVAL, "prefill: null pointer argument");
    if (dtype != MI355_BF16) return set_error(MI355_EDTYPE, "prefill: dtype must be MI355_BF16");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq_max <= 0 || Sk_max <= 0)
        return set_error(MI355_EINVAL, "prefill: B, Hq, Hkv, Sq_max and Sk_max must be positive");
    if (Hq % Hkv != 0) return set_error(MI355_EINVAL, "prefill: Hq must be a multiple of Hkv");
    if (!(D == 128 || D == 64 || D == 32)) return set_error(MI355_EINVAL, "prefill: head_dim must be 32, 64 or 128");
    if (Hq > 65535 || B > 65535) return set_error(MI355_EINVAL, "prefill: Hq and B must be <= 65535");
    if ((cu_seqlens_q == nullptr) != (cu_seqlens_k == nullptr))
        return set_error(MI355_EINVAL, "prefill: cu_seqlens_q and cu_seqlens_k must be given together");
    if (mask_mode < MI355_MASK_NONE || mask_mode > MI355_MASK_BOOL)
        return set_error(MI355_EINVAL, "prefill: unknown mask_mode");
    if (mask_mode == MI355_MASK_BOOL && (!mask || !mask_strides || cu_seqlens_q))
        return set_error(MI355_EINVAL, "prefill: MI355_MASK_BOOL needs mask + mask_strides and the dense layout");
    for (int i = 0; i < 3; ++i) {
        if ((q_strides[i] | k_strides[i] | v_strides[i] | o_strides[i]) & 7)
            return set_error(MI355_EINVAL, "prefill: strides must be multiples of 8 elements (16-byte rows)");
    }
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15)
        return set_error(MI355_EINVAL, "prefill: q, k, v and out must be 16-byte aligned");

    PrefillParams p;
    p.q = (const __bf16*)q;
    p.k = (const __bf16*)k;
    p.v = (const __bf16*)v;
    p.out = (__bf16*)out;
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = q_strides[i];
        p.ks[i] = k_strides[i];
        p.vs[i] = v_strides[i];
        p.os[i] = o_strides[i];
        p.ms[i] = mask_strides ? mask_strides[i] : 0;
    }
    p.cu_q = cu_seqlens_q;
    p.cu_k = cu_seqlens_k;
    p.mask = mask;
    p.B = B;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.Sq = Sq_max;
    p.Sk = Sk_max;
    p.scale_log2 = softmax_scale * kLog2e;
    p.mask_mode = mask_mode;
    p.n_qtiles = (Sq_max + kBM - 1) / kBM;

    hipStream_t s = (hipStream_t)stream;
    int rc = D == 128 ? launch_prefill<128>(p, s) : (D == 64 ? launch_prefill<64>(p, s) : launch_prefill<32>(p, s));
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}
