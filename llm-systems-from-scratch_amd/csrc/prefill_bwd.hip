// FlashAttention-style prefill backward for gfx950 (bf16, MFMA 32x32x16): dQ, dK, dV from
// q, k, v, out, dout and the forward's log-sum-exp.  No atomics; results are deterministic.
//
//   delta_i = sum_d dO[i,d] * O[i,d]                       (computed, and stored, by the dQ kernel)
//   P_ij    = exp(scale * q_i.k_j - lse_i)                 (recomputed, never stored)
//   dV_j    = sum_i P_ij dO_i                              (bwd_dkv_kernel: one workgroup per key tile,
//   dP_ij   = dO_i . v_j                                    summing over the query heads of a GQA group;
//   dS_ij   = P_ij (dP_ij - delta_i)                        dV on half of its wavefronts, dK on the other half)
//   dK_j    = scale * sum_i dS_ij q_i
//   dQ_i    = scale * sum_j dS_ij k_j                      (bwd_dq_kernel: one workgroup per query tile)
//
// Both kernels work on transposed problems, like the forward: the wavefront owns 32 columns
// (queries in the dQ kernel, keys in the dK/dV kernel) whose operand fragments stay in
// registers; the other side streams through LDS tiles of 64 rows.  The accumulator of the first
// MFMA (S or dP, column = lane) is, converted to bf16, directly the B operand of the second
// (dQ^T += K^T dS^T; dV^T += dO^T P, dK^T += Q^T dS), and the matching A operand is a transposed
// LDS read (ds_read_b64_tr_b16) of the streamed tile with the same row permutation.
// 7 GEMM-sized products are executed (S and dP in both kernels) where 5 are needed.
//
// Masks: none, causal (bottom-right aligned, as in the forward), or an explicit boolean keep-mask (the mask argument
// of llm-core/llm_core/model.py:308-325, which its non-flash branch passes at model.py:384-385).  The explicit mask is
// the general, slower path: every tile takes the per-element select and reads its mask bytes from global memory.
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"
#include "prefill_tile.hpp"

namespace mi355 {

constexpr int kBwWaves = 8;
constexpr int kBwCols = 32 * kBwWaves;   // query columns per workgroup of the dQ kernel (one workgroup of 8 wavefronts per CU)
constexpr int kBwRows = 64;              // rows of a streamed LDS tile

struct BwdParams {
    const __bf16* q;
    const __bf16* k;
    const __bf16* v;
    const __bf16* out;
    const __bf16* dout;
    const float* lse;
    float* delta;
    __bf16* dq;
    __bf16* dk;
    __bf16* dv;
    int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3];   // batch, head, row strides (elements)
    int64_t ls[2];                                                          // lse / delta: batch, head strides
    const int32_t* cu_q;
    const int32_t* cu_k;
    const uint8_t* mask;          // MI355_MASK_BOOL: (B, Hq, Sq, Sk) bytes, non-zero = keep; rows 4-byte aligned
    int64_t ms[3];                // batch, head, row strides of the mask in bytes (0 = broadcast), multiples of 4
    int B, Hq, Hkv, Sq, Sk;
    float scale, scale_log2;
    int n_qtiles, n_ktiles;
};

// Loader of a 64-row tile (rows of D bf16, row stride `stride` elements) into swizzled LDS:
// wavefront w, instruction j covers LDS chunks (w*NI + j)*64 .. +63; rows past `last` re-read row `last`.
template <int D, int NW>
struct TileLoader {
    static constexpr int CPR = D / 8;
    static constexpr int TOTAL = kBwRows * CPR / 64;            // 1 KiB instructions per tile
    static constexpr int NI = (TOTAL + NW - 1) / NW;            // per wavefront (the last wavefronts may have none)
    int row[NI], col[NI];
    bool active;
    __device__ __forceinline__ void init(int wave, int lane) {
        active = wave * NI < TOTAL;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int idx = (wave * NI + j) * 64 + lane;
            row[j] = idx / CPR;
            col[j] = ((idx % CPR) ^ swz<D>(idx / CPR)) * 16;
        }
    }
    __device__ __forceinline__ void issue(const __bf16* first_row, int stride, int last, uint32_t lds_wave_base) const {
        if (!active) return;
#pragma unroll
        for (int j = 0; j < NI; ++j)
            dma_to_lds_16(first_row, (uint32_t)(min(row[j], last) * stride * 2 + col[j]), lds_wave_base + j * 1024);
    }
};

// Per-lane LDS offsets of the two read patterns of a swizzled 64 x D tile.
template <int D>
struct TileReads {
    static constexpr int NS = D / 16, NDT = D / 32, kRow = D * 2;
    int row_off[NS];        // A fragment "row n of the tile, k = 16s + 8kg ..": add 32*t*kRow
    int tr_off[2][NDT];     // transposed fragment of d-tile dt for a 16-row slice: add 16*u*kRow
    __device__ __forceinline__ void init(int lane) {
        const int n = lane & 31, kg = lane >> 5;
#pragma unroll
        for (int s = 0; s < NS; ++s) row_off[s] = n * kRow + (((2 * s + kg) ^ swz<D>(n)) << 4);
        const int g16 = lane >> 4, s16 = lane & 15;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int row = 4 * (g16 >> 1) + (s16 >> 2) + 8 * e;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const int d = 32 * dt + 16 * (g16 & 1) + 4 * (s16 & 3);
                tr_off[e][dt] = row * kRow + (((d >> 3) ^ swz<D>(row)) << 4) + (d & 7) * 2;
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// dQ: one workgroup per tile of 128 queries of one (batch, query head); K/V stream through LDS.
// Per wavefront: Q and dO fragments of its 32 query columns in registers (64), dQ^T accumulators (64).
template <int D, int MODE>
__global__ __launch_bounds__(kBwWaves * 64, 1) void bwd_dq_kernel(BwdParams p) {
    constexpr bool CAUSAL = MODE == MI355_MASK_CAUSAL, BOOLM = MODE == MI355_MASK_BOOL;
    constexpr int NWV = kBwWaves;
    using R = TileReads<D>;
    constexpr int NS = R::NS, NDT = R::NDT, kRow = R::kRow, kTile = kBwRows * kRow;
    // [K buffer 0][K buffer 1][V buffer 0][V buffer 1]
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * kTile];

    // Workgroup ids are dealt round-robin to the 8 XCDs (private L2s) and, in order, to their shader
    // engines: workgroups must carry EQUAL work (a periodic heavy/light pattern starves the engines that
    // always draw the light ones), and the workgroups that stream the same K/V should share an XCD.  So a
    // workgroup takes the query-tile PAIR (nq-1-i, i), and the pairs and query heads of one kv head -- a chunk
    // of the logical order (pair, query head, batch) -- run on one XCD.
    const int n_pairs = (p.n_qtiles + 1) / 2;
    const int lid = xcd_chunked_id(blockIdx.x, gridDim.x, n_pairs * (p.Hq / p.Hkv));
    const int pair = lid % n_pairs;
    const int h = (lid / n_pairs) % p.Hq;
    const int b = lid / (n_pairs * p.Hq);
    const int hk = h / (p.Hq / p.Hkv);
    int sq, sk;
    int64_t q_base, k_base, v_base, do_base, dq_base, l_base, o_base;
    if (p.cu_q) {
        const int q_start = p.cu_q[b], k_start = p.cu_k[b];
        sq = p.cu_q[b + 1] - q_start;
        sk = p.cu_k[b + 1] - k_start;
        o_base = (int64_t)q_start * p.os[2] + (int64_t)h * p.os[1];
        q_base = (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
        do_base = (int64_t)q_start * p.dos[2] + (int64_t)h * p.dos[1];
        dq_base = (int64_t)q_start * p.dqs[2] + (int64_t)h * p.dqs[1];
        k_base = (int64_t)k_start * p.ks[2] + (int64_t)hk * p.ks[1];
        v_base = (int64_t)k_start * p.vs[2] + (int64_t)hk * p.vs[1];
        l_base = q_start + (int64_t)h * p.ls[1];
    } else {
        sq = p.Sq;
        sk = p.Sk;
        o_base = (int64_t)b * p.os[0] + (int64_t)h * p.os[1];
        q_base = (int64_t)b * p.qs[0] + (int64_t)h * p.qs[1];
        do_base = (int64_t)b * p.dos[0] + (int64_t)h * p.dos[1];
        dq_base = (int64_t)b * p.dqs[0] + (int64_t)h * p.dqs[1];
        k_base = (int64_t)b * p.ks[0] + (int64_t)hk * p.ks[1];
        v_base = (int64_t)b * p.vs[0] + (int64_t)hk * p.vs[1];
        l_base = (int64_t)b * p.ls[0] + (int64_t)h * p.ls[1];
    }
    const int nq = (sq + kBwCols - 1) / kBwCols;
    if (2 * pair >= nq) return;                                         // (a sequence without keys still gets dq = 0 written)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, kg = lane >> 5;
    const int coff = sk - sq;

    TileLoader<D, NWV> ld;
    ld.init(wave, lane);
    R rd;
    rd.init(lane);
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds) + wave * TileLoader<D, NWV>::NI * 1024);

    for (int half = 0; half < 2; ++half) {
        const int qtile = half == 0 ? nq - 1 - pair : pair;
        if (half == 1 && qtile == nq - 1 - pair) break;                 // odd tile count: the middle tile has no partner
        const int q0 = qtile * kBwCols;
        const int qw0 = q0 + 32 * wave;
        const int qi = qw0 + n;
        const bool q_ok = qi < sq;
        __syncthreads();                                                // the previous half's readers are done with the LDS buffers

        // fragments of this lane's query column: step s covers d = 16s + 8kg + j
        bf16x8 qf[NS], dof[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            u32x4 a = {0u, 0u, 0u, 0u}, g = {0u, 0u, 0u, 0u};
            if (q_ok) {
                a = *reinterpret_cast<const u32x4*>(p.q + q_base + (int64_t)qi * p.qs[2] + 16 * s + 8 * kg);
                g = *reinterpret_cast<const u32x4*>(p.dout + do_base + (int64_t)qi * p.dos[2] + 16 * s + 8 * kg);
            }
            qf[s] = as_bf16x8(a);
            dof[s] = as_bf16x8(g);
        }
        // a padded query column gets lse = +inf, i.e. P = 0 everywhere
        const float lse2 = q_ok ? p.lse[l_base + qi] * kLog2e : INFINITY;
        // delta = rowsum(dO * O) of this lane's query: each lane of the pair (kg = 0, 1) covers half of d.
        // It is also written out: the dK kernel, launched after this one, reads it per row.
        float delta = 0.f;
        if (q_ok) {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const bf16x8 o8 = as_bf16x8(*reinterpret_cast<const u32x4*>(p.out + o_base + (int64_t)qi * p.os[2] + 16 * s + 8 * kg));
#pragma unroll
                for (int e = 0; e < 8; ++e) delta += (float)o8[e] * (float)dof[s][e];
            }
        }
        delta = xor32_sum(delta);
        if (q_ok && kg == 0) p.delta[l_base + qi] = delta;

        f32x16 dq[NDT];
#pragma unroll
        for (int i = 0; i < NDT; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) dq[i][j] = 0.f;
        const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // dP - delta comes straight out of the MFMAs: -delta (one value per lane: its query) is their C operand
        f32x16 neg_delta16;
#pragma unroll
        for (int j = 0; j < 16; ++j) neg_delta16[j] = -delta;

        int kv_end = sk;
        if (CAUSAL) kv_end = max(0, min(sk, min(sq, q0 + kBwCols) + coff));
        const int n_tiles = (kv_end + kBwRows - 1) / kBwRows;
        const int last_key = CAUSAL ? min(sk - 1, qi + coff) : sk - 1;      // last key this lane's query sees
        const int wave_last_key = CAUSAL ? min(sk - 1, qw0 + coff) : sk - 1;   // ... and the last one ALL queries of the wavefront see
        // explicit mask: the row of this lane's query (a padded lane re-reads the last row; its lse keeps P at 0);
        // four keys at a time as one 32-bit word (rows are 4-byte aligned; a word past the last key is the last word)
        const uint8_t* mrow = nullptr;
        if constexpr (BOOLM) mrow = p.mask + (int64_t)b * p.ms[0] + (int64_t)h * p.ms[1] + (int64_t)min(qi, sq - 1) * p.ms[2];
        const int last_word = (sk - 1) & ~3;
        const auto issue = [&](int tile) {
            const int r0 = tile * kBwRows, buf = (tile & 1) * kTile;
            ld.issue(p.k + k_base + (int64_t)r0 * p.ks[2], (int)p.ks[2], sk - 1 - r0, dst + buf);
            ld.issue(p.v + v_base + (int64_t)r0 * p.vs[2], (int)p.vs[2], sk - 1 - r0, dst + 2 * kTile + buf);
        };
        // The LDS fragments of every MFMA are read kDepth MFMAs ahead, in program order, fenced by scheduling
        // barriers: left alone the compiler puts each read, and a full wait, directly in front of its MFMA,
        // and the wavefront then sits through the LDS latency once per MFMA.
        constexpr int kDepth = 2;
        // (32 rows of the tile at a_lds) x (this lane's query column, fragments b)
        const auto scores = [&](const unsigned char* a_lds, const bf16x8 (&bfr)[NS], const f32x16& c0) {
            u32x4 a[NS];
#pragma unroll
            for (int s = 0; s < kDepth && s < NS; ++s) a[s] = *reinterpret_cast<const u32x4*>(a_lds + rd.row_off[s]);
            f32x16 r = c0;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                if (s + kDepth < NS) a[s + kDepth] = *reinterpret_cast<const u32x4*>(a_lds + rd.row_off[s + kDepth]);
                r = mfma32(as_bf16x8(a[s]), bfr[s], r);
                __builtin_amdgcn_sched_barrier(0);
            }
            return r;
        };
        const auto step = [&](auto masked_c, int tile) {
            constexpr bool MASKED = decltype(masked_c)::value;
            const int k0 = tile * kBwRows;
            const unsigned char* k_lds = lds + (tile & 1) * kTile;
            const unsigned char* v_lds = k_lds + 2 * kTile;
            const int key_lim = last_key - k0 - 4 * kg;      // element (t,i) is kept iff its tile-relative key index <= key_lim
            u32x4 ds[4];
            uint32_t mw[8] = {};
            if constexpr (BOOLM && MASKED) {
#pragma unroll
                for (int g = 0; g < 8; ++g)      // keys k0 + 32(g/4) + 8(g%4) + 4kg .. + 3
                    mw[g] = *reinterpret_cast<const uint32_t*>(mrow + min(k0 + 32 * (g >> 2) + 8 * (g & 3) + 4 * kg, last_word));
            }
            // one 32-key half at a time: element i of this lane is key k0 + 32t + 8(i/4) + 4kg + i%4, query qi
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const f32x16 s_acc = scores(k_lds + t * 32 * kRow, qf, zero16);
                const f32x16 dp_acc = scores(v_lds + t * 32 * kRow, dof, neg_delta16);             // dP - delta
                float x[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float pr = fast_exp2(fmaf(s_acc[i], p.scale_log2, -lse2));
                    x[i] = pr * dp_acc[i];                                             // dS (without the scale factor)
                    if constexpr (MASKED) {
                        // key index relative to the tile (compile-time part) against this lane's last visible key
                        bool keep = 32 * t + 8 * (i >> 2) + (i & 3) <= key_lim;
                        if constexpr (BOOLM) keep = keep & (((mw[4 * t + (i >> 2)] >> (8 * (i & 3))) & 0xffu) != 0u);
                        x[i] = keep ? x[i] : 0.f;
                    }
                }
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    ds[2 * t][w] = pack_bf16(x[2 * w], x[2 * w + 1]);
                    ds[2 * t + 1][w] = pack_bf16(x[8 + 2 * w], x[8 + 2 * w + 1]);
                }
            }
            // dQ^T (D x 32 queries) += K^T . dS^T, 16 keys at a time
            constexpr int NC = 4 * NDT;
            i16x4 lo[NC], hi[NC];
            const auto read = [&](int c) {
                const int u = c / NDT, dt = c % NDT;
                lo[c] = lds_read_tr16(k_lds + 16 * u * kRow + rd.tr_off[0][dt]);
                hi[c] = lds_read_tr16(k_lds + 16 * u * kRow + rd.tr_off[1][dt]);
            };
#pragma unroll
            for (int c = 0; c < kDepth && c < NC; ++c) read(c);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (c + kDepth < NC) read(c + kDepth);
                dq[c % NDT] = mfma32(join_bf16x8(lo[c], hi[c]), as_bf16x8(ds[c / NDT]), dq[c % NDT]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        // Two loops over the tile stream: first the tiles that every query of the wavefront sees in full, then
        // those that reach past wave_last_key (the diagonal, a ragged end), which run the instantiation with the
        // per-element compare/select.  (Two loops, not a branch in one: each loop body is scheduled on its own.)
        const int n_full = BOOLM ? 0 : min(n_tiles, max(0, wave_last_key + 1) / kBwRows);
        if (n_tiles > 0) issue(0);
        for (int tile = 0; tile < n_full; ++tile) {
            wait_vmcnt<0>();                                   // this wavefront's share of tile `tile` has landed
            __syncthreads();                                   // ... and everybody's; all are done reading the other buffer
            if (tile + 1 < n_tiles) issue(tile + 1);
            step(std::false_type{}, tile);
        }
        for (int tile = n_full; tile < n_tiles; ++tile) {
            wait_vmcnt<0>();
            __syncthreads();
            if (tile + 1 < n_tiles) issue(tile + 1);
            if (CAUSAL && tile * kBwRows > qw0 + 31 + coff) continue;      // wholly above this wavefront's diagonal (uniform)
            step(std::true_type{}, tile);
        }

        // store: lane owns query qi, d = 32dt + 8(i/4) + 4kg + i%4
        if (q_ok) {
            __bf16* row = p.dq + dq_base + (int64_t)qi * p.dqs[2];
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = pack_bf16(dq[dt][4 * g + 0] * p.scale, dq[dt][4 * g + 1] * p.scale);
                    w[1] = pack_bf16(dq[dt][4 * g + 2] * p.scale, dq[dt][4 * g + 3] * p.scale);
                    *reinterpret_cast<u32x2*>(row + 32 * dt + 8 * g + 4 * kg) = w;
                }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dK and dV in one kernel, the two roles on different wavefronts: a workgroup owns 128 keys of one
// (batch, kv head); wavefronts 0-3 (role A) hold the K fragments of 32 keys each and the dV
// accumulators, wavefronts 4-7 (role B) hold the V fragments of the same keys and the dK accumulators
// (each role fits 256 registers, so two wavefronts share a SIMD - an A and a B wavefront).  Per step
// (64 query rows of one query head):
//   A:  S = Q K^T,  P = exp2(S c - lse)  -> LDS (fp32, for B) and registers (bf16),  dV^T += dO^T P
//   B:  dP = dO V^T,  dS = P (dP - delta)  with A's P from LDS,                        dK^T += Q^T dS
// so S is computed once for both gradients (4 GEMM-sized products per step instead of 2 + 3 in two
// kernels).  A runs one step ahead of B with its P: at iteration i, A produces P(i+1) while B consumes
// P(i), and the only synchronisation is the one workgroup barrier per iteration that the tile stream
// needs anyway.  Q tiles therefore live for three iterations (landing, read by A, read by B): a ring
// of three; dO tiles, read by both roles in the same iteration, alternate between two buffers.
constexpr int kFuPairs = 4;
constexpr int kFuCols = 32 * kFuPairs;

template <int D, int MODE>
__global__ __launch_bounds__(2 * kFuPairs * 64, 1) void bwd_dkv_kernel(BwdParams p) {
    constexpr bool CAUSAL = MODE == MI355_MASK_CAUSAL, BOOLM = MODE == MI355_MASK_BOOL;
    constexpr int NWV = 2 * kFuPairs;
    using R = TileReads<D>;
    constexpr int NS = R::NS, NDT = R::NDT, kRow = R::kRow, kTile = kBwRows * kRow;
    constexpr int kPSlab = 64 * 32 * 4;                              // one wavefront's P of one step, fp32
    // [Q ring 0..2][dO buffer 0..1][P: 2 x kFuPairs slabs]
    __shared__ __attribute__((aligned(1024))) unsigned char lds[5 * kTile + 2 * kFuPairs * kPSlab];
    __shared__ __attribute__((aligned(16))) float lse_lds2[2 * kBwRows];
    __shared__ __attribute__((aligned(16))) float delta_lds2[2 * kBwRows];

    // (the key-tile pairs of one (batch, kv head), which stream the same Q and dO tiles, run on one XCD)
    const int n_pairs = (p.n_ktiles + 1) / 2;
    const int lid = xcd_chunked_id(blockIdx.x, gridDim.x, n_pairs);
    const int pair = lid % n_pairs;
    const int hk = (lid / n_pairs) % p.Hkv;
    const int b = lid / (n_pairs * p.Hkv);
    const int G = p.Hq / p.Hkv;
    int sq, sk, q_start = 0;
    int64_t k_base, v_base, dk_base, dv_base;
    if (p.cu_q) {
        q_start = p.cu_q[b];
        const int k_start = p.cu_k[b];
        sq = p.cu_q[b + 1] - q_start;
        sk = p.cu_k[b + 1] - k_start;
        k_base = (int64_t)k_start * p.ks[2] + (int64_t)hk * p.ks[1];
        v_base = (int64_t)k_start * p.vs[2] + (int64_t)hk * p.vs[1];
        dk_base = (int64_t)k_start * p.dks[2] + (int64_t)hk * p.dks[1];
        dv_base = (int64_t)k_start * p.dvs[2] + (int64_t)hk * p.dvs[1];
    } else {
        sq = p.Sq;
        sk = p.Sk;
        k_base = (int64_t)b * p.ks[0] + (int64_t)hk * p.ks[1];
        v_base = (int64_t)b * p.vs[0] + (int64_t)hk * p.vs[1];
        dk_base = (int64_t)b * p.dks[0] + (int64_t)hk * p.dks[1];
        dv_base = (int64_t)b * p.dvs[0] + (int64_t)hk * p.dvs[1];
    }
    const int nk = (sk + kFuCols - 1) / kFuCols;
    if (2 * pair >= nk) return;                                         // (a sequence without queries still gets dk = dv = 0 written)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool role_b = wave >= kFuPairs;
    const int pw = wave & (kFuPairs - 1);
    const int n = lane & 31, kg = lane >> 5;
    const int coff = sk - sq;

    TileLoader<D, NWV> ld;
    ld.init(wave, lane);
    R rd;
    rd.init(lane);
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds) + wave * TileLoader<D, NWV>::NI * 1024);
    unsigned char* const p_lds = lds + 5 * kTile + pw * kPSlab + lane * 16;       // + parity * kFuPairs * kPSlab + 1024 * vector
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    for (int half = 0; half < 2; ++half) {
        const int ktile = half == 0 ? pair : nk - 1 - pair;
        if (half == 1 && ktile == pair) break;                          // odd tile count: the middle tile has no partner
        const int k0 = ktile * kFuCols;
        const int kw0 = k0 + 32 * pw;
        const int kj = kw0 + n;
        const bool k_ok = kj < sk;
        __syncthreads();                                                // the previous half's readers are done with the LDS buffers

        // fragments of this lane's key column (K for role A, V for role B): step s covers d = 16s + 8kg + j
        bf16x8 frag[NS];
        {
            const __bf16* src = role_b ? p.v + v_base + (int64_t)kj * p.vs[2] : p.k + k_base + (int64_t)kj * p.ks[2];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                u32x4 a = {0u, 0u, 0u, 0u};
                if (k_ok) a = *reinterpret_cast<const u32x4*>(src + 16 * s + 8 * kg);
                frag[s] = as_bf16x8(a);
            }
        }
        f32x16 acc[NDT];
#pragma unroll
        for (int i = 0; i < NDT; ++i) acc[i] = zero16;

        int first_tile = 0;
        if (CAUSAL) first_tile = max(0, k0 - coff) / kBwRows;
        const int n_tiles = (sq + kBwRows - 1) / kBwRows;
        // Steps: (query head of the group, row tile), heads innermost; the first key tile of the pair walks
        // its row tiles from the last one down, the second from its first one up, which keeps all workgroups
        // of a (batch, kv head) on the same Q/dO tiles at the same time (they share them through the L2).
        const int n_steps = G * max(0, n_tiles - first_tile);
        // position of a step: first row of its tile and query head within the group; advanced incrementally
        // (steps i, i+1 and i+2 are in flight at any time; no division per step)
        struct Pos {
            int r0, hq;
        };
        const int r_step = half == 0 ? -kBwRows : kBwRows;
        const auto advance = [&](Pos ps) {
            ++ps.hq;
            if (ps.hq == G) {
                ps.hq = 0;
                ps.r0 += r_step;
            }
            return ps;
        };
        // a step whose rows all lie above this wavefront's first key column has nothing for it (uniform)
        const auto idle = [&](Pos ps) { return CAUSAL && kw0 > ps.r0 + kBwRows - 1 + coff; };

        float pend_lse = 0.f, pend_delta = 0.f;      // (delta_lds2 holds -delta)
        const auto bases = [&](Pos ps, int64_t& q_base, int64_t& do_base, int64_t& l_base) {
            const int h = hk * G + ps.hq;
            if (p.cu_q) {
                q_base = (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
                do_base = (int64_t)q_start * p.dos[2] + (int64_t)h * p.dos[1];
                l_base = q_start + (int64_t)h * p.ls[1];
            } else {
                q_base = (int64_t)b * p.qs[0] + (int64_t)h * p.qs[1];
                do_base = (int64_t)b * p.dos[0] + (int64_t)h * p.dos[1];
                l_base = (int64_t)b * p.ls[0] + (int64_t)h * p.ls[1];
            }
        };
        // Q tile of step st (at ps) into ring slot `slot`; its lse into a register
        const auto issue_q = [&](Pos ps, int slot) {
            int64_t q_base, do_base, l_base;
            bases(ps, q_base, do_base, l_base);
            const int r0 = ps.r0;
            ld.issue(p.q + q_base + (int64_t)r0 * p.qs[2], (int)p.qs[2], sq - 1 - r0, dst + slot * kTile);
            const float* rows = p.lse + l_base + r0;                                   // uniform base, 32-bit lane offset
            if (tid < kBwRows) pend_lse = rows[(unsigned)min(tid, sq - 1 - r0)];       // consumed only by publish_lse
        };
        const auto issue_do = [&](int st, Pos ps) {
            int64_t q_base, do_base, l_base;
            bases(ps, q_base, do_base, l_base);
            const int r0 = ps.r0;
            ld.issue(p.dout + do_base + (int64_t)r0 * p.dos[2], (int)p.dos[2], sq - 1 - r0, dst + (3 + (st & 1)) * kTile);
            const float* rows = p.delta + l_base + r0;
            if (tid < kBwRows) pend_delta = rows[(unsigned)min(tid, sq - 1 - r0)];
        };
        // (the values are scaled and masked here, not where they are loaded: consuming them there would put a
        // wait for all outstanding loads - the tiles just issued - in front of the step's arithmetic)
        const auto publish_lse = [&](int st, Pos ps) {
            if (tid < kBwRows) lse_lds2[(st & 1) * kBwRows + tid] = ps.r0 + tid < sq ? pend_lse * kLog2e : INFINITY;
        };
        const auto publish_delta = [&](int st, Pos ps) {
            // a causal row that sees no key has out = NaN, hence delta = NaN, and P = 0 everywhere: any finite
            // delta gives the dS = 0 it must have
            if (tid < kBwRows)
                delta_lds2[(st & 1) * kBwRows + tid] = (ps.r0 + tid < sq && pend_delta == pend_delta) ? -pend_delta : 0.f;
        };

        // second GEMM of either role: acc^T (D x 32 keys) += tile^T . W, 16 query rows at a time.
        // The transposed fragments are read kDepth MFMAs ahead, in this order, fenced by scheduling barriers:
        // left alone the compiler puts each pair of reads, and a full wait, directly in front of its MFMA.
        constexpr int kDepth = 2;
        const auto update = [&](const unsigned char* a_lds, const u32x4 (&w)[4]) {
            constexpr int NC = 4 * NDT;
            i16x4 lo[NC], hi[NC];
            const auto read = [&](int c) {
                const int u = c / NDT, dt = c % NDT;
                lo[c] = lds_read_tr16(a_lds + 16 * u * kRow + rd.tr_off[0][dt]);
                hi[c] = lds_read_tr16(a_lds + 16 * u * kRow + rd.tr_off[1][dt]);
            };
#pragma unroll
            for (int c = 0; c < kDepth && c < NC; ++c) read(c);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (c + kDepth < NC) read(c + kDepth);
                acc[c % NDT] = mfma32(join_bf16x8(lo[c], hi[c]), as_bf16x8(w[c / NDT]), acc[c % NDT]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // first GEMM of either role: (32 rows of the tile at a_lds) x (this lane's key column), fragments read ahead likewise
        const auto scores = [&](const unsigned char* a_lds, const f32x16& c0) {
            u32x4 a[NS];
#pragma unroll
            for (int s = 0; s < kDepth && s < NS; ++s) a[s] = *reinterpret_cast<const u32x4*>(a_lds + rd.row_off[s]);
            f32x16 r = c0;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                if (s + kDepth < NS) a[s + kDepth] = *reinterpret_cast<const u32x4*>(a_lds + rd.row_off[s + kDepth]);
                r = mfma32(as_bf16x8(a[s]), frag[s], r);
                __builtin_amdgcn_sched_barrier(0);
            }
            return r;
        };
        // role A: P of step st from the Q tile in ring slot `slot`: fp32 to LDS for role B, bf16 into p_cur
        u32x4 p_cur[4];
        const auto make_p = [&](auto masked_c, int st, Pos ps, int slot) {
            constexpr bool MASKED = decltype(masked_c)::value;
            const unsigned char* q_lds = lds + slot * kTile;
            const float* lse_lds = lse_lds2 + (st & 1) * kBwRows;
            unsigned char* out = p_lds + (st & 1) * (kFuPairs * kPSlab);
            const int row_lim = CAUSAL ? kj - coff - ps.r0 - 4 * kg : -1;
            // explicit mask: the bytes (row, this lane's key) of the step's 64 rows (a row or key past the end re-reads
            // the last one: its P is 0 through lse = inf, or its column is never stored)
            uint8_t mb[32] = {};
            if constexpr (BOOLM && MASKED) {
                const uint8_t* mcol = p.mask + (int64_t)b * p.ms[0] + (int64_t)(hk * G + ps.hq) * p.ms[1] + min(kj, sk - 1);
#pragma unroll
                for (int e = 0; e < 32; ++e)     // row r0 + 32(e/16) + 8((e/4)%4) + 4kg + e%4
                    mb[e] = mcol[(int64_t)min(ps.r0 + 32 * (e >> 4) + 8 * ((e >> 2) & 3) + 4 * kg + (e & 3), sq - 1) * p.ms[2]];
            }
            // one 32-row half at a time: element i of this lane is query row r0 + 32t + 8(i/4) + 4kg + i%4, key kj
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const f32x16 s_acc = scores(q_lds + t * 32 * kRow, zero16);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_lds + 32 * t + 8 * j + 4 * kg);
                    f32x4 x4;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float x = fast_exp2(fmaf(s_acc[4 * j + r], p.scale_log2, -l4[r]));
                        // kept iff kj <= row + coff, i.e. the tile-relative row (compile-time part) >= row_lim
                        if constexpr (MASKED) {
                            bool keep = 32 * t + 8 * j + r >= row_lim;
                            if constexpr (BOOLM) keep = keep & (mb[16 * t + 4 * j + r] != 0);
                            x = keep ? x : 0.f;
                        }
                        x4[r] = x;
                    }
                    *reinterpret_cast<f32x4*>(out + (4 * t + j) * 1024) = x4;
                    p_cur[2 * t + (j >> 1)][2 * (j & 1)] = pack_bf16(x4[0], x4[1]);
                    p_cur[2 * t + (j >> 1)][2 * (j & 1) + 1] = pack_bf16(x4[2], x4[3]);
                }
            }
        };
        // role B: dS of step st (Q tile in ring slot `slot`), dK^T += Q^T dS
        const auto step_b = [&](int st, int slot) {
            const unsigned char* q_lds = lds + slot * kTile;
            const unsigned char* do_lds = lds + (3 + (st & 1)) * kTile;
            const float* delta_lds = delta_lds2 + (st & 1) * kBwRows;
            const unsigned char* in = p_lds + (st & 1) * (kFuPairs * kPSlab);
            u32x4 ds[4];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                // dP - delta comes straight out of the MFMAs: the -delta of the rows (as published) is their C operand
                f32x16 c0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_lds + 32 * t + 8 * j + 4 * kg);
#pragma unroll
                    for (int r = 0; r < 4; ++r) c0[4 * j + r] = d4[r];
                }
                const f32x16 dp_acc = scores(do_lds + t * 32 * kRow, c0);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const f32x4 p4 = *reinterpret_cast<const f32x4*>(in + (4 * t + j) * 1024);
                    float x[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) x[r] = p4[r] * dp_acc[4 * j + r];                 // dS without the scale factor
                    ds[2 * t + (j >> 1)][2 * (j & 1)] = pack_bf16(x[0], x[1]);
                    ds[2 * t + (j >> 1)][2 * (j & 1) + 1] = pack_bf16(x[2], x[3]);
                }
            }
            update(q_lds, ds);
        };

        // iteration i = -1 .. n_steps-1; ring slots: Q(i) in s_b, Q(i+1) in s_a, Q(i+2) lands in s_l;
        // positions: ps0 of step i, ps1 of step i+1, ps2 of step i+2
        Pos ps1 = {(half == 0 ? n_tiles - 1 : first_tile) * kBwRows, 0};
        Pos ps0 = ps1, ps2 = advance(ps1);
        if (n_steps > 0) {
            issue_q(ps1, 0);
            publish_lse(0, ps1);
        }
        int s_b = 2, s_a = 0, s_l = 1;
        // what every wavefront does around its role's work in an iteration (the same number of barriers in both loops)
        const auto open_iteration = [&](int i) {
            wait_vmcnt<0>();                                   // this wavefront's share of the tiles issued one iteration ago has landed
            __syncthreads();                                   // ... and everybody's; P(i), lse(i+1), delta(i) are visible; older buffers are free
            if (i + 2 < n_steps) issue_q(ps2, s_l);
            if (i + 1 < n_steps) issue_do(i + 1, ps1);
        };
        const auto close_iteration = [&](int i) {
            if (i + 2 < n_steps) publish_lse(i + 2, ps2);
            if (i + 1 < n_steps) publish_delta(i + 1, ps1);
            const int t3 = s_b;
            s_b = s_a;
            s_a = s_l;
            s_l = t3;
            ps0 = ps1;
            ps1 = ps2;
            ps2 = advance(ps2);
        };
        // One loop per role: in a shared loop the accumulators of the two branches meet again after every
        // iteration, and the compiler then copies all 64 of them, and more, each time round.
        if (!role_b) {
            for (int i = -1; i < n_steps; ++i) {
                open_iteration(i);
                if (i >= 0 && !idle(ps0)) update(lds + (3 + (i & 1)) * kTile, p_cur);      // dV^T += dO(i)^T P(i)
                if (i + 1 < n_steps && !idle(ps1)) make_p(std::integral_constant<bool, CAUSAL || BOOLM>{}, i + 1, ps1, s_a);
                close_iteration(i);
            }
        } else {
            for (int i = -1; i < n_steps; ++i) {
                open_iteration(i);
                if (i >= 0 && !idle(ps0)) step_b(i, s_b);
                close_iteration(i);
            }
        }

        // store: lane owns key kj, d = 32dt + 8(i/4) + 4kg + i%4
        if (k_ok) {
            const float f = role_b ? p.scale : 1.0f;
            __bf16* row = role_b ? p.dk + dk_base + (int64_t)kj * p.dks[2] : p.dv + dv_base + (int64_t)kj * p.dvs[2];
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = pack_bf16(acc[dt][4 * g + 0] * f, acc[dt][4 * g + 1] * f);
                    w[1] = pack_bf16(acc[dt][4 * g + 2] * f, acc[dt][4 * g + 3] * f);
                    *reinterpret_cast<u32x2*>(row + 32 * dt + 8 * g + 4 * kg) = w;
                }
        }
    }
}

template <int D>
static int launch_bwd(const BwdParams& p, int mask_mode, hipStream_t stream) {
    const dim3 block(kBwWaves * 64), block_kv(2 * kFuPairs * 64);
    const dim3 grid_q((unsigned)((p.n_qtiles + 1) / 2 * p.Hq * p.B)), grid_k((unsigned)((p.n_ktiles + 1) / 2 * p.Hkv * p.B));
    if (mask_mode == MI355_MASK_CAUSAL) {
        hipLaunchKernelGGL((bwd_dq_kernel<D, MI355_MASK_CAUSAL>), grid_q, block, 0, stream, p);        // dQ, writes delta
        hipLaunchKernelGGL((bwd_dkv_kernel<D, MI355_MASK_CAUSAL>), grid_k, block_kv, 0, stream, p);    // dK and dV, reads delta
    } else if (mask_mode == MI355_MASK_BOOL) {
        hipLaunchKernelGGL((bwd_dq_kernel<D, MI355_MASK_BOOL>), grid_q, block, 0, stream, p);
        hipLaunchKernelGGL((bwd_dkv_kernel<D, MI355_MASK_BOOL>), grid_k, block_kv, 0, stream, p);
    } else {
        hipLaunchKernelGGL((bwd_dq_kernel<D, MI355_MASK_NONE>), grid_q, block, 0, stream, p);
        hipLaunchKernelGGL((bwd_dkv_kernel<D, MI355_MASK_NONE>), grid_k, block_kv, 0, stream, p);
    }
    return (int)hipGetLastError();
}

}  // namespace mi355

using namespace mi355;

static int prefill_bwd_common(const void* q, const void* k, const void* v, const void* out, const void* dout,
                              const float* lse, float* delta, void* dq, void* dk, void* dv,
                              const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                              const int64_t dk_strides[3], const int64_t dv_strides[3], const int64_t lse_strides[2],
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const uint8_t* mask,
                              const int64_t* mask_strides, int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                              float softmax_scale, int mask_mode, int dtype, void* stream) {
    if (!q || !k || !v || !out || !dout || !lse || !delta || !dq || !dk || !dv)
        return set_error(MI355_EINVAL, "prefill_bwd: null pointer argument");
    if (!q_strides || !k_strides || !v_strides || !o_strides || !do_strides || !dq_strides || !dk_strides || !dv_strides ||
        !lse_strides)
        return set_error(MI355_EINVAL, "prefill_bwd: null stride argument");
    if (dtype != MI355_BF16) return set_error(MI355_EDTYPE, "prefill_bwd: dtype must be MI355_BF16");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq_max <= 0 || Sk_max <= 0)
        return set_error(MI355_EINVAL, "prefill_bwd: B, Hq, Hkv, Sq_max and Sk_max must be positive");
    if (Hq % Hkv != 0) return set_error(MI355_EINVAL, "prefill_bwd: Hq must be a multiple of Hkv");
    if (!(D == 128 || D == 64 || D == 32)) return set_error(MI355_EINVAL, "prefill_bwd: head_dim must be 32, 64 or 128");
    if ((cu_seqlens_q == nullptr) != (cu_seqlens_k == nullptr))
        return set_error(MI355_EINVAL, "prefill_bwd: cu_seqlens_q and cu_seqlens_k must be given together");
    if (mask_mode < MI355_MASK_NONE || mask_mode > MI355_MASK_BOOL) return set_error(MI355_EINVAL, "prefill_bwd: unknown mask_mode");
    if (mask_mode == MI355_MASK_BOOL) {
        if (!mask || !mask_strides || cu_seqlens_q)
            return set_error(MI355_EINVAL, "prefill_bwd: MI355_MASK_BOOL needs mask + mask_strides and the dense layout");
        if (((uintptr_t)mask | (uintptr_t)mask_strides[0] | (uintptr_t)mask_strides[1] | (uintptr_t)mask_strides[2]) & 3)
            return set_error(MI355_EINVAL, "prefill_bwd: the mask and its strides must be multiples of 4 bytes");
        if (mask_strides[0] < 0 || mask_strides[1] < 0 || mask_strides[2] < 0)
            return set_error(MI355_EINVAL, "prefill_bwd: mask strides must not be negative");
    }
    const int64_t* all[8] = {q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides};
    for (const int64_t* st : all)
        for (int i = 0; i < 3; ++i)
            if (st[i] & 7) return set_error(MI355_EINVAL, "prefill_bwd: strides must be multiples of 8 elements (16-byte rows)");
    const int64_t* rows[4] = {q_strides, k_strides, v_strides, do_strides};
    for (const int64_t* st : rows)
        if (st[2] <= 0 || st[2] >= (1 << 24))
            return set_error(MI355_EINVAL, "prefill_bwd: row strides must be positive and below 2^24 elements");
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk |
         (uintptr_t)dv) & 15)
        return set_error(MI355_EINVAL, "prefill_bwd: tensors must be 16-byte aligned");

    BwdParams p;
    p.q = (const __bf16*)q;
    p.k = (const __bf16*)k;
    p.v = (const __bf16*)v;
    p.out = (const __bf16*)out;
    p.dout = (const __bf16*)dout;
    p.lse = lse;
    p.delta = delta;
    p.dq = (__bf16*)dq;
    p.dk = (__bf16*)dk;
    p.dv = (__bf16*)dv;
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = q_strides[i];
        p.ks[i] = k_strides[i];
        p.vs[i] = v_strides[i];
        p.os[i] = o_strides[i];
        p.dos[i] = do_strides[i];
        p.dqs[i] = dq_strides[i];
        p.dks[i] = dk_strides[i];
        p.dvs[i] = dv_strides[i];
    }
    p.ls[0] = lse_strides[0];
    p.ls[1] = lse_strides[1];
    p.cu_q = cu_seqlens_q;
    p.cu_k = cu_seqlens_k;
    p.mask = mask_mode == MI355_MASK_BOOL ? mask : nullptr;
    for (int i = 0; i < 3; ++i) p.ms[i] = mask_mode == MI355_MASK_BOOL ? mask_strides[i] : 0;
    p.B = B;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.Sq = Sq_max;
    p.Sk = Sk_max;
    p.scale = softmax_scale;
    p.scale_log2 = softmax_scale * kLog2e;
    p.n_qtiles = (Sq_max + kBwCols - 1) / kBwCols;
    p.n_ktiles = (Sk_max + kFuCols - 1) / kFuCols;
    if ((int64_t)p.n_qtiles * Hq * B > 0x7fffffffLL || (int64_t)p.n_ktiles * Hkv * B > 0x7fffffffLL)
        return set_error(MI355_EINVAL, "prefill_bwd: too many workgroups");

    hipStream_t s = (hipStream_t)stream;
    int rc = D == 128 ? launch_bwd<128>(p, mask_mode, s)
                      : (D == 64 ? launch_bwd<64>(p, mask_mode, s) : launch_bwd<32>(p, mask_mode, s));
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" int mi355_prefill_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout,
                                 const float* lse, float* delta, void* dq, void* dk, void* dv,
                                 const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                 const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                                 const int64_t dk_strides[3], const int64_t dv_strides[3], const int64_t lse_strides[2],
                                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int B, int Hq,
                                 int Hkv, int Sq_max, int Sk_max, int D, float softmax_scale, int mask_mode, int dtype,
                                 void* stream) {
    if (mask_mode == MI355_MASK_BOOL)
        return set_error(MI355_EINVAL, "prefill_bwd: mask_mode must be MI355_MASK_NONE or MI355_MASK_CAUSAL (an explicit mask goes through mi355_prefill_bwd_mask)");
    return prefill_bwd_common(q, k, v, out, dout, lse, delta, dq, dk, dv, q_strides, k_strides, v_strides, o_strides,
                              do_strides, dq_strides, dk_strides, dv_strides, lse_strides, cu_seqlens_q, cu_seqlens_k,
                              nullptr, nullptr, B, Hq, Hkv, Sq_max, Sk_max, D, softmax_scale, mask_mode, dtype, stream);
}

extern "C" int mi355_prefill_bwd_mask(const void* q, const void* k, const void* v, const void* out, const void* dout,
                                      const float* lse, float* delta, void* dq, void* dk, void* dv,
                                      const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                      const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                                      const int64_t dk_strides[3], const int64_t dv_strides[3],
                                      const int64_t lse_strides[2], const uint8_t* mask, const int64_t mask_strides[3],
                                      int B, int Hq, int Hkv, int Sq, int Sk, int D, float softmax_scale, int dtype,
                                      void* stream) {
    return prefill_bwd_common(q, k, v, out, dout, lse, delta, dq, dk, dv, q_strides, k_strides, v_strides, o_strides,
                              do_strides, dq_strides, dk_strides, dv_strides, lse_strides, nullptr, nullptr, mask,
                              mask_strides, B, Hq, Hkv, Sq, Sk, D, softmax_scale, MI355_MASK_BOOL, dtype, stream);
}
