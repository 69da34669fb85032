// Paged-KV decode attention for gfx950: split-K pass + combine.
//
// Work item of the split-K pass = (sequence, kv head, chunk of 4 * tokens_per_wave tokens).
// One workgroup of 4 wavefronts per work item; each wavefront streams its own
// quarter of the chunk, 32 keys (two 16-token cache blocks) per step:
//
//   S^T (keys x queries) = K . Q^T      v_mfma_f32_16x16x32_bf16, the Hq/Hkv query
//                                       heads that share the kv head are the N
//                                       columns (padded to 16), so every KV byte
//                                       is fetched once per GQA group (once per 16
//                                       query heads when a group has more)
//   online softmax on S^T               each lane owns ONE query column and 8 keys;
//                                       max/sum across the 4 lanes of a column
//   O^T (d x queries) += V^T . P^T      V^T fragments come from a wavefront-private
//                                       LDS tile through ds_read_b64_tr_b16
//
// K and V both go global -> registers (fully coalesced, non-temporal, 1 KiB per
// instruction) -> wavefront-private LDS tile; K fragments come back with
// ds_read_b128 in MFMA A-operand layout, V^T fragments with the transposed read.
// The next step's loads are issued as soon as the staging registers are free, so
// they fly during the whole step.  (Direct global->LDS loads are not used: an LDS
// read of a wavefront waits for every direct-to-LDS load it issued earlier, which
// would serialise a wavefront-private pipeline.)
// The four wavefronts merge their (m, l, O) in LDS; a sequence that fits one
// chunk is normalised and written straight to `out`, otherwise the chunk's
// partial goes to the workspace and the combine kernel finishes it:
//   o = sum_c 2^(m_c - m) o_c / sum_c 2^(m_c - m) l_c      (m = max_c m_c).
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace mi355 {

constexpr int kDecodeWaves = 4;
constexpr int kMaxTokensPerWave = 1024;                 // 64 cache blocks: one block id per lane
constexpr int kBlock = 16;                              // tokens per cache block
constexpr int kStage = 32;                              // keys per step (2 blocks)

struct DecodeParams {
    const __bf16* q;
    const void* k_cache;
    const void* v_cache;
    __bf16* out;
    const int32_t* block_tables;
    int64_t bt_row_stride;
    int num_blocks;
    const int32_t* context_lens;
    const float* k_scale;
    const float* v_scale;
    float* ws_o;
    float* ws_m;
    float* ws_l;
    int B, Hq, Hkv, max_chunks, max_ctx;
    int n_groups;             // ceil((Hq / Hkv) / 16): a kv head with more than 16 query heads is served 16 at a time
    int tokens_per_wave;      // 256, 512 or 1024: a long stream per wavefront amortises its start-up latency
    float scale_log2;
};

template <int D, bool FP8>
struct DecodeLds {
    static constexpr int kVRow = D * 2 + 32;                 // bytes per staged V row (bf16, padded)
    static constexpr int kVBytes = kStage * kVRow;           // per-wavefront V tile
    static constexpr int kKRow = FP8 ? D : D * 2;            // bytes per staged K row (raw cache bytes, swizzled)
    static constexpr int kKBytes = kStage * kKRow;           // per-wavefront K tile
    static constexpr int kPartRow = D + 4;                   // floats per row of a wavefront's partial O: the padding puts the
                                                             // 16-byte pieces that 16 lanes write together into 16 bank groups
    static constexpr int kPartFloats = 16 * kPartRow + 32;   // per-wavefront (O, m, l)
    static constexpr int kTiles = kVBytes + kKBytes;
    static constexpr int kWaveBytes = kTiles > kPartFloats * 4 ? kTiles : kPartFloats * 4;
};

// Occupancy: the fp8 instance is held to the registers of three wavefronts per SIMD (164 used, no spills) so
// that three workgroups share a CU (3 x 52 KiB of LDS): with ragged lengths many workgroups have idle
// wavefronts, and a third resident workgroup fills in (+1 % on a log-uniform batch, -0.7 % on equal lengths).
// The bf16 instance needs 70 KiB of LDS per workgroup: two per CU whatever the registers.
template <int D, bool FP8>
__global__ __launch_bounds__(kDecodeWaves * 64) __attribute__((amdgpu_waves_per_eu(FP8 ? 3 : 2, FP8 ? 3 : 2)))
void paged_decode_split_kernel(DecodeParams p) {
    constexpr int NS = D / 32;                       // MFMA k-steps of K.Q^T
    constexpr int NT = D / 16;                       // 16-row tiles of O^T
    constexpr int VL = FP8 ? (D / 64) : (D / 32);    // 16-byte loads per lane per block (K and V alike)
    constexpr int KL = VL;
    constexpr int kVRow = DecodeLds<D, FP8>::kVRow;
    constexpr int kVBytes = DecodeLds<D, FP8>::kVBytes;
    constexpr int kKRow = DecodeLds<D, FP8>::kKRow;
    constexpr int kKChunks = kKRow / 16;              // 16-byte chunks per staged K row
    constexpr int kKRowsPer256 = 256 / kKRow > 0 ? 256 / kKRow : 1;
    constexpr int kWaveBytes = DecodeLds<D, FP8>::kWaveBytes;
    constexpr int kPartRow = DecodeLds<D, FP8>::kPartRow;
    static_assert(!FP8 || D >= 64, "fp8 KV needs head_dim >= 64");

    __shared__ __attribute__((aligned(16))) unsigned char smem[kDecodeWaves * kWaveBytes];

    // 1-D grid, kv head fastest, then sequence, chunk slowest.  Workgroup ids are dealt
    // round-robin to the 8 XCDs, so the low bits of the id must not select the chunk:
    // with ragged lengths late chunks are mostly empty and the XCDs that own them would idle.
    // Chunks are dealt in DESCENDING order: the full chunks of the long sequences start first
    // and the first chunks of the short sequences (the smallest work items) form the tail.
    // A kv head with more than 16 query heads is served by several workgroups per (sequence, chunk), 16 query heads
    // each, which read the same K/V: they sit eight ids apart, i.e. on one XCD and next to each other in time, so that
    // the stream comes from HBM once and from that XCD's L2 afterwards.
    const int wg = blockIdx.x;
    int item = wg, grp = 0;                               // item = (kv head, sequence, chunk); grp = which 16 query heads
    if (p.n_groups > 1) {
        const int items = gridDim.x / p.n_groups, whole = items / 8 * 8;
        if (wg < whole * p.n_groups) {
            const int within = wg % (8 * p.n_groups);
            grp = within / 8;
            item = wg / (8 * p.n_groups) * 8 + within % 8;
        } else {
            const int rest = wg - whole * p.n_groups;
            grp = rest % p.n_groups;
            item = whole + rest / p.n_groups;
        }
    }
    const int hk = item % p.Hkv;
    const int b = (item / p.Hkv) % p.B;
    const int chunk = p.max_chunks - 1 - item / (p.Hkv * p.B);
    const int ctx = min(p.context_lens[b], p.max_ctx);     // a length beyond the promised bound is truncated, never chased
    const int chunk_tokens = kDecodeWaves * p.tokens_per_wave;
    const int chunk_start = chunk * chunk_tokens;
    if (chunk_start >= ctx) return;

    const int h0 = hk * (p.Hq / p.Hkv) + 16 * grp;       // first query head of this work item
    const int G = min(16, p.Hq / p.Hkv - 16 * grp);      // ... and how many it serves
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15;          // key row of K / query column of S^T / d row of V^T
    const int kg = lane >> 4;         // 0..3

    unsigned char* wsm = smem + wave * kWaveBytes;      // this wavefront's V tile (then its K tile)
    unsigned char* ksm = wsm + kVBytes;
    // K rows are stored unpadded; the 16-byte chunk c of row q lives in slot c ^ kswz(q) so that the
    // 16 lanes reading one chunk column of 16 consecutive rows hit 16 different bank groups
    auto kswz = [&](int row) { return (row / kKRowsPer256) % kKChunks; };

    // ---- Q^T B-operand fragments (zero for padded query columns) ----------
    // bf16 cache: step s covers d = 32s + 8kg + j.
    // fp8 cache : one 16-byte K load carries d = 64t + 16kg + (0..15); step s = 2t+e
    //             covers d = 64t + 16kg + 8e + j, so Q uses the same d order.
    bf16x8 qf[NS];
    {
        const __bf16* qrow = p.q + ((int64_t)b * p.Hq + h0 + r) * D;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int d0 = FP8 ? (64 * (s >> 1) + 16 * kg + 8 * (s & 1)) : (32 * s + 8 * kg);
            u32x4 t = {0u, 0u, 0u, 0u};
            if (r < G) t = *reinterpret_cast<const u32x4*>(qrow + d0);
            qf[s] = as_bf16x8(t);
        }
    }

    const int t0 = chunk_start + wave * p.tokens_per_wave;
    const int t1 = min(ctx, t0 + p.tokens_per_wave);
    const int n_iter = t1 > t0 ? (t1 - t0 + kStage - 1) / kStage : 0;
    const int last_blk = (ctx - 1) / kBlock;
    const int32_t* bt = p.block_tables + (int64_t)b * p.bt_row_stride;

    // Block ids (and fp8 scales) of this wavefront's token range, one block per lane, fetched
    // once: lane l holds logical block t0/16 + l, clamped to the sequence's last block so that
    // every id is a real block.  The step loop reads them with v_readlane, so no dependent
    // table load sits between two steps.
    // a block id outside the pool (a corrupted table) is clamped into it: wrong numbers, never a wild read
    const int my_phys = min(max(bt[min(t0 / kBlock + lane, last_blk)], 0), p.num_blocks - 1);
    float my_ks = 1.0f, my_vs = 1.0f;
    if constexpr (FP8) {
        my_ks = p.k_scale[(int64_t)my_phys * p.Hkv + hk];
        my_vs = p.v_scale[(int64_t)my_phys * p.Hkv + hk];
    }

    u32x4 kreg[2][KL];
    u32x4 vreg[2][VL];

    auto slab_of = [&](int blk) -> int64_t {     // element offset of (block, kv head) in the cache
        const int64_t phys = __builtin_amdgcn_readlane(my_phys, blk);
        return (phys * p.Hkv + hk) * (int64_t)(kBlock * D);
    };
    // K and V are both fetched as fully contiguous 1 KiB per instruction (streaming, non-temporal):
    // partial-line patterns measurably lose HBM bandwidth.  Lane l of load j holds bytes
    // (64j + l)*16 .. +15 of the (block, kv head) slab.
    auto load_k = [&](int it) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const unsigned char* kb = reinterpret_cast<const unsigned char*>(p.k_cache) + slab_of(2 * it + t) * (FP8 ? 1 : 2);
#pragma unroll
            for (int j = 0; j < KL; ++j)
                kreg[t][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kb + (j * 64 + lane) * 16));
        }
    };
    auto load_v = [&](int it) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int64_t slab = slab_of(2 * it + t);
            if constexpr (FP8) {
                const unsigned char* vb = reinterpret_cast<const unsigned char*>(p.v_cache) + slab;
#pragma unroll
                for (int j = 0; j < VL; ++j)
                    vreg[t][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vb + (j * 64 + lane) * 16));
            } else {
                const __bf16* vb = reinterpret_cast<const __bf16*>(p.v_cache) + slab;
#pragma unroll
                for (int j = 0; j < VL; ++j)
                    vreg[t][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vb + (j * 64 + lane) * 8));
            }
        }
    };

    float m_run = -INFINITY;      // exponent reference (log2 domain) of this lane's query column: >= its running max - slack
    float l_run = 0.0f;           // this lane's share of the running sum
    f32x4 o[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Software pipeline without double buffering: the registers of step `it` are refilled for
    // step it+1 as soon as they have been consumed (V after its copy to LDS, K after K.Q^T), so
    // the next step's loads fly during this step's softmax and P.V.  The last step "prefetches"
    // itself again (cache hits, never used): an unconditional prefetch keeps the loop free of
    // branches, so the wait counts stay exact.
    if (n_iter > 0) {
        load_v(0);
        load_k(0);
    }
    // One step; TAIL selects the code that blanks the keys past the end of the range (only the last step
    // of a wavefront can need it, so the other steps carry no compare/select per element).
    const auto step = [&](int it, auto tail_c) {
        constexpr bool tail = decltype(tail_c)::value;
        const int kbase = t0 + it * kStage;

        // ---- V: registers -> wavefront-private LDS tile (bf16, row = key) --
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int j = 0; j < VL; ++j) {
                if constexpr (FP8) {
                    const int e = (j * 64 + lane) * 16;     // element index in the block slab
                    const int row = e / D, col = e % D;
                    u32x4 raw = vreg[t][j];
                    if (tail && kbase + 16 * t + row >= t1) raw = u32x4{0u, 0u, 0u, 0u};
                    u32x2 a = fp8x4_to_bf16x4(raw[0]), bq = fp8x4_to_bf16x4(raw[1]);
                    u32x2 c = fp8x4_to_bf16x4(raw[2]), dq = fp8x4_to_bf16x4(raw[3]);
                    unsigned char* dst = wsm + (16 * t + row) * kVRow + col * 2;
                    *reinterpret_cast<u32x4*>(dst) = u32x4{a[0], a[1], bq[0], bq[1]};
                    *reinterpret_cast<u32x4*>(dst + 16) = u32x4{c[0], c[1], dq[0], dq[1]};
                } else {
                    const int e = (j * 64 + lane) * 8;
                    const int row = e / D, col = e % D;
                    u32x4 raw = vreg[t][j];
                    if (tail && kbase + 16 * t + row >= t1) raw = u32x4{0u, 0u, 0u, 0u};
                    *reinterpret_cast<u32x4*>(wsm + (16 * t + row) * kVRow + col * 2) = raw;
                }
            }
        }
        // ---- K: registers -> wavefront-private LDS tile (raw cache bytes, swizzled chunks) --
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int j = 0; j < KL; ++j) {
                const int cidx = j * 64 + lane;                       // 16-byte chunk index inside the slab
                const int row = 16 * t + cidx / kKChunks, c = cidx % kKChunks;
                *reinterpret_cast<u32x4*>(ksm + row * kKRow + ((c ^ kswz(row)) << 4)) = kreg[t][j];
            }
        }
        // The staging registers are free again: fetch the next step now, so that its loads
        // fly during everything below.  The scheduling barriers keep the compiler from sinking
        // the loads towards their (next-iteration) uses.
        __builtin_amdgcn_sched_barrier(0);
        load_v(min(it + 1, n_iter - 1));
        load_k(min(it + 1, n_iter - 1));
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T = K . Q^T ---------------------------------------------------
        // A fragment of step s, key row 16t + r: bf16 cache: chunk 4s + kg (d = 32s + 8kg ..);
        // fp8 cache: chunk 4j + kg holds d = 64j + 16kg .. +15, i.e. the two steps 2j and 2j+1.
        f32x4 s_acc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s_acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            const int row = 16 * t + r;
            const unsigned char* krow = ksm + row * kKRow;
            if constexpr (FP8) {
#pragma unroll
                for (int j = 0; j < D / 64; ++j) {
                    const u32x4 raw = *reinterpret_cast<const u32x4*>(krow + (((4 * j + kg) ^ kswz(row)) << 4));
                    u32x2 a = fp8x4_to_bf16x4(raw[0]), bq = fp8x4_to_bf16x4(raw[1]);
                    u32x2 c = fp8x4_to_bf16x4(raw[2]), dq = fp8x4_to_bf16x4(raw[3]);
                    s_acc[t] = mfma16(as_bf16x8(u32x4{a[0], a[1], bq[0], bq[1]}), qf[2 * j], s_acc[t]);
                    s_acc[t] = mfma16(as_bf16x8(u32x4{c[0], c[1], dq[0], dq[1]}), qf[2 * j + 1], s_acc[t]);
                }
            } else {
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const u32x4 kf = *reinterpret_cast<const u32x4*>(krow + (((4 * s + kg) ^ kswz(row)) << 4));
                    s_acc[t] = mfma16(as_bf16x8(kf), qf[s], s_acc[t]);
                }
            }
        }

        // ---- online softmax (lane: query column r, keys 16t + 4kg + i) -------
        float ks2[2] = {1.0f, 1.0f}, vs2[2] = {1.0f, 1.0f};
        if constexpr (FP8) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                ks2[t] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_ks), 2 * it + t));
                vs2[t] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_vs), 2 * it + t));
            }
        }
        float x[8];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const float sc = p.scale_log2 * ks2[t];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = s_acc[t][i] * sc;
                if (tail && kbase + 16 * t + 4 * kg + i >= t1) v = -INFINITY;
                x[4 * t + i] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = xor_max_16_32(mx);
        // Lazy rescaling: m_run is the exponent reference, not the running maximum; it moves only when some
        // query's maximum outgrows it by more than 2^kSlack (weights up to 2^kSlack are exact in the fp32
        // sums and harmless in bf16), so the common step neither multiplies O nor touches l.
        constexpr float kSlack = 8.0f;
        if (__builtin_amdgcn_ballot_w64(!(mx - m_run <= kSlack)) != 0) {       // also taken while m_run = -inf
            const float m_new = fmaxf(m_run, mx);
            const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2(m_run - m_new);   // 0 the first time a key is seen
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < NT; ++i) o[i] *= alpha;
        }
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            x[i] = fast_exp2(x[i] - m_run);
            psum += x[i];
        }
        l_run += psum;
        u32x4 pp;
        pp[0] = pack_bf16(x[0] * vs2[0], x[1] * vs2[0]);
        pp[1] = pack_bf16(x[2] * vs2[0], x[3] * vs2[0]);
        pp[2] = pack_bf16(x[4] * vs2[1], x[5] * vs2[1]);
        pp[3] = pack_bf16(x[6] * vs2[1], x[7] * vs2[1]);
        const bf16x8 pf = as_bf16x8(pp);

        // ---- O^T += V^T . P^T -------------------------------------------------
        // source lane s of group kg addresses key row 4kg + s/4, columns 16dt + 4(s%4)..+3
        const unsigned char* vsrc = wsm + (4 * kg + (r >> 2)) * kVRow + (r & 3) * 8;
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) {
            i16x4 lo = lds_read_tr16(vsrc + dt * 32);
            i16x4 hi = lds_read_tr16(vsrc + 16 * kVRow + dt * 32);
            o[dt] = mfma16(join_bf16x8(lo, hi), pf, o[dt]);
        }
        // Compiler barrier: without a may-write instruction after the prefetch loads, the
        // optimiser turns "phi of loads" into "load of phi" and the loads land at the top of
        // the NEXT iteration, i.e. the prefetch is undone.
        asm volatile("" ::: "memory");
    };
    for (int it = 0; it + 1 < n_iter; ++it) step(it, std::false_type{});
    if (n_iter > 0) {
        if ((t1 - t0) % kStage == 0) step(n_iter - 1, std::false_type{});
        else step(n_iter - 1, std::true_type{});
    }

    // ---- merge the four wavefronts ------------------------------------------
    l_run = xor_sum_16_32(l_run);
    {
        // (one 16-byte write per d-tile; with unpadded rows of D floats the sixteen lanes of a query column group
        // all wrote the same bank: a third of this kernel's LDS time on short streams)
        float* part = reinterpret_cast<float*>(wsm);
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) *reinterpret_cast<f32x4*>(part + r * kPartRow + 16 * dt + 4 * kg) = o[dt];
        if (kg == 0) {
            part[16 * kPartRow + r] = m_run;
            part[16 * kPartRow + 16 + r] = l_run;
        }
    }
    __syncthreads();

    const int n_chunks = (ctx + chunk_tokens - 1) / chunk_tokens;
    for (int idx = threadIdx.x; idx < G * D; idx += kDecodeWaves * 64) {
        const int qi = idx / D, d = idx % D;
        float mw[kDecodeWaves];
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; ++w) {
            mw[w] = reinterpret_cast<const float*>(smem + w * kWaveBytes)[16 * kPartRow + qi];
            M = fmaxf(M, mw[w]);
        }
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; ++w) {
            const float* part = reinterpret_cast<const float*>(smem + w * kWaveBytes);
            const float f = fast_exp2(mw[w] - M);       // a wavefront without keys has m = -inf -> 0
            num += f * part[qi * kPartRow + d];
            den += f * part[16 * kPartRow + 16 + qi];
        }
        const int64_t row = (int64_t)b * p.Hq + h0 + qi;
        if (n_chunks == 1) {
            p.out[row * D + d] = (__bf16)(num / den);
        } else {
            const int64_t slot = row * p.max_chunks + chunk;
            p.ws_o[slot * D + d] = num;
            if (d == 0) {
                p.ws_m[slot] = M;
                p.ws_l[slot] = den;
            }
        }
    }
}

// Combine: one thread per (row = sequence x query head, 4 adjacent d), 256 / (D / 4) rows per workgroup.
constexpr int kCombineThreads = 256;

template <int D>
__global__ __launch_bounds__(kCombineThreads) void paged_decode_combine_kernel(DecodeParams p) {
    constexpr int kLanesPerRow = D / 4;
    const int row = blockIdx.x * (kCombineThreads / kLanesPerRow) + threadIdx.x / kLanesPerRow;      // b * Hq + h
    if (row >= p.B * p.Hq) return;
    const int b = row / p.Hq;
    const int ctx = min(p.context_lens[b], p.max_ctx);
    const int chunk_tokens = kDecodeWaves * p.tokens_per_wave;
    const int n_chunks = (ctx + chunk_tokens - 1) / chunk_tokens;
    if (n_chunks <= 1) return;                   // written by the split pass (or empty)
    const int d = (threadIdx.x % kLanesPerRow) * 4;
    const int64_t base = (int64_t)row * p.max_chunks;
    float M = -INFINITY;
    for (int c = 0; c < n_chunks; ++c) M = fmaxf(M, p.ws_m[base + c]);
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int c = 0; c < n_chunks; ++c) {
        const float f = fast_exp2(p.ws_m[base + c] - M);
        const f32x4 o = *reinterpret_cast<const f32x4*>(p.ws_o + (base + c) * D + d);
#pragma unroll
        for (int i = 0; i < 4; ++i) num[i] += f * o[i];
        den += f * p.ws_l[base + c];
    }
    u32x2 w;
    w[0] = pack_bf16(num[0] / den, num[1] / den);
    w[1] = pack_bf16(num[2] / den, num[3] / den);
    *reinterpret_cast<u32x2*>(p.out + (int64_t)row * D + d) = w;
}

// Combine for sequences of many chunks (a small batch of long contexts runs short chunks, see tokens_per_wave_for: one
// sequence of 32 K tokens has 128 of them): one workgroup per row, the chunks dealt to 256 / (D / 4) groups of lanes
// that each reduce every kGroups-th chunk; the groups' partial sums meet in LDS.  (One thread walking 128 chunks took
// 12 us of that sequence's 35 us step.)
template <int D>
__global__ __launch_bounds__(kCombineThreads) void paged_decode_combine_wide_kernel(DecodeParams p) {
    constexpr int kLanesPerRow = D / 4;
    constexpr int kGroups = kCombineThreads / kLanesPerRow;
    __shared__ float s_m[kGroups], s_den[kGroups];
    __shared__ f32x4 s_num[kGroups][kLanesPerRow];
    const int row = blockIdx.x;                    // b * Hq + h
    const int b = row / p.Hq;
    const int ctx = min(p.context_lens[b], p.max_ctx);
    const int chunk_tokens = kDecodeWaves * p.tokens_per_wave;
    const int n_chunks = (ctx + chunk_tokens - 1) / chunk_tokens;
    if (n_chunks <= 1) return;                   // written by the split pass (or empty); the whole workgroup leaves
    const int g = threadIdx.x / kLanesPerRow, ln = threadIdx.x % kLanesPerRow, d = ln * 4;
    const int64_t base = (int64_t)row * p.max_chunks;
    float M = -INFINITY;
    for (int c = g; c < n_chunks; c += kGroups) M = fmaxf(M, p.ws_m[base + c]);
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int c = g; c < n_chunks; c += kGroups) {
        const float f = fast_exp2(p.ws_m[base + c] - M);
        const f32x4 o = *reinterpret_cast<const f32x4*>(p.ws_o + (base + c) * D + d);
#pragma unroll
        for (int i = 0; i < 4; ++i) num[i] += f * o[i];
        den += f * p.ws_l[base + c];
    }
    if (ln == 0) {
        s_m[g] = M;                                // -inf for a group without chunks: its weight below is 0
        s_den[g] = den;
    }
    s_num[g][ln] = num;
    __syncthreads();
    if (g != 0) return;
    float Mall = s_m[0];
#pragma unroll
    for (int i = 1; i < kGroups; ++i) Mall = fmaxf(Mall, s_m[i]);
    f32x4 tot = {0.f, 0.f, 0.f, 0.f};
    float dtot = 0.f;
#pragma unroll
    for (int i = 0; i < kGroups; ++i) {
        const float f = fast_exp2(s_m[i] - Mall);      // (group 0 always has a chunk, so Mall is finite)
        const f32x4 o = s_num[i][ln];
#pragma unroll
        for (int e = 0; e < 4; ++e) tot[e] += f * o[e];
        dtot += f * s_den[i];
    }
    u32x2 w;
    w[0] = pack_bf16(tot[0] / dtot, tot[1] / dtot);
    w[1] = pack_bf16(tot[2] / dtot, tot[3] / dtot);
    *reinterpret_cast<u32x2*>(p.out + (int64_t)row * D + d) = w;
}

// The wide combine serves launches of more than kWideCombineChunks chunks per sequence and at most kWideCombineRows rows
// (a workgroup per row: with thousands of rows of eight chunks -- 16 384 at 256 sequences of 64 query heads -- the
// narrow kernel's eight rows per workgroup are 8 us against 15).
constexpr int kWideCombineChunks = 4;
constexpr int kWideCombineRows = 2048;

template <int D, bool FP8>
static int launch_decode(const DecodeParams& p, hipStream_t stream) {
    dim3 grid((unsigned)p.max_chunks * p.Hkv * p.n_groups * p.B);
    hipLaunchKernelGGL((paged_decode_split_kernel<D, FP8>), grid, dim3(kDecodeWaves * 64), 0, stream, p);
    if (p.max_chunks > kWideCombineChunks && (int64_t)p.B * p.Hq <= kWideCombineRows) {
        hipLaunchKernelGGL((paged_decode_combine_wide_kernel<D>), dim3((unsigned)(p.B * p.Hq)), dim3(kCombineThreads), 0,
                           stream, p);
    } else if (p.max_chunks > 1) {
        const int rows_per_wg = kCombineThreads / (D / 4);
        hipLaunchKernelGGL((paged_decode_combine_kernel<D>), dim3((p.B * p.Hq + rows_per_wg - 1) / rows_per_wg),
                           dim3(kCombineThreads), 0, stream, p);
    }
    return (int)hipGetLastError();
}

}  // namespace mi355

using namespace mi355;

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Tokens per wavefront grow with the longest context: short batches keep all four wavefronts of
// a workgroup busy, long ones get long uninterrupted streams.  A small batch then has too few workgroups
// for the GPU -- one sequence of 8192 tokens on 8 kv heads: 16 -- and gets shorter streams until there is
// about a workgroup per compute unit (the same sequence: 256 workgroups of 4 x 64 tokens).
// items = B * Hkv * (groups of 16 query heads per kv head): the workgroups per chunk.
constexpr int kMinTokensPerWave = 64;
constexpr int kTargetWorkgroups = 256;
static int tokens_per_wave_for(int max_ctx, int64_t items) {
    int tpw = max_ctx >= 4096 ? kMaxTokensPerWave : (max_ctx >= 2048 ? 512 : 256);
    // (up to 1024 tokens one chunk serves a sequence and no combine pass is needed: worth more than shorter streams)
    if (max_ctx <= kDecodeWaves * 256) return tpw;
    while (tpw > kMinTokensPerWave && items * ((max_ctx + kDecodeWaves * tpw - 1) / (kDecodeWaves * tpw)) < kTargetWorkgroups) tpw /= 2;
    return tpw;
}
static int n_groups_of(int Hq, int Hkv) { return (Hq / Hkv + 15) / 16; }

extern "C" int mi355_paged_decode_chunk_tokens(int B, int Hq, int Hkv, int max_ctx) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || max_ctx <= 0) return 0;
    return kDecodeWaves * tokens_per_wave_for(max_ctx, (int64_t)B * Hkv * n_groups_of(Hq, Hkv));
}

// Bytes of split-K partials for `rows` (sequence, query head, chunk) triples: O (D fp32), m, l.
static size_t workspace_layout_bytes(size_t rows, size_t D) {
    return align_up(rows * D * 4, 256) + 2 * align_up(rows * 4, 256);
}

// The chunk size depends on max_ctx (1024, 2048, 4096 tokens) and shrinks for small batches, so the number of
// chunks a launch really uses is not monotonic in max_ctx or B.  The requirement reported here bounds it for every
// launch with a batch up to B and a bound up to max_ctx: chunks of the full size need at most 2 per sequence below
// 4096 tokens and ceil(max_ctx / 4096) from there on; shrunken chunks mean fewer than 2 * kTargetWorkgroups
// workgroups, i.e. fewer than 32 * kTargetWorkgroups rows (a workgroup serves at most 16 query heads), and never
// more than ceil(max_ctx / 256) per sequence.  A workspace sized for a caller's largest batch and longest context
// therefore serves every smaller call.
extern "C" size_t mi355_paged_decode_workspace_bytes(int B, int Hq, int D, int max_ctx) {
    if (B <= 0 || Hq <= 0 || D <= 0 || max_ctx <= 0) return 0;
    const size_t big = ((size_t)max_ctx + 4 * kMaxTokensPerWave - 1) / (4 * kMaxTokensPerWave);
    const size_t small = max_ctx > 4 * 256 ? 2 : 1;
    const size_t full = (size_t)B * Hq * (big > small ? big : small);
    const size_t finest = (size_t)B * Hq * (((size_t)max_ctx + kDecodeWaves * kMinTokensPerWave - 1) / (kDecodeWaves * kMinTokensPerWave));
    const size_t shrunk = finest < (size_t)32 * kTargetWorkgroups ? finest : (size_t)32 * kTargetWorkgroups;
    return workspace_layout_bytes(full > shrunk ? full : shrunk, (size_t)D);
}

// Argument checks and launches shared by the two entry points.  `static_scratch`: the workspace is the library's
// own device array (its capacity is `workspace_bytes`), fetched only once the arguments have passed the checks.
static int scratch_for_current_device(void** ptr);

static int decode_common(const void* q, const void* k_cache, const void* v_cache, void* out,
                         const int32_t* block_tables, int64_t bt_row_stride, const int32_t* context_lens,
                         const float* k_scale, const float* v_scale, void* workspace, size_t workspace_bytes,
                         bool static_scratch, int B, int Hq, int Hkv, int D, int block_size, int64_t num_blocks,
                         int max_ctx, float softmax_scale, int kv_dtype, void* stream) {
    if (!q || !k_cache || !v_cache || !out || !block_tables || !context_lens)
        return set_error(MI355_EINVAL, "paged_decode: null pointer argument");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || max_ctx <= 0)
        return set_error(MI355_EINVAL, "paged_decode: B, Hq, Hkv and max_ctx must be positive");
    if (Hq % Hkv != 0) return set_error(MI355_EINVAL, "paged_decode: Hq must be a multiple of Hkv");
    const int n_groups = n_groups_of(Hq, Hkv);
    if (block_size != kBlock) return set_error(MI355_EINVAL, "paged_decode: block_size must be 16");
    if (num_blocks <= 0 || num_blocks > 0x7fffffffLL)
        return set_error(MI355_EINVAL, "paged_decode: num_blocks must be positive (and below 2^31)");
    const int chunk = mi355_paged_decode_chunk_tokens(B, Hq, Hkv, max_ctx);
    if ((int64_t)((max_ctx + chunk - 1) / chunk) * Hkv * n_groups * B > 0x7fffffffLL)
        return set_error(MI355_EINVAL, "paged_decode: chunks * Hkv * B exceeds the grid limit");
    if (kv_dtype != MI355_BF16 && kv_dtype != MI355_FP8_E4M3)
        return set_error(MI355_EDTYPE, "paged_decode: kv_dtype must be MI355_BF16 or MI355_FP8_E4M3");
    const bool fp8 = kv_dtype == MI355_FP8_E4M3;
    if (fp8 && (!k_scale || !v_scale))
        return set_error(MI355_EINVAL, "paged_decode: fp8 KV cache needs k_scale and v_scale");
    if (!(D == 128 || D == 64 || (D == 32 && !fp8)))
        return set_error(MI355_EINVAL, "paged_decode: head_dim must be 64 or 128 (or 32 with a bf16 cache)");
    const int max_chunks = (max_ctx + chunk - 1) / chunk;
    const size_t need = workspace_layout_bytes((size_t)B * Hq * max_chunks, (size_t)D);   // <= the reported bound
    if (static_scratch) {
        if (max_chunks > 1 && need > workspace_bytes)
            return set_error(MI355_EWORKSPACE,
                             "paged_decode_static: B * Hq * chunks(max_ctx) * (D + 2) * 4 bytes of split-K partials exceed the "
                             "library's static scratch (MI355_STATIC_SCRATCH_BYTES); use "
                             "mi355_paged_decode_fwd with a caller-provided workspace");
        if (max_chunks > 1) {
            const int rc = scratch_for_current_device(&workspace);
            if (rc != 0) return rc;
        }
    } else if (max_chunks > 1 && (!workspace || workspace_bytes < need)) {
        return set_error(MI355_EWORKSPACE, "paged_decode: workspace smaller than mi355_paged_decode_workspace_bytes()");
    }

    DecodeParams p;
    p.q = (const __bf16*)q;
    p.k_cache = k_cache;
    p.v_cache = v_cache;
    p.out = (__bf16*)out;
    p.block_tables = block_tables;
    p.bt_row_stride = bt_row_stride;
    p.num_blocks = (int)num_blocks;
    p.context_lens = context_lens;
    p.k_scale = k_scale;
    p.v_scale = v_scale;
    const size_t rows = (size_t)B * Hq * max_chunks;
    char* ws = (char*)workspace;
    p.ws_o = (float*)ws;
    p.ws_m = (float*)(ws + align_up(rows * D * 4, 256));
    p.ws_l = (float*)(ws + align_up(rows * D * 4, 256) + align_up(rows * 4, 256));
    p.B = B;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.max_chunks = max_chunks;
    p.max_ctx = max_ctx;
    p.n_groups = n_groups;
    p.tokens_per_wave = chunk / kDecodeWaves;
    p.scale_log2 = softmax_scale * kLog2e;

    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (fp8) {
        rc = D == 128 ? launch_decode<128, true>(p, s) : launch_decode<64, true>(p, s);
    } else {
        rc = D == 128 ? launch_decode<128, false>(p, s)
                      : (D == 64 ? launch_decode<64, false>(p, s) : launch_decode<32, false>(p, s));
    }
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" int mi355_paged_decode_fwd(const void* q, const void* k_cache, const void* v_cache, void* out,
                                      const int32_t* block_tables, int64_t bt_row_stride,
                                      const int32_t* context_lens, const float* k_scale,
                                      const float* v_scale, void* workspace, size_t workspace_bytes, int B,
                                      int Hq, int Hkv, int D, int block_size, int64_t num_blocks, int max_ctx,
                                      float softmax_scale, int kv_dtype, void* stream) {
    return decode_common(q, k_cache, v_cache, out, block_tables, bt_row_stride, context_lens, k_scale, v_scale, workspace,
                         workspace_bytes, false, B, Hq, Hkv, D, block_size, num_blocks, max_ctx, softmax_scale, kv_dtype,
                         stream);
}

// ---- the variant that allocates nothing -------------------------------------------------------------------
// Split-K partials live in a file-scope device array instead of a caller-provided workspace.  Every GPU that
// loads the library holds its own copy of the array (at its own address) until the process ends.  In host code
// the array's name is only a stand-in for the symbol, not a device address: the address on a device is asked for
// once per device, with that device current, and kept; kernels only ever see that pointer.
constexpr size_t kStaticScratchBytes = MI355_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];            // device address of `scratch`, per device (null: not asked yet)
static std::mutex g_scratch_mutex;

static int scratch_for_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error((int)e, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return set_error(MI355_EINVAL, "paged_decode_static: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            return set_error(e != hipSuccess ? (int)e : MI355_EINVAL,
                             e != hipSuccess ? hipGetErrorString(e) : "paged_decode_static: no address for the static scratch");
        }
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return MI355_OK;
}

extern "C" int mi355_paged_decode_fwd_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                             const int32_t* block_tables, int64_t bt_row_stride,
                                             const int32_t* context_lens, const float* k_scale,
                                             const float* v_scale, int B, int Hq, int Hkv, int D, int block_size,
                                             int64_t num_blocks, int max_ctx, float softmax_scale, int kv_dtype,
                                             void* stream) {
    return decode_common(q, k_cache, v_cache, out, block_tables, bt_row_stride, context_lens, k_scale, v_scale, nullptr,
                         kStaticScratchBytes, true, B, Hq, Hkv, D, block_size, num_blocks, max_ctx, softmax_scale,
                         kv_dtype, stream);
}
