// FlashAttention-style prefill forward for gfx950 (bf16, MFMA 32x32x16).
//
// One workgroup = 8 wavefronts (two per SIMD, one workgroup per CU) = one tile of 256 queries
// of one (batch, head); each wavefront owns 32 query rows.  K/V tiles of 64 keys are double-buffered in
// LDS and shared by the eight wavefronts (256 queries per loaded tile: half the L2->LDS
// traffic per MFMA of a 128-query workgroup, worth +1.5 %).  Per wavefront and KV tile:
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
//
// Tiles travel global -> LDS with global_load_lds_dwordx4 (no staging registers).
// Such a load writes 1 KiB of consecutive LDS per wavefront, so rows cannot be
// padded; bank conflicts are avoided by an XOR swizzle instead: the 16-byte chunk
// c of row r is stored in slot c ^ swz(r), applied on the global-address side.
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"
#include "prefill_params.hpp"
#include "prefill_tile.hpp"

namespace mi355 {

constexpr int kPfWaves = 8;
constexpr int kBM = 256;   // queries per workgroup
constexpr int kBN = 64;    // keys per LDS tile


// PAGED: keys and values are read from a paged cache through a block table (16 rows per block, so
// every direct-to-LDS instruction -- 4, 8 or 16 whole rows -- stays inside one block and needs one
// table entry, a scalar load); queries and outputs are packed.
// Occupancy: at head_dim 64 the kernel is held to the registers of four wavefronts per SIMD (128; left alone the
// compiler takes 163 and a compute unit then holds ONE workgroup, whose barriers and waits nobody fills): two
// workgroups per compute unit, 7-8 % faster at throughput shapes and 14 % on short sequences, a handful of spilled
// registers outside the tile loop.  Head_dim 32 has two workgroups per compute unit as it is (117 registers; a third
// would need 85 and spills by the hundred: three to four times slower), head_dim 128 needs its 250.
template <int D, int MODE, bool PAGED = false>
__global__ __launch_bounds__(kPfWaves * 64, D == 64 ? 4 : 1) void prefill_fwd_kernel(PrefillParams p) {
    constexpr int NS = D / 16;                    // MFMA k-steps of K.Q^T
    constexpr int NDT = D / 32;                   // 32-row tiles of O^T
    constexpr int CPR = D / 8;                    // 16-byte chunks per row
    constexpr int kRow = D * 2;                   // bytes per LDS row
    constexpr int kTile = kBN * kRow;             // bytes per K (or V) tile
    constexpr int NT = kBN * CPR / 64;            // direct-to-LDS instructions per tile and tensor
    constexpr int NI = (NT + kPfWaves - 1) / kPfWaves;   // ... per wavefront (the last wavefronts may have none)

    // K/V tile buffers: tile t lives in buffer t % NB, and while tile t is computed tile t+1 is landing.  (Four buffers
    // with three tiles in flight were tried for head_dim 64 and 32, where a tile is only a few hundred cycles of work:
    // the larger LDS footprint leaves room for fewer workgroups per compute unit, and every shape but the smallest
    // launches ran 10-23 % slower.  The code below is written for any power of two.)
    constexpr int NB = 2;
    constexpr int kAhead = NB - 1;
    constexpr float kBias = 32.0f;             // first attempt: the weight of a score x (log2 domain) is 2^(x - kBias)
    constexpr float kUnderflow = 0x1p-92f;     // a final row sum below this may have lost terms
    constexpr float kOverflow = 0x1p40f;       // ... above this (or NaN) may have overflowed somewhere
    __shared__ __attribute__((aligned(1024))) unsigned char k_lds[NB * kTile];
    __shared__ __attribute__((aligned(1024))) unsigned char v_lds[NB * kTile];
    // Staging of the query rows on their way in and of the output rows on their way out, one private slab per
    // wavefront (32 rows of D bf16, rows padded by 16 bytes): fragments and accumulators hold a query per lane,
    // so direct accesses would touch 16- or 8-byte pieces of 32 different rows per instruction; through the
    // slab every global instruction moves whole 2*D-byte rows (+2.4 % for the stores alone at D = 128).
    constexpr int kORow = D * 2 + 16;
    __shared__ __attribute__((aligned(16))) unsigned char o_lds[kPfWaves * 32 * kORow];

    // Logical order: pair fastest, then the query heads of one kv head, then kv head, then batch.  The workgroups
    // that stream the same K/V -- the pairs and query heads of one kv head -- form a chunk of that order and run on
    // one XCD.
    const int lid = xcd_chunked_id(blockIdx.x, gridDim.x, p.n_pairs * (p.Hq / p.Hkv));
    const int split = blockIdx.y;                    // share of the keys this workgroup serves (gridDim.y = n_split)
    const int pair0 = lid % p.n_pairs;
    const int h = (lid / p.n_pairs) % p.Hq;
    const int b = lid / (p.n_pairs * p.Hq);
    const int hk = h / (p.Hq / p.Hkv);

    int sq, sk;
    const __bf16 *qb, *kb, *vb;
    __bf16* ob;
    float* lb;
    int64_t part_row0 = (int64_t)b * p.Sq;          // first row of this sequence in the partial buffers
    if (PAGED || p.cu_q) part_row0 = p.cu_q[b];
    if constexpr (PAGED) {
        const int q_start = p.cu_q[b];
        sq = p.cu_q[b + 1] - q_start;
        sk = min(p.ctx_lens[b], 16 * p.max_blocks);      // a length beyond what the table row addresses is cut, never chased
        qb = p.q + (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
        kb = vb = nullptr;
        ob = p.out + (int64_t)q_start * p.os[2] + (int64_t)h * p.os[1];
        lb = nullptr;
    } else if (p.cu_q) {
        const int q_start = p.cu_q[b], k_start = p.cu_k[b];
        sq = p.cu_q[b + 1] - q_start;
        sk = p.cu_k[b + 1] - k_start;
        qb = p.q + (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
        kb = p.k + (int64_t)k_start * p.ks[2] + (int64_t)hk * p.ks[1];
        vb = p.v + (int64_t)k_start * p.vs[2] + (int64_t)hk * p.vs[1];
        ob = p.out + (int64_t)q_start * p.os[2] + (int64_t)h * p.os[1];
        lb = p.lse ? p.lse + q_start + (int64_t)h * p.ls[1] : nullptr;
    } else {
        sq = p.Sq;
        sk = p.Sk;
        qb = p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[1];
        kb = p.k + (int64_t)b * p.ks[0] + (int64_t)hk * p.ks[1];
        vb = p.v + (int64_t)b * p.vs[0] + (int64_t)hk * p.vs[1];
        ob = p.out + (int64_t)b * p.os[0] + (int64_t)h * p.os[1];
        lb = p.lse ? p.lse + (int64_t)b * p.ls[0] + (int64_t)h * p.ls[1] : nullptr;
    }
    // Causal work grows with the query-tile index, so a workgroup takes the tiles
    // (nq-1-pair) and (pair): every workgroup of a sequence then carries the same load.
    // (A launch that would leave compute units without a workgroup deals single query tiles instead, heaviest first:
    // p.n_pairs then counts tiles.)
    const int nq = (sq + kBM - 1) / kBM;
    const bool singles = p.single_tiles != 0;
    if ((singles ? pair0 : 2 * pair0) >= nq) return;         // (a sequence without keys still gets its rows written: no key kept -> NaN)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;          // query column of S^T / O^T, key row of K, d row of V^T
    const int kg = lane >> 5;         // 0..1

    constexpr bool causal = MODE == MI355_MASK_CAUSAL;
    constexpr bool boolmask = MODE == MI355_MASK_BOOL;
    const int coff = sk - sq;                          // bottom-right aligned causal diagonal

    // ---- tile loader: wavefront w, instruction j covers LDS chunks (w*NI + j)*64 .. +63 -----
    // lane -> (row, slot); it fetches global chunk slot ^ swz(row) of that row.  The per-lane
    // part of the address is a constant byte offset; the tile's first row is a scalar base.
    int ld_row[NI], ld_col[NI];
    uint32_t k_voff[NI], v_voff[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int idx = (wave * NI + j) * 64 + lane;
        ld_row[j] = idx / CPR;
        ld_col[j] = ((idx % CPR) ^ swz<D>(idx / CPR)) * 16;      // byte offset inside the row
        k_voff[j] = (uint32_t)(ld_row[j] * (int)p.ks[2] * 2 + ld_col[j]);
        v_voff[j] = (uint32_t)(ld_row[j] * (int)p.vs[2] * 2 + ld_col[j]);
    }
    const bool ld_active = wave * NI < NT;
    auto issue_tile = [&](int tile, int buf) {
        if (!ld_active) return;
        if constexpr (PAGED) {
            const uint32_t kdst = __builtin_amdgcn_readfirstlane(lds_address(k_lds + buf * kTile + wave * NI * 1024));
            const uint32_t vdst = __builtin_amdgcn_readfirstlane(lds_address(v_lds + buf * kTile + wave * NI * 1024));
            const int last = sk - 1, last_b = last >> 4;            // last valid key and its logical block
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                // the instruction's rows (64 / CPR of them, aligned) lie in logical block bidx of the sequence;
                // rows past the last key re-read the last key's row (finite; their scores are masked), and a
                // block past the last one is never looked up (its table entry need not exist)
                int bidx = tile * (kBN / 16) + (((wave * NI + j) * (64 / CPR)) >> 4);
                int rin = ld_row[j] & 15;
                if (bidx > last_b) {
                    bidx = last_b;
                    rin = last & 15;
                } else if (bidx == last_b) {
                    rin = min(rin, last & 15);
                }
                int phys = p.block_table[(int64_t)b * p.table_stride + bidx];
                phys = min(max(phys, 0), p.num_blocks - 1);           // a corrupt table cannot leave the pool
                const int64_t base = ((int64_t)phys * p.Hkv + hk) * (16 * D);
                const uint32_t voff = (uint32_t)(rin * kRow + ld_col[j]);
                dma_to_lds_16(reinterpret_cast<const unsigned char*>(p.k + base), voff, kdst + j * 1024);
                dma_to_lds_16(reinterpret_cast<const unsigned char*>(p.v + base), voff, vdst + j * 1024);
            }
            return;
        }
        const unsigned char* kbase = reinterpret_cast<const unsigned char*>(kb + (int64_t)tile * kBN * p.ks[2]);
        const unsigned char* vbase = reinterpret_cast<const unsigned char*>(vb + (int64_t)tile * kBN * p.vs[2]);
        const uint32_t kdst = __builtin_amdgcn_readfirstlane(lds_address(k_lds + buf * kTile + wave * NI * 1024));
        const uint32_t vdst = __builtin_amdgcn_readfirstlane(lds_address(v_lds + buf * kTile + wave * NI * 1024));
        if (tile * kBN + kBN <= sk) {
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                dma_to_lds_16(kbase, k_voff[j], kdst + j * 1024);
                dma_to_lds_16(vbase, v_voff[j], vdst + j * 1024);
            }
        } else {
            // last, partial tile: rows past the end re-read the last row (finite; their scores are masked)
            const int last = sk - 1 - tile * kBN;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int row = min(ld_row[j], last);
                dma_to_lds_16(kbase, (uint32_t)(row * (int)p.ks[2] * 2 + ld_col[j]), kdst + j * 1024);
                dma_to_lds_16(vbase, (uint32_t)(row * (int)p.vs[2] * 2 + ld_col[j]), vdst + j * 1024);
            }
        }
    };

    // ---- per-lane LDS read offsets (tile- and buffer-independent parts) ------
    // K fragment of step s, key row 32t + n: logical chunk 2s + kg -> slot (2s + kg) ^ swz(n)
    // (swz depends on the row only through bits that 32t does not touch).
    int k_off[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) k_off[s] = n * kRow + (((2 * s + kg) ^ swz<D>(n)) << 4);
    // V^T fragment of O^T tile dt: source lane s16 of 16-lane group g16 addresses key row
    // 4*(g16>>1) + (s16>>2) (+8 for the upper half), d = 32dt + 16*(g16&1) + 4*(s16&3) .. +3
    const int g16 = lane >> 4, s16 = lane & 15;
    int v_off[2][NDT];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const int row = 4 * (g16 >> 1) + (s16 >> 2) + 8 * e;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const int d = 32 * dt + 16 * (g16 & 1) + 4 * (s16 & 3);
            v_off[e][dt] = row * kRow + ((((d >> 3)) ^ swz<D>(row)) << 4) + (d & 7) * 2;
        }
    }
    const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};

    // The grid holds n_pairs workgroups per (batch, head), sized from the caller's Sq_max.  A packed sequence that is
    // longer than that promise is still computed in full: its workgroups walk on through the remaining tile pairs
    // (with a correct Sq_max this loop runs once).
    for (int pair = pair0; (singles ? pair : 2 * pair) < nq; pair += p.n_pairs)
    for (int half = 0; half < (singles ? 1 : 2); ++half) {
        const int qtile = half == 0 ? nq - 1 - pair : pair;
        if (half == 1 && qtile == nq - 1 - pair) break;         // odd tile count: the middle tile has no partner
        const int q0 = qtile * kBM;
        const int qw0 = q0 + 32 * wave;                    // first query of this wavefront
        const int qi = qw0 + n;                            // this lane's query
        const bool q_ok = qi < sq;

        int kv_end = sk;
        if (causal) kv_end = max(0, min(sk, min(sq, q0 + kBM) + coff));
        const int n_tiles = (kv_end + kBN - 1) / kBN;
        int t0 = 0, t1 = n_tiles;                  // this workgroup's tiles
        if (p.n_split > 1) {
            const int per = (n_tiles + p.n_split - 1) / p.n_split;
            t0 = min(n_tiles, split * per);
            t1 = min(n_tiles, t0 + per);
        }

        // the first K/V tiles are requested before the query rows, so that the latencies overlap
        __syncthreads();                     // the previous query tile's readers are done with the LDS buffers
#pragma unroll
        for (int i = 0; i < kAhead; ++i)
            if (t0 + i < t1) issue_tile(t0 + i, (t0 + i) & (NB - 1));

        // ---- Q^T fragments: step s covers d = 16s + 8kg + j ----------------------
        // rows come in whole (CPR lanes per row) and go through the wavefront's slab (private, and LDS operations
        // of a wavefront execute in order: no barrier); rows past the end of the sequence are zero
        bf16x8 qf[NS];
        {
            unsigned char* slab = o_lds + wave * (32 * kORow);
            constexpr int kRowsPerPass = 64 / CPR;
            const int c = lane % CPR, r0 = lane / CPR;
            u32x4 rows[32 / kRowsPerPass];
#pragma unroll
            for (int i = 0; i < 32 / kRowsPerPass; ++i) {
                const int r = i * kRowsPerPass + r0;
                rows[i] = u32x4{0u, 0u, 0u, 0u};
                if (qw0 + r < sq) rows[i] = *reinterpret_cast<const u32x4*>(qb + (int64_t)(qw0 + r) * p.qs[2] + c * 8);
            }
#pragma unroll
            for (int i = 0; i < 32 / kRowsPerPass; ++i)
                *reinterpret_cast<u32x4*>(slab + (i * kRowsPerPass + r0) * kORow + c * 16) = rows[i];
#pragma unroll
            for (int s = 0; s < NS; ++s)
                qf[s] = as_bf16x8(*reinterpret_cast<const u32x4*>(slab + n * kORow + (16 * s + 8 * kg) * 2));
        }

        f32x16 o[NDT];
#pragma unroll
        for (int i = 0; i < NDT; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) o[i][j] = 0.f;
        // m_ref: exponent reference of this lane's query row, in RAW score units (>= row max - slack);
        // neg_ref = -m_ref * scale_log2 is the additive term of the exponent
        float m_ref = -INFINITY, neg_ref = 0.f, l_run = 0.f;
        bool redo = false;                   // a row sum overflowed on the way (first attempt)

        const uint8_t* mrow = nullptr;
        if (boolmask)     // rows of padded query lanes alias the last real row (their results are never stored)
            mrow = p.mask + (int64_t)b * p.ms[0] + (int64_t)h * p.ms[1] + (int64_t)min(qi, sq - 1) * p.ms[2];

        // Leading tiles whose keys are all visible to every query of this wavefront need no
        // mask code at all; only the tiles on the diagonal / at the ragged end take the masked path.
        int n_plain = sk / kBN;
        if (causal) n_plain = min(n_plain, max(0, qw0 + coff + 1) / kBN);
        if (boolmask) n_plain = 0;
        n_plain = min(n_plain, n_tiles);

        f32x16 s_acc[2];
        float mx = 0.f;
        // the per-lane read offsets carry the LDS buffer of the tile being read
        const auto set_buf = [&](int buf) {
#pragma unroll
            for (int s = 0; s < NS; ++s) k_off[s] = (k_off[s] & (kTile - 1)) | (buf * kTile);
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) v_off[e][dt] = (v_off[e][dt] & (kTile - 1)) | (buf * kTile);
        };
        int cur_tile = t0;                   // the tile the offsets point at
        const auto flip = [&]() {            // on to the next tile's buffer
            ++cur_tile;
            if constexpr (NB == 2) {
#pragma unroll
                for (int s = 0; s < NS; ++s) k_off[s] ^= kTile;
#pragma unroll
                for (int e = 0; e < 2; ++e)
#pragma unroll
                    for (int dt = 0; dt < NDT; ++dt) v_off[e][dt] ^= kTile;
            } else {
                set_buf(cur_tile & (NB - 1));
            }
        };

        // First half of a KV tile: wait for it, start the next one, S^T = K . Q^T, mask, row max.
        // Returns false when the whole tile lies above this wavefront's diagonal (nothing to add).
        auto head = [&](auto masked_c, auto track_c, int tile) -> bool {
            constexpr bool MASKED = decltype(masked_c)::value;
            constexpr bool TRACK = decltype(track_c)::value;
            // this wavefront's share of tile `tile` has landed: its loads are older than those of the tiles requested
            // after it (2 * NI instructions each), which may stay in flight
            if constexpr (NB == 2) {
                wait_vmcnt<0>();
            } else {
                const int younger = min(kAhead - 1, t1 - 1 - tile);
                if (younger >= 2) wait_vmcnt<4 * NI>();
                else if (younger == 1) wait_vmcnt<2 * NI>();
                else wait_vmcnt<0>();
            }
            __syncthreads();                 // ... and everybody's; also: all are done reading the buffer of the tile before

            // The loads of the tile that takes that buffer go out first: the work of kAhead tiles hides their latency.
            if (tile + kAhead < t1) issue_tile(tile + kAhead, (tile + kAhead) & (NB - 1));

            const int k0 = tile * kBN;
            if (causal && MASKED && k0 > qw0 + 31 + coff) return false;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int j = 0; j < 16; ++j) s_acc[t][j] = 0.f;
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const u32x4 kf = *reinterpret_cast<const u32x4*>(k_lds + t * 32 * kRow + k_off[s]);
                    s_acc[t] = mfma32(as_bf16x8(kf), qf[s], s_acc[t]);
                }
            }
            // element (t,i) of this lane: key k0 + 32t + 8(i/4) + 4kg + i%4, query qi
            if constexpr (MASKED) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int key = k0 + 32 * t + 8 * (i >> 2) + 4 * kg + (i & 3);
                        bool keep = key < sk;
                        if constexpr (causal) keep = keep & (key <= qi + coff);
                        // unconditional, clamped byte load: no divergent control flow around the select
                        if constexpr (boolmask) keep = keep & (mrow[min(key, sk - 1)] != 0);
                        s_acc[t][i] = keep ? s_acc[t][i] : -INFINITY;
                    }
            }
            if constexpr (TRACK) {
                mx = s_acc[0][0];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_acc[t][i]);
                mx = xor32_max(mx);
            }
            return true;
        };

        // Second half: P = 2^(S*scale - ref), row sums, O^T += V^T . P^T.
        // 16-key slice u: P^T fragment = accumulator registers 8(u%2).. of tile u/2, i.e.
        // keys 16u + 4kg + (0..3) and 16u + 8 + 4kg + (0..3); the V^T read mirrors it.
        // The row sum adds the bf16-rounded weights, i.e. exactly what multiplies V.
        auto accumulate = [&]() {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int t = u >> 1, e0 = 8 * (u & 1);
                u32x4 pw;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float a0 = fast_exp2(fmaf(s_acc[t][e0 + 2 * w], p.scale_log2, neg_ref));
                    const float a1 = fast_exp2(fmaf(s_acc[t][e0 + 2 * w + 1], p.scale_log2, neg_ref));
                    pw[w] = pack_bf16(a0, a1);
                    const uint32_t pwv = pw[w];
                    l_run = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pwv), ones2, l_run, false);
                }
                const bf16x8 pf = as_bf16x8(pw);
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    const i16x4 lo = lds_read_tr16(v_lds + 16 * u * kRow + v_off[0][dt]);
                    const i16x4 hi = lds_read_tr16(v_lds + 16 * u * kRow + v_off[1][dt]);
                    o[dt] = mfma32(join_bf16x8(lo, hi), pf, o[dt]);
                }
            }
        };

        // Lazy rescaling: the exponent reference m_ref only moves when some row's maximum
        // outgrows it by more than 2^kSlack; until then weights are at most 2^kSlack (exact in
        // the fp32 sums, harmless in bf16) and the O accumulators need no per-tile multiply.
        // The fast loop below therefore only accumulates in place; a tile that needs the
        // reference moved leaves it, rescales, and re-enters.
        constexpr float kSlack = 8.0f;
        // The first attempt at a query tile does not look at row maxima at all (MODE NONE / CAUSAL): the reference is
        // preset to 0 (weights 2^(x - kBias), x the score in the log2 domain), and what is watched is the row SUM: a
        // partial sum that reaches 2 moves the row's reference up by the exponent of its sum, an exact rescaling by a
        // power of two.  Scores between -60 and +72 binary orders need nothing else.  A row whose final sum left
        // [2^-92, 2^40] (or is NaN) may have lost terms: the workgroup then runs the query tile again with the
        // reference tracked from the row maxima (below).  What this saves is the maximum itself: 32 v_max and a
        // cross-lane step per tile, a tenth of the vector work, which is what bounds head_dim 64 and 32.
        auto run_tiles_preset = [&](auto masked_c, int tile, const int tile_end) {
            while (tile < tile_end) {
                if (head(masked_c, std::false_type{}, tile)) {
                    accumulate();
                    if (__builtin_amdgcn_ballot_w64(!(l_run < 2.0f)) != 0) {
                        const float l = xor32_sum(l_run);                  // the row's sum (its keys are dealt to two lanes)
                        if (!(l <= kOverflow)) redo = true;
                        const int expo = (int)((__builtin_bit_cast(uint32_t, l) >> 23) & 0xffu) - 127;
                        const int k = min(max(expo + (int)kBias, 0), 126);
                        const float alpha = __builtin_bit_cast(float, (uint32_t)(127 - k) << 23);      // 2^-k
                        neg_ref -= (float)k;
                        l_run *= alpha;
#pragma unroll
                        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                            for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
                    }
                }
                flip();
                ++tile;
            }
        };
        auto run_tiles = [&](auto masked_c, int tile, const int tile_end) {
            for (;;) {
                bool pending = false;
                while (tile < tile_end) {
                    if (head(masked_c, std::true_type{}, tile)) {
                        const bool grow = !((mx - m_ref) * p.scale_log2 <= kSlack);   // also true while m_ref = -inf
                        if (__builtin_amdgcn_ballot_w64(grow) != 0) {
                            pending = true;
                            break;
                        }
                        accumulate();
                    }
                    flip();
                    ++tile;
                }
                if (!pending) break;
                const float m_new = fmaxf(m_ref, mx);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;    // row with no key yet: keep p = 0, not NaN
                const float alpha = fast_exp2((m_ref - m_use) * p.scale_log2);
                m_ref = m_new;
                neg_ref = -m_use * p.scale_log2;
                l_run *= alpha;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
                accumulate();
                flip();
                ++tile;
            }
        };

        bool tracked = boolmask;             // explicit masks: tracked from the start
        if constexpr (!boolmask) {
            neg_ref = -kBias;
            set_buf(t0 & (NB - 1));          // the offsets start at the first tile's buffer
            cur_tile = t0;
            run_tiles_preset(std::false_type{}, t0, min(n_plain, t1));
            run_tiles_preset(std::true_type{}, max(n_plain, t0), t1);
            const float l = xor32_sum(l_run);
            // (a query that sees none of this share's keys -- causal with fewer keys than queries, or a share of split
            // keys that lies past its diagonal -- has a sum of zero by right)
            const int k_first = t0 * kBN;
            const bool sees = t0 < t1 && k_first < sk && (!causal || k_first <= qi + coff);
            const bool bad = redo || (sees && !(l >= kUnderflow)) || !(l <= kOverflow);
            // the workgroup meets (everybody is done with the K/V buffers) and votes
            if (__syncthreads_or(bad ? 1 : 0)) {
                tracked = true;
#pragma unroll
                for (int i = 0; i < kAhead; ++i)
                    if (t0 + i < t1) issue_tile(t0 + i, (t0 + i) & (NB - 1));
#pragma unroll
                for (int i = 0; i < NDT; ++i)
#pragma unroll
                    for (int j = 0; j < 16; ++j) o[i][j] = 0.f;
                m_ref = -INFINITY;
                neg_ref = 0.f;
                l_run = 0.f;
            }
        }
        if (tracked) {
            set_buf(t0 & (NB - 1));
            cur_tile = t0;
            run_tiles(std::false_type{}, t0, min(n_plain, t1));
            run_tiles(std::true_type{}, max(n_plain, t0), t1);
        }

        // ---- normalise and store: lane owns query qi, d = 32dt + 8(i/4) + 4kg + i%4 ---
        l_run = xor32_sum(l_run);
        if (p.n_split > 1) {
            // partial result of this share of the keys: normalised fp32 rows and their log-sum-exp (-inf and
            // zeros when the share kept no key for the row); the merge kernel weighs them
            const float inv_p = l_run > 0.f ? 1.0f / l_run : 0.f;
            if (q_ok) {
                const int64_t prow = ((int64_t)split * p.Hq + h) * p.part_rows + part_row0 + qi;
                if (kg == 0)
                    p.part_lse[prow] = l_run > 0.f ? 0.69314718056f * (__log2f(l_run) - neg_ref) : -INFINITY;
                float* po = p.part_o + prow * D + 4 * kg;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        f32x4 w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = o[dt][4 * g + e] * inv_p;
                        *reinterpret_cast<f32x4*>(po + 32 * dt + 8 * g) = w;
                    }
            }
            continue;
        }
        const float inv = 1.0f / l_run;          // l == 0 (no key kept) -> NaN row, like the reference softmax
        // sum_j exp(scale * s_j) = 2^(-neg_ref) * l  ->  lse = ln2 * (log2 l - neg_ref)
        if (lb && q_ok && kg == 0)
            lb[qi] = l_run > 0.f ? 0.69314718056f * (__log2f(l_run) - neg_ref) : -INFINITY;
        {
            // (the slab is private to the wavefront and LDS operations of a wavefront execute in order: no barrier)
            unsigned char* slab = o_lds + wave * (32 * kORow);
            unsigned char* mine = slab + n * kORow + 8 * kg;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = pack_bf16(o[dt][4 * g + 0] * inv, o[dt][4 * g + 1] * inv);
                    w[1] = pack_bf16(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
                    *reinterpret_cast<u32x2*>(mine + (32 * dt + 8 * g) * 2) = w;
                }
            // read back row-wise: 16-byte chunk c of row r, CPR lanes per row
            constexpr int kRowsPerPass = 64 / CPR;
            const int c = lane % CPR, r0 = lane / CPR;
#pragma unroll
            for (int i = 0; i < 32 / kRowsPerPass; ++i) {
                const int r = i * kRowsPerPass + r0;
                const u32x4 w = *reinterpret_cast<const u32x4*>(slab + r * kORow + c * 16);
                if (qw0 + r < sq) *reinterpret_cast<u32x4*>(ob + (int64_t)(qw0 + r) * p.os[2] + c * 8) = w;
            }
        }
    }
}

// Pairs of query tiles carry equal causal work, but a launch with fewer pairs than the GPU can hold at once (two
// workgroups per compute unit) leaves compute units idle and makes every workgroup walk two tiles: such a launch
// deals single tiles instead.
static PrefillParams with_units(const PrefillParams& p0) {
    PrefillParams p = p0;
    p.single_tiles = 0;
    int dev = 0, n_cu = 0;
    if (p.n_qtiles > 1 && hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) {
        const int64_t wgs = (int64_t)p.n_pairs * p.Hq * p.B * (p.n_split > 1 ? p.n_split : 1);
        if (wgs < 2 * (int64_t)n_cu) {
            p.single_tiles = 1;
            p.n_pairs = p.n_qtiles;
        }
    }
    return p;
}

template <int D>
static int launch_prefill(const PrefillParams& p0, hipStream_t stream) {
    const PrefillParams p = with_units(p0);
    // one workgroup per PAIR of query tiles (or per tile), 1-D in x (see the id remap); y = share of the keys
    dim3 grid((unsigned)(p.n_pairs * p.Hq * p.B), (unsigned)(p.n_split > 1 ? p.n_split : 1));
    dim3 block(kPfWaves * 64);
    if (p.mask_mode == MI355_MASK_CAUSAL)
        hipLaunchKernelGGL((prefill_fwd_kernel<D, MI355_MASK_CAUSAL>), grid, block, 0, stream, p);
    else if (p.mask_mode == MI355_MASK_BOOL)
        hipLaunchKernelGGL((prefill_fwd_kernel<D, MI355_MASK_BOOL>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((prefill_fwd_kernel<D, MI355_MASK_NONE>), grid, block, 0, stream, p);
    return (int)hipGetLastError();
}

// Merge of the split-key partials: one wavefront per (query row, head).
//   out = sum_c w_c O_c / sum_c w_c,  w_c = exp(lse_c - max_c lse_c);  no share kept a key -> NaN, like the reference
struct MergeParams {
    const float* part_o;
    const float* part_lse;
    __bf16* out;
    int64_t os[3];
    int64_t part_rows;
    int n_split, Hq, D, Sq_dense;        // Sq_dense: rows per batch entry of the dense layout, 0 = packed
};
// One (query row, head) per D/4 lanes: a lane owns four adjacent d of the row (16-byte loads of the partial rows, an
// 8-byte store), and the partial rows of up to eight shares are in flight together.
__global__ __launch_bounds__(256) void prefill_merge_kernel(MergeParams p) {
    const int lanes_per_row = p.D / 4, rows_per_wave = 64 / lanes_per_row;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t item = wave * rows_per_wave + lane / lanes_per_row;
    if (item >= p.part_rows * p.Hq) return;
    const int d = 4 * (lane % lanes_per_row);
    const int h = (int)(item % p.Hq);
    const int64_t row = item / p.Hq;
    const int64_t share_stride = (int64_t)p.Hq * p.part_rows;          // rows from one share to the next
    const int64_t prow0 = (int64_t)h * p.part_rows + row;
    float m = -INFINITY;
    for (int c = 0; c < p.n_split; ++c) m = fmaxf(m, p.part_lse[prow0 + c * share_stride]);
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int c0 = 0; c0 < p.n_split; c0 += 8) {
        float wgt[8];
        f32x4 part[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t prow = prow0 + (int64_t)min(c0 + i, p.n_split - 1) * share_stride;
            const float l = p.part_lse[prow];
            // (a share that kept no key for the row has -inf here, and its partial row may never have been written)
            wgt[i] = c0 + i < p.n_split && l != -INFINITY ? __expf(l - m) : 0.f;
            part[i] = wgt[i] != 0.f ? *reinterpret_cast<const f32x4*>(p.part_o + prow * p.D + d) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (wgt[i] != 0.f) {
#pragma unroll
                for (int e = 0; e < 4; ++e) num[e] += wgt[i] * part[i][e];
                den += wgt[i];
            }
        }
    }
    __bf16* dst = p.Sq_dense ? p.out + (row / p.Sq_dense) * p.os[0] + (int64_t)h * p.os[1] + (row % p.Sq_dense) * p.os[2]
                             : p.out + row * p.os[2] + (int64_t)h * p.os[1];
    const float none = __builtin_nanf("");
    u32x2 packed;
    packed[0] = m == -INFINITY ? pack_bf16(none, none) : pack_bf16(num[0] / den, num[1] / den);
    packed[1] = m == -INFINITY ? pack_bf16(none, none) : pack_bf16(num[2] / den, num[3] / den);
    *reinterpret_cast<u32x2*>(dst + d) = packed;
}

static int launch_merge(const PrefillParams& p, int D, hipStream_t stream) {
    MergeParams m;
    m.part_o = p.part_o;
    m.part_lse = p.part_lse;
    m.out = p.out;
    for (int i = 0; i < 3; ++i) m.os[i] = p.os[i];
    m.part_rows = p.part_rows;
    m.n_split = p.n_split;
    m.Hq = p.Hq;
    m.D = D;
    m.Sq_dense = (p.cu_q || p.block_table) ? 0 : p.Sq;
    const int64_t per_wg = 4 * (64 / (D / 4));                  // (row, head) items per workgroup of four wavefronts
    const int64_t wgs = (p.part_rows * p.Hq + per_wg - 1) / per_wg;
    if (wgs > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(prefill_merge_kernel, dim3((unsigned)wgs), dim3(256), 0, stream, m);
    return (int)hipGetLastError();
}

template <int D>
static int launch_prefill_paged(const PrefillParams& p0, hipStream_t stream) {
    const PrefillParams p = with_units(p0);
    dim3 grid((unsigned)(p.n_pairs * p.Hq * p.B), (unsigned)(p.n_split > 1 ? p.n_split : 1));
    hipLaunchKernelGGL((prefill_fwd_kernel<D, MI355_MASK_CAUSAL, true>), grid, dim3(kPfWaves * 64), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace mi355

using namespace mi355;

static size_t split_workspace_bytes(int64_t total_q_rows, int Hq, int D, int n_split) {
    return (size_t)n_split * (size_t)Hq * (size_t)total_q_rows * (size_t)(D + 1) * sizeof(float);
}

// Split-key fields of the parameters (n_split <= 1: none).  `expected_rows` >= 0: what total_q_rows must equal.
static int set_split(PrefillParams& p, int D, int n_split, int64_t total_q_rows, void* workspace, size_t workspace_bytes,
                     int64_t expected_rows) {
    p.n_split = 1;
    p.part_o = nullptr;
    p.part_lse = nullptr;
    p.part_rows = 0;
    if (n_split <= 1) return 0;
    if (n_split > 64) return set_error(MI355_EINVAL, "prefill: n_split must be at most 64");
    if (total_q_rows <= 0 || (expected_rows >= 0 && total_q_rows != expected_rows))
        return set_error(MI355_EINVAL, "prefill: total_q_rows must be the number of query rows (B * Sq, or the packed total)");
    if (!workspace || ((uintptr_t)workspace & 15))
        return set_error(MI355_EINVAL, "prefill: split keys need a 16-byte aligned workspace");
    if (workspace_bytes < split_workspace_bytes(total_q_rows, p.Hq, D, n_split))
        return set_error(MI355_EWORKSPACE, "prefill: workspace smaller than mi355_prefill_splitkv_workspace_bytes()");
    p.n_split = n_split;
    p.part_rows = total_q_rows;
    p.part_o = (float*)workspace;
    p.part_lse = p.part_o + (size_t)n_split * p.Hq * total_q_rows * D;
    return 0;
}

static int prefill_common(const void* q, const void* k, const void* v, void* out, const int64_t q_strides[3],
                          const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const uint8_t* mask,
                          const int64_t mask_strides[3], int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                          float softmax_scale, int mask_mode, int dtype, float* lse, const int64_t* lse_strides,
                          void* stream, int n_split = 1, int64_t total_q_rows = 0, void* workspace = nullptr,
                          size_t workspace_bytes = 0) {
    if (!q || !k || !v || !out || !q_strides || !k_strides || !v_strides || !o_strides)
        return set_error(MI355_EINVAL, "prefill: null pointer argument");
    if (dtype != MI355_BF16) return set_error(MI355_EDTYPE, "prefill: dtype must be MI355_BF16");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq_max <= 0 || Sk_max <= 0)
        return set_error(MI355_EINVAL, "prefill: B, Hq, Hkv, Sq_max and Sk_max must be positive");
    if (Hq % Hkv != 0) return set_error(MI355_EINVAL, "prefill: Hq must be a multiple of Hkv");
    if (!(D == 128 || D == 64 || D == 32)) return set_error(MI355_EINVAL, "prefill: head_dim must be 32, 64 or 128");
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
    if (k_strides[2] <= 0 || v_strides[2] <= 0 || k_strides[2] >= (1 << 24) || v_strides[2] >= (1 << 24))
        return set_error(MI355_EINVAL, "prefill: k/v row strides must be positive and below 2^24 elements");
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
    p.lse = lse;
    p.ls[0] = lse ? lse_strides[0] : 0;
    p.ls[1] = lse ? lse_strides[1] : 0;
    p.B = B;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.Sq = Sq_max;
    p.Sk = Sk_max;
    p.scale_log2 = softmax_scale * kLog2e;
    p.mask_mode = mask_mode;
    p.n_qtiles = (Sq_max + kBM - 1) / kBM;
    p.n_pairs = (p.n_qtiles + 1) / 2;
    p.single_tiles = 0;
    p.block_table = nullptr;
    p.ctx_lens = nullptr;
    p.table_stride = 0;
    p.num_blocks = 0;
    p.max_blocks = 0;
    if (int e = set_split(p, D, n_split, total_q_rows, workspace, workspace_bytes, cu_seqlens_q ? -1 : (int64_t)B * Sq_max))
        return e;
    if ((int64_t)p.n_pairs * Hq * B > 0x7fffffffLL) return set_error(MI355_EINVAL, "prefill: too many workgroups");

    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (p.n_split > 1) {
        if (D == 128 && mask_mode != MI355_MASK_BOOL && prefill_w64_takes(p)) rc = launch_prefill_w64(p, s);
        else rc = D == 128 ? launch_prefill<128>(p, s) : (D == 64 ? launch_prefill<64>(p, s) : launch_prefill<32>(p, s));
        if (rc == 0) rc = launch_merge(p, D, s);
        if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
        return MI355_OK;
    }
    // head_dim 128 without an explicit mask: the kernel with 64 queries per wavefront and a hand-scheduled tile loop
    if (D == 128 && mask_mode != MI355_MASK_BOOL && prefill_w64_takes(p)) rc = launch_prefill_w64(p, s);
    else rc = D == 128 ? launch_prefill<128>(p, s) : (D == 64 ? launch_prefill<64>(p, s) : launch_prefill<32>(p, s));
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" int mi355_prefill_fwd(const void* q, const void* k, const void* v, void* out,
                                 const int64_t q_strides[3], const int64_t k_strides[3],
                                 const int64_t v_strides[3], const int64_t o_strides[3],
                                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                 const uint8_t* mask, const int64_t mask_strides[3], int B, int Hq, int Hkv,
                                 int Sq_max, int Sk_max, int D, float softmax_scale, int mask_mode, int dtype,
                                 void* stream) {
    return prefill_common(q, k, v, out, q_strides, k_strides, v_strides, o_strides, cu_seqlens_q, cu_seqlens_k, mask,
                          mask_strides, B, Hq, Hkv, Sq_max, Sk_max, D, softmax_scale, mask_mode, dtype, nullptr, nullptr,
                          stream);
}

extern "C" int mi355_prefill_fwd_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                                     const int64_t q_strides[3], const int64_t k_strides[3],
                                     const int64_t v_strides[3], const int64_t o_strides[3],
                                     const int64_t lse_strides[2], const int32_t* cu_seqlens_q,
                                     const int32_t* cu_seqlens_k, int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                                     float softmax_scale, int mask_mode, int dtype, void* stream) {
    if (!lse || !lse_strides) return set_error(MI355_EINVAL, "prefill_fwd_lse: null lse argument");
    if (mask_mode == MI355_MASK_BOOL)
        return set_error(MI355_EINVAL, "prefill_fwd_lse: mask_mode must be MI355_MASK_NONE or MI355_MASK_CAUSAL");
    return prefill_common(q, k, v, out, q_strides, k_strides, v_strides, o_strides, cu_seqlens_q, cu_seqlens_k, nullptr,
                          nullptr, B, Hq, Hkv, Sq_max, Sk_max, D, softmax_scale, mask_mode, dtype, lse, lse_strides,
                          stream);
}

extern "C" int mi355_prefill_fwd_mask_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                                          const int64_t q_strides[3], const int64_t k_strides[3],
                                          const int64_t v_strides[3], const int64_t o_strides[3],
                                          const int64_t lse_strides[2], const uint8_t* mask,
                                          const int64_t mask_strides[3], int B, int Hq, int Hkv, int Sq, int Sk, int D,
                                          float softmax_scale, int dtype, void* stream) {
    if (!lse || !lse_strides) return set_error(MI355_EINVAL, "prefill_fwd_mask_lse: null lse argument");
    return prefill_common(q, k, v, out, q_strides, k_strides, v_strides, o_strides, nullptr, nullptr, mask, mask_strides,
                          B, Hq, Hkv, Sq, Sk, D, softmax_scale, MI355_MASK_BOOL, dtype, lse, lse_strides, stream);
}

extern "C" int mi355_prefill_paged_fwd(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       int64_t q_token_stride, int64_t out_token_stride, const int32_t* cu_seqlens_q,
                                       const int32_t* block_tables, int64_t table_stride, int64_t max_blocks,
                                       const int32_t* context_lens,
                                       int B, int Hq, int Hkv, int Sq_max, int D, int block_size, int64_t num_blocks,
                                       float softmax_scale, int kv_dtype, int n_split, int64_t total_q_rows,
                                       void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k_cache || !v_cache || !out || !cu_seqlens_q || !block_tables || !context_lens)
        return set_error(MI355_EINVAL, "prefill_paged: null pointer argument");
    if (kv_dtype != MI355_BF16) return set_error(MI355_EDTYPE, "prefill_paged: the cache must be MI355_BF16");
    if (block_size != 16) return set_error(MI355_EINVAL, "prefill_paged: block_size must be 16");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq_max <= 0) return set_error(MI355_EINVAL, "prefill_paged: B, Hq, Hkv and Sq_max must be positive");
    if (Hq % Hkv != 0) return set_error(MI355_EINVAL, "prefill_paged: Hq must be a multiple of Hkv");
    if (!(D == 128 || D == 64 || D == 32)) return set_error(MI355_EINVAL, "prefill_paged: head_dim must be 32, 64 or 128");
    if (num_blocks <= 0 || num_blocks > 0x7fffffffLL || table_stride <= 0)
        return set_error(MI355_EINVAL, "prefill_paged: num_blocks and table_stride must be positive");
    if (max_blocks <= 0 || max_blocks > table_stride || max_blocks > 0x7ffffff)
        return set_error(MI355_EINVAL, "prefill_paged: max_blocks must be in 1..table_stride");
    if ((q_token_stride | out_token_stride) & 7)
        return set_error(MI355_EINVAL, "prefill_paged: token strides must be multiples of 8 elements (16-byte rows)");
    if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
        return set_error(MI355_EINVAL, "prefill_paged: q, caches and out must be 16-byte aligned");
    PrefillParams p{};
    p.q = (const __bf16*)q;
    p.k = (const __bf16*)k_cache;
    p.v = (const __bf16*)v_cache;
    p.out = (__bf16*)out;
    p.qs[1] = D;
    p.qs[2] = q_token_stride;
    p.os[1] = D;
    p.os[2] = out_token_stride;
    p.ks[1] = p.vs[1] = 16 * D;
    p.ks[2] = p.vs[2] = D;
    p.cu_q = cu_seqlens_q;
    p.B = B;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.Sq = Sq_max;
    p.Sk = 0;
    p.scale_log2 = softmax_scale * kLog2e;
    p.mask_mode = MI355_MASK_CAUSAL;
    p.n_qtiles = (Sq_max + kBM - 1) / kBM;
    p.n_pairs = (p.n_qtiles + 1) / 2;
    p.single_tiles = 0;
    p.block_table = block_tables;
    p.ctx_lens = context_lens;
    p.table_stride = table_stride;
    p.num_blocks = (int)num_blocks;
    p.max_blocks = (int)max_blocks;
    if (int e = set_split(p, D, n_split, total_q_rows, workspace, workspace_bytes, -1)) return e;
    if ((int64_t)p.n_pairs * Hq * B > 0x7fffffffLL) return set_error(MI355_EINVAL, "prefill_paged: too many workgroups");
    hipStream_t s = (hipStream_t)stream;
    // head_dim 128: the kernel with 64 queries per wavefront, which reads the block table too
    int rc;
    if (D == 128 && prefill_w64_takes(p)) rc = launch_prefill_w64(p, s);
    else rc = D == 128 ? launch_prefill_paged<128>(p, s) : (D == 64 ? launch_prefill_paged<64>(p, s) : launch_prefill_paged<32>(p, s));
    if (rc == 0 && p.n_split > 1) rc = launch_merge(p, D, s);
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" size_t mi355_prefill_splitkv_workspace_bytes(int64_t total_q_rows, int Hq, int D, int n_split) {
    if (total_q_rows <= 0 || Hq <= 0 || D <= 0 || n_split <= 1) return 0;
    return split_workspace_bytes(total_q_rows, Hq, D, n_split);
}

// Cost model behind mi355_prefill_suggest_kv_splits, in microseconds, from timings on an MI355X (32 and 8 query
// heads, head_dim 128, 64..2048 query rows over 1.5K..32K keys): a workgroup spends about 1.5 us per K/V tile of 64
// keys (1.6 us in the split kernel) and 5 us per query tile outside the tile loop; the partial rows cost their bytes
// twice (written, then read by the merge) at about 2.5 TB/s, plus 8 us for the second launch.  Head_dim 128 runs on
// the persistent 64-query kernel, split or not, and has figures of its own (below).
extern "C" int mi355_prefill_suggest_kv_splits(int B, int Hq, int D, int Sq_max, int Sk_max, int64_t total_q_rows,
                                               int causal, int n_compute_units) {
    if (B <= 0 || Hq <= 0 || D <= 0 || Sq_max <= 0 || Sk_max <= 0 || total_q_rows <= 0) return 1;
    int n_cu = n_compute_units;
    if (n_cu <= 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
            return 1;
    }
    const int nq = (Sq_max + kBM - 1) / kBM, n_pairs = (nq + 1) / 2;
    const double over = causal && Sk_max > Sq_max ? Sk_max - Sq_max : 0;            // keys every query sees (causal)
    // K/V tiles of the heaviest single query tile and of the heaviest pair (causal: bottom-right diagonal)
    double keys_single = Sk_max, keys_pair = (nq >= 2 ? 2.0 : 1.0) * Sk_max;
    if (causal) {
        keys_single = over + Sq_max;
        keys_pair = nq >= 2 ? 2.0 * over + Sq_max + kBM : over + (Sq_max < kBM ? Sq_max : kBM);
        if (keys_single > Sk_max) keys_single = Sk_max;
        if (keys_pair > (nq >= 2 ? 2.0 : 1.0) * Sk_max) keys_pair = (nq >= 2 ? 2.0 : 1.0) * Sk_max;
    }
    const double halves = nq >= 2 ? 2.0 : 1.0;
    const auto rounds = [&](double wgs) { return (double)(int64_t)((wgs + n_cu - 1) / n_cu); };
    const auto partials = [&](int n) { return 8.0 + 2.0 * ((double)total_q_rows * Hq * (D + 1) * 4.0 * n) / 3.0e6; };
    double plain;
    int best_n = 1;
    static const int kCandidates[] = {2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64};
    if (D == 128) {
        // The persistent 64-query kernel serves both: a workgroup per query tile and share while there are compute units
        // for all of them, per pair of query tiles otherwise; 1.45 us per K/V tile on a busy GPU, 1.25 us when at most
        // three quarters of the compute units have a workgroup (the clock is higher then), 5 us per query tile around
        // the tile loop.
        const auto time_of = [&](int n) {
            const double singles = (double)nq * Hq * B * n;
            if (singles <= n_cu) return keys_single / n / kBN * (singles >= 0.75 * n_cu ? 1.45 : 1.25) + 5.0;
            const double wgs = (double)n_pairs * Hq * B * n;
            return rounds(wgs) * (keys_pair / n / kBN * (wgs >= 0.75 * n_cu ? 1.45 : 1.25) + 5.0 * halves);
        };
        plain = time_of(1);
        double best = plain * 0.85;                   // a split must win clearly
        for (int n : kCandidates) {
            if (keys_single / kBN / n < 2.0) break;   // at least two tiles per share and query tile
            const double t = time_of(n) + partials(n);
            if (t < best) {
                best = t;
                best_n = n;
            }
        }
        return best_n;
    }
    // the 8-wavefront kernel: a K/V tile of 64 keys takes a workgroup about 1.5 / 0.9 / 0.6 us at head_dim 128 / 64 / 32
    // (one 4096-token prompt with 16 heads of 64: 72 us unsplit, 84 us with two shares)
    const double tile_us = D >= 128 ? 1.5 : (D >= 64 ? 0.9 : 0.6);
    const double jobs = (double)n_pairs * Hq * B;
    const double tiles = keys_pair / kBN;
    plain = rounds(jobs) * (tiles * tile_us + 5.0 * halves);
    double best = plain * 0.85;                       // a split must win clearly
    for (int n : kCandidates) {
        if (tiles / n < 2.0 * halves) break;          // at least two tiles per share and query tile
        const double t = rounds(jobs * n) * (tiles / n * tile_us * 1.07 + 5.0 * halves) + partials(n);
        if (t < best) {
            best = t;
            best_n = n;
        }
    }
    return best_n;
}

extern "C" int mi355_prefill_fwd_splitkv(const void* q, const void* k, const void* v, void* out,
                                         const int64_t q_strides[3], const int64_t k_strides[3],
                                         const int64_t v_strides[3], const int64_t o_strides[3],
                                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int B, int Hq, int Hkv,
                                         int Sq_max, int Sk_max, int D, float softmax_scale, int mask_mode, int dtype,
                                         int n_split, int64_t total_q_rows, void* workspace, size_t workspace_bytes,
                                         void* stream) {
    if (mask_mode == MI355_MASK_BOOL)
        return set_error(MI355_EINVAL, "prefill_fwd_splitkv: mask_mode must be MI355_MASK_NONE or MI355_MASK_CAUSAL");
    if (n_split < 1) return set_error(MI355_EINVAL, "prefill_fwd_splitkv: n_split must be at least 1");
    return prefill_common(q, k, v, out, q_strides, k_strides, v_strides, o_strides, cu_seqlens_q, cu_seqlens_k, nullptr,
                          nullptr, B, Hq, Hkv, Sq_max, Sk_max, D, softmax_scale, mask_mode, dtype, nullptr, nullptr, stream,
                          n_split, total_q_rows, workspace, workspace_bytes);
}
