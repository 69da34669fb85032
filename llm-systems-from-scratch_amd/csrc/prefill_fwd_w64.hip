// Prefill forward for head_dim 128 (no mask or causal; optional log-sum-exp output; K/V packed, dense, or read through
// the block table of a paged cache), one wavefront per SIMD, 64 queries per wavefront.
//
// One workgroup = 4 wavefronts = one tile of 256 queries of one (batch, head); a wavefront owns 64 query rows as two
// column blocks A and B of 32.  It runs alone on its SIMD with the whole register file: the output accumulators
// (2 x 4 x 16 registers) live in AGPRs, everything the vector unit touches in VGPRs.  K/V tiles of 64 keys are
// double-buffered in LDS (direct-to-LDS loads, XOR-swizzled rows) and shared by the four wavefronts; every K
// fragment and every V^T fragment read from LDS feeds two MFMAs (one per column block).
//
// The mathematics is that of prefill_fwd.hip (transposed problem: S^T = K . Q^T, O^T += V^T . P^T, one query per
// lane, weights 2^(s * scale * log2(e) + nb) with one fma and one exp2 per score), with two changes that take vector
// work out of the loop: row sums come from a 16x16x32 MFMA against a 0/1 operand instead of adds, and the exponent
// reference is looked at only through the weights themselves.  A query tile starts with the reference preset to 0
// (nb = -32: the weight of a score x is 2^(x - 32)) and the loop watches for a row sum that reaches 2: only then
// ordinary code moves the reference of that row up, rescales and
// resumes.  For scores between -60 and +33 binary orders -- anything a trained model produces -- no row maximum is
// ever computed.  The loop notices a row sum >= 2 at the end of a tile: the tile is already accumulated (weights up
// to 2^40 are harmless in fp32 sums), the reference of every row is then moved by the exponent of its row sum, a
// rescaling by an exact power of two.  A row whose sum left [2^-92, 2^40] may have lost terms to underflow or
// overflow; the workgroup then computes the whole query tile again with references taken from the data.
// (Folding the scale into the Q fragments would save the fma too, but rounds Q once more: the error of a score then
// grows with the score, and outlier keys came out 3x less accurate.  Not done.)
//
// What differs most from prefill_fwd.hip is who schedules the instructions.  The loop over the K/V tiles of a query
// tile is hand-scheduled assembly (prefill_w64_asm.inc, written by gen_prefill_w64_loop.py: vector and LDS
// instructions sit at fixed places in the shadow of the MFMAs, which one wavefront per SIMD cannot leave to chance,
// and unmasked tiles run as a software pipeline across tiles); it covers unmasked tiles, the tiles on the causal
// diagonal and the tiles above it.  Ragged ends and the recomputation go through step_cxx below, ordinary HIP code
// on the same state.
//
// Between query tiles: a workgroup is persistent and works through (batch, head, query tile) jobs.  The 64 query rows
// of a wavefront reach its own part of LDS by direct-to-LDS loads (laid out like a K tile) and go from there into
// AGPRs once per job; the output rows are normalised 32 at a time and leave whole through the wavefront's own shares
// of the second K and V buffers, which nobody needs between the last tile of a job and the first boundary of the
// next.  The next job is worked out at the top of the current one, and its first requests (K[0], query rows, V[0],
// then K[1]) go out between the pieces of output work -- the query rows earlier still where a causal mask leaves
// wavefronts without work in the last tiles of a job: they request them then, also for the others.  No ordinary
// vector load sits in the job loop of the packed forms, so the only waits on memory are the ones written here (the
// compiler would add s_waitcnt vmcnt(0), which also waits for every request in flight, in front of the first use of
// a loaded register).  The block-table form has one such load, of the block ids of the next 64 tiles, directly in
// front of the tile loop: its wait lands where the first hand-over would wait for the same requests anyway.
//
// Hand-over protocol between the two (and between tiles), one "boundary" per tile t and wavefront: K[t] and V[t]
// live in LDS buffers t % 2.  When tile t starts, K[t] has landed and the workgroup has met since; K[t+1] and V[t]
// are in flight.  At boundary(t) the wavefront has read what it needs of K[t] and V[t-1]; it waits for its own
// shares of K[t+1] and V[t], meets the others at the barrier and requests K[t+2] and V[t+1] into the buffers just
// freed.  Only after boundary(t) may it read V[t].
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"
#include "prefill_params.hpp"
#include "prefill_tile.hpp"
#include "prefill_w64_asm.inc"

namespace mi355 {

// ---- the accumulators in the AGPRs, as ordinary code sees them ------------------------------------------------
// O^T (2 column blocks x 4 d-tiles x 16 registers) and the row sums (2 x 4 registers) stay in a[0:135] for a whole
// query tile.  This file is compiled with its builtin MFMAs in VGPR form (see build.py), so the compiler allocates no
// AGPR of its own, and every statement below names the registers it touches as clobbered.
template <int C, int DT>
__device__ __forceinline__ void acc_pv(bf16x8 vt, bf16x8 pt) {      // O^T(C, DT) += vt . pt
    if constexpr (C == 0 && DT == 0) asm volatile(W64_PV_0_0 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 1) asm volatile(W64_PV_0_1 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 2) asm volatile(W64_PV_0_2 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 3) asm volatile(W64_PV_0_3 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 0) asm volatile(W64_PV_1_0 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 1) asm volatile(W64_PV_1_1 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 2) asm volatile(W64_PV_1_2 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 3) asm volatile(W64_PV_1_3 : : "v"(vt), "v"(pt) : W64_CLOBBER_ACC);
}
template <int C>
__device__ __forceinline__ void acc_sum(bf16x8 sum_a, bf16x8 pt) {  // row sums of block C += sum_a . pt
    if constexpr (C == 0) asm volatile(W64_SUM_0 : : "v"(sum_a), "v"(pt) : W64_CLOBBER_ACC);
    else asm volatile(W64_SUM_1 : : "v"(sum_a), "v"(pt) : W64_CLOBBER_ACC);
}
// scores of one 32-key half against column block C: sum over the eight steps of K fragment . Q^T fragment
template <int C>
__device__ __forceinline__ f32x16 qk_scores(const u32x4 (&kf)[8]) {
    f32x16 s;
    if constexpr (C == 0)
        asm volatile(W64_QK_0 : "=&v"(s) : "v"(kf[0]), "v"(kf[1]), "v"(kf[2]), "v"(kf[3]), "v"(kf[4]), "v"(kf[5]), "v"(kf[6]), "v"(kf[7]) : W64_CLOBBER_ACC);
    else
        asm volatile(W64_QK_1 : "=&v"(s) : "v"(kf[0]), "v"(kf[1]), "v"(kf[2]), "v"(kf[3]), "v"(kf[4]), "v"(kf[5]), "v"(kf[6]), "v"(kf[7]) : W64_CLOBBER_ACC);
    return s;
}
template <int C>
__device__ __forceinline__ void acc_scale(float alpha, float a_lo, float a_hi) {   // O^T(C, .) *= alpha, row sums likewise
    float scratch;
    if constexpr (C == 0) asm volatile(W64_SCALE_0 : "=&v"(scratch) : "v"(alpha), "v"(a_lo), "v"(a_hi) : W64_CLOBBER_ACC);
    else asm volatile(W64_SCALE_1 : "=&v"(scratch) : "v"(alpha), "v"(a_lo), "v"(a_hi) : W64_CLOBBER_ACC);
}
#define W64_OUT16(x) "=v"(x[0]), "=v"(x[1]), "=v"(x[2]), "=v"(x[3]), "=v"(x[4]), "=v"(x[5]), "=v"(x[6]), "=v"(x[7]), \
                     "=v"(x[8]), "=v"(x[9]), "=v"(x[10]), "=v"(x[11]), "=v"(x[12]), "=v"(x[13]), "=v"(x[14]), "=v"(x[15])
template <int C, int DT>
__device__ __forceinline__ void acc_read(float (&x)[16]) {
    if constexpr (C == 0 && DT == 0) asm volatile(W64_READ_0_0 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 1) asm volatile(W64_READ_0_1 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 2) asm volatile(W64_READ_0_2 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 0 && DT == 3) asm volatile(W64_READ_0_3 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 0) asm volatile(W64_READ_1_0 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 1) asm volatile(W64_READ_1_1 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 2) asm volatile(W64_READ_1_2 : W64_OUT16(x) : : W64_CLOBBER_ACC);
    if constexpr (C == 1 && DT == 3) asm volatile(W64_READ_1_3 : W64_OUT16(x) : : W64_CLOBBER_ACC);
}
template <int C>
__device__ __forceinline__ void acc_read_sums(float& lo, float& hi) {
    if constexpr (C == 0) asm volatile(W64_READL_0 : "=v"(lo), "=v"(hi) : : W64_CLOBBER_ACC);
    else asm volatile(W64_READL_1 : "=v"(lo), "=v"(hi) : : W64_CLOBBER_ACC);
}

constexpr int kWWaves = 4;
constexpr int kWBM = 256;            // queries per workgroup
constexpr int kWBN = 64;             // keys per LDS tile
constexpr int kWD = 128;
constexpr int kWRow = kWD * 2;       // bytes per LDS row
constexpr int kWTile = kWBN * kWRow; // bytes per K (or V) tile
constexpr int kWMaxSeqs = 4096;      // sequences of a packed batch

// Direct-to-LDS load of 16 bytes per lane (see dma_to_lds_16 in common.hpp).  This variant writes m0 inside the
// statement: the assembly loop of this kernel writes m0 too, behind the compiler's back, so nothing here may rely on
// the compiler's idea of what m0 holds.  (m0 cannot be named in a clobber list -- the compiler treats it as reserved
// and warns that clobbering it is undefined -- and it needs no naming: the compiler keeps nothing in m0 across
// statements, it writes m0 directly in front of each of its own instructions that read it.)
// The s_nop 3 makes five wait states between anything in front of the statement and the load: a scalar register
// that a vector instruction wrote (v_readlane restoring a spilled `gbase`, v_readfirstlane) may be read as a
// vector-memory address only five states later, and the compiler does not see the load inside the statement.
__device__ __forceinline__ void dma_to_lds_16_m0(const void* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(gbase), "s"(lds_addr)
                 : "memory");
}

// cu_q[b], cu_q[b+1], cu_k[b], cu_k[b+1] through the scalar cache (the arrays do not change while the kernel runs;
// the compiler, seeing stores all around, would fetch them one after the other with vector loads)
__device__ __forceinline__ void load_bounds(const int32_t* cu_q, const int32_t* cu_k, int b, int& q_lo, int& q_hi, int& k_lo, int& k_hi) {
    typedef int i32x2 __attribute__((ext_vector_type(2)));
    i32x2 qb, kb;
    asm volatile("s_load_dwordx2 %0, %2, 0x0\n\ts_load_dwordx2 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(qb), "=&s"(kb)
                 : "s"(cu_q + b), "s"(cu_k + b)
                 : "memory");
    q_lo = qb[0];
    q_hi = qb[1];
    k_lo = kb[0];
    k_hi = kb[1];
}

// One int32 through the scalar cache (block-table entries and context lengths: they do not change while the kernel
// runs).  An ordinary load here would be a vector load, and the wait the compiler puts in front of its use would also
// wait for every direct-to-LDS request in flight.
__device__ __forceinline__ int load_scalar_i32(const int32_t* ptr) {
    int v;
    asm volatile("s_nop 4\n\ts_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=&s"(v) : "s"(ptr) : "memory");
    return v;
}

// heads_per_wg: how the four wavefronts of a workgroup divide a job.
//   1: a job is 256 query rows of one head, 64 rows per wavefront.  Under a causal mask the wavefronts then see
//      different numbers of K/V tiles -- in the last four tile steps of a job one to three of them have nothing to
//      compute and wait at the hand-over for the one with the lowest rows.
//   4: a job is 64 query rows of FOUR query heads that share a K/V head, one head per wavefront.  The same K/V tiles
//      serve all four, every wavefront sees the same keys, nobody waits: the launch code takes this whenever a K/V
//      head has a multiple of four query heads and the mask is causal.
// PAGED: K and V are pools of 16-row blocks (num_blocks, Hkv, 16, D) read through a block table (queries and outputs
// packed; always causal, bottom-right aligned).  A wavefront's share of a K/V tile -- 16 rows -- is exactly one
// block, so a tile costs every wavefront one table entry: ordinary code fetches it with a scalar load, the assembly
// loop takes it from a register that holds the entries of the next 64 tiles, one per lane (the loop then runs at
// most 63 tiles per entry and is entered again with the next window).
template <bool CAUSAL, bool PAGED>
__global__ __launch_bounds__(kWWaves * 64, 1) void prefill_fwd_w64_kernel(PrefillParams p, int tiles_per_unit, int heads_per_wg) {
    static_assert(CAUSAL || !PAGED, "the block-table variant is causal");
    constexpr int D = kWD, NS = D / 16, NDT = D / 32, CPR = D / 8;
    constexpr float kBias = 32.0f;             // the largest weight sits at 2^-kBias when a reference is set
    constexpr float kUnderflow = 0x1p-92f;     // a row sum below this may have lost terms (see the file header)
    constexpr float kOverflow = 0x1p40f;       // a row sum above this (or NaN) may have overflowed somewhere

    // K buffers 0,1 then V buffers 0,1 (the assembly loop addresses all four relative to one base)
    __shared__ __attribute__((aligned(1024))) unsigned char kv_lds[4 * kWTile];
    // the four wavefronts' 64 query rows each, laid out like a K tile
    __shared__ __attribute__((aligned(1024))) unsigned char q_lds[kWWaves * 64 * kWRow];
    // the number of query tiles of every sequence of a packed batch (see the jobs below)
    __shared__ int nq_lds[kWMaxSeqs];
    unsigned char* const k_lds = kv_lds;
    unsigned char* const v_lds = kv_lds + 2 * kWTile;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;          // query column inside a block / key row of K / d row of V^T
    const int kg = lane >> 5;
    const bool by_head = heads_per_wg == kWWaves;
    const int bm = by_head ? 64 : kWBM;               // query rows of a job
    const int wave_rows = by_head ? 0 : 64;           // rows from one wavefront's first query to the next one's

    // ---- jobs: a workgroup works through query tiles, one "job" each.  What is dealt to workgroups are UNITS of one
    // (sequence, head [, share of the keys]), all units of the launch forming one list sorted by cost, in one of two
    // ways that the launch code chooses between:
    //   pairs (tiles_per_unit == 2): a unit is the PAIR of query tiles (n-1-i, i), n the number of query tiles of the
    //     sequence: under a causal mask every pair of a sequence costs the same.  The list: sequences by their number
    //     of query tiles, the longest class first; inside a class by sequence; inside a sequence by share of the keys,
    //     K/V head, pair, query head of that K/V head.  Neighbours in the list read the same K/V.
    //   single tiles (tiles_per_unit == 1): the list goes by tile index from the highest down -- "class c" is then
    //     every sequence with at least c query tiles, and its unit the tile c-1 -- inside a class by sequence, share,
    //     K/V head, query head.  Finer units: this is for launches of few rounds, where a round of pairs more or
    //     less for some workgroups would be felt.
    // The list is dealt in rounds of one unit per workgroup, every other round in reverse order: each workgroup gets
    // the same number of units from every part of the list, whatever the lengths of the sequences are.  Nothing of
    // this lives in memory: a workgroup walks down the classes and counts the sequences of a class (their numbers of
    // query tiles sit in LDS, 64 per instruction), and finds the sequence of its unit by the same count.
    // In pairs mode the 32 workgroups of an XCD (workgroup ids are dealt round-robin to the 8 XCDs) take 32 neighbours
    // of the list: the pairs and query heads of one K/V head, as far as the numbers allow, which stream the same K/V
    // tiles through that XCD's L2 at the same time. ----
    struct Job {
        const __bf16 *qb, *kb, *vb;
        __bf16* ob;
        float* lb;                       // row 0 of this (sequence, head) in the log-sum-exp output, or null
        const int32_t* tab;              // PAGED: the sequence's row of the block table (kb, vb: block 0 of the K/V head)
        int sq, sk, q0;
        int split;                       // which share of the query tile's K/V tiles (0 when the keys are not split)
    };
    // Split keys (p.n_split > 1): a job works on its share of the K/V tiles and writes, instead of output rows, a
    // normalised fp32 partial row and its log-sum-exp per query, which a second kernel merges.  `ob` and `lb` of such
    // a job point at row 0 of its (share, head, sequence) in the two partial buffers.
    const int n_split = p.n_split > 1 ? p.n_split : 1;
    // head and row strides fit 32 bits (the host checks), so an address takes two scalar multiplications
    const int qs2 = (int)p.qs[2], ks2 = (int)p.ks[2], vs2 = (int)p.vs[2], os2 = (int)p.os[2];
    // (the "query head" digit of a unit counts whole workgroups: single heads, or sets of four heads of one K/V head)
    const int Hq = p.Hq, Hkv = p.Hkv, Hu = by_head ? Hq / kWWaves : Hq, inner = Hu * n_split;
    const int group = Hu / Hkv, group_shift = (group & (group - 1)) == 0 ? __builtin_ctz(group) : -1;
    const bool packed = p.cu_q != nullptr;
    const int n_seq_chunks = (p.B + 63) / 64;
    // numbers of query tiles per sequence (packed layout; zero past the last sequence) and the first class
    int cls;
    if (packed) {
        for (int b = tid; b < 64 * n_seq_chunks; b += kWWaves * 64)
            nq_lds[b] = b < p.B ? (p.cu_q[b + 1] - p.cu_q[b] + bm - 1) / bm : 0;
        __syncthreads();
    }
    const bool pairs = tiles_per_unit == 2;
    // the class after class `c` (0: none): the largest number of query tiles below c that a sequence has, or c - 1
    auto class_below = [&](int c) -> int {
        if (!pairs) return c - 1;
        if (!packed) return 0;
        int most = 0;
        for (int m = 0; m < n_seq_chunks; ++m) {
            const int v = nq_lds[64 * m + lane];
            most = max(most, v < c ? v : 0);
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) most = max(most, __shfl_xor(most, d, 64));
        return __builtin_amdgcn_readfirstlane(most);
    };
    // the sequences of class c, 64 at a time as a bit mask; their number; the `rank`-th of them
    auto members = [&](int c, int m) -> uint64_t {
        const int v = nq_lds[64 * m + lane];
        return __builtin_amdgcn_ballot_w64(pairs ? v == c : v >= c);
    };
    auto seqs_of = [&](int c) -> int {
        if (!packed) return p.B;
        int count = 0;
        for (int m = 0; m < n_seq_chunks; ++m) count += __builtin_popcountll(members(c, m));
        return __builtin_amdgcn_readfirstlane(count);
    };
    auto seq_of = [&](int c, int rank) -> int {
        if (!packed) return rank;
        for (int m = 0; m < n_seq_chunks; ++m) {
            const uint64_t mask = members(c, m);
            const int count = __builtin_popcountll(mask);
            if (rank < count) {               // position of set bit number `rank`: halving by counts
                int pos = 0;
#pragma unroll
                for (int w = 32; w >= 1; w >>= 1) {
                    const int below = __builtin_popcountll((mask >> pos) & ((1ull << w) - 1));
                    const bool skip = rank >= below;
                    rank -= skip ? below : 0;
                    pos += skip ? w : 0;
                }
                return 64 * m + pos;
            }
            rank -= count;
        }
        return 0;
    };
    auto units_of = [&](int c) { return pairs ? (c + 1) / 2 : 1; };      // units of one (sequence, head, share) in class c
    if (packed) {                             // the first class: the largest number of query tiles
        int most = 0;
        for (int m = 0; m < n_seq_chunks; ++m) most = max(most, nq_lds[64 * m + lane]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) most = max(most, __shfl_xor(most, d, 64));
        cls = __builtin_amdgcn_readfirstlane(most);
    } else {
        cls = (p.Sq + bm - 1) / bm;
    }
    // place of this workgroup in a round: neighbours of the list go to the workgroups of one XCD -- in pairs mode
    // as many as the XCD has workgroups; in single-tile mode, where neighbours cost the same, only the query heads
    // of one K/V head, so that the dearest units of the launch are spread over all XCDs
    const int G = gridDim.x, bid = blockIdx.x;
    int place = bid;
    if (G % 8 == 0) {
        const int xcd = bid % 8, local = bid / 8;
        const int chunk = min(group & -group, 32);
        if (pairs) place = (G / 8) * xcd + local;
        else if ((G / 8) % chunk == 0) place = chunk * ((local / chunk) * 8 + xcd) + local % chunk;
    }
    int round = 0;
    int64_t cls_first = 0;                    // position in the list of the first unit of the class
    int per_seq = units_of(cls) * inner;      // units of one sequence of the class
    int cls_units = cls > 0 ? seqs_of(cls) * per_seq : 0;
    int job_tiles = 0, job_unit = 0, job_half = 1;      // the current job: tiles of its sequence, its unit, which tile of the pair
    // next_job(j, prev): the job after `prev` (whatever `prev` holds before the first).
    // What only a new unit needs -- tensor addresses, batch strides, the bounds arrays -- is read from the kernel
    // arguments (first argument, offset 0 of the segment) where it is needed, through an offset the compiler cannot
    // trace: two scalar loads per unit instead of three dozen scalar registers held, and spilled, for the whole kernel.
    typedef const __attribute__((address_space(4))) PrefillParams* ParamsPtr;
    auto args = [&]() -> ParamsPtr {
        size_t off = 0;
        asm volatile("" : "+s"(off));
        return (ParamsPtr)((const __attribute__((address_space(4))) char*)__builtin_amdgcn_kernarg_segment_ptr() + off);
    };
    auto next_job = [&](Job& j, const Job& prev) -> bool {
        j = prev;                             // the sequence-level fields stay while the unit stays
        if (pairs && job_half == 0 && job_unit != job_tiles - 1 - job_unit) {      // second query tile of the pair
            job_half = 1;
            j.q0 = job_unit * bm;
            return true;
        }
        const int64_t at = (int64_t)round * G + ((round & 1) ? G - 1 - place : place);
        ++round;
        while (cls > 0 && at >= cls_first + cls_units) {
            cls_first += cls_units;
            cls = class_below(cls);
            per_seq = units_of(cls) * inner;
            cls_units = cls > 0 ? seqs_of(cls) * per_seq : 0;
        }
        if (cls <= 0) return false;
        // (the compiler divides on the vector unit)
        const int local = (int)(at - cls_first);
        const int seq_rank = __builtin_amdgcn_readfirstlane(local / per_seq), rest = local - seq_rank * per_seq;
        const int units = units_of(cls);
        const int g = group_shift >= 0 ? rest & (group - 1) : rest % group;
        const int above = group_shift >= 0 ? rest >> group_shift : __builtin_amdgcn_readfirstlane(rest / group);      // (share, K/V head, unit)
        const int head_share = __builtin_amdgcn_readfirstlane(above / units), unit = above - head_share * units;
        const int share = n_split > 1 ? __builtin_amdgcn_readfirstlane(head_share / Hkv) : 0, hk = head_share - share * Hkv;
        const int h = by_head ? (hk * group + g) * kWWaves + wave : hk * group + g;     // (this wavefront's query head)
        const int b = __builtin_amdgcn_readfirstlane(seq_of(cls, seq_rank));
        const ParamsPtr a = args();
        const int qs1 = (int)a->qs[1], ks1 = (int)a->ks[1], vs1 = (int)a->vs[1], os1 = (int)a->os[1], ls1 = (int)a->ls[1];
        if (a->cu_q) {
            int q_start, q_end, k_start, k_end;
            load_bounds(a->cu_q, PAGED ? a->cu_q : a->cu_k, b, q_start, q_end, k_start, k_end);
            j.sq = q_end - q_start;
            j.sk = k_end - k_start;
            if constexpr (PAGED) {
                // a length beyond what the table row addresses is cut, never chased
                j.sk = max(0, min(load_scalar_i32(a->ctx_lens + b), 16 * a->max_blocks));
                j.tab = a->block_table + (int64_t)b * a->table_stride;
                k_start = 0;
            }
            j.qb = a->q + ((int64_t)q_start * qs2 + (int64_t)h * qs1);
            j.kb = a->k + ((int64_t)k_start * ks2 + (int64_t)hk * ks1);
            j.vb = a->v + ((int64_t)k_start * vs2 + (int64_t)hk * vs1);
            j.ob = a->out + ((int64_t)q_start * os2 + (int64_t)h * os1);
            j.lb = a->lse ? a->lse + (q_start + (int64_t)h * ls1) : nullptr;
            if (n_split > 1) {
                const int64_t prow = ((int64_t)share * Hq + h) * a->part_rows + q_start;
                j.ob = reinterpret_cast<__bf16*>(a->part_o + prow * kWD);
                j.lb = a->part_lse + prow;
            }
        } else {
            j.sq = a->Sq;
            j.sk = a->Sk;
            j.qb = a->q + ((int64_t)b * a->qs[0] + (int64_t)h * qs1);
            j.kb = a->k + ((int64_t)b * a->ks[0] + (int64_t)hk * ks1);
            j.vb = a->v + ((int64_t)b * a->vs[0] + (int64_t)hk * vs1);
            j.ob = a->out + ((int64_t)b * a->os[0] + (int64_t)h * os1);
            j.lb = a->lse ? a->lse + ((int64_t)b * a->ls[0] + (int64_t)h * ls1) : nullptr;
            if (n_split > 1) {
                const int64_t prow = ((int64_t)share * Hq + h) * a->part_rows + (int64_t)b * a->Sq;
                j.ob = reinterpret_cast<__bf16*>(a->part_o + prow * kWD);
                j.lb = a->part_lse + prow;
            }
        }
        j.split = share;
        job_tiles = cls;
        job_unit = unit;
        job_half = 0;
        j.q0 = (cls - 1 - unit) * bm;
        return true;
    };

    // ---- tile loader: wavefront w, instruction j covers LDS chunks (4w + j)*64 .. +63, i.e. rows 16w + 4j + lane/16;
    // the lane fetches global chunk (lane%16) ^ swz(row) of its row, and swz(row) = ((lane/16) << 2) | j here ----
    const int ld_q = lane >> 4;
    const int ld_c0 = (lane & 15) ^ (ld_q << 2);
    // byte offset of the lane's 16 bytes from the wavefront's first row of step j: row part + ((ld_c0 ^ j) << 4)
    const uint32_t dma_row_k = (uint32_t)(ld_q * ks2 * 2), dma_row_v = (uint32_t)(ld_q * vs2 * 2);
    const uint32_t lds_dst = __builtin_amdgcn_readfirstlane(lds_address(kv_lds + wave * 4096));
    const uint32_t k_step = (uint32_t)(4 * ks2 * 2), v_step = (uint32_t)(4 * vs2 * 2);   // 4 rows, in bytes
    const int blk_elems = Hkv * 16 * kWD;      // PAGED: elements from one block of the pool to the next
    // K (which == 0) or V (which == 1) rows of tile `tile` into that tensor's LDS buffer `buf`
    auto issue_rows = [&](const Job& jb, int which, int tile, int buf) {
        const __bf16* src = which ? jb.vb : jb.kb;
        const int stride = which ? vs2 : ks2;
        const uint32_t step = which ? v_step : k_step, dma_row = which ? dma_row_v : dma_row_k;
        const uint32_t dst = lds_dst + (2 * which + buf) * kWTile;
        if constexpr (PAGED) {
            // this wavefront's 16 rows are logical block 4 * tile + wave of the sequence.  Rows past the last key
            // re-read the last key's row (finite; their scores are masked); a block past the last one is never looked
            // up (its table entry need not exist); an entry that points outside the pool is pulled back into it.
            int last = max(jb.sk - 1, 0);
            asm volatile("" : "+s"(last));          // (keeps this arithmetic at the request, see below)
            const int last_b = last >> 4;
            int bidx = tile * (kWBN / 16) + wave, rin_max = 15;
            if (bidx >= last_b) {
                bidx = last_b;
                rin_max = last & 15;
            }
            int phys = load_scalar_i32(jb.tab + bidx);
            phys = min(max(phys, 0), args()->num_blocks - 1);
            const unsigned char* base = reinterpret_cast<const unsigned char*>(src + (int64_t)phys * blk_elems);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t row = (uint32_t)min(4 * j + ld_q, rin_max);
                dma_to_lds_16_m0(base, row * (uint32_t)kWRow + (uint32_t)((ld_c0 ^ j) << 4), dst + j * 1024);
            }
            return;
        }
        if (tile * kWBN + kWBN <= jb.sk) {
            const unsigned char* base = reinterpret_cast<const unsigned char*>(src + (int64_t)(tile * kWBN + 16 * wave) * stride);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                dma_to_lds_16_m0(base + (size_t)j * step, dma_row + ((ld_c0 ^ j) << 4), dst + j * 1024);
        } else {
            // last, partial tile: rows past the end re-read the last row (finite; their scores are masked).
            // (The empty statement keeps the address arithmetic of this rare path inside the branch: hoisted to
            // the top of the job it occupied two dozen registers that then lived in scratch memory.)
            int last = jb.sk - 1 - tile * kWBN;
            asm volatile("" : "+s"(last));
            const unsigned char* t0 = reinterpret_cast<const unsigned char*>(src + (int64_t)(tile * kWBN) * stride);
            const uint32_t row_bytes = (uint32_t)stride * 2u;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t row = (uint32_t)min(16 * wave + 4 * j + ld_q, last);   // row inside the tile
                dma_to_lds_16_m0(t0, row * row_bytes + (uint32_t)((ld_c0 ^ j) << 4), dst + j * 1024);
            }
        }
    };
    auto issue_k = [&](const Job& jb, int tile, int buf) { issue_rows(jb, 0, tile, buf); };
    auto issue_v = [&](const Job& jb, int tile, int buf) { issue_rows(jb, 1, tile, buf); };
    // number of K/V tiles of a job (the same for the four wavefronts)
    auto tiles_of = [&](const Job& jb) {
        int kv_end = jb.sk;
        if (CAUSAL) kv_end = max(0, min(jb.sk, min(jb.sq, jb.q0 + bm) + (jb.sk - jb.sq)));
        return (kv_end + kWBN - 1) / kWBN;
    };

    // first and one-past-last tile of a job's share
    auto share_of = [&](const Job& jb, int& t0, int& t1) {
        const int nt = tiles_of(jb);
        t0 = 0;
        t1 = nt;
        if (n_split > 1) {
            const int per = (nt + n_split - 1) / n_split;
            t0 = min(nt, jb.split * per);
            t1 = min(nt, t0 + per);
        }
    };

    // ---- per-lane LDS read addresses for buffer 0 (absolute: the assembly loop uses them as they are) ----
    // K fragment of step s, key row 32t + n: chunk (2s + kg) ^ swz(n);  V^T fragment of d-tile dt: source lane s16 of
    // group g16 addresses key row 4(g16>>1) + (s16>>2) (+8 for the upper half), d = 32dt + 16(g16&1) + 4(s16&3)..+3
    // Only the addresses of step 0 / d-tile 0 are kept: the one of step s / d-tile dt is that with s << 5 / dt << 6
    // XORed in (the swizzle XORs exactly those bits).  (The empty statements keep the other fifteen from being
    // computed once and held in registers for the whole kernel, where they pushed other values into scratch memory.)
    uint32_t rd_k0, rd_vlo0, rd_vhi0;
    {
        const int g16 = lane >> 4, s16 = lane & 15;
        const int row = 4 * (g16 >> 1) + (s16 >> 2), d = 16 * (g16 & 1) + 4 * (s16 & 3);
        rd_k0 = lds_address(k_lds) + n * kWRow + ((kg ^ swz<D>(n)) << 4);
        rd_vlo0 = lds_address(v_lds) + row * kWRow + (((d >> 3) ^ swz<D>(row)) << 4) + (d & 7) * 2;
        rd_vhi0 = lds_address(v_lds) + (row + 8) * kWRow + (((d >> 3) ^ swz<D>(row + 8)) << 4) + (d & 7) * 2;
    }
    auto rd_k = [&](int s) {
        uint32_t a = rd_k0;
        asm volatile("" : "+v"(a));
        return a ^ (uint32_t)(s << 5);
    };
    auto rd_v = [&](int e, int dt) {
        uint32_t a = e ? rd_vhi0 : rd_vlo0;
        asm volatile("" : "+v"(a));
        return a ^ (uint32_t)(dt << 6);
    };

    // A operand of the row-sum MFMA (see prefill_fwd.hip): row 0 sums k = 0..7, 16..23 (query c), row 1 the rest (c + 16)
    uint32_t sum_word;
    {
        const int r16 = lane & 15, g = (lane >> 4) & 1;
        sum_word = ((r16 == 0 && g == 0) || (r16 == 1 && g == 1)) ? 0x3f803f80u : 0u;     // bf16 1.0 twice
    }
    const bf16x8 sum_a = as_bf16x8(u32x4{sum_word, sum_word, sum_word, sum_word});

    // ---- query rows: the wavefront's 64 rows go to its own part of q_lds with sixteen direct-to-LDS loads of four
    // rows each, swizzled like a K tile (load i covers rows 4i + lane/16, and swz of that row is ((lane/16) << 2) |
    // (i & 3)); a row past the end of the sequence re-reads the last row (finite; nothing of it is ever stored) ----
    const uint32_t q_dst = __builtin_amdgcn_readfirstlane(lds_address(q_lds + wave * (64 * kWRow)));
    // (loads 4 * part .. 4 * part + 3: rows 16 * part .. 16 * part + 15 of wavefront `to`; a wavefront may request
    // another one's rows, see the early requests below)
    auto issue_q = [&](const Job& jb, int to, int part) {
        const int qw0 = jb.q0 + wave_rows * to;
        const uint32_t row_bytes = (uint32_t)qs2 * 2u;
        const uint32_t dst = q_dst + (uint32_t)((to - wave) * (64 * kWRow) + 4 * part * 1024);
        // (jb.qb is this wavefront's head; another wavefront's rows may be another head's)
        const __bf16* qb_to = jb.qb;
        if (by_head && to != wave) qb_to += (int64_t)(to - wave) * (int)args()->qs[1];
        if (qw0 + 64 <= jb.sq) {
            const unsigned char* base = reinterpret_cast<const unsigned char*>(qb_to + (int64_t)(qw0 + 16 * part) * qs2);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                dma_to_lds_16_m0(base + (size_t)(4 * j) * row_bytes, (uint32_t)ld_q * row_bytes + ((ld_c0 ^ j) << 4), dst + j * 1024);
        } else {
            // (the empty statement keeps the arithmetic of this rare path inside the branch)
            int last = jb.sq - 1;
            asm volatile("" : "+s"(last));
            const int first = min(qw0, last);              // (a wavefront wholly past the end reads the last row 64 times)
            const unsigned char* base = reinterpret_cast<const unsigned char*>(qb_to + (int64_t)first * qs2);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t row = (uint32_t)(min(qw0 + 16 * part + 4 * j + ld_q, last) - first);
                dma_to_lds_16_m0(base, row * row_bytes + (uint32_t)((ld_c0 ^ j) << 4), dst + j * 1024);
            }
        }
    };
    // Q^T fragment of step s in block c: row 32c + n, chunk (2s + kg) ^ swz(n), as for K
    const uint32_t q_rd0 = q_dst + n * kWRow + ((kg ^ swz<D>(n)) << 4);

    // ---- output rows leave whole, 32 at a time, through LDS: through the wavefront's own shares of the second K and
    // V buffers (the 16 rows each that its own direct-to-LDS loads fill), which are idle between the last tile of a
    // job and the requests of K[1] / V[1] of the next.  Rows of 256 bytes, chunk c of row r at c ^ swz(r).
    // (Jobs on split keys, whose first tile may live in either buffer, write fp32 partial rows straight from their
    // registers instead.) ----
    constexpr int kRowsPerPass = 64 / CPR;           // a store instruction takes 4 whole rows
    const int c16 = lane % CPR, r0 = lane / CPR;
    unsigned char* const stage_w = kv_lds + ((n < 16) ? 1 : 3) * kWTile + wave * 4096 + (n & 15) * kWRow + 8 * kg;   // the lane's row n
    const int stage_wx = swz<D>(n);
    unsigned char* const stage_r = kv_lds + kWTile + wave * 4096 + r0 * kWRow;        // row r0 of pass 0

    // What a job needs before it can start is requested as early as possible -- for the first job right away, for
    // every other one while the job before it normalises and stores its output: K[0], the query rows, V[0], and K[1]
    // once the output rows have left its buffer.  Six groups of four requests and a seventh: in the epilogue of a job
    // they go out one group at a time between pieces of vector work, so that the wavefront does not sit behind a
    // full request queue (the four wavefronts all do this at the same time).
    // (n_early: how many of the job's sixteen parts of query rows -- part p = rows 16 (p % 4) .. of wavefront
    // 3 - p / 4 -- were requested already, while the job before was still in its tile loop: see the early requests)
    auto prefetch_group = [&](const Job& jb, int group, int n_early) {
        int t0, t1;
        share_of(jb, t0, t1);
        if (group == 0) {
            if (t1 > t0) issue_k(jb, t0, t0 & 1);
        } else if (group <= 4) {
            if (4 * (3 - wave) + group - 1 >= n_early) issue_q(jb, wave, group - 1);
        } else if (group == 5) {
            if (t1 > t0) issue_v(jb, t0, t0 & 1);
        } else {
            if (t1 > t0 + 1) issue_k(jb, t0 + 1, (t0 + 1) & 1);
        }
    };
    // number of output row stores a job issues at its end (four whole rows each): a pass whose four rows all lie
    // past the end of the sequence is jumped over, so the count is known here.  (The one or two stores of a
    // log-sum-exp output are not counted: a count that is too low only makes a wait take a little more than it must.)
    auto row_passes = [&](const Job& jb) {
        return min(max((jb.sq - (jb.q0 + wave_rows * wave) + kRowsPerPass - 1) / kRowsPerPass, 0), 64 / kRowsPerPass);
    };
    // waits until at most `young` (rounded down to a multiple of 4) of this wavefront's vector-memory operations
    // are in flight; they complete in order, so everything older than the youngest `young` has then arrived
    auto wait_all_but = [&](int young) {
        switch (young >> 2) {
            case 0: wait_vmcnt<0>(); break;
            case 1: wait_vmcnt<4>(); break;
            case 2: wait_vmcnt<8>(); break;
            case 3: wait_vmcnt<12>(); break;
            case 4: wait_vmcnt<16>(); break;
            case 5: wait_vmcnt<20>(); break;
            case 6: wait_vmcnt<24>(); break;
            case 7: wait_vmcnt<28>(); break;
            case 8: wait_vmcnt<32>(); break;
            case 9: wait_vmcnt<36>(); break;
            default: wait_vmcnt<40>(); break;
        }
    };

    Job cur{}, nxt{};
    bool have = next_job(cur, cur);
    if (have) {
#pragma unroll
        for (int group = 0; group < 7; ++group) prefetch_group(cur, group, 0);
    }
    int prev_stores = 0;       // output row stores of the job before `cur` that are younger than the requests for `cur`
    while (have) {
        const int sq = cur.sq, sk = cur.sk, q0 = cur.q0;
        const int coff = sk - sq;                          // bottom-right aligned causal diagonal
        const int qw0 = q0 + wave_rows * wave;             // first query of this wavefront
        // the job's tiles are [t_first, n_tiles): all of the query tile's, or its share of them
        int t_first, n_tiles;
        share_of(cur, t_first, n_tiles);
        // tile kinds of this wavefront: [0, n_plain) every key visible to each of its queries, [n_plain, n_mask) some,
        // [n_mask, n_tiles) none (the wavefront then only takes part in the hand-over)
        int n_plain = sk / kWBN, n_mask = n_tiles;
        if (CAUSAL) {
            n_plain = min(n_plain, max(0, qw0 + coff + 1) / kWBN);
            n_mask = min(n_tiles, max(0, qw0 + 63 + coff + kWBN) / kWBN);      // first tile whose first key is past query qw0+63
        }
        n_plain = min(n_plain, n_tiles);
        // diagonal aligned with the tiles: query i of the wavefront sees key j of its one masked tile iff j <= i
        const int aligned = CAUSAL && n_mask == n_plain + 1 && qw0 + coff == n_plain * kWBN && (n_plain + 1) * kWBN <= sk;
        // the assembly loop requests tile+2 with whole-tile loads: it may run tile t only if tile t+2 is a whole tile
        // (or does not exist), so it stops three tiles before a partial last tile
        const int n_asm = n_tiles > sk / kWBN ? max(0, n_tiles - 3) : n_tiles;
        const int share_tiles = n_tiles - t_first;
        // the job after this one (scalar work, done while the first tile is still landing)
        const bool have_next = next_job(nxt, cur);
        // Early requests.  Under a causal mask the wavefronts with the upper rows of the query tile have nothing to
        // compute in its last tiles ("hidden" steps: they only take part in the hand-over, in ordinary code) while
        // the one with the lowest rows sets the pace.  In such a step a wavefront requests query rows of the NEXT
        // job -- anybody's: the place in LDS is free once every wavefront has its fragments in registers, which the
        // first hand-over of the job guarantees -- three parts per step, in an order every wavefront can work out
        // (step by step, wavefront by wavefront; part p = rows 16 (p % 4) .. of wavefront 3 - p / 4, so the rows of
        // the wavefront that is busiest at the end of a job go first).  What is left goes out after the tile loop.
        const auto first_hidden_of = [&](int q_tile0, int off, int first, int tiles, int w) {
            const int hidden = CAUSAL ? min(tiles, max(0, q_tile0 + wave_rows * w + 63 + off + kWBN) / kWBN) : tiles;
            return max(hidden, first);
        };
        // number of (step, wavefront) slots in front of slot (tile, w)
        const auto slots_before = [&](int q_tile0, int off, int first, int tiles, int tile, int w) {
            int slots = 0;
#pragma unroll
            for (int other = 0; other < kWWaves; ++other) {
                const int hidden = first_hidden_of(q_tile0, off, first, tiles, other);
                slots += max(0, min(tile, tiles) - hidden) + (other < w && hidden <= tile ? 1 : 0);
            }
            return slots;
        };
        constexpr int kPartsPerSlot = 3;
        const int n_early = have_next ? min(16, kPartsPerSlot * slots_before(q0, coff, t_first, n_tiles, n_tiles, 0)) : 0;

        // per column block: r_ref exponent reference in the log2 domain (-inf: none yet), nb = -r_ref - kBias
        float r_ref[2], nb[2], l_row[2];
        bool redo = false;                    // a row sum left the range in which no term can have been lost
        const int young_dma = (share_tiles > 1 ? 4 : 0) + (share_tiles > 0 ? 4 : 0);      // requests of the first V and the second K tile

        // Ordinary code for single tiles.  Everything it derives from the job goes through `fresh`, a copy of the few
        // values it needs that the compiler cannot trace back: what could be computed once per job would otherwise
        // be computed at the top of every job and wait in registers (spilled ones, mostly) for a tile that rarely comes.
        struct Fresh {
            int sk, qw0, coff, n_tiles, q0, t_first, early;
        };
        // Scores of one 32-key half of a tile for one column block (reads K[tile]).
        auto scores = [&](auto c_c, int tile, int t) {
            constexpr int c = decltype(c_c)::value;
            const int buf = tile & 1;
            // (all fragment reads first, then the MFMAs: one LDS latency instead of eight)
            u32x4 kf[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) kf[s] = lds_load_at<u32x4>(rd_k(s) + buf * kWTile + t * 32 * kWRow);
            return qk_scores<c>(kf);
        };
        // The rest of that half: mask, reference move, weights, accumulation (reads V[tile]).
        auto finish = [&](const Fresh& fr, auto c_c, int tile, int t, bool masked, f32x16 s_acc) {
            constexpr int c = decltype(c_c)::value;
            const int buf = tile & 1;
            const int k0 = tile * kWBN + 32 * t;
            const int qi = fr.qw0 + 32 * c + n;
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float x = fmaf(s_acc[i], p.scale_log2, nb[c]);
                if (masked) {
                    const int key = k0 + 8 * (i >> 2) + 4 * kg + (i & 3);
                    bool keep = key < fr.sk;
                    if (CAUSAL) keep = keep & (key <= qi + fr.coff);
                    x = keep ? x : -INFINITY;
                }
                s_acc[i] = x;
                mx = fmaxf(mx, x);
            }
            mx = xor32_max(mx);
            const float r_new = fmaxf(r_ref[c], mx - nb[c]);
            const float alpha = r_ref[c] == -INFINITY ? 1.0f : fast_exp2(r_ref[c] - r_new);
            const float nb_new = r_new == -INFINITY ? 0.f : -r_new - kBias;
            const float delta = nb_new - nb[c];
            r_ref[c] = r_new;
            nb[c] = nb_new;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0)      // (lanes 0..15 hold the sums of queries c and c + 16)
                acc_scale<c>(alpha, __shfl(alpha, lane & 15, 64), __shfl(alpha, (lane & 15) + 16, 64));
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int u = 2 * t + hf;
                u32x4 pw;
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    pw[w] = pack_bf16(fast_exp2(s_acc[8 * hf + 2 * w] + delta), fast_exp2(s_acc[8 * hf + 2 * w + 1] + delta));
                const bf16x8 pf = as_bf16x8(pw);
                bf16x8 vf[NDT];
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
                    vf[dt] = join_bf16x8(lds_read_tr16_at(rd_v(0, dt) + buf * kWTile + 16 * u * kWRow),
                                         lds_read_tr16_at(rd_v(1, dt) + buf * kWTile + 16 * u * kWRow));
                acc_sum<c>(sum_a, pf);
                acc_pv<c, 0>(vf[0], pf);
                acc_pv<c, 1>(vf[1], pf);
                acc_pv<c, 2>(vf[2], pf);
                acc_pv<c, 3>(vf[3], pf);
            }
        };
        // boundary(tile): see the protocol in the file header
        auto boundary = [&](const Fresh& fr, int tile) {
            wait_vmcnt<0>();
            __syncthreads();
            Job jc = cur;
            asm volatile("" : "+s"(jc.kb), "+s"(jc.vb));
            jc.sk = fr.sk;
            if (tile + 1 < fr.n_tiles) issue_v(jc, tile + 1, (tile + 1) & 1);
            if (tile + 2 < fr.n_tiles) issue_k(jc, tile + 2, tile & 1);
        };
        // a whole tile in ordinary code: scores from K[tile], boundary, everything else from V[tile]
        // (a tile past n_mask has nothing for this wavefront: it only takes part in the boundary)
        auto step_cxx = [&](int tile, bool early) {
            Fresh fr{sk, qw0, coff, n_tiles, q0, t_first, early ? n_early : 0};
            int first_masked = n_plain, first_hidden = n_mask;
            asm volatile("" : "+s"(fr.sk), "+s"(fr.qw0), "+s"(fr.coff), "+s"(fr.n_tiles), "+s"(first_masked), "+s"(first_hidden), "+s"(tile),
                         "+s"(fr.q0), "+s"(fr.t_first), "+s"(fr.early));
            const bool visible = tile < first_hidden, masked = tile >= first_masked;
            constexpr std::integral_constant<int, 0> A{};
            constexpr std::integral_constant<int, 1> B{};
            f32x16 sa0{}, sb0{}, sa1{}, sb1{};
            if (visible) {
                sa0 = scores(A, tile, 0);
                sb0 = scores(B, tile, 0);
                sa1 = scores(A, tile, 1);
                sb1 = scores(B, tile, 1);
            }
            boundary(fr, tile);
            if (!visible && fr.early > 0) {           // a hidden step of the first attempt: early requests
                const int slot = slots_before(fr.q0, fr.coff, fr.t_first, fr.n_tiles, tile, wave);
                Job jn = nxt;
                asm volatile("" : "+s"(jn.qb), "+s"(jn.q0), "+s"(jn.sq));
#pragma unroll 1
                for (int i = 0; i < kPartsPerSlot; ++i) {
                    const int part = kPartsPerSlot * slot + i;
                    if (part < fr.early) issue_q(jn, 3 - part / 4, part % 4);
                }
            }
            if (visible) {
                finish(fr, A, tile, 0, masked, sa0);
                finish(fr, B, tile, 0, masked, sb0);
                finish(fr, A, tile, 1, masked, sa1);
                finish(fr, B, tile, 1, masked, sb1);
            }
        };
        // The assembly loop saw a row sum reach 2: every row's reference moves up by the exponent of its sum (the sum,
        // and with it every weight so far, lands in [2^-32, 2^-31)); an exact rescaling by a power of two.
        auto move_references = [&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            float s_lo, s_hi;
            acc_read_sums<c>(s_lo, s_hi);
            const float l_lo = __shfl(s_lo, lane & 15, 64), l_hi = __shfl(s_hi, lane & 15, 64);
            const float l = (n & 16) ? l_hi : l_lo;
            if (!(l <= kOverflow)) redo = true;
            const int expo = (int)((__builtin_bit_cast(uint32_t, l) >> 23) & 0xffu) - 127;
            const int k = min(max(expo + (int)kBias, 0), 126);
            const float alpha = __builtin_bit_cast(float, (uint32_t)(127 - k) << 23);      // 2^-k
            if (__builtin_amdgcn_ballot_w64(k != 0) != 0)
                acc_scale<c>(alpha, __shfl(alpha, lane & 15, 64), __shfl(alpha, (lane & 15) + 16, 64));
            r_ref[c] += (float)k;
            nb[c] -= (float)k;
        };

        // Two attempts at most: the first with the references preset to 0 and the hand-scheduled loop wherever it can
        // run; the second -- only if some row's sum came out suspiciously small or large -- entirely in ordinary code
        // with references taken from the data.
        for (int attempt = 0; attempt < 2; ++attempt) {
        const bool preset = attempt == 0;
        // (What this loop would let the compiler compute once, before it -- the addresses of the tiles requested
        // again -- it would compute at the top of every job and park in spilled registers; the copy below, which it
        // cannot trace, keeps that arithmetic where it is used.)
        if (!preset) {                        // start over: the buffers are free (everybody passed the vote below)
            Job jc = cur;
            asm volatile("" : "+s"(jc.kb), "+s"(jc.vb), "+s"(jc.sk));
            if (share_tiles > 0) issue_k(jc, t_first, t_first & 1);
            if (share_tiles > 1) issue_k(jc, t_first + 1, (t_first + 1) & 1);
            if (share_tiles > 0) issue_v(jc, t_first, t_first & 1);
        }
        asm volatile(W64_ZERO : : "v"(as_bf16x8(u32x4{0u, 0u, 0u, 0u})) : W64_CLOBBER_ACC);      // O^T and the row sums
        r_ref[0] = r_ref[1] = preset ? 0.f : -INFINITY;
        nb[0] = nb[1] = preset ? -kBias : 0.f;
        // Wait for K[0] and the query rows.  Younger than the last request of those are the requests of V[0] and K[1]
        // and, the first time, the last output row stores of the job before this one.
        wait_all_but(young_dma + (preset ? prev_stores : 0));
        __syncthreads();                      // everybody's share of K[0] and of the query rows is in
        if (preset) {                         // the query rows go to their registers
            uint32_t scratch;
            asm volatile(W64_QFRAGS : "=&v"(scratch) : "v"(q_rd0) : "memory", W64_CLOBBER_ACC);
        }
        int tile = t_first;
        // (the hand-scheduled loop ends where the wavefront's hidden steps begin: those run in ordinary code)
        const int n_loop = preset ? min(n_asm, n_mask) : 0;
        while (tile < n_tiles) {
            if (tile >= n_loop) {
                step_cxx(tile, preset);
                ++tile;
                continue;
            }
            // ---- the hand-scheduled loop over tiles [tile, n_loop); leaves after a tile that took a row sum to 2 ----
            // (PAGED: at most 63 tiles per entry, see the block ids below; the loop is then entered again)
            const int n_stop = PAGED ? min(n_loop, tile + 63) : n_loop;
            uint64_t kptr, vptr;
            int v_ids = 0;
            if constexpr (PAGED) {
                // Block ids of this wavefront's shares of tiles tile + 1 + lane (the loop requests V[t+1] and K[t+2]),
                // never from past the sequence's last block, pulled into the pool.  The bases are block 0 of the K/V head.
                int last = max(sk - 1, 0), first = tile + 1;
                asm volatile("" : "+s"(last), "+s"(first));
                const int bidx = min((first + lane) * (kWBN / 16) + wave, last >> 4);
                v_ids = min(max(cur.tab[bidx], 0), args()->num_blocks - 1);
                kptr = (uint64_t)(uintptr_t)cur.kb;
                vptr = (uint64_t)(uintptr_t)cur.vb;
            } else {
                kptr = (uint64_t)(uintptr_t)(cur.kb + (int64_t)((tile + 2) * kWBN + 16 * wave) * ks2);
                vptr = (uint64_t)(uintptr_t)(cur.vb + (int64_t)((tile + 1) * kWBN + 16 * wave) * vs2);
            }
            // mask thresholds for the first masked tile the loop will meet: a key at index j of that tile is kept by
            // query i of the wavefront iff j <= i + (qw0 + coff - k0) and j < sk - k0 (the lane part 4*kg of a key's
            // index is folded in)
            const int k0m = max(tile, n_plain) * kWBN;
            const int diag = CAUSAL ? qw0 + coff - k0m : (1 << 20);
            // vector operands: read once when the block starts, scratch registers of the block afterwards
            float v_nb0 = nb[0], v_nb1 = nb[1];
            int v_thr0 = min(n + diag, sk - 1 - k0m) - 4 * kg, v_thr1 = min(n + 32 + diag, sk - 1 - k0m) - 4 * kg;
            uint32_t v_sum = sum_word, v_k0 = rd_k0, v_vlo = rd_vlo0, v_vhi = rd_vhi0;
            uint32_t v_rowk = dma_row_k, v_rowv = dma_row_v, v_c0s = (uint32_t)(ld_c0 << 4);
            int status;
            int tile_s = __builtin_amdgcn_readfirstlane(tile);
#define W64_LOOP_OUTPUTS                                                                                              \
    [tile] "+&s"(tile_s), [t2] "=&s"(status), [nb0] "+v"(v_nb0), [nb1] "+v"(v_nb1), [suma] "+v"(v_sum),               \
        [k0] "+v"(v_k0), [vlo0] "+v"(v_vlo), [vhi0] "+v"(v_vhi), [rowk] "+v"(v_rowk), [rowv] "+v"(v_rowv),            \
        [c0s] "+v"(v_c0s), [thr0] "+v"(v_thr0), [thr1] "+v"(v_thr1)
#define W64_LOOP_INPUTS                                                                                               \
    [n_tiles] "s"(__builtin_amdgcn_readfirstlane(n_tiles)), [n_end] "s"(__builtin_amdgcn_readfirstlane(n_stop)),      \
        [n_pipe] "s"(__builtin_amdgcn_readfirstlane(min(n_plain, n_stop))),                                           \
        [n_mask] "s"(__builtin_amdgcn_readfirstlane(n_mask)), [aligned] "s"(__builtin_amdgcn_readfirstlane(aligned)), \
        [kstep] "s"(__builtin_amdgcn_readfirstlane(k_step)), [vstep] "s"(__builtin_amdgcn_readfirstlane(v_step)),     \
        [ldsdst] "s"(lds_dst), [scale] "s"(__builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, p.scale_log2))), \
        [klo] "s"(__builtin_amdgcn_readfirstlane((uint32_t)kptr)),                                                    \
        [khi] "s"(__builtin_amdgcn_readfirstlane((uint32_t)(kptr >> 32))),                                            \
        [vlo] "s"(__builtin_amdgcn_readfirstlane((uint32_t)vptr)),                                                    \
        [vhi] "s"(__builtin_amdgcn_readfirstlane((uint32_t)(vptr >> 32)))
#define W64_LOOP_CLOBBERS "memory", "vcc", "scc", "s36", "s37", "s38", "s39", "s40", "s41", "s42", W64_CLOBBER_ACC, W64_CLOBBER_LOOP_VGPRS
            if constexpr (PAGED) {
                asm volatile(W64_LOOP_PAGED
                             : W64_LOOP_OUTPUTS
                             : W64_LOOP_INPUTS, [ids] "v"(v_ids),
                               [blk] "s"(__builtin_amdgcn_readfirstlane((uint32_t)blk_elems * 2u))
                             : W64_LOOP_CLOBBERS, "s43", "s44");
            } else {
                asm volatile(W64_LOOP : W64_LOOP_OUTPUTS : W64_LOOP_INPUTS : W64_LOOP_CLOBBERS);
            }
#undef W64_LOOP_OUTPUTS
#undef W64_LOOP_INPUTS
#undef W64_LOOP_CLOBBERS
            tile = tile_s;
            // status 0: tiles up to n_loop done.  1: tiles up to `tile` done, and the last of them took a row sum to 2.
            if (status != 0) {
                move_references(std::integral_constant<int, 0>{});
                move_references(std::integral_constant<int, 1>{});
            }
        }
        // row sums
        const auto read_sums = [&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            float s_lo, s_hi;
            acc_read_sums<c>(s_lo, s_hi);
            const float l_lo = __shfl(s_lo, lane & 15, 64), l_hi = __shfl(s_hi, lane & 15, 64);
            l_row[c] = (n & 16) ? l_hi : l_lo;
        };
        read_sums(std::integral_constant<int, 0>{});
        read_sums(std::integral_constant<int, 1>{});
        // ---- the workgroup meets (everybody is done with the K/V buffers) and, the first time, votes: if some row's
        // sum came out suspiciously small or large, the query tile is done again (rows past the end of the sequence
        // count too: they repeat the last row) ----
        if (!preset) {
            __syncthreads();
            break;
        }
        // (a query that sees none of the job's keys -- causal with fewer keys than queries, or a share of split keys
        // that lies past its diagonal -- has a sum of zero by right)
        const int k_first = t_first * kWBN;
        const bool sees0 = k_first < sk && (!CAUSAL || k_first <= qw0 + n + coff);
        const bool sees1 = k_first < sk && (!CAUSAL || k_first <= qw0 + 32 + n + coff);
        const bool bad = redo || (sees0 && !(l_row[0] >= kUnderflow)) || (sees1 && !(l_row[1] >= kUnderflow)) ||
                         !(l_row[0] <= kOverflow) || !(l_row[1] <= kOverflow);
        if (!__syncthreads_or(bad ? 1 : 0)) break;
        redo = false;
        }   // attempts

        // ---- normalise: lane owns query qw0 + 32c + n, d = 32dt + 8(i/4) + 4kg + i%4; the rows of a block leave
        // whole (written once, never read here: non-temporal, so that the K/V tiles keep the L2 to themselves).  The
        // next job's first requests go out in between. ----
        if (n_split > 1) {
            // partial result of this share of the keys: normalised fp32 rows and their log-sum-exp (-inf and zeros when
            // the share kept no key for the row), straight from the registers; the merge kernel weighs them
            float* const part = reinterpret_cast<float*>(cur.ob);
            const auto partial_block = [&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                const int qi = qw0 + 32 * c + n;
                const bool q_ok = qi < sq;
                const float inv_p = l_row[c] > 0.f ? 1.0f / l_row[c] : 0.f;
                if (q_ok && kg == 0)
                    cur.lb[qi] = l_row[c] > 0.f ? 0.69314718056f * (__log2f(l_row[c]) - nb[c]) : -INFINITY;
                float* const po = part + (int64_t)qi * D + 4 * kg;
                const auto store_dt = [&](auto dt_c) {
                    constexpr int dt = decltype(dt_c)::value;
                    float x[16];
                    acc_read<c, dt>(x);
                    if (q_ok) {
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            *reinterpret_cast<f32x4*>(po + 32 * dt + 8 * g) =
                                f32x4{x[4 * g] * inv_p, x[4 * g + 1] * inv_p, x[4 * g + 2] * inv_p, x[4 * g + 3] * inv_p};
                    }
                    if (have_next && 4 * c + dt < 6) prefetch_group(nxt, 4 * c + dt, n_early);
                };
                store_dt(std::integral_constant<int, 0>{});
                store_dt(std::integral_constant<int, 1>{});
                store_dt(std::integral_constant<int, 2>{});
                store_dt(std::integral_constant<int, 3>{});
            };
            partial_block(std::integral_constant<int, 0>{});
            partial_block(std::integral_constant<int, 1>{});
            if (have_next) prefetch_group(nxt, 6, n_early);
            prev_stores = 0;                   // (the stores above are not counted: the next wait takes a few of them along)
            cur = nxt;
            have = have_next;
            continue;
        }
        __bf16* const wave_out = cur.ob + (int64_t)qw0 * os2;                              // (wave-uniform)
        const uint32_t lane_out = (uint32_t)(r0 * os2 + c16 * 8) * 2u;                     // bytes from there
        auto out_row = [&](int r) {           // the lane's 16 bytes of the wavefront's row r + r0
            return reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(wave_out + (int64_t)r * os2) + lane_out);
        };
        auto staged_row = [&](int i) {
            // row 4i + r0 of the block: in the K share for i < 4, in the V share after; swz of it is (r0 << 2) | (i & 3)
            return *reinterpret_cast<const u32x4*>(stage_r + (i / 4) * (2 * kWTile) + (i & 3) * (kRowsPerPass * kWRow) +
                                                   ((c16 ^ ((r0 << 2) | (i & 3))) << 4));
        };
        const auto store_block = [&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            const float inv = 1.0f / l_row[c];     // l == 0 (no key kept) -> NaN row, like the reference softmax
            // sum_j exp(scale * s_j) = l * 2^(-nb)  ->  lse = ln2 * (log2 l - nb); no key kept -> -inf
            if (cur.lb && kg == 0 && qw0 + 32 * c + n < sq)
                cur.lb[qw0 + 32 * c + n] = l_row[c] > 0.f ? 0.69314718056f * (__log2f(l_row[c]) - nb[c]) : -INFINITY;
            const auto stage_dt = [&](auto dt_c) {
                constexpr int dt = decltype(dt_c)::value;
                float x[16];
                acc_read<c, dt>(x);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = pack_bf16(x[4 * g + 0] * inv, x[4 * g + 1] * inv);
                    w[1] = pack_bf16(x[4 * g + 2] * inv, x[4 * g + 3] * inv);
                    *reinterpret_cast<u32x2*>(stage_w + (((4 * dt + g) ^ stage_wx) << 4)) = w;
                }
                if (have_next && 4 * c + dt < 6) prefetch_group(nxt, 4 * c + dt, n_early);
            };
            stage_dt(std::integral_constant<int, 0>{});
            stage_dt(std::integral_constant<int, 1>{});
            stage_dt(std::integral_constant<int, 2>{});
            stage_dt(std::integral_constant<int, 3>{});
            if (qw0 + 64 <= sq) {                  // all rows exist: reads first, then the stores
                u32x4 w[32 / kRowsPerPass];
#pragma unroll
                for (int i = 0; i < 32 / kRowsPerPass; ++i) w[i] = staged_row(i);
#pragma unroll
                for (int i = 0; i < 32 / kRowsPerPass; ++i) __builtin_nontemporal_store(w[i], out_row(32 * c + i * kRowsPerPass));
            } else {
#pragma unroll
                for (int i = 0; i < 32 / kRowsPerPass; ++i) {
                    const u32x4 w = staged_row(i);
                    const int r = 32 * c + i * kRowsPerPass;
                    if (qw0 + r < sq) {                    // (wave-uniform: see row_passes)
                        if (qw0 + r + r0 < sq) __builtin_nontemporal_store(w, out_row(r));
                    }
                }
            }
        };
        store_block(std::integral_constant<int, 0>{});
        store_block(std::integral_constant<int, 1>{});
        // (the stores above took their data from the staged rows, so every read of them has returned)
        if (have_next) prefetch_group(nxt, 6, n_early);
        // (the rows of block A leave before the last query rows of the next job are requested; those of block B after)
        prev_stores = max(row_passes(cur) - 32 / kRowsPerPass, 0);
        cur = nxt;
        have = have_next;
    }
}

// The kernel multiplies head and row strides as 32-bit numbers (batch strides stay 64-bit), and keeps one number per
// sequence of a packed batch in LDS.
bool prefill_w64_takes(const PrefillParams& p) {
    const int64_t strides[] = {p.qs[1], p.qs[2], p.ks[1], p.ks[2], p.vs[1], p.vs[2], p.os[1], p.os[2], p.lse ? p.ls[1] : 0};
    for (int64_t v : strides)
        if (v < 0 || v > 0x7fffffffLL) return false;
    if (p.cu_q && p.B > kWMaxSeqs) return false;
    // a row offset inside a tile of 64 rows, in bytes, is a 32-bit number as well
    return p.qs[2] < (1 << 23) && p.ks[2] < (1 << 23) && p.vs[2] < (1 << 23) && p.os[2] < (1 << 23);
}

int launch_prefill_w64(const PrefillParams& p, hipStream_t stream) {
    // One resident workgroup per compute unit (fewer when there are fewer jobs), each working through its share of
    // the (sequence, head, query tiles [, share of the keys]) units.  The kernel finds them from the sequence
    // lengths themselves; Sq_max only bounds their number here.
    int dev = 0, n_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    const int n_split = p.n_split > 1 ? p.n_split : 1;
    // Causal mask and a multiple of four query heads per K/V head: the four wavefronts of a workgroup take the same 64
    // rows of four heads (every wavefront then sees the same keys); otherwise 4 x 64 rows of one head.
    const bool by_head = p.mask_mode == MI355_MASK_CAUSAL && (p.Hq / p.Hkv) % kWWaves == 0;
    const int heads_per_wg = by_head ? kWWaves : 1;
    const int64_t n_qtiles = by_head ? (p.Sq + 63) / 64 : p.n_qtiles, n_heads = p.Hq / heads_per_wg;
    // Units are pairs of query tiles (equal causal work per unit of a sequence, neighbours that share K/V) unless
    // pairs would leave compute units idle: when every single tile can have a compute unit of its own, or when the
    // pairs make few rounds and the last of them is far from full (judged for sequences of Sq_max rows; then single
    // tiles, dealt by cost, fill the gap better than half as many pairs).
    const int64_t most_tiles = n_qtiles * n_heads * p.B * n_split;
    const int64_t most_pairs = (n_qtiles + 1) / 2 * n_heads * p.B * n_split;
    const int64_t rounds = (most_pairs + n_cu - 1) / n_cu;
    const bool singles = most_tiles <= n_cu || (rounds < 8 && most_pairs * 100 < rounds * n_cu * 97);
    const int tiles_per_unit = singles ? 1 : 2;
    const int64_t most_units = singles ? most_tiles : most_pairs;
    if (most_units <= 0) return 0;
    if (most_units > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    int grid = most_units < n_cu ? (int)most_units : n_cu;
    if (grid >= 8) grid -= grid % 8;          // whole number of workgroups per XCD
    dim3 block(kWWaves * 64);
    if (p.block_table)
        hipLaunchKernelGGL((prefill_fwd_w64_kernel<true, true>), dim3((unsigned)grid), block, 0, stream, p, tiles_per_unit, heads_per_wg);
    else if (p.mask_mode == MI355_MASK_CAUSAL)
        hipLaunchKernelGGL((prefill_fwd_w64_kernel<true, false>), dim3((unsigned)grid), block, 0, stream, p, tiles_per_unit, heads_per_wg);
    else
        hipLaunchKernelGGL((prefill_fwd_w64_kernel<false, false>), dim3((unsigned)grid), block, 0, stream, p, tiles_per_unit, heads_per_wg);
    return (int)hipGetLastError();
}

}  // namespace mi355
