// Prefill forward for head_dim 128 (no mask or causal; optional log-sum-exp output), one wavefront per SIMD, 64
// queries per wavefront.
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
constexpr int kWORow = kWD * 2 + 16; // bytes per row of the query/output staging slab

// Direct-to-LDS load of 16 bytes per lane (see dma_to_lds_16 in common.hpp).  This variant writes m0 inside the
// statement: the assembly loop of this kernel writes m0 too, behind the compiler's back, so nothing here may rely on
// the compiler's idea of what m0 holds.  (m0 cannot be named in a clobber list -- the compiler treats it as reserved
// and warns that clobbering it is undefined -- and it needs no naming: the compiler keeps nothing in m0 across
// statements, it writes m0 directly in front of each of its own instructions that read it.)
__device__ __forceinline__ void dma_to_lds_16_m0(const void* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(gbase), "s"(lds_addr)
                 : "memory");
}

template <bool CAUSAL>
__global__ __launch_bounds__(kWWaves * 64, 1) void prefill_fwd_w64_kernel(PrefillParams p, int n_logical) {
    constexpr int D = kWD, NS = D / 16, NDT = D / 32, CPR = D / 8;
    constexpr float kBias = 32.0f;             // the largest weight sits at 2^-kBias when a reference is set
    constexpr float kUnderflow = 0x1p-92f;     // a row sum below this may have lost terms (see the file header)
    constexpr float kOverflow = 0x1p40f;       // a row sum above this (or NaN) may have overflowed somewhere

    // K buffers 0,1 then V buffers 0,1 (the assembly loop addresses all four relative to one base)
    __shared__ __attribute__((aligned(1024))) unsigned char kv_lds[4 * kWTile];
    __shared__ __attribute__((aligned(16))) unsigned char o_lds[kWWaves * 64 * kWORow];
    unsigned char* const k_lds = kv_lds;
    unsigned char* const v_lds = kv_lds + 2 * kWTile;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;          // query column inside a block / key row of K / d row of V^T
    const int kg = lane >> 5;

    // ---- jobs: a workgroup works through query tiles, one "job" each.  Logical id = (batch, head, tile pair); a
    // pair is the query tiles (nq-1-i, i) of a sequence, so that causal work is the same for every id.  The ids are
    // dealt so that the workgroups resident on one XCD (workgroup ids are dealt round-robin to the 8 XCDs) walk
    // through one contiguous range of ids together and stream the same K/V through that XCD's L2. ----
    struct Job {
        const __bf16 *qb, *kb, *vb;
        __bf16* ob;
        float* lb;                       // row 0 of this (sequence, head) in the log-sum-exp output, or null
        int sq, sk, q0;
    };
    const int G = gridDim.x, bid = blockIdx.x;
    const bool by_xcd = (n_logical % 8 == 0) && (G % 8 == 0);
    int job_k = -1, job_nq = 0, job_pair = 0, job_half = 1;      // position: "after the last query tile of id number job_k"
    Job job_seq{};                                               // sequence-level fields of the current id
    auto next_job = [&](Job& j) -> bool {
        if (job_half == 0 && job_pair != job_nq - 1 - job_pair) {           // second query tile of the pair
            job_half = 1;
            j = job_seq;
            j.q0 = job_pair * kWBM;
            return true;
        }
        job_pair += p.n_pairs;                // a further pair of the same sequence: only if it is longer than Sq_max promised
        while (!(job_k >= 0 && 2 * job_pair < job_nq)) {
            ++job_k;
            int lid;
            if (by_xcd) {
                const int per = n_logical / 8, slot = bid / 8 + job_k * (G / 8);
                if (slot >= per) return false;
                lid = (bid % 8) * per + slot;
            } else {
                lid = bid + job_k * G;
                if (lid >= n_logical) return false;
            }
            const int h = (lid / p.n_pairs) % p.Hq, b = lid / (p.n_pairs * p.Hq), hk = h / (p.Hq / p.Hkv);
            if (p.cu_q) {
                const int q_start = p.cu_q[b], k_start = p.cu_k[b];
                job_seq.sq = p.cu_q[b + 1] - q_start;
                job_seq.sk = p.cu_k[b + 1] - k_start;
                job_seq.qb = p.q + (int64_t)q_start * p.qs[2] + (int64_t)h * p.qs[1];
                job_seq.kb = p.k + (int64_t)k_start * p.ks[2] + (int64_t)hk * p.ks[1];
                job_seq.vb = p.v + (int64_t)k_start * p.vs[2] + (int64_t)hk * p.vs[1];
                job_seq.ob = p.out + (int64_t)q_start * p.os[2] + (int64_t)h * p.os[1];
                job_seq.lb = p.lse ? p.lse + q_start + (int64_t)h * p.ls[1] : nullptr;
            } else {
                job_seq.sq = p.Sq;
                job_seq.sk = p.Sk;
                job_seq.qb = p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[1];
                job_seq.kb = p.k + (int64_t)b * p.ks[0] + (int64_t)hk * p.ks[1];
                job_seq.vb = p.v + (int64_t)b * p.vs[0] + (int64_t)hk * p.vs[1];
                job_seq.ob = p.out + (int64_t)b * p.os[0] + (int64_t)h * p.os[1];
                job_seq.lb = p.lse ? p.lse + (int64_t)b * p.ls[0] + (int64_t)h * p.ls[1] : nullptr;
            }
            job_nq = (job_seq.sq + kWBM - 1) / kWBM;
            job_pair = lid % p.n_pairs;
        }
        job_half = 0;
        j = job_seq;
        j.q0 = (job_nq - 1 - job_pair) * kWBM;
        return true;
    };

    // ---- tile loader: wavefront w, instruction j covers LDS chunks (4w + j)*64 .. +63, i.e. rows 16w + 4j + lane/16;
    // the lane fetches global chunk (lane%16) ^ swz(row) of its row, and swz(row) = ((lane/16) << 2) | j here ----
    const int ld_q = lane >> 4;
    const int ld_c0 = (lane & 15) ^ (ld_q << 2);
    // byte offset of the lane's 16 bytes from the wavefront's first row of step j: row part + ((ld_c0 ^ j) << 4)
    const uint32_t dma_row_k = (uint32_t)(ld_q * (int)p.ks[2] * 2), dma_row_v = (uint32_t)(ld_q * (int)p.vs[2] * 2);
    const uint32_t lds_dst = __builtin_amdgcn_readfirstlane(lds_address(kv_lds + wave * 4096));
    const uint32_t k_step = (uint32_t)(4 * p.ks[2] * 2), v_step = (uint32_t)(4 * p.vs[2] * 2);   // 4 rows, in bytes
    // K (which == 0) or V (which == 1) rows of tile `tile` into that tensor's LDS buffer `buf`
    auto issue_rows = [&](const Job& jb, int which, int tile, int buf) {
        const __bf16* src = which ? jb.vb : jb.kb;
        const int64_t stride = which ? p.vs[2] : p.ks[2];
        const uint32_t step = which ? v_step : k_step, dma_row = which ? dma_row_v : dma_row_k;
        const uint32_t dst = lds_dst + (2 * which + buf) * kWTile;
        if (tile * kWBN + kWBN <= jb.sk) {
            const unsigned char* base = reinterpret_cast<const unsigned char*>(src + ((int64_t)tile * kWBN + 16 * wave) * stride);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                dma_to_lds_16_m0(base + (size_t)j * step, dma_row + ((ld_c0 ^ j) << 4), dst + j * 1024);
        } else {
            // last, partial tile: rows past the end re-read the last row (finite; their scores are masked).
            // (The empty statement keeps the address arithmetic of this rare path inside the branch: hoisted to
            // the top of the job it occupied two dozen registers that then lived in scratch memory.)
            int last = jb.sk - 1 - tile * kWBN;
            asm volatile("" : "+s"(last));
            const unsigned char* t0 = reinterpret_cast<const unsigned char*>(src + (int64_t)tile * kWBN * stride);
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
        if (CAUSAL) kv_end = max(0, min(jb.sk, min(jb.sq, jb.q0 + kWBM) + (jb.sk - jb.sq)));
        return (kv_end + kWBN - 1) / kWBN;
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

    // The staging slab of the wavefront: its 64 query rows during a job (the assembly loop loads its fragments from
    // here whenever it starts, ordinary code reads them as it needs them), the output rows at the end of the job.
    unsigned char* const slab = o_lds + wave * (64 * kWORow);
    const uint32_t q_addr = lds_address(slab + n * kWORow + 8 * kg * 2);
    auto qfrag = [&](int c, int s) { return as_bf16x8(lds_load_at<u32x4>(q_addr + c * 32 * kWORow + 32 * s)); };
    constexpr int kRowsPerPass = 64 / CPR;           // the slab is filled and emptied 4 whole rows at a time, 16 passes
    const int c16 = lane % CPR, r0 = lane / CPR;

    // What a job needs before it can start is requested as early as possible -- for the first job right here, for
    // every other one while the job before it normalises and stores its output: K[0] (direct-to-LDS), the wavefront's
    // query rows (into registers; rows past the end of the sequence are zero), then K[1] and V[0].
    u32x4 q_rows[64 / kRowsPerPass];
    auto prefetch = [&](const Job& jb) {
        const int nt = tiles_of(jb);
        if (nt > 0) issue_k(jb, 0, 0);
        const int qw0 = jb.q0 + 64 * wave;
        // (the row addresses are derived from a value the compiler cannot trace, so that it computes them here and
        // not at the top of the job, where sixteen 64-bit addresses would have to wait in registers)
        // (an offset, not the pointer, goes through the empty statement: a pointer would come back without its
        // address space and the loads would become flat ones, which also count as LDS operations)
        int64_t my_off = (int64_t)(qw0 + r0) * p.qs[2] + c16 * 8;
        asm volatile("" : "+v"(my_off));
        const __bf16* my_rows = jb.qb + my_off;
#pragma unroll
        for (int i = 0; i < 64 / kRowsPerPass; ++i) {
            const int r = i * kRowsPerPass + r0;
            q_rows[i] = u32x4{0u, 0u, 0u, 0u};
            if (qw0 + i * kRowsPerPass < jb.sq) {          // (wave-uniform: see row_passes)
                if (qw0 + r < jb.sq) q_rows[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(my_rows + (int64_t)(i * kRowsPerPass) * p.qs[2]));
            }
        }
        if (nt > 1) issue_k(jb, 1, 1);
        if (nt > 0) issue_v(jb, 0, 0);
    };
    // number of row instructions (loads of query rows, stores of output rows: four rows each) a job issues: a pass
    // whose four rows all lie past the end of the sequence is jumped over, so the count is known here
    auto row_passes = [&](const Job& jb) {
        return min(max((jb.sq - (jb.q0 + 64 * wave) + kRowsPerPass - 1) / kRowsPerPass, 0), 64 / kRowsPerPass);
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
    bool have = next_job(cur);
    if (have) prefetch(cur);
    int prev_stores = 0;                                   // output row stores of the job before `cur`
    while (have) {
        const int sq = cur.sq, sk = cur.sk, q0 = cur.q0;
        const int coff = sk - sq;                          // bottom-right aligned causal diagonal
        const int qw0 = q0 + 64 * wave;                    // first query of this wavefront
        const int n_tiles = tiles_of(cur);
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
        const int young_rows = row_passes(cur) + prev_stores;

        // query rows: registers -> slab (the previous job has read its output rows back from the slab by now: LDS
        // operations of a wavefront execute in order)
#pragma unroll
        for (int i = 0; i < 64 / kRowsPerPass; ++i)
            *reinterpret_cast<u32x4*>(slab + (i * kRowsPerPass + r0) * kWORow + c16 * 16) = q_rows[i];

        // Two attempts at most: the first with the references preset to 0, the second -- only if some row's sum came
        // out suspiciously small or large -- entirely in ordinary code with references taken from the data.
        bool have_next = false;
        for (int attempt = 0; attempt < 2; ++attempt) {
        const bool preset = attempt == 0;
        const int young_dma = (n_tiles > 1 ? 4 : 0) + (n_tiles > 0 ? 4 : 0);      // requests of K[1] and V[0]
        if (!preset) {                        // start over: the buffers are free (everybody passed the vote below)
            if (n_tiles > 0) issue_k(cur, 0, 0);
            if (n_tiles > 1) issue_k(cur, 1, 1);
            if (n_tiles > 0) issue_v(cur, 0, 0);
        }
        asm volatile(W64_ZERO : : "v"(as_bf16x8(u32x4{0u, 0u, 0u, 0u})) : W64_CLOBBER_ACC);      // O^T and the row sums
        // per column block: r_ref exponent reference in the log2 domain (-inf: none yet), nb = -r_ref - kBias
        float r_ref[2], nb[2];
        r_ref[0] = r_ref[1] = preset ? 0.f : -INFINITY;
        nb[0] = nb[1] = preset ? -kBias : 0.f;
        bool redo = false;                    // a row sum left the range in which no term can have been lost
        // The first boundary of a query tile need not wait for the row stores of the query tile before it: they
        // are younger than every request in flight (first attempt only, and only when their number is the usual 16).
        bool first_boundary = preset && prev_stores == 16;

        // Wait for K[0] and meet the others.  Younger than its request are: on the first attempt this job's query row
        // loads and the previous job's output row stores (each issued once per four rows that exist), and on both
        // the requests of K[1] and V[0].
        wait_all_but(young_dma + (preset ? young_rows : 0));
        __syncthreads();

        // Scores of one 32-key half of a tile for one column block, in ordinary code (reads K[tile]).
        auto scores = [&](auto c_c, int tile, int t) {
            constexpr int c = decltype(c_c)::value;
            const int buf = tile & 1;
            f32x16 s_acc;
#pragma unroll
            for (int j = 0; j < 16; ++j) s_acc[j] = 0.f;
            // (all fragment reads first, then the MFMAs: one LDS latency instead of eight)
            u32x4 kf[NS];
            bf16x8 qf[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                kf[s] = lds_load_at<u32x4>(rd_k(s) + buf * kWTile + t * 32 * kWRow);
                qf[s] = qfrag(c, s);
            }
#pragma unroll
            for (int s = 0; s < NS; ++s) s_acc = mfma32(as_bf16x8(kf[s]), qf[s], s_acc);
            return s_acc;
        };
        // The rest of that half: mask, reference move, weights, accumulation (reads V[tile]).
        auto finish = [&](auto c_c, int tile, int t, bool masked, f32x16 s_acc) {
            constexpr int c = decltype(c_c)::value;
            const int buf = tile & 1;
            const int k0 = tile * kWBN + 32 * t;
            const int qi = qw0 + 32 * c + n;
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float x = fmaf(s_acc[i], p.scale_log2, nb[c]);
                if (masked) {
                    const int key = k0 + 8 * (i >> 2) + 4 * kg + (i & 3);
                    bool keep = key < sk;
                    if (CAUSAL) keep = keep & (key <= qi + coff);
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
        auto boundary = [&](int tile) {
            if (first_boundary) wait_vmcnt<16>(); else wait_vmcnt<0>();
            first_boundary = false;
            __syncthreads();
            if (tile + 1 < n_tiles) issue_v(cur, tile + 1, (tile + 1) & 1);
            if (tile + 2 < n_tiles) issue_k(cur, tile + 2, tile & 1);
        };
        // a whole tile in ordinary code: scores from K[tile], boundary, everything else from V[tile]
        // (a tile past n_mask has nothing for this wavefront: it only takes part in the boundary)
        auto step_cxx = [&](int tile) {
            const bool visible = tile < n_mask, masked = tile >= n_plain;
            constexpr std::integral_constant<int, 0> A{};
            constexpr std::integral_constant<int, 1> B{};
            f32x16 sa0{}, sb0{}, sa1{}, sb1{};
            if (visible) {
                sa0 = scores(A, tile, 0);
                sb0 = scores(B, tile, 0);
                sa1 = scores(A, tile, 1);
                sb1 = scores(B, tile, 1);
            }
            boundary(tile);
            if (visible) {
                finish(A, tile, 0, masked, sa0);
                finish(B, tile, 0, masked, sb0);
                finish(A, tile, 1, masked, sa1);
                finish(B, tile, 1, masked, sb1);
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

        int tile = 0;
        const int n_loop = preset ? n_asm : 0;
        while (tile < n_tiles) {
            if (tile >= n_loop) {
                step_cxx(tile);
                ++tile;
                continue;
            }
            // ---- the hand-scheduled loop over tiles [tile, n_loop); leaves after a tile that took a row sum to 2 ----
            const uint64_t kptr = (uint64_t)(uintptr_t)(cur.kb + ((int64_t)(tile + 2) * kWBN + 16 * wave) * p.ks[2]);
            const uint64_t vptr = (uint64_t)(uintptr_t)(cur.vb + ((int64_t)(tile + 1) * kWBN + 16 * wave) * p.vs[2]);
            // mask thresholds for the first masked tile the loop will meet: a key at index j of that tile is kept by
            // query i of the wavefront iff j <= i + (qw0 + coff - k0) and j < sk - k0 (the lane part 4*kg of a key's
            // index is folded in)
            const int k0m = max(tile, n_plain) * kWBN;
            const int diag = CAUSAL ? qw0 + coff - k0m : (1 << 20);
            // vector operands: read once when the block starts, scratch registers of the block afterwards
            float v_nb0 = nb[0], v_nb1 = nb[1];
            int v_thr0 = min(n + diag, sk - 1 - k0m) - 4 * kg, v_thr1 = min(n + 32 + diag, sk - 1 - k0m) - 4 * kg;
            uint32_t v_sum = sum_word, v_k0 = rd_k0, v_vlo = rd_vlo0, v_vhi = rd_vhi0;
            uint32_t v_rowk = dma_row_k, v_rowv = dma_row_v, v_c0s = (uint32_t)(ld_c0 << 4), v_q = q_addr;
            int status;
            int tile_s = __builtin_amdgcn_readfirstlane(tile);
            asm volatile(W64_LOOP
                : [tile] "+&s"(tile_s), [t2] "=&s"(status),
                  [nb0] "+v"(v_nb0), [nb1] "+v"(v_nb1), [suma] "+v"(v_sum), [k0] "+v"(v_k0), [vlo0] "+v"(v_vlo),
                  [vhi0] "+v"(v_vhi), [rowk] "+v"(v_rowk), [rowv] "+v"(v_rowv), [c0s] "+v"(v_c0s), [qaddr] "+v"(v_q),
                  [thr0] "+v"(v_thr0), [thr1] "+v"(v_thr1)
                : [n_tiles] "s"(__builtin_amdgcn_readfirstlane(n_tiles)), [n_end] "s"(__builtin_amdgcn_readfirstlane(n_loop)),
                  [n_pipe] "s"(__builtin_amdgcn_readfirstlane(min(n_plain, n_loop))), [n_mask] "s"(__builtin_amdgcn_readfirstlane(n_mask)),
                  [aligned] "s"(__builtin_amdgcn_readfirstlane(aligned)), [first] "s"(__builtin_amdgcn_readfirstlane((int)first_boundary)),
                  [kstep] "s"(__builtin_amdgcn_readfirstlane(k_step)), [vstep] "s"(__builtin_amdgcn_readfirstlane(v_step)),
                  [ldsdst] "s"(lds_dst), [scale] "s"(__builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, p.scale_log2))),
                  [klo] "s"(__builtin_amdgcn_readfirstlane((uint32_t)kptr)), [khi] "s"(__builtin_amdgcn_readfirstlane((uint32_t)(kptr >> 32))),
                  [vlo] "s"(__builtin_amdgcn_readfirstlane((uint32_t)vptr)), [vhi] "s"(__builtin_amdgcn_readfirstlane((uint32_t)(vptr >> 32)))
                : "memory", "vcc", "scc", "s36", "s37", "s38", "s39", "s40", "s41", "s42", "s43", W64_CLOBBER_ACC, W64_CLOBBER_LOOP_VGPRS);
            if (tile_s > tile) first_boundary = false;      // (every tile the block ran had its boundary)
            tile = tile_s;
            // status 0: tiles up to n_loop done.  1: tiles up to `tile` done, and the last of them took a row sum to 2.
            if (status != 0) {
                move_references(std::integral_constant<int, 0>{});
                move_references(std::integral_constant<int, 1>{});
            }
        }

        // ---- row sums; the workgroup meets (everybody is done with the K/V buffers) and, on the first attempt,
        // votes on doing the query tile again ----
        float l_row[2];
        const auto read_sums = [&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            float s_lo, s_hi;
            acc_read_sums<c>(s_lo, s_hi);
            const float l_lo = __shfl(s_lo, lane & 15, 64), l_hi = __shfl(s_hi, lane & 15, 64);
            l_row[c] = (n & 16) ? l_hi : l_lo;
        };
        read_sums(std::integral_constant<int, 0>{});
        read_sums(std::integral_constant<int, 1>{});
        if (preset) {
            // (rows past the end of the sequence count too: their sums are sk * 2^-32, far above the lower limit)
            const bool bad = redo || !(l_row[0] >= kUnderflow) || !(l_row[1] >= kUnderflow) || !(l_row[0] <= kOverflow) ||
                             !(l_row[1] <= kOverflow);
            if (__syncthreads_or(bad ? 1 : 0)) continue;
        } else {
            __syncthreads();
        }

        // the next job's first tiles and query rows are on their way while this one finishes
        have_next = next_job(nxt);
        if (have_next) prefetch(nxt);

        // ---- normalise: lane owns query qw0 + 32c + n, d = 32dt + 8(i/4) + 4kg + i%4 ----
        const auto store_block = [&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            const float inv = 1.0f / l_row[c];     // l == 0 (no key kept) -> NaN row, like the reference softmax
            // sum_j exp(scale * s_j) = l * 2^(-nb)  ->  lse = ln2 * (log2 l - nb); no key kept -> -inf
            if (cur.lb && kg == 0 && qw0 + 32 * c + n < sq)
                cur.lb[qw0 + 32 * c + n] = l_row[c] > 0.f ? 0.69314718056f * (__log2f(l_row[c]) - nb[c]) : -INFINITY;
            unsigned char* mine = slab + (32 * c + n) * kWORow + 8 * kg;
            const auto store_dt = [&](auto dt_c) {
                constexpr int dt = decltype(dt_c)::value;
                float x[16];
                acc_read<c, dt>(x);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = pack_bf16(x[4 * g + 0] * inv, x[4 * g + 1] * inv);
                    w[1] = pack_bf16(x[4 * g + 2] * inv, x[4 * g + 3] * inv);
                    *reinterpret_cast<u32x2*>(mine + (32 * dt + 8 * g) * 2) = w;
                }
            };
            store_dt(std::integral_constant<int, 0>{});
            store_dt(std::integral_constant<int, 1>{});
            store_dt(std::integral_constant<int, 2>{});
            store_dt(std::integral_constant<int, 3>{});
        };
        store_block(std::integral_constant<int, 0>{});
        store_block(std::integral_constant<int, 1>{});
        break;
        }   // attempts
        // ---- output rows leave whole, through the slab (written once, never read here: non-temporal, like the
        // query rows, so that the K/V tiles keep the L2 to themselves) ----
        int64_t out_off = (int64_t)(qw0 + r0) * p.os[2] + c16 * 8;
        asm volatile("" : "+v"(out_off));                  // (as for the query rows: addresses computed here, not earlier)
        __bf16* my_out = cur.ob + out_off;
#pragma unroll
        for (int i = 0; i < 64 / kRowsPerPass; ++i) {
            const int r = i * kRowsPerPass + r0;
            const u32x4 w = *reinterpret_cast<const u32x4*>(slab + r * kWORow + c16 * 16);
            if (qw0 + i * kRowsPerPass < sq) {             // (wave-uniform: see row_passes)
                if (qw0 + r < sq) __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(my_out + (int64_t)(i * kRowsPerPass) * p.os[2]));
            }
        }
        prev_stores = row_passes(cur);
        cur = nxt;
        have = have_next;
    }
}

int launch_prefill_w64(const PrefillParams& p, hipStream_t stream) {
    // One resident workgroup per compute unit, each working through its share of the (batch, head, tile pair) ids.
    int dev = 0, n_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    const int n_logical = p.n_pairs * p.Hq * p.B;
    if (n_logical <= 0) return 0;
    int grid = n_logical < n_cu ? n_logical : n_cu;
    if (n_logical % 8 == 0 && grid >= 8) grid -= grid % 8;          // whole number of workgroups per XCD
    dim3 block(kWWaves * 64);
    if (p.mask_mode == MI355_MASK_CAUSAL)
        hipLaunchKernelGGL((prefill_fwd_w64_kernel<true>), dim3((unsigned)grid), block, 0, stream, p, n_logical);
    else
        hipLaunchKernelGGL((prefill_fwd_w64_kernel<false>), dim3((unsigned)grid), block, 0, stream, p, n_logical);
    return (int)hipGetLastError();
}

}  // namespace mi355
