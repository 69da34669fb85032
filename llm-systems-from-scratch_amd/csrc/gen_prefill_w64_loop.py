#!/usr/bin/env python3
"""Writes prefill_w64_asm.inc: the hand-scheduled tile loop of prefill_fwd_w64.hip as inline-assembly text.

Why assembly: with one wavefront per SIMD and 64 query columns per wavefront the output accumulators (128 registers)
and the query fragments (64) must live in AGPRs while the score accumulators must live in VGPRs (the exponentials read
them), and the vector and LDS instructions must sit in the shadow of the MFMAs at a fixed rhythm.  The compiler offers
neither (it picks one register form for every MFMA of a function and clusters the vector work), so the loop over the
K/V tiles of a query tile is generated here, instruction by instruction, and included by the kernel as a string.
What stays ordinary HIP C++: prologue, epilogue, ragged ends, and moving a row's exponent reference.

One tile = 64 keys; a wavefront owns 64 queries = column blocks A and B of 32; head_dim 128.  Per 32-key half h of
tile t there are three pieces of work (each for both blocks):
  S(t,h)  scores   = K[t][32h:32h+32] . Q^T         16 MFMA 32x32x16 (8 per block), K fragments from LDS
  E(t,h)  weights  = bf16(2^(S * scale + nb))       32 v_fma, 32 v_exp, 16 cvt (a masked tile adds a compare and a
                                                    select per score)
  O(t,h)  O^T     += V[t][32h:32h+32]^T . P, l += row sums   16 MFMA + 4 row-sum MFMA 16x16x32, V^T fragments from LDS
With one wavefront per SIMD the vector work of a half hides only behind MFMAs of the same wavefront that do not
depend on it.  Unmasked tiles therefore run as a software pipeline across tiles, two half-steps per tile:
  H0(t):  S(t,1)   | E(t,0) | O(t-1,1)
  H1(t):  S(t+1,0) | E(t,1) | O(t,0)
so every half-step carries 36 MFMAs and one half's vector work.  The pipeline is filled by a prologue (S(t,0), then
H0 without its O part) and emptied by an epilogue (H1 without its S part, then O(t,1)).  Masked tiles (the causal
diagonal) run one at a time: S(t,0); S(t,1) | E(t,0); O(t,0) | E(t,1); O(t,1).

Tile hand-over ("boundary") -- the protocol every wavefront of the workgroup follows once per tile, here and in the
C++ steps of the kernel.  K[t] and V[t] live in LDS buffers t % 2 (one pair of buffers for K, one for V).
  when tile t starts: K[t] has landed and the workgroup has met since; K[t+1] and V[t] are in flight
  boundary(t):        this wavefront has read all it needs of K[t] and V[t-1]; it waits for its own shares of
                      K[t+1] and V[t], meets the others at a barrier, and requests K[t+2] and V[t+1] into the
                      buffers just freed
  afterwards:         it reads V[t] (and K[t+1])
In the pipeline the boundary sits inside H0(t), behind three quarters of its MFMAs; the last quarter (whose
fragments are in registers by then) covers the latency of the first reads of K[t+1] and V[t], and the requests are
issued between its MFMAs.

Weights are 2^(score * scale + nb) with nb preset by the caller (see the kernel); nothing here looks at row maxima.
At the end of each tile the row sums are looked at, and a sum >= 2 ends the block after that tile with status 1: the
caller lowers nb of the rows that need it, rescales, and re-enters.

Tiles come in three kinds, by index: [0, n_plain) every key visible to every query; [n_plain, n_mask) masked (causal
diagonal: key <= threshold of the lane's query; the threshold moves down by 64 per tile); [n_mask, n_end) nothing
visible for this wavefront -- it only takes part in the boundary.  When the diagonal is aligned with the tiles
(operand `aligned`: query i of the wavefront sees key j of the one masked tile iff j <= i) that tile takes a cheaper
body: only the two triangular 32x32 sub-blocks get mask code, and the invisible one is neither scored nor accumulated.

Register map (physical, fixed; the block loads them itself from its operands, see entry()):
  v[0:31]   S(A,0), S(B,0)     v[32:63]  S(A,1), S(B,1)
  v[64:79]  P(.,0): A slices 0,1 then B slices 0,1 (a slice = 16 keys = 4 registers)     v[80:95] P(.,1)
  v96 / v97 nb (the additive term of the exponent) of this lane's query in block A / B
  v98 -inf, v99 / v100 mask threshold of the lane's query in block A / B (key index inside the tile, minus 4*(lane/32))
  v[102:105] A operand of the row-sum MFMA
  v[106:113] K fragment LDS addresses per step, v[114:121] V^T LDS addresses [half][d-tile] (both for buffer 0; the
  buffer and the position inside the tile are immediates; V tiles sit two tile sizes behind the K tiles),
  v[122:129] lane offsets of the direct-to-LDS loads (K steps 0..3, V steps 0..3)
  twelve more registers, wherever the compiler puts the block's vector operands: after entry() they serve as scratch
  (exponentials on their way to packing)
  a[0:63] O^T of block A (d-tile dt = a[16dt:16dt+15]), a[64:127] block B, a[128:131] / a[132:135] row sums:
  these live in the AGPRs for a whole query tile and are touched only by the assembly snippets below (the kernel
  is compiled with its builtin MFMAs in VGPR form, so the compiler has no use for AGPRs of its own)
  a[136:167] Q^T fragments of block A (step s = a[136+4s:139+4s]), a[168:199] block B: loaded from LDS by the
  W64_QFRAGS statement before the block first runs for a query tile; they stay across re-entries
  a[200:215] K fragments (4 in flight), a[216:247] V^T fragments (8: 2 slices x 4 d-tiles): LDS reads land in
  AGPRs directly and the MFMAs take them as A operands, which leaves the vector registers to the compiler
  s[36:37] / s[38:39] global address of the wavefront's first DMA row of K[t+2] / V[t+1] (advanced per tile),
  s40 / s41 bytes from one tile to the next in K / V, s42 "a row sum reached 2"; every other scalar is a named operand

The block-table variant (W64_LOOP_PAGED: K and V live in a paged cache of 16-row blocks, and a wavefront's share of a
tile -- 16 rows -- is exactly one block).  It differs in where the two addresses come from, nothing else: operand
`ids` holds, in lane l, the physical block of this wavefront's share of tile (first tile of this entry) + 1 + l;
s40 / s41 are the lanes of K[t+2] / V[t+1]; after a tensor's four requests its lane moves on by one and the address
becomes base (operands klo:khi / vlo:vhi: block 0 of the K/V head) + id * blk (operand: bytes per block), s43 / s44
scratch.  The caller sizes an entry so that no lane beyond 63 is ever used for a request: at most 63 tiles per entry.
"""
import os
import sys

EXP = "v_exp_f32"
S = {("A", 0): 0, ("B", 0): 16, ("A", 1): 32, ("B", 1): 48}
P = {0: {"A": 64, "B": 72}, 1: {"A": 80, "B": 88}}          # + 4 * slice inside the half
KF = 200                            # AGPRs: LDS reads land there directly, the MFMAs take them as A operands
VF = 216                            # AGPRs: fragment j (slice j // 4 of the half, d-tile j % 4) at VF + 4j
NB = {"A": 96, "B": 97}
NEGINF = 98
THR = {"A": 99, "B": 100}
SUMA = 102                          # (register tuples of MFMA operands start at even registers)
KOFF, VOFF, DMAOFF = 106, 114, 122
N_FIXED_VGPRS = 130
# Scratch registers are the block's vector operands themselves: each is read once by entry() and is free from then on
# (the operands are declared in/out), so the block needs no register beyond v[0:129] and its operands.
ETMP = ["%[nb0]", "%[nb1]", "%[suma]", "%[k0]", "%[vlo0]", "%[vhi0]", "%[rowk]", "%[rowv]"]   # exponentials on their way to packing
TMP = "v0"                          # scratch of entry() (the score registers hold nothing yet)
OREG = {"A": 0, "B": 64}
LREG = {"A": 128, "B": 132}
QREG = {"A": 136, "B": 168}
N_ACC = 136                         # a[0:135]: what ordinary code reaches through the snippets
N_AGPRS = 248
KPTR, VPTR, FLAG, KSTEP16, VSTEP16 = 36, 38, 42, 40, 41
KLANE, VLANE, PTMP = 40, 41, 43     # block-table variant: lanes of `ids` for K[t+2] / V[t+1]; two scratch registers
PAGED = False                       # which variant is being generated
K_TILE = 16384                      # bytes of one K (or V) tile in LDS: 64 rows x 256 bytes
ROW = 256
NONE = {"A": False, "B": False}


def rng(base, n):
    return f"[{base}:{base + n - 1}]"


class Emitter:
    """Collects instructions and keeps count of the LDS reads in flight, so that every consumer of a fragment is
    preceded by the s_waitcnt that its own read needs and no more."""

    def __init__(self):
        self.lines = []
        self.pending = []            # destination base registers of LDS reads in flight, oldest first

    def raw(self, text):
        self.lines.append(text)

    def lds_read(self, text, dst):
        if len(self.pending) == 15:          # the counter holds 15: retire the oldest read (issued long ago) first
            self.lines.append("s_waitcnt lgkmcnt(14)")
            self.pending.pop(0)
        self.lines.append(text)
        self.pending.append(dst)

    def need(self, *regs):
        """Wait until the reads into the given destination registers have returned."""
        last = -1
        for i, d in enumerate(self.pending):
            if d in regs:
                last = i
        if last >= 0:
            left = len(self.pending) - 1 - last
            self.lines.append(f"s_waitcnt lgkmcnt({left})")
            self.pending = self.pending[last + 1:]

    def drain(self):
        if self.pending:
            self.lines.append("s_waitcnt lgkmcnt(0)")
            self.pending = []


def mfma_s(c, h, slot, s):
    """S(c,h) (+)= K fragment in `slot` . Q^T fragment of step s."""
    dst = S[(c, h)]
    cs = "0" if s == 0 else f"v{rng(dst, 16)}"
    return f"v_mfma_f32_32x32x16_bf16 v{rng(dst, 16)}, a{rng(KF + 4 * slot, 4)}, a{rng(QREG[c] + 4 * s, 4)}, {cs}"


def mfma_o(c, j, p):
    """O^T(c, d-tile j % 4) += V^T fragment j . P words at p."""
    acc = OREG[c] + 16 * (j % 4)
    return f"v_mfma_f32_32x32x16_bf16 a{rng(acc, 16)}, a{rng(VF + 4 * j, 4)}, v{rng(p, 4)}, a{rng(acc, 16)}"


def mfma_sum(c, p):
    acc = LREG[c]
    return f"v_mfma_f32_16x16x32_bf16 a{rng(acc, 4)}, v{rng(SUMA, 4)}, v{rng(p, 4)}, a{rng(acc, 4)}"


def k_read(e, buf, h, s, slot):
    e.lds_read(f"ds_read_b128 a{rng(KF + 4 * slot, 4)}, v{KOFF + s} offset:{buf * K_TILE + h * 32 * ROW}", KF + 4 * slot)


def v_read(e, buf, h, j):
    """V^T fragment j of half h (16-key slice 2h + j // 4, d-tile j % 4) into its registers (two transposed 64-bit reads)."""
    off = buf * K_TILE + 16 * (2 * h + j // 4) * ROW
    base, dt = VF + 4 * j, j % 4
    e.lds_read(f"ds_read_b64_tr_b16 a{rng(base, 2)}, v{VOFF + dt} offset:{off}", base)
    e.lds_read(f"ds_read_b64_tr_b16 a{rng(base + 2, 2)}, v{VOFF + 4 + dt} offset:{off}", base + 2)


def vneeds(j):
    return (VF + 4 * j, VF + 4 * j + 2)


def exp_ops(h, mask, blocks="AB"):
    """Vector work that turns S(c,h), c in `blocks`, into packed bf16 weights P(c,h).  The result of a transcendental
    may not feed the next vector instruction, so the packing of a pair trails its exponentials.  Accumulator register
    i of a lane holds key 32h + 8(i/4) + 4(lane/32) + i%4 of the tile; where mask[c] is set the score is kept only if
    that index is <= the lane's threshold (the lane part of the index is folded into the threshold)."""
    ops, pend = [], []
    i = 0
    for c in blocks:
        dst = P[h][c]
        for w in range(8):                      # packed word w of the block: accumulator registers 2w, 2w+1
            t0, t1 = ETMP[2 * (i % 4)], ETMP[2 * (i % 4) + 1]
            for tmp, r in ((t0, 2 * w), (t1, 2 * w + 1)):
                ops.append(f"v_fma_f32 {tmp}, v{S[(c, h)] + r}, %[scale], v{NB[c]}")
                if mask[c]:
                    ops.append(f"v_cmp_le_i32_e64 vcc, {32 * h + 8 * (r // 4) + r % 4}, v{THR[c]}")
                    ops.append(f"v_cndmask_b32 {tmp}, v{NEGINF}, {tmp}, vcc")
            ops.append(f"{EXP} {t0}, {t0}")
            ops.append(f"{EXP} {t1}, {t1}")
            ops += pend
            pend = [f"v_cvt_pk_bf16_f32 v{dst + w}, {t0}, {t1}"]
            i += 1
    ops += pend          # (the packing of the word before sits between the last exponentials and their packing)
    return ops


def issue_cost(text):
    """Issue time of a non-MFMA instruction in cycles, as the microbenchmarks show it next to an MFMA stream."""
    return 8 if text.startswith("v_exp") else 4


def plan(e, mfmas, valu, hold=0, span=None):
    """Distributes the vector instructions behind the MFMAs so that every gap between two MFMAs carries about the same
    issue time (a wavefront issues one instruction per four cycles, and what does not fit under an MFMA delays the
    next one): the LDS reads and waits that belong to fixed MFMAs are counted first, the vector instructions fill
    up to the average.  None goes behind the first `hold` MFMAs -- the vector work reads accumulators that the MFMAs
    just before it wrote, and the hardware does not interlock that dependency (a result is visible 8 passes after
    its MFMA started; `hold` MFMAs of other chains in between cover that) -- and none behind MFMA `span` and later.
    `mfmas` entries are (text, needs, post): registers whose LDS reads must have returned, and a callback run right
    after the MFMA (it issues the LDS reads that refill the registers the MFMA has just consumed).
    Returns entries (text, needs, post, vector instructions that follow, issue time of the gap's fixed part --
    doubled behind the short row-sum MFMAs)."""
    n = len(mfmas)
    span = n if span is None else span
    fixed = [0] * n
    for i, (text, needs, post) in enumerate(mfmas):
        if post:                                   # dry run of the callback: how many instructions does it issue?
            n0, p0 = len(e.lines), list(e.pending)
            post()
            fixed[i] += sum(issue_cost(t) for t in e.lines[n0:])
            del e.lines[n0:]
            e.pending = p0
        if needs and i:
            fixed[i - 1] += 4                      # the wait in front of this MFMA sits in the previous gap
    weight = [0.5 if "16x16x32" in t or t.startswith("s_nop") else 1.0 for t, _, _ in mfmas]
    elig = range(hold, span)
    total = sum(fixed[i] for i in elig) + sum(issue_cost(v) for v in valu)
    wsum = sum(weight[i] for i in elig) or 1.0
    out, vi, cum, wcum = [], 0, 0.0, 0.0
    for i, (text, needs, post) in enumerate(mfmas):
        mine = []
        if hold <= i < span:
            cum += fixed[i]
            wcum += weight[i]
            target = total * wcum / wsum
            while vi < len(valu) and (i == span - 1 or cum + issue_cost(valu[vi]) / 2 <= target):
                mine.append(valu[vi])
                cum += issue_cost(valu[vi])
                vi += 1
        out.append((text, needs, post, mine, fixed[i] * (2.0 if weight[i] < 1.0 else 1.0)))
    assert vi == len(valu)
    return out


def emit(e, entries, extras=()):
    """Emits planned entries; `extras` (groups of instructions that must stay together, e.g. the m0 write and its
    direct-to-LDS load) go behind the MFMAs too, again so that the gaps carry equal issue time."""
    extras = list(extras)
    cost_x = [sum(issue_cost(t) for t in x) for x in extras]
    gap = [f + sum(issue_cost(v) for v in valu) for (_, _, _, valu, f) in entries]
    total = sum(gap) + sum(cost_x)
    n, xi, cum = len(entries), 0, 0.0
    for i, (text, needs, post, valu, _) in enumerate(entries):
        if needs:
            e.need(*needs)
        e.raw(text)
        if post:
            post()
        for v in valu:
            e.raw(v)
        cum += gap[i]
        target = total * (i + 1) / n
        while xi < len(extras) and (i == n - 1 or cum + cost_x[xi] / 2 <= target):
            for x in extras[xi]:
                e.raw(x)
            cum += cost_x[xi]
            xi += 1


def check_sums(e, flagged_label):
    """End of a tile: has a row sum reached 2 (or become NaN)?  Then control goes to `flagged_label`.  Lanes 0..15 of
    the first two registers of each row-sum accumulator hold the sums, everything else there is zero; the last
    row-sum MFMA was issued at least eight MFMAs ago."""
    t = ETMP
    e.raw(f"v_accvgpr_read_b32 {t[0]}, a{LREG['A']}")
    e.raw(f"v_accvgpr_read_b32 {t[1]}, a{LREG['A'] + 1}")
    e.raw(f"v_accvgpr_read_b32 {t[2]}, a{LREG['B']}")
    e.raw(f"v_accvgpr_read_b32 {t[3]}, a{LREG['B'] + 1}")
    e.raw(f"v_max3_f32 {t[0]}, {t[0]}, {t[1]}, {t[2]}")
    e.raw(f"v_max_f32 {t[0]}, {t[0]}, {t[3]}")
    e.raw(f"v_cmp_nlt_f32_e64 vcc, {t[0]}, 2.0")
    e.raw("s_nop 1")
    e.raw(f"s_cbranch_vccnz {flagged_label}")


def dma_chunks(which, buf):
    """Instruction groups that request K[t+2] into K buffer `buf` ("k" in which) and V[t+1] into V buffer buf ^ 1
    ("v" in which), and advance the pointers by a tile.  The four loads of a tensor share the scalar base: the
    distance between them (four rows) is part of the lane offsets."""
    chunks = []
    for name, j0, ptr, step, lds0 in (("v", 4, VPTR, VSTEP16, 2 * K_TILE + (buf ^ 1) * K_TILE), ("k", 0, KPTR, KSTEP16, buf * K_TILE)):
        if name not in which:
            continue
        for j in range(4):
            c = [f"s_add_u32 m0, %[ldsdst], {lds0 + j * 1024}", "s_nop 0"]
            c.append(f"global_load_lds_dwordx4 v{DMAOFF + j0 + j}, s[{ptr}:{ptr + 1}]")
            chunks.append(c)
        if PAGED:
            lane = KLANE if name == "k" else VLANE
            addr = block_address(name)
            chunks.append([f"s_add_u32 s{lane}, s{lane}, 1"] + addr[:2])
            chunks.append(addr[2:])
        else:
            chunks.append([f"s_add_u32 s{ptr}, s{ptr}, s{step}", f"s_addc_u32 s{ptr + 1}, s{ptr + 1}, 0"])
    return chunks


def block_address(name):
    """Block-table variant: s[ptr:ptr+1] of tensor `name` <- base + ids[lane] * blk.  (A scalar instruction may read
    the register that v_readlane wrote right away; the address is read by a memory instruction only much later.)"""
    ptr, lane, lo, hi = (KPTR, KLANE, "%[klo]", "%[khi]") if name == "k" else (VPTR, VLANE, "%[vlo]", "%[vhi]")
    return [f"v_readlane_b32 s{PTMP}, %[ids], s{lane}",
            f"s_mul_hi_u32 s{PTMP + 1}, s{PTMP}, %[blk]",
            f"s_mul_i32 s{PTMP}, s{PTMP}, %[blk]",
            f"s_add_u32 s{ptr}, {lo}, s{PTMP}",
            f"s_addc_u32 s{ptr + 1}, {hi}, s{PTMP + 1}"]


def wait_and_meet(e):
    """First half of a boundary: all LDS reads of this wavefront have returned, its shares of K[t+1] and V[t] have
    landed, and every wavefront of the workgroup is here."""
    e.raw("; boundary")
    e.drain()
    e.raw("s_waitcnt vmcnt(0)")
    e.raw("s_barrier")


def boundary_plain(e, buf, tag, after):
    """A whole boundary with nothing to interleave: the requests are jumped over when their tiles do not exist.
    `after` emits what follows the barrier and precedes the requests (LDS reads of the data that has just landed)."""
    wait_and_meet(e)
    after()
    e.raw("s_add_u32 %[t2], %[tile], 1")
    e.raw("s_cmp_ge_u32 %[t2], %[n_tiles]")
    e.raw(f"s_cbranch_scc1 6{tag}f")                       # no tile t+1: nothing to request
    for c in dma_chunks("v", buf):
        for x in c:
            e.raw(x)
    e.raw("s_add_u32 %[t2], %[tile], 2")
    e.raw("s_cmp_ge_u32 %[t2], %[n_tiles]")
    e.raw(f"s_cbranch_scc1 6{tag}f")
    for c in dma_chunks("k", buf):
        for x in c:
            e.raw(x)
    e.raw(f"6{tag}:")


KINDS = {"masked": 1, "diag": 3}


def single_tile(e, buf, kind, start):
    """A masked tile on its own (no pipelining across tiles).  kind: "masked" every score against its threshold;
    "diag" the tile on an ALIGNED causal diagonal (query i of the wavefront sees key j of the tile iff j <= i):
    S(A,0) and S(B,1) are triangular, S(B,0) is fully visible, and S(A,1) is not computed at all -- block A neither
    scores nor accumulates keys 32..63.  Arrives with K fragments 0..3 of half 0 in flight; leaves likewise for the
    next tile."""
    tag = f"{buf}{KINDS[kind]}"
    diag = kind == "diag"
    h1_blocks = "B" if diag else "AB"
    mask0 = {"A": True, "B": kind == "masked"}
    mask1 = {"A": kind == "masked", "B": True}
    e.raw(f"; ---- {kind} tile in buffers {buf}: S(.,0)")
    m = []
    for s in range(8):
        slot = s % 4

        def refill(s=s, slot=slot):
            if s < 4:
                k_read(e, buf, 0, s + 4, slot)
            else:
                k_read(e, buf, 1, s - 4, slot)
        m.append((mfma_s("A", 0, slot, s), (KF + 4 * slot,), None))
        m.append((mfma_s("B", 0, slot, s), None, refill))
    emit(e, plan(e, m, []))
    e.raw("; S(.,1) | E(.,0)")
    m = []
    for s in range(8):
        slot = s % 4

        def refill(s=s, slot=slot):
            if s < 4:
                k_read(e, buf, 1, s + 4, slot)
        for ci, c in enumerate(h1_blocks):
            m.append((mfma_s(c, 1, slot, s), (KF + 4 * slot,) if ci == 0 else None,
                      refill if ci == len(h1_blocks) - 1 else None))
    emit(e, plan(e, m, exp_ops(0, mask0), hold=1 if diag else 3))

    def first_v_reads():
        for j in range(8):
            v_read(e, buf, 0, j)
    boundary_plain(e, buf, tag, first_v_reads)
    e.raw("; O(.,0) | E(.,1)")
    m = []
    for j in range(8):
        if j % 4 == 0:
            m.append((mfma_sum("A", P[0]["A"] + 4 * (j // 4)), None, None))
            m.append((mfma_sum("B", P[0]["B"] + 4 * (j // 4)), None, None))

        def refill(j=j):
            v_read(e, buf, 1, j)
        m.append((mfma_o("A", j, P[0]["A"] + 4 * (j // 4)), vneeds(j), None))
        m.append((mfma_o("B", j, P[0]["B"] + 4 * (j // 4)), None, refill))
    emit(e, plan(e, m, exp_ops(1, mask1, h1_blocks), hold=3))
    e.raw("s_nop 1")
    e.raw("; O(.,1); the next tile's first K fragments are requested half way")
    m = []
    for j in range(8):
        if j % 4 == 0:
            for c in h1_blocks:
                m.append((mfma_sum(c, P[1][c] + 4 * (j // 4)), None, None))

        def next_k(j=j):
            if j == 3:
                for s in range(4):
                    k_read(e, buf ^ 1, 0, s, s)
        for ci, c in enumerate(h1_blocks):
            m.append((mfma_o(c, j, P[1][c] + 4 * (j // 4)), vneeds(j) if ci == 0 else None,
                      next_k if ci == len(h1_blocks) - 1 else None))
    emit(e, plan(e, m, []))
    e.raw(f"v_subrev_u32 v{THR['A']}, 64, v{THR['A']}")     # the next tile's keys are 64 further along
    e.raw(f"v_subrev_u32 v{THR['B']}, 64, v{THR['B']}")
    e.raw("s_add_u32 %[tile], %[tile], 1")
    assert e.pending == start, (e.pending, start)
    check_sums(e, "80f")
    e.raw("s_branch 20b")


def half_step(e, *, s_part, o_part, valu, hold, span=None, a_posts=None):
    """The MFMAs of one pipeline half-step as planned entries.
    s_part: (K buffer, half, k_next(i, slot) called after step i >= 4) -- S(., half) of the tile in that buffer; the
            fragments of steps 0..3 are in flight, those of steps 4..7 are requested as the slots come free
    o_part: (P half, v_next(j) called after fragment j is consumed) -- O += V^T fragments 0..7 (already requested)
            . P(., half)
    a_posts: {("S", i) or ("O", i): callback} run behind the block-A MFMA of step i
    Order: per step i the two score MFMAs (blocks A, B), then the two (with row sums: four) accumulations of
    fragment i."""
    a_posts = a_posts or {}
    m = []
    for i in range(8):
        slot = i % 4
        # the fragments of steps i and i + 1 are waited for together (they were requested long ago: half as many
        # wait instructions)
        pair_needs = None
        if i % 2 == 0:
            pair_needs = ()
            for k in (i, i + 1):
                if s_part:
                    pair_needs += (KF + 4 * (k % 4),)
                if o_part:
                    pair_needs += vneeds(k)
        if s_part:
            kbuf, kh, k_next = s_part

            def k_refill(i=i, slot=slot, kbuf=kbuf, kh=kh, k_next=k_next):
                if i < 4:
                    k_read(e, kbuf, kh, i + 4, slot)
                elif k_next:
                    k_next(i, slot)
            m.append((mfma_s("A", kh, slot, i), pair_needs, a_posts.get(("S", i))))
            pair_needs = None
            m.append((mfma_s("B", kh, slot, i), None, k_refill))
        if o_part:
            ph, v_next = o_part
            if i % 4 == 0:
                m.append((mfma_sum("A", P[ph]["A"] + 4 * (i // 4)), None, None))
                m.append((mfma_sum("B", P[ph]["B"] + 4 * (i // 4)), None, None))

            def v_refill(i=i, v_next=v_next):
                if v_next:
                    v_next(i)
            m.append((mfma_o("A", i, P[ph]["A"] + 4 * (i // 4)), pair_needs, a_posts.get(("O", i))))
            m.append((mfma_o("B", i, P[ph]["B"] + 4 * (i // 4)), None, v_refill))
    return plan(e, m, valu, hold, span)


def pipeline(e, b, start, h0_start, dry=False):
    """The software pipeline over unmasked tiles for tiles whose buffers are `b` (code for both parities is
    generated; a tile step ends by jumping to the other parity's H0).  Returns the reads H1 leaves in flight."""
    o = b ^ 1
    # After the barrier of boundary(t) the first reads of what has landed -- K[t+1] half 0 and V[t] half 0 -- go out
    # between the last eight MFMAs of H0 (steps 6, 7, whose own fragments are in registers): fragments 0, 1 of both at
    # once, the others one per MFMA, K slots 2, 3 and V^T fragments 6, 7 as those steps free their registers.  The
    # order of the reads is the same in the prologue, which has only the score MFMAs to put them behind.
    def k_after(i, slot):
        if i >= 6:
            k_read(e, o, 0, slot, slot)

    def v_after(j):
        if j >= 6:
            v_read(e, b, 0, j)

    tail_posts = {("S", 6): lambda: v_read(e, b, 0, 2), ("O", 6): lambda: v_read(e, b, 0, 3),
                  ("S", 7): lambda: v_read(e, b, 0, 4), ("O", 7): lambda: v_read(e, b, 0, 5)}

    def k_after_pro(i, slot):
        if i >= 6:
            k_read(e, o, 0, slot, slot)
            v_read(e, b, 0, 2 * i - 9)          # 3 behind step 6, 5 behind step 7
            v_read(e, b, 0, i)

    pro_posts = {("S", 6): tail_posts[("S", 6)], ("S", 7): tail_posts[("S", 7)]}

    def first_reads():
        k_read(e, o, 0, 0, 0)
        k_read(e, o, 0, 1, 1)
        v_read(e, b, 0, 0)
        v_read(e, b, 0, 1)

    def tail_variants(entries, tagbase, join_label):
        """boundary(t) and the rest of the half-step, in two variants: with and without the request of K[t+2]
        (V[t+1] is requested in H1)."""
        wait_and_meet(e)
        first_reads()
        e.raw("s_add_u32 %[t2], %[tile], 2")
        e.raw("s_cmp_lt_u32 %[t2], %[n_tiles]")
        e.raw(f"s_cbranch_scc1 {tagbase}1f")
        saved, result = list(e.pending), None
        for vi, which in ((0, ""), (1, "k")):
            e.pending = list(saved)
            if vi:
                e.raw(f"{tagbase}{vi}:")
            emit(e, entries, dma_chunks(which, b))
            e.raw(f"s_branch {join_label}")
            assert result is None or result == e.pending
            result = list(e.pending)
        return result

    # ---------------- prologue: S(t,0), then H0 without its O part ----------------
    e.pending = list(start)
    e.raw(f"4{b}0:")
    e.raw(f"; ---- pipeline prologue, tile in buffers {b}: S(t,0)")
    emit(e, half_step(e, s_part=(b, 0, lambda i, slot: k_read(e, b, 1, i - 4, slot)), o_part=None, valu=[], hold=0))
    e.raw("; S(t,1) | E(t,0), boundary inside")
    pro = half_step(e, s_part=(b, 1, k_after_pro), o_part=None, valu=exp_ops(0, NONE), hold=3, span=12, a_posts=pro_posts)
    emit(e, pro[:12])                                      # steps 0..5
    at_m = tail_variants(pro[12:], f"5{b}0", f"4{b}4f")

    # ---------------- H0(t): S(t,1) | E(t,0) | O(t-1,1) ----------------
    e.raw(f"4{b}1:")
    e.raw(f"; ---- H0, tile in buffers {b}: S(t,1) | E(t,0) | O(t-1,1), boundary inside")
    e.pending = list(h0_start)
    h0 = half_step(e, s_part=(b, 1, k_after), o_part=(1, v_after), valu=exp_ops(0, NONE), hold=0, span=28,
                   a_posts=tail_posts)
    emit(e, h0[:28])                                       # steps 0..5
    at_m2 = tail_variants(h0[28:], f"5{b}1", f"4{b}4f")
    assert dry or at_m == at_m2, (at_m, at_m2)

    # ---------------- H1 ----------------
    e.raw(f"4{b}4:")
    e.pending = list(at_m2)
    e.raw("s_add_u32 %[t2], %[tile], 1")
    e.raw("s_cmp_ge_u32 %[t2], %[n_pipe]")
    e.raw(f"s_cbranch_scc1 4{b}6f")
    e.raw(f"; ---- H1, tile in buffers {b}: S(t+1,0) | E(t,1) | O(t,0); V[t+1] (it exists) is requested on the way")
    emit(e, half_step(e, s_part=(o, 0, lambda i, slot: k_read(e, o, 1, i - 4, slot)),
                      o_part=(0, lambda j: v_read(e, b, 1, j)), valu=exp_ops(1, NONE), hold=0), dma_chunks("v", b))
    leaves = list(e.pending)
    check_sums(e, f"4{b}7f")
    e.raw("s_add_u32 %[tile], %[tile], 1")
    e.raw(f"s_branch 4{o}1b" if o < b else f"s_branch 4{o}1f")
    e.raw(f"4{b}7:")                                       # a row sum reached 2: finish this tile, then leave
    e.raw(f"s_mov_b32 s{FLAG}, 1")
    e.raw(f"s_branch 4{b}5f")
    # ---------------- H1 without its S part (the last unmasked tile the block may run) ----------------
    e.raw(f"4{b}6:")
    e.pending = list(at_m2)
    e.raw(f"; ---- H1 tail, tile in buffers {b}: E(t,1) | O(t,0)")
    e.raw("s_cmp_ge_u32 %[t2], %[n_tiles]")               # (t2 = t + 1) no tile t+1: no V[t+1] to request
    e.raw(f"s_cbranch_scc1 6{b}9f")
    for c in dma_chunks("v", b):
        for x in c:
            e.raw(x)
    e.raw(f"6{b}9:")
    emit(e, half_step(e, s_part=None, o_part=(0, lambda j: v_read(e, b, 1, j)), valu=exp_ops(1, NONE), hold=0))
    check_sums(e, f"4{b}9f")
    e.raw(f"s_branch 4{b}5f")
    e.raw(f"4{b}9:")
    e.raw(f"s_mov_b32 s{FLAG}, 1")
    # ---------------- epilogue: O(t,1); the next tile's first K fragments are requested first ----------------
    e.raw(f"4{b}5:")
    e.raw("; ---- pipeline epilogue: O(t,1)")
    e.raw("s_waitcnt lgkmcnt(0)")
    e.pending = []
    for s in range(4):
        k_read(e, o, 0, s, s)
    epi = half_step(e, s_part=None, o_part=(1, None), valu=[], hold=0)
    emit(e, [(t, None, p_, v, f) for (t, _, p_, v, f) in epi])
    e.raw("s_add_u32 %[tile], %[tile], 1")
    assert e.pending == start, (e.pending, start)
    e.raw("s_branch 20b")
    return leaves


def entry(e):
    """Loads the fixed registers from the block's operands: nb, the row-sum operand, LDS read addresses (the address of step s / d-tile dt is the one of step 0 / d-tile 0 with s << 5 /
    dt << 6 XORed in: the swizzle XORs exactly those bits), DMA lane offsets and pointers, mask thresholds."""
    e.raw(f"v_mov_b32 v{NB['A']}, %[nb0]")
    e.raw(f"v_mov_b32 v{NB['B']}, %[nb1]")
    e.raw(f"v_mov_b32 v{NEGINF}, 0xff800000")
    e.raw(f"v_mov_b32 v{THR['A']}, %[thr0]")
    e.raw(f"v_mov_b32 v{THR['B']}, %[thr1]")
    for i in range(4):
        e.raw(f"v_mov_b32 v{SUMA + i}, %[suma]")
    for s_ in range(8):
        e.raw(f"v_xor_b32 v{KOFF + s_}, {hex(s_ << 5)}, %[k0]")
    for dt in range(4):
        e.raw(f"v_xor_b32 v{VOFF + dt}, {hex(dt << 6)}, %[vlo0]")
        e.raw(f"v_xor_b32 v{VOFF + 4 + dt}, {hex(dt << 6)}, %[vhi0]")
    for j in range(4):                                 # load j of a tile: swizzled chunk, row part, and j * four rows
        e.raw(f"v_xor_b32 {TMP}, {hex(j << 4)}, %[c0s]")
        e.raw(f"v_add_u32 v{DMAOFF + j}, {TMP}, %[rowk]")
        e.raw(f"v_add_u32 v{DMAOFF + 4 + j}, {TMP}, %[rowv]")
        if j:
            e.raw(f"s_mul_i32 s{KSTEP16}, %[kstep], {j}")
            e.raw(f"s_mul_i32 s{VSTEP16}, %[vstep], {j}")
            e.raw(f"v_add_u32 v{DMAOFF + j}, s{KSTEP16}, v{DMAOFF + j}")
            e.raw(f"v_add_u32 v{DMAOFF + 4 + j}, s{VSTEP16}, v{DMAOFF + 4 + j}")
    if PAGED:                                              # lane 0 of `ids` is tile + 1: V[t+1] lane 0, K[t+2] lane 1
        e.raw(f"s_mov_b32 s{KLANE}, 1")
        e.raw(f"s_mov_b32 s{VLANE}, 0")
        for name in "kv":
            for x in block_address(name):
                e.raw(x)
    else:
        e.raw(f"s_lshl_b32 s{KSTEP16}, %[kstep], 4")          # a tile is 64 rows = 16 steps of 4 rows
        e.raw(f"s_lshl_b32 s{VSTEP16}, %[vstep], 4")
        e.raw(f"s_mov_b32 s{KPTR}, %[klo]")
        e.raw(f"s_mov_b32 s{KPTR + 1}, %[khi]")
        e.raw(f"s_mov_b32 s{VPTR}, %[vlo]")
        e.raw(f"s_mov_b32 s{VPTR + 1}, %[vhi]")
    e.raw(f"s_mov_b32 s{FLAG}, 0")


def generate(paged=False):
    global PAGED
    PAGED = paged
    e = Emitter()
    entry(e)
    # first K fragments of the tile the block starts with (its buffer is the tile's parity)
    e.raw("s_bitcmp1_b32 %[tile], 0")
    e.raw("s_cbranch_scc1 11f")
    for s in range(4):
        k_read(e, 0, 0, s, s)
    e.raw("s_branch 20f")
    start = list(e.pending)
    e.pending = []
    e.raw("11:")
    for s in range(4):
        k_read(e, 1, 0, s, s)
    assert e.pending == start
    # ---- loop head: which kind of tile, which buffer.  Every path arrives here with those four reads in flight. ----
    e.raw("20:")
    e.raw(f"s_cmp_lg_u32 s{FLAG}, 0")
    e.raw("s_cbranch_scc1 91f")
    e.raw("s_cmp_ge_u32 %[tile], %[n_end]")
    e.raw("s_cbranch_scc1 90f")
    e.raw("s_bitcmp1_b32 %[tile], 0")
    e.raw("s_cbranch_scc1 21f")
    for buf, lab in ((0, None), (1, "21")):
        if lab:
            e.raw(f"{lab}:")
        e.raw("s_cmp_lt_u32 %[tile], %[n_pipe]")
        e.raw(f"s_cbranch_scc1 4{buf}0f")
        e.raw("s_cmp_ge_u32 %[tile], %[n_mask]")
        e.raw(f"s_cbranch_scc1 3{buf}2f")
        e.raw("s_cmp_lg_u32 %[aligned], 0")              # masked: on an aligned diagonal the cheaper body
        e.raw(f"s_cbranch_scc1 3{buf}3f")
        e.raw(f"s_branch 3{buf}1f")
    # what H1 leaves in flight for H0 (the same for both parities): from a dry run
    dry = Emitter()
    h0_start = pipeline(dry, 0, start, [], dry=True)
    for buf in (0, 1):
        leaves = pipeline(e, buf, start, h0_start)
        assert leaves == h0_start, (leaves, h0_start)
        for kind in ("masked", "diag"):
            e.pending = list(start)
            e.raw(f"3{buf}{KINDS[kind]}:")
            single_tile(e, buf, kind, start)
        # nothing visible in this tile: the wavefront only takes part in the boundary
        e.pending = list(start)
        e.raw(f"3{buf}2:")

        def next_k(buf=buf):
            for s in range(4):
                k_read(e, buf ^ 1, 0, s, s)
        boundary_plain(e, buf, f"{buf}2", next_k)
        e.raw("s_add_u32 %[tile], %[tile], 1")
        assert e.pending == start
        e.raw("s_branch 20b")
    # exits
    e.raw("80:")                                       # a masked tile took a row sum to 2
    e.raw(f"s_mov_b32 s{FLAG}, 1")
    e.raw("s_branch 20b")
    e.raw("90:")
    e.raw("s_mov_b32 %[t2], 0")                        # %[t2] doubles as the status the block returns
    e.raw("s_branch 99f")
    e.raw("91:")
    e.raw("s_mov_b32 %[t2], 1")
    e.raw("99:")
    e.raw("s_waitcnt lgkmcnt(0)")
    e.raw("s_nop 15")                                  # the last MFMA results are read by ordinary code next
    return e.lines


def acc_of(c, dt):
    return (OREG["A"], OREG["B"])[c] + 16 * dt


def snippets():
    """Small assembly statements through which ordinary code reaches the accumulators in the AGPRs."""
    out = {}
    # operand %0: four registers of zeros.  The products land long before anything reads the accumulators, and the
    # wavefront spends ten issue slots instead of 136 register writes.
    # (The s_nop: the compiler may have written the operand in the instruction just before this statement, and
    # cannot see that an MFMA reads it here.)
    out["W64_ZERO"] = (["s_nop 3"] + [f"v_mfma_f32_32x32x16_bf16 a{rng(16 * i, 16)}, %0, %0, 0" for i in range(8)] +
                       [f"v_mfma_f32_16x16x32_bf16 a{rng(LREG[c], 4)}, %0, %0, 0" for c in "AB"])
    # Q^T fragments from the wavefront's query rows in LDS (64 rows of 256 bytes, swizzled like a K tile) into their
    # AGPRs.  Operands: %0 scratch (early-clobber output), %1 LDS address of the lane's piece of step 0 in block A
    # (the one of step s is that with s << 5 XORed in; block B sits 32 rows further).
    lines = []
    for s_ in range(8):
        lines.append(f"v_xor_b32 %0, {hex(s_ << 5)}, %1")
        lines += [f"ds_read_b128 a{rng(QREG[c] + 4 * s_, 4)}, %0 offset:{(c == 'B') * 32 * ROW}" for c in "AB"]
        if s_ == 5:
            lines.append("s_waitcnt lgkmcnt(4)")           # (the counter of LDS operations in flight holds 15)
    lines.append("s_waitcnt lgkmcnt(0)")
    out["W64_QFRAGS"] = lines
    for c in range(2):
        # scores of one 32-key half in ordinary code: %0 = sum over steps of K fragment %(1+s) . Q^T fragment s
        q = (QREG["A"], QREG["B"])[c]
        out[f"W64_QK_{c}"] = (["s_nop 3"] +
                              [f"v_mfma_f32_32x32x16_bf16 %0, %{1 + s_}, a{rng(q + 4 * s_, 4)}, {'%0' if s_ else '0'}"
                               for s_ in range(8)] + ["s_nop 15"])
        for dt in range(4):
            a = acc_of(c, dt)
            # operands: %0 V^T fragment (4 registers), %1 P^T fragment (4 registers), both ready when the statement
            # starts (the compiler waits for the LDS reads behind its operands; the s_nop covers a vector
            # instruction that wrote an operand just before the statement, which the compiler's hazard
            # bookkeeping cannot relate to an MFMA inside it)
            out[f"W64_PV_{c}_{dt}"] = ["s_nop 3",
                                       f"v_mfma_f32_32x32x16_bf16 a{rng(a, 16)}, %0, %1, a{rng(a, 16)}"]
            # 16 outputs %0..%15 <- the accumulator (after the last MFMA on it has finished)
            out[f"W64_READ_{c}_{dt}"] = ["s_nop 15"] + [f"v_accvgpr_read_b32 %{i}, a{a + i}" for i in range(16)]
        la = (LREG["A"], LREG["B"])[c]
        out[f"W64_SUM_{c}"] = ["s_nop 3", f"v_mfma_f32_16x16x32_bf16 a{rng(la, 4)}, %0, %1, a{rng(la, 4)}"]
        out[f"W64_READL_{c}"] = ["s_nop 15", f"v_accvgpr_read_b32 %0, a{la}", f"v_accvgpr_read_b32 %1, a{la + 1}"]
        # operands: %0 scratch (early-clobber output), %1 alpha of the lane's query, %2 / %3 alpha of queries c and c+16
        # as the row-sum accumulator holds them
        lines = ["s_nop 15"]
        for i in range(64):
            a = acc_of(c, 0) + i
            lines += [f"v_accvgpr_read_b32 %0, a{a}", f"v_mul_f32 %0, %0, %1", f"v_accvgpr_write_b32 a{a}, %0"]
        for i, op in ((0, "%2"), (1, "%3")):
            lines += [f"v_accvgpr_read_b32 %0, a{la + i}", f"v_mul_f32 %0, %0, {op}", f"v_accvgpr_write_b32 a{la + i}, %0"]
        lines.append("s_nop 4")
        out[f"W64_SCALE_{c}"] = lines
    return out


HEADER = '''// GENERATED by gen_prefill_w64_loop.py -- do not edit; change the generator and run it again.
// Assembly of prefill_fwd_w64.hip: W64_LOOP is the hand-scheduled loop over the K/V tiles (register map, pipeline
// and hand-over protocol: see the generator), W64_LOOP_PAGED the same loop with K and V read through a block table;
// the other macros are the small statements through which ordinary code reaches the accumulators that live in the
// AGPRs.
'''


def as_macro(name, lines):
    body = " \\\n".join('    "%s\\n"' % l for l in lines)
    return f"#define {name} \\\n{body}\n\n"


def main(out_path=None):
    """Writes the include file next to this script, or to `out_path` (first command-line argument)."""
    here = os.path.dirname(os.path.abspath(__file__))
    out_path = out_path or os.path.join(here, "prefill_w64_asm.inc")
    lines = generate()
    paged = generate(paged=True)
    with open(out_path, "w") as f:
        f.write(HEADER)
        f.write(as_macro("W64_LOOP", lines))
        f.write(as_macro("W64_LOOP_PAGED", paged))
        for name, body in snippets().items():
            f.write(as_macro(name, body))
        acc = ", ".join('"a%d"' % i for i in range(N_AGPRS))
        f.write(f"#define W64_CLOBBER_ACC {acc}\n")
        f.write("#define W64_CLOBBER_LOOP_VGPRS " + ", ".join('"v%d"' % i for i in range(N_FIXED_VGPRS)) + "\n")
    n_mfma = sum(1 for l in lines if l.startswith("v_mfma"))
    print(f"wrote {out_path}: loop of {len(lines)} lines, {n_mfma} MFMAs")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else None)
