#!/usr/bin/env python3
"""Writes prefill_w64_asm.inc: the hand-scheduled tile loop of prefill_fwd_w64.hip as inline-assembly text.

Why assembly: with one wavefront per SIMD and 64 query columns per wavefront the output accumulators (128 registers)
must live in AGPRs while the score accumulators must live in VGPRs (the exponentials read them), and the vector and
LDS instructions must sit in the shadow of the MFMAs at a fixed rhythm.  The compiler offers neither (it picks one
register form for every MFMA of a function and clusters the vector work), so the loop over the K/V tiles of a query
tile is generated here, instruction by instruction, and included by the kernel as a string.  What stays ordinary HIP
C++: prologue, epilogue, ragged ends, and the rare tile in which a row maximum outgrows its exponent reference.

One tile (64 keys) of one wavefront (64 queries = column blocks A and B, head_dim 128):
  phase 1   S(.,0) = K[0:32] . Q^T               16 MFMA 32x32x16 (8 per block), K fragments one step ahead
  phase 2   S(.,1) = K[32:64] . Q^T              16 MFMA | P(.,0) = bf16(2^(S(.,0) * scale + nb)): 32 v_fma, 32 v_exp,
                                                           16 cvt, 8 or3 (a masked tile adds a compare and a select
                                                           per score: key index against a per-lane threshold)
  check     some weight >= 2 (top exponent bit of its bf16 pattern)?  -> leave, status 1 (nothing of the tile accumulated)
  phase 3   O += V[0:32]^T . P(.,0), l += sums   16 MFMA + 4 row-sum MFMA 16x16x32 | P(.,1) likewise from S(.,1)
  check     -> leave, status 2 (keys 0..31 of the tile are accumulated, 32..63 are not)
  phase 4a  O += V[32:48]^T . P(.,1)             8 + 2 MFMA (fragments already in registers)
  hand-over every wavefront is done reading the tile; the next tile has landed; the tile after it is requested
            (direct-to-LDS loads into the buffer just freed) and the next tile's first K fragments are read
  phase 4b  O += V[48:64]^T . P(.,1)             8 + 2 MFMA: covers the latency of those reads
Tiles come in three kinds, by index: [0, n_plain) every key visible to every query; [n_plain, n_mask) masked (causal
diagonal: key <= threshold of the lane's query; the threshold moves down by 64 per tile); [n_mask, n_end) nothing
visible for this wavefront -- it only takes part in the hand-over.  When the diagonal is aligned with the tiles
(operand `aligned`: query i of the wavefront sees key j of the one masked tile iff j <= i) that tile takes a cheaper
body: only the two triangular 32x32 sub-blocks get mask code, and the invisible one is neither scored nor accumulated.

Register map (physical, fixed; the block loads them itself from its operands, see entry()):
  v[0:31] Q^T fragments of block A (step s = v[4s:4s+3]), v[32:63] block B
  v[64:95]  S(A,0), S(B,0); dead after the first check: v[64:79] then hold P(.,1), v[80:95] V^T fragments
  v[96:127] S(A,1), S(B,1)
  v128 / v129 nb (the additive term of the exponent) of this lane's query in block A / B
  v130 -inf, v131 / v132 mask threshold of the lane's query in block A / B (key index inside the tile, minus 4*(lane/32))
  v[134:149] P(.,0): A slices 0,1 then B slices 0,1
  v[150:165] K fragments (4 in flight), v[166:181] V^T fragments (4 d-tiles of one 16-key slice)
  v[182:185] A operand of the row-sum MFMA
  v[186:193] K fragment LDS addresses per step, v[194:201] V^T LDS addresses [half][d-tile] (both for buffer 0; the
  buffer and the position inside the tile are immediates; V tiles sit two tile sizes behind the K tiles),
  v[202:209] lane offsets of the direct-to-LDS loads (K steps 0..3, V steps 0..3)
  twelve more registers, wherever the compiler puts the block's vector operands: after entry() they serve as scratch
  (collected weight bits, exponentials on their way to packing)
  a[0:63] O^T of block A (d-tile dt = a[16dt:16dt+15]), a[64:127] block B, a[128:131] / a[132:135] row sums:
  these live in the AGPRs for a whole query tile and are touched only by the assembly snippets below (the kernel
  is compiled with its builtin MFMAs in VGPR form, so the compiler has no use for AGPRs of its own)
  s[36:37] / s[38:39] global address of the wavefront's first DMA row of the K / V tile after next (advanced per tile),
  s[40:41] scratch; every other scalar is a named operand
"""
import os

ABL = os.environ.get("W64_ABL", "").split(",")       # timing experiments only (results wrong): nobarrier, nodma, nocheck

QA, QB = 0, 32
S = {("A", 0): 64, ("B", 0): 80, ("A", 1): 96, ("B", 1): 112}
NB = {"A": 128, "B": 129}
NEGINF = 130
THR = {"A": 131, "B": 132}
PW0 = {"A": 134, "B": 142}          # + 4*slice
PW1 = {"A": 64, "B": 72}            # aliases S(A,0)
VF1 = 80                            # aliases S(B,0): 4 d-tiles x 4 registers
KF = 150
VF0 = 166
SUMA = 182
KOFF, VOFF, DMAOFF = 186, 194, 202
N_FIXED_VGPRS = 210
# Scratch registers are the block's vector operands themselves: each is read once by entry() and is free from then on
# (the operands are declared in/out), so the block needs no register beyond v[0:209] and its operands.
ETMP = ["%[nb0]", "%[nb1]", "%[suma]", "%[k0]", "%[vlo0]", "%[vhi0]", "%[rowk]", "%[rowv]"]   # exponentials on their way to packing
ANY, TMP = "%[c0s]", "%[qaddr]"     # collected weight bits; scratch
OA, OB, LA, LB = 0, 64, 128, 132
KPTR, VPTR, PTMP = 36, 38, 40       # SGPR pairs: global address of this wavefront's share of the tile after next (K, V); scratch
Q_SLAB_ROW = 272                    # bytes per row of the query staging slab (256 + 16 of padding)
K_TILE = 16384                      # bytes of one K (or V) tile in LDS: 64 rows x 256 bytes
ROW = 256


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


def mfma32_v(dst, a, b, c):
    cs = "0" if c is None else f"v{rng(c, 16)}"
    return f"v_mfma_f32_32x32x16_bf16 v{rng(dst, 16)}, v{rng(a, 4)}, v{rng(b, 4)}, {cs}"


def mfma32_a(acc, a, b):
    return f"v_mfma_f32_32x32x16_bf16 a{rng(acc, 16)}, v{rng(a, 4)}, v{rng(b, 4)}, a{rng(acc, 16)}"


def mfma16_a(acc, a, b):
    return f"v_mfma_f32_16x16x32_bf16 a{rng(acc, 4)}, v{rng(a, 4)}, v{rng(b, 4)}, a{rng(acc, 4)}"


def k_read(e, buf, t, s, slot):
    e.lds_read(f"ds_read_b128 v{rng(KF + 4 * slot, 4)}, v{KOFF + s} offset:{buf * K_TILE + t * 32 * ROW}", KF + 4 * slot)


def v_read(e, buf, u, dt, base):
    """V^T fragment of 16-key slice u, d-tile dt into registers base..base+3 (two transposed 64-bit reads)."""
    off = buf * K_TILE + 16 * u * ROW
    e.lds_read(f"ds_read_b64_tr_b16 v{rng(base, 2)}, v{VOFF + dt} offset:{off}", base)
    e.lds_read(f"ds_read_b64_tr_b16 v{rng(base + 2, 2)}, v{VOFF + 4 + dt} offset:{off}", base + 2)


def exp_ops(t, dst, mask, blocks="AB"):
    """Vector work that turns S(c,t), c in `blocks`, into packed bf16 weights in dst[c] (+ slice * 4).  The result of
    a transcendental may not feed the next vector instruction, so the packing of a pair trails its exponentials.
    Accumulator register i of a lane holds key 32t + 8(i/4) + 4(lane/32) + i%4 of the tile; where mask[c] is set the
    score is kept only if that index is <= the lane's threshold (the lane part of the index is folded into the
    threshold)."""
    ops, pend = [], []
    i = 0
    for c in blocks:
        for w in range(8):                      # packed word w of the block: accumulator registers 2w, 2w+1
            t0, t1 = ETMP[2 * (i % 4)], ETMP[2 * (i % 4) + 1]
            for tmp, r in ((t0, 2 * w), (t1, 2 * w + 1)):
                ops.append(f"v_fma_f32 {tmp}, v{S[(c, t)] + r}, %[scale], v{NB[c]}")
                if mask[c]:
                    ops.append(f"v_cmp_le_i32_e64 vcc, {32 * t + 8 * (r // 4) + r % 4}, v{THR[c]}")
                    ops.append(f"v_cndmask_b32 {tmp}, v{NEGINF}, {tmp}, vcc")
            ops.append(f"v_exp_f32 {t0}, {t0}")
            ops.append(f"v_exp_f32 {t1}, {t1}")
            ops += pend
            pend = [f"v_cvt_pk_bf16_f32 v{dst[c] + w}, {t0}, {t1}"]
            if w % 2 == 1:
                pend.append(f"v_or3_b32 {ANY}, {ANY}, v{dst[c] + w - 1}, v{dst[c] + w}")
            i += 1
    ops += ["s_nop 0"] + pend
    return ops


def spread(e, mfmas, valu, hold=0):
    """Emit the MFMAs in order with the vector instructions spread evenly behind them, none behind the first
    `hold` MFMAs: the vector work reads accumulators that the MFMAs just before this phase wrote, and the hardware
    does not interlock that dependency (a result is visible 8 passes after its MFMA started; `hold` MFMAs of other
    chains in between cover that).  `mfmas` entries are (text, needs, post): registers whose LDS reads must have
    returned, and a callback run right after the MFMA (it issues the LDS reads that refill the registers the MFMA
    has just consumed)."""
    n, nv, vi = len(mfmas), len(valu), 0
    for i, (text, needs, post) in enumerate(mfmas):
        if needs:
            e.need(*needs)
        e.raw(text)
        if post:
            post()
        upto = (i + 1 - hold) * nv // (n - hold) if i >= hold else 0
        while vi < upto:
            e.raw(valu[vi])
            vi += 1


def check(e, label):
    e.raw(f"v_and_b32 {TMP}, 0x40004000, {ANY}")
    e.raw(f"v_cmp_ne_u32 vcc, 0, {TMP}")
    e.raw(f"v_mov_b32 {ANY}, 0")
    e.raw("s_nop 1")
    if "nocheck" not in ABL:
        e.raw(f"s_cbranch_vccnz {label}")


def hand_over(e, buf, tag):
    """End of the LDS reads of the tile in buffer `buf`: count the tile, meet the other wavefronts once the own share
    of the next tile has landed, request the tile after next into this buffer, read the next tile's first K fragments."""
    nxt = buf ^ 1
    e.raw("; tile hand-over")
    e.drain()
    e.raw("s_add_u32 %[tile], %[tile], 1")
    e.raw("s_cmp_ge_u32 %[tile], %[n_tiles]")          # no next tile: nothing to wait for, nobody to meet
    e.raw(f"s_cbranch_scc1 7{tag}f")
    e.raw("s_waitcnt vmcnt(0)")
    if "nobarrier" not in ABL:
        e.raw("s_barrier")
    e.raw("s_add_u32 %[t2], %[tile], 1")
    e.raw("s_cmp_ge_u32 %[t2], %[n_tiles]")
    e.raw(f"s_cbranch_scc1 6{tag}f")
    for name, j0, ptr, lds0 in (("k", 0, KPTR, 0), ("v", 4, VPTR, 2 * K_TILE)):
        e.raw(f"s_mov_b64 s[{PTMP}:{PTMP + 1}], s[{ptr}:{ptr + 1}]")
        for j in range(4):
            e.raw(f"s_add_u32 m0, %[ldsdst], {lds0 + buf * K_TILE + j * 1024}")
            e.raw("s_nop 0")
            if "nodma" not in ABL:
                e.raw(f"global_load_lds_dwordx4 v{DMAOFF + j0 + j}, s[{PTMP}:{PTMP + 1}]")
            if j < 3:
                e.raw(f"s_add_u32 s{PTMP}, s{PTMP}, %[{name}step]")
                e.raw(f"s_addc_u32 s{PTMP + 1}, s{PTMP + 1}, 0")
        e.raw(f"s_lshl_b32 %[t2], %[{name}step], 4")          # a tile is 64 rows = 16 DMA steps of 4 rows
        e.raw(f"s_add_u32 s{ptr}, s{ptr}, %[t2]")
        e.raw(f"s_addc_u32 s{ptr + 1}, s{ptr + 1}, 0")
    e.raw(f"6{tag}:")
    for s in range(4):
        k_read(e, nxt, 0, s, s)
    e.raw(f"7{tag}:")


KINDS = {"plain": 0, "masked": 1, "diag": 3}


def tile_body(e, buf, kind):
    """kind: "plain" no mask; "masked" every score against its threshold; "diag" the tile on an ALIGNED causal
    diagonal (query i of the wavefront sees key j of the tile iff j <= i): S(A,0) and S(B,1) are triangular, S(B,0)
    is fully visible, and S(A,1) is not computed at all -- block A neither scores nor accumulates keys 32..63."""
    tag = f"{buf}{KINDS[kind]}"
    diag = kind == "diag"
    t1_blocks = "B" if diag else "AB"
    mask0 = {"A": kind != "plain", "B": kind == "masked"}
    mask1 = {"A": kind == "masked", "B": kind != "plain"}
    qreg = {"A": QA, "B": QB}
    oreg = {"A": OA, "B": OB}
    lreg = {"A": LA, "B": LB}
    # ---- phase 1: scores of keys 0..31.  K fragments 0..3 of this tile are in flight (or in registers) ----
    e.raw(f"; ---- {kind} tile in buffer {buf}: phase 1")
    m = []
    for s in range(8):
        slot = s % 4

        def refill(s=s, slot=slot):
            if s < 4:
                k_read(e, buf, 0, s + 4, slot)
            else:
                k_read(e, buf, 1, s - 4, slot)
        m.append((mfma32_v(S[("A", 0)], KF + 4 * slot, QA + 4 * s, None if s == 0 else S[("A", 0)]), (KF + 4 * slot,), None))
        m.append((mfma32_v(S[("B", 0)], KF + 4 * slot, QB + 4 * s, None if s == 0 else S[("B", 0)]), None, refill))
    spread(e, m, [])
    # ---- phase 2: scores of keys 32..63 | weights of keys 0..31; V^T fragments of slice 0 requested ----
    e.raw("; phase 2")
    m = []
    for s in range(8):
        slot = s % 4

        def refill(s=s, slot=slot):
            if s < 4:
                k_read(e, buf, 1, s + 4, slot)
            else:
                dt = s - 4
                v_read(e, buf, 0, dt, VF0 + 4 * dt)
        for ci, c in enumerate(t1_blocks):
            m.append((mfma32_v(S[(c, 1)], KF + 4 * slot, qreg[c] + 4 * s, None if s == 0 else S[(c, 1)]),
                      (KF + 4 * slot,) if ci == 0 else None, refill if ci == len(t1_blocks) - 1 else None))
    spread(e, m, exp_ops(0, PW0, mask0), hold=1 if diag else 3)
    check(e, "91f")
    # ---- phase 3: values of keys 0..31 | weights of keys 32..63 ----
    e.raw("; phase 3")
    e.need(VF0, VF0 + 2)                         # (keeps the number of reads in flight countable)
    for dt in range(4):                          # slice 1 goes into the registers S(B,0) has just vacated
        v_read(e, buf, 1, dt, VF1 + 4 * dt)
    m = []
    for u, vf in ((0, VF0), (1, VF1)):
        m.append((mfma16_a(LA, SUMA, PW0["A"] + 4 * u), None, None))
        m.append((mfma16_a(LB, SUMA, PW0["B"] + 4 * u), None, None))
        for dt in range(4):
            def refill(u=u, dt=dt, vf=vf):
                v_read(e, buf, u + 2, dt, vf + 4 * dt)
            m.append((mfma32_a(OA + 16 * dt, vf + 4 * dt, PW0["A"] + 4 * u), (vf + 4 * dt, vf + 4 * dt + 2), None))
            m.append((mfma32_a(OB + 16 * dt, vf + 4 * dt, PW0["B"] + 4 * u), None, refill))
    spread(e, m, exp_ops(1, PW1, mask1, t1_blocks), hold=3)
    check(e, "92f")
    # ---- phase 4a: values of keys 32..47 (fragments are in registers or about to arrive) ----
    e.raw("; phase 4a")
    m = [(mfma16_a(lreg[c], SUMA, PW1[c]), None, None) for c in t1_blocks]
    for dt in range(4):
        for ci, c in enumerate(t1_blocks):
            m.append((mfma32_a(oreg[c] + 16 * dt, VF0 + 4 * dt, PW1[c]), (VF0 + 4 * dt, VF0 + 4 * dt + 2) if ci == 0 else None, None))
    spread(e, m, [])
    if kind != "plain":                          # the next tile's keys are 64 further along: thresholds move down
        e.raw(f"v_subrev_u32 v{THR['A']}, 64, v{THR['A']}")
        e.raw(f"v_subrev_u32 v{THR['B']}, 64, v{THR['B']}")
    hand_over(e, buf, tag)
    # ---- phase 4b: values of keys 48..63 ----
    e.raw("; phase 4b")
    m = [(mfma16_a(lreg[c], SUMA, PW1[c] + 4), None, None) for c in t1_blocks]
    for dt in range(4):
        for c in t1_blocks:
            m.append((mfma32_a(oreg[c] + 16 * dt, VF1 + 4 * dt, PW1[c] + 4), None, None))
    spread(e, m, [])
    e.raw("s_branch 20b")


def entry(e):
    """Loads the fixed registers from the block's operands: the Q^T fragments from the staging slab, nb, the row-sum
    operand, LDS read addresses (the address of step s / d-tile dt is the one of step 0 / d-tile 0 with s << 5 /
    dt << 6 XORed in: the swizzle XORs exactly those bits), DMA lane offsets and pointers, mask thresholds."""
    for c, q in ((0, QA), (1, QB)):
        for s_ in range(8):
            e.lines.append(f"ds_read_b128 v{rng(q + 4 * s_, 4)}, %[qaddr] offset:{c * 32 * Q_SLAB_ROW + 32 * s_}")
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
    e.raw("s_waitcnt lgkmcnt(0)")                      # the Q^T fragments are in; %[qaddr] is scratch from here on
    for j in range(4):
        e.raw(f"v_xor_b32 {TMP}, {hex(j << 4)}, %[c0s]")
        e.raw(f"v_add_u32 v{DMAOFF + j}, {TMP}, %[rowk]")
        e.raw(f"v_add_u32 v{DMAOFF + 4 + j}, {TMP}, %[rowv]")
    e.raw(f"s_mov_b32 s{KPTR}, %[klo]")
    e.raw(f"s_mov_b32 s{KPTR + 1}, %[khi]")
    e.raw(f"s_mov_b32 s{VPTR}, %[vlo]")
    e.raw(f"s_mov_b32 s{VPTR + 1}, %[vhi]")
    e.raw(f"v_mov_b32 {ANY}, 0")


def generate():
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
    e.raw("s_cmp_ge_u32 %[tile], %[n_end]")
    e.raw("s_cbranch_scc1 90f")
    e.raw("s_bitcmp1_b32 %[tile], 0")
    e.raw("s_cbranch_scc1 21f")
    for buf, lab in ((0, None), (1, "21")):
        if lab:
            e.raw(f"{lab}:")
        e.raw("s_cmp_lt_u32 %[tile], %[n_plain]")
        e.raw(f"s_cbranch_scc1 3{buf}0f")
        e.raw("s_cmp_ge_u32 %[tile], %[n_mask]")
        e.raw(f"s_cbranch_scc1 3{buf}2f")
        e.raw("s_cmp_lg_u32 %[aligned], 0")              # masked: on an aligned diagonal the cheaper body
        e.raw(f"s_cbranch_scc1 3{buf}3f")
        e.raw(f"s_branch 3{buf}1f")
    for buf in (0, 1):
        for kind in ("plain", "masked", "diag"):
            e.pending = list(start)
            e.raw(f"3{buf}{KINDS[kind]}:")
            tile_body(e, buf, kind)
            assert e.pending == start, (e.pending, start)
        # nothing visible in this tile: the wavefront only takes part in the hand-over
        e.pending = list(start)
        e.raw(f"3{buf}2:")
        hand_over(e, buf, f"{buf}2")
        assert e.pending == start
        e.raw("s_branch 20b")
    # exits
    e.raw("90:")
    e.raw("s_mov_b32 %[t2], 0")                        # %[t2] doubles as the status the block returns
    e.raw("s_branch 99f")
    e.raw("91:")
    e.raw("s_mov_b32 %[t2], 1")
    e.raw("s_branch 99f")
    e.raw("92:")
    e.raw("s_mov_b32 %[t2], 2")
    e.raw("99:")
    e.raw("s_waitcnt lgkmcnt(0)")
    e.raw("s_nop 15")                                  # the last MFMA results are read by ordinary code next
    return e.lines


def acc_of(c, dt):
    return (OA, OB)[c] + 16 * dt


def snippets():
    """Small assembly statements through which ordinary code reaches the accumulators in the AGPRs."""
    out = {}
    out["W64_ZERO"] = [f"v_accvgpr_write_b32 a{i}, 0" for i in range(LB + 4)]
    for c in range(2):
        for dt in range(4):
            a = acc_of(c, dt)
            # operands: %0 V^T fragment (4 registers), %1 P^T fragment (4 registers), both ready when the statement
            # starts (the compiler waits for the LDS reads behind its operands)
            out[f"W64_PV_{c}_{dt}"] = ["s_nop 1",
                                       f"v_mfma_f32_32x32x16_bf16 a{rng(a, 16)}, %0, %1, a{rng(a, 16)}"]
            # 16 outputs %0..%15 <- the accumulator (after the last MFMA on it has finished)
            out[f"W64_READ_{c}_{dt}"] = ["s_nop 15"] + [f"v_accvgpr_read_b32 %{i}, a{a + i}" for i in range(16)]
        la = (LA, LB)[c]
        out[f"W64_SUM_{c}"] = ["s_nop 1", f"v_mfma_f32_16x16x32_bf16 a{rng(la, 4)}, %0, %1, a{rng(la, 4)}"]
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
// Assembly of prefill_fwd_w64.hip: W64_LOOP is the hand-scheduled loop over the K/V tiles (register map and
// phases: see the generator); the other macros are the small statements through which ordinary code reaches the
// accumulators that live in the AGPRs.
'''


def as_macro(name, lines):
    body = " \\\n".join('    "%s\\n"' % l for l in lines)
    return f"#define {name} \\\n{body}\n\n"


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    lines = generate()
    with open(os.path.join(here, "prefill_w64_asm.inc"), "w") as f:
        f.write(HEADER)
        f.write(as_macro("W64_LOOP", lines))
        for name, body in snippets().items():
            f.write(as_macro(name, body))
        acc = ", ".join('"a%d"' % i for i in range(LB + 4))
        f.write(f"#define W64_CLOBBER_ACC {acc}\n")
        f.write("#define W64_CLOBBER_LOOP_VGPRS " + ", ".join('"v%d"' % i for i in range(N_FIXED_VGPRS)) + "\n")
    n_mfma = sum(1 for l in lines if l.startswith("v_mfma"))
    print(f"wrote prefill_w64_asm.inc: loop of {len(lines)} lines, {n_mfma} MFMAs (four tile bodies)")


if __name__ == "__main__":
    main()
