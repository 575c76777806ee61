#!/usr/bin/env python3
"""Generator of the hand-scheduled main loop of the fp16 FMHA forward kernel on 16x16x32 MFMAs
(fmha_fwd_kernel16a.h), head dim 128, 256 query rows per workgroup (8 waves x 32 rows, two waves per SIMD).

    python3 gen_fmha_loop16.py            # rewrites fmha_fwd_loop16_d128.inc beside this file

Why a generator: the loop is one inline-asm statement of ~2800 instructions with every register assigned by hand.
Left to the compiler, the step comes out as blocks (all MFMAs of a GEMM, then all of the softmax), the two waves of
a SIMD run those blocks in lockstep and the matrix pipe idles during the softmax; at 256 registers any attempt to
make it interleave spills.  Here each wave's instruction stream is uniform: every MFMA is followed by its share of
the softmax's vector instructions (about 1.5 per MFMA) and of the LDS operand reads, operands are requested
LOOKAHEAD fragments ahead through a ring of registers, and nothing spills.

What the loop computes (same mathematics and data layout as fmha_fwd_kernel16.h; reference:
src/fmha-pipeline/fmha_consumer.h:8-73, online_softmax.h:87-207, fmha_pipe_ws.h:245-296):
  for key tile t (64 keys):  S(t)^T = K(t) . Q^T ;  P(t) = fp16(exp2(c S(t) - m)) ;  l += rowsum P(t) ;
                             O^T += V(t)^T . P(t)^T
with the reference point m fixed by the first tile's row max (no rescale inside the loop: the caller checks l for
overflow afterwards and falls back to a loop that tracks the max).  S(0) is computed by the caller.

Timeline.  One MFMA "slot" = one v_mfma_f32_16x16x32_f16 (16 cycles of the matrix pipe).  Tile t owns 64 slots:
  slots 64t+[0,32)   S(t+1) = K(t+1).Q^T      (4 K-steps x 4 key blocks x 2 query blocks)
  slots 64t+[32,64)  O += V(t).P(t)           (2 K-steps x 8 d blocks x 2 query blocks)
The vector work of softmax(t+1) is spread over slots 64t+[48,105): it starts when P(t)'s first half has been consumed
(its registers are reused) and ends before slot 64t+112 needs P(t+1)'s second half.
A super-step = two tiles = 128 slots = one s_barrier.  K and V tiles live in rings of four 16 KB LDS slots (tile t
in slot t % 4); super-step J (tiles 2J, 2J+1) issues the global->LDS copies of K tiles 2J+3, 2J+4 and V tiles 2J+2,
2J+3 into the slots that the previous super-step read.  The barrier of a super-step sits HOLD MFMAs before its end:
those MFMAs have their operands in registers already and cover the LDS latency of the next super-step's first K
fragments, which may only be read after the barrier.

Registers (VGPRs, fixed):
  v[192:255] O^T accumulators   o[db][qb]  at 192 + 4 (2 db + qb)
  v[128:159] S set A            s[kb][qb]  at base + 4 (2 kb + qb)     (even tiles)
  v[160:191] S set B                                                    (odd tiles)
  v[96:127]  Q                  q[qb][s]   at 96 + 4 (4 qb + s)
  v[80:95]   P                  p[qb][ps]  at 80 + 4 (2 qb + ps)
  v[48:79]   operand ring, 8 fragments of 4 registers (a K fragment = one ds_read_b128, a V fragment = two
             ds_read_b64_tr_b16); each fragment feeds two MFMAs (query blocks 0 and 1)
  v[24:27] K read addresses per K-step, v[28:35] V read addresses per d block, v[36:37] / v[38:39] lane offsets of
  the K / V copies, v[40:41] m per query block, v[42:43] l, v[44:45] / v[46:47] the two partial row sums of the tile
SGPRs: s[40:41] / s[42:43] global address of the next K / V tile to copy; the rest are compiler-chosen operands.
"""
import os
import re
import sys

# ---- shape (head dim 128, 64-key tiles, 8 waves) ---------------------------------------------------------------
D, BN, NWAVES = 128, 64, 8
KB, KS, DB, PS, QB = BN // 16, D // 32, D // 16, BN // 32, 2
K_PITCH = V_PITCH = D * 2
K_TILE = V_TILE = BN * K_PITCH          # 16384
NSLOT = 4
K_ST0, V_ST0 = 0, NSLOT * K_TILE        # LDS map: K slots, then V slots (the read addresses include these bases)
IPW = 2                                  # copies per wave and tile (K and V alike)

# ---- registers ---------------------------------------------------------------------------------------------------
O0, SA0, SB0, Q0, P0, RING0 = 192, 128, 160, 96, 80, 48
KRD0, VRD0, GOK0, GOV0, M0R, L0, RS0, RS20 = 24, 28, 36, 38, 40, 42, 44, 46
RING = 8
LOOKAHEAD = 7      # fragments requested ahead of use
HOLD = 8           # MFMAs of a super-step issued behind its barrier
VALU_START = 48    # slot (within the previous tile's period) where softmax(t) starts
VALU_RATE = 2.25   # issue slots (4 cycles each; v_exp_f32 counts two) per MFMA slot
# Ablation switches for timing experiments (the results are then wrong); never set in the committed include.
ABLATE = set(os.environ.get("LOOP16_ABLATE", "").split(",")) - {""}


def o_reg(db, qb): return O0 + 4 * (2 * db + qb)
def s_reg(t, kb, qb): return (SA0 if t % 2 == 0 else SB0) + 4 * (2 * kb + qb)
def q_reg(qb, s): return Q0 + 4 * (4 * qb + s)
def p_reg(qb, ps): return P0 + 4 * (2 * qb + ps)
def vr(r, n=4): return "v[%d:%d]" % (r, r + n - 1)


class Frag:
    """one MFMA operand fragment: 4 registers of the ring, consumed by the two MFMAs of slots slot0, slot0+1"""
    def __init__(self, kind, t, a, b, slot0, idx):
        self.kind, self.t, self.a, self.b, self.slot0, self.idx = kind, t, a, b, slot0, idx
        self.reg = RING0 + 4 * (idx % RING)

    def reads(self):
        slot = self.t % NSLOT
        if self.kind == 'K':   # K-step a, key block b
            return ["ds_read_b128 %s, v%d offset:%d" % (vr(self.reg), KRD0 + self.a, slot * K_TILE + self.b * 16 * K_PITCH)]
        off = slot * V_TILE + self.a * 32 * V_PITCH  # K-step (ps) a, d block b
        return ["ds_read_b64_tr_b16 %s, v%d offset:%d" % (vr(self.reg, 2), VRD0 + self.b, off),
                "ds_read_b64_tr_b16 %s, v%d offset:%d" % (vr(self.reg + 2, 2), VRD0 + self.b, off + 16 * V_PITCH)]

    def mfma(self, qb):
        if self.kind == 'K':
            d = s_reg(self.t, self.b, qb)
            return "v_mfma_f32_16x16x32_f16 %s, %s, %s, %s" % (vr(d), vr(self.reg), vr(q_reg(qb, self.a)), "0" if self.a == 0 else vr(d))
        d = o_reg(self.b, qb)
        return "v_mfma_f32_16x16x32_f16 %s, %s, %s, %s" % (vr(d), vr(self.reg), vr(p_reg(qb, self.a)), vr(d))


def softmax_ops(t):
    """vector instructions of softmax(t) in issue order: (text, issue slots)"""
    ops = []
    for kb in range(KB):
        for qb in range(QB):
            s = s_reg(t, kb, qb)
            p = p_reg(qb, kb // 2) + 2 * (kb % 2)
            for i in range(4): ops.append(("v_fma_f32 v%d, v%d, %%[c], -v%d" % (s + i, s + i, M0R + qb), 1))
            for i in range(4): ops.append(("v_exp_f32 v%d, v%d" % (s + i, s + i), 2))
            ops.append(("v_cvt_pk_f16_f32 v%d, v%d, v%d" % (p, s, s + 1), 1))
            ops.append(("v_cvt_pk_f16_f32 v%d, v%d, v%d" % (p + 1, s + 2, s + 3), 1))
            if kb == 0:  # the tile's partial sums start from zero (same order of summation as fmha_fwd_kernel16.h)
                ops.append(("v_dot2_f32_f16 v%d, %%[ones], v%d, 0" % (RS0 + qb, p), 1))
                ops.append(("v_dot2_f32_f16 v%d, %%[ones], v%d, 0" % (RS20 + qb, p + 1), 1))
            else:
                ops.append(("v_dot2c_f32_f16 v%d, %%[ones], v%d" % (RS0 + qb, p), 1))
                ops.append(("v_dot2c_f32_f16 v%d, %%[ones], v%d" % (RS20 + qb, p + 1), 1))
    return ops


def tile_sum_ops():
    """l += (rs + rs2) per query block; issued a few instructions after the tile's last v_dot2c"""
    ops = []
    for qb in range(QB): ops.append(("v_add_f32 v%d, v%d, v%d" % (RS0 + qb, RS0 + qb, RS20 + qb), 1))
    for qb in range(QB): ops.append(("v_add_f32 v%d, v%d, v%d" % (L0 + qb, L0 + qb, RS0 + qb), 1))
    return ops


def copy_ops(kind, slot):
    """the wave's two global->LDS copies of one tile into ring slot `slot`, then the pointer moves on one tile"""
    base = (K_ST0 if kind == 'K' else V_ST0) + slot * K_TILE
    go, sp = (GOK0, 40) if kind == 'K' else (GOV0, 42)
    ops = []
    for i in range(IPW):
        ops.append(["s_add_u32 m0, %%[ldsw], %d" % (base + i * NWAVES * 1024), "s_nop 0",
                    "global_load_lds_dwordx4 v%d, s[%d:%d]" % (go + i, sp, sp + 1)])
    ops[-1] += ["s_add_u32 s%d, s%d, %%[stride]" % (sp, sp), "s_addc_u32 s%d, s%d, 0" % (sp + 1, sp + 1)]
    return ops


def schedule(n_tiles):
    """straight-line program for n_tiles key tiles (a multiple of 4, at least 8), as a list of segments, one per
    super-step; a segment ends with its barrier (the last one has none)"""
    assert n_tiles % 4 == 0 and n_tiles >= 8
    n_slots = 64 * n_tiles
    n_steps = n_tiles // 2
    # ---- MFMA slots and fragments
    slot_frag = [None] * n_slots           # slot -> (frag, qb)
    frags = []
    for t in range(n_tiles):
        base = 64 * t
        if t + 1 < n_tiles:
            for s in range(KS):
                for kb in range(KB):
                    f = Frag('K', t + 1, s, kb, base + 2 * (s * KB + kb), len(frags)); frags.append(f)
                    for qb in range(QB): slot_frag[f.slot0 + qb] = (f, qb)
        for ps in range(PS):
            for db in range(DB):
                f = Frag('V', t, ps, db, base + 32 + 2 * (ps * DB + db), len(frags)); frags.append(f)
                for qb in range(QB): slot_frag[f.slot0 + qb] = (f, qb)
    # ---- vector work: slot -> [text]; positions before slot 0 are issued ahead of it
    valu_at = {}
    for t in range(n_tiles):
        start = 64 * (t - 1) + VALU_START
        ops = softmax_ops(t)
        cum = 0.0
        for i, (txt, cost) in enumerate(ops):
            valu_at.setdefault(max(int(start + cum / VALU_RATE), -1), []).append(txt)
            cum += cost
        # the tile's sums join l a few instructions into the next tile's softmax (or right after, for the last tile)
        for txt, cost in tile_sum_ops():
            valu_at.setdefault(max(int(start + cum / VALU_RATE) + 2, -1), []).append(txt)
    # ---- copies: super-step J, one copy instruction group every fourth slot from its second slot on
    copies_at = {}
    for J in range(n_steps):
        todo = [('K', 2 * J + 3), ('K', 2 * J + 4), ('V', 2 * J + 2), ('V', 2 * J + 3)]
        groups = []
        for kind, t in todo:
            if t < n_tiles: groups += copy_ops(kind, t % NSLOT)
        for i, g in enumerate(groups): copies_at[128 * J + 1 + 4 * i] = g
    # ---- emission
    segs, cur = [], []
    issued = []           # fragments whose reads have been issued, in order
    nread = 0             # LDS read instructions issued so far
    done_reads = 0        # ... known complete (by the last wait)
    read_end = {}         # frag idx -> nread after its last read
    next_frag = 0         # next fragment to request

    def barrier_passed_for(f, slot):
        # a K fragment of tile t >= 2 (first read in super-step (t-1)/2) needs the barrier of the super-step before
        if f.kind != 'K' or f.t < 2: return True
        J = (f.t - 1) // 2
        return slot > 128 * J - HOLD   # `slot` is the slot after the MFMA just issued
    def request(slot, limit):
        nonlocal next_frag, nread
        n = 0
        while next_frag < len(frags) and n < limit:
            f = frags[next_frag]
            cur_frag = slot // 2
            # ring entry free: the fragment RING places earlier has been consumed (both MFMAs issued)
            if next_frag >= RING and frags[next_frag - RING].slot0 + 1 >= slot: break
            if f.slot0 // 2 > cur_frag + LOOKAHEAD: break
            if not barrier_passed_for(f, slot): break
            for r in f.reads():
                if "reads" not in ABLATE: cur.append(r); nread += 1
            read_end[f.idx] = nread
            next_frag += 1; n += 1
    # ahead of slot 0: first operand requests, then the vector work that precedes the timeline
    cur.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    cur.append("s_nop 7"); cur.append("s_nop 7")   # MFMA results of the caller's S(0) are read by vector instructions
    for r in range(O0, O0 + 64): cur.append("v_mov_b32 v%d, 0" % r)
    for qb in range(QB): cur.append("v_mov_b32 v%d, 0" % (L0 + qb))
    request(0, LOOKAHEAD)
    for txt in valu_at.get(-1, []): cur.append(txt)
    for slot in range(n_slots):
        J = slot // 128
        if slot % 128 == 128 - HOLD and J < n_steps - 1:
            cur.append("s_waitcnt lgkmcnt(0)" if "vmwait" in ABLATE else "s_waitcnt vmcnt(0) lgkmcnt(0)")
            if "barrier" not in ABLATE: cur.append("s_barrier")
            done_reads = nread
            segs.append(cur); cur = []
        sf = slot_frag[slot]
        if sf is not None and "mfma" not in ABLATE:
            f, qb = sf
            if qb == 0 and read_end[f.idx] > done_reads:
                out = nread - read_end[f.idx]
                assert out <= 15
                if "reads" not in ABLATE: cur.append("s_waitcnt lgkmcnt(%d)" % out)
                done_reads = read_end[f.idx]
            cur.append(f.mfma(qb))
        if "valu" not in ABLATE:
            for txt in valu_at.get(slot, []): cur.append(txt)
        request(slot + 1, 1)
        if "copies" not in ABLATE:
            for txt in copies_at.get(slot, []): cur.append(txt)
    assert next_frag == len(frags)
    cur.append("s_nop 7"); cur.append("s_nop 7")   # the accumulators are read by the caller's vector instructions
    segs.append(cur)
    assert len(segs) == n_steps
    return segs


def folded():
    """(head, loop body, tail): head = super-steps 0,1; body = 2,3 (repeated); tail = the last two"""
    segs = schedule(16)
    assert segs[2] + segs[3] == segs[4] + segs[5], "the schedule is not periodic"
    # the same schedule for other lengths must be made of the same pieces
    for n in (8, 12, 24):
        other = schedule(n)
        assert other[0] + other[1] == segs[0] + segs[1] and other[-2] + other[-1] == segs[6] + segs[7]
        for j in range(2, n // 2 - 2, 2): assert other[j] + other[j + 1] == segs[2] + segs[3]
    return segs[0] + segs[1], segs[2] + segs[3], segs[6] + segs[7]


def program(n_tiles):
    """the instruction sequence a wave executes for n_tiles key tiles (loop unrolled): what the checker walks"""
    head, body, tail = folded()
    return head + body * ((n_tiles // 2 - 4) // 2) + tail


def render():
    head, body, tail = folded()
    lines = []
    lines.append("// GENERATED by gen_fmha_loop16.py -- do not edit.  The hand-scheduled main loop of fmha_fwd_kernel16a (head dim")
    lines.append("// 128, 256 x 128): %d + %d (loop) + %d instructions.  Operands: see the asm statement in fmha_fwd_kernel16a.h." % (len(head), len(body), len(tail)))
    def emit(ins): lines.append('"%s\\n"' % ins)
    for i in head: emit(i)
    emit("s_cmp_eq_u32 %[nloop], 0")
    emit("s_cbranch_scc1 2f")
    emit("1:")
    for i in body: emit(i)
    emit("s_sub_u32 %[nloop], %[nloop], 1")
    emit("s_cmp_lg_u32 %[nloop], 0")
    emit("s_cbranch_scc1 1b")
    emit("2:")
    for i in tail: emit(i)
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fmha_fwd_loop16_d128.inc")
    txt = render()
    if "--check" in sys.argv:
        sys.exit(0 if open(out).read() == txt else 1)
    open(out, "w").write(txt)
    print("wrote", out, len(txt.splitlines()), "lines")
