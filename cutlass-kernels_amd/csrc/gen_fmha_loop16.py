#!/usr/bin/env python3
"""Generator of the hand-scheduled main loops of the fp16 FMHA forward kernel on 16x16x32 MFMAs (fmha_fwd_kernel16p.h,
FmhaCfg::ASM), in three shapes:
  d128  head dim 128, 64-key tiles, 256 query rows per workgroup (8 waves x 32 rows, two waves per SIMD)
  d128w4, d64w4  the d128 / d64 loops for 128 query rows per workgroup: 4 waves, one per SIMD, O in the accumulation
        registers (for problems with too few 256-row work items to go round)
  d64   head dim 64, 64-key tiles of 8 KB, 256 query rows per workgroup (8 waves, two per SIMD); 36 MFMA slots per tile:
        here the softmax (112 vector instructions beside 32 MFMAs) is what fills the issue port, so the row sum goes to
        the matrix pipe (ROWSUM = "mfma")
  d256  head dim 256, 32-key tiles, 128 query rows per workgroup (4 waves x 32 rows, one wave per SIMD: Q and O alone
        are 192 registers per lane; O lives in the accumulation registers a[0:127])
d128 and d256 have the same timeline (64 MFMA slots and 16 KB of K and of V per tile); the text below describes d128.

    python3 gen_fmha_loop16.py            # rewrites fmha_fwd_loop16_{d128,d128w4,d256,d64,d64w4}.inc beside this file
    python3 gen_fmha_loop16.py --check    # exit status 1 if those files are not what the generator produces

Why a generator: the loop is one inline-asm statement of ~2800 instructions with every register assigned by hand.
Left to the compiler, the step comes out as blocks (all MFMAs of a GEMM, then all of the softmax), the two waves of
a SIMD run those blocks in lockstep and the matrix pipe idles during the softmax; at 256 registers any attempt to
make it interleave spills.  Here each wave's instruction stream is uniform: every MFMA is followed by its share of
the softmax's vector instructions and of the LDS operand reads, operands are requested LOOKAHEAD fragments ahead
through a ring of registers, and nothing spills.

What the vector pipe can take beside the MFMAs was measured with register-only loops (two waves per SIMD, cycles of
the SIMD per v_mfma_f32_16x16x32_f16, 16.3 with nothing else): an MFMA holds the issue port for 8 cycles, an ordinary
vector instruction for 4, v_exp_f32 for 8 -- up to two ordinary instructions per MFMA are free (16.5, 16.7), three
are not (21.8), one exponential plus one multiply-add is not either (21.7); and a v_dot2c_f32_f16 between MFMAs
waits for the matrix pipe to drain (32.5 with one per MFMA).  The softmax of a 64-key tile is 32 multiply-adds, 32
exponentials and 16 packed converts per wave beside 64 MFMAs: 7 of the 8 free cycles per MFMA.  The row sum
therefore does not go through the vector pipe at all (ROWSUM = "mfma"): four more MFMAs per tile multiply P by an
all-ones operand, which also leaves every lane with the complete sum of its query.

What the loop computes (same mathematics and data layout as the rest of fmha_fwd_kernel16.h; reference:
src/fmha-pipeline/fmha_consumer.h:8-73, online_softmax.h:87-207, fmha_pipe_ws.h:245-296):
  for key tile t (64 keys):  S(t)^T = K(t) . Q^T ;  P(t) = fp16(exp2(c S(t) - m)) ;  l += rowsum P(t) ;
                             O^T += V(t)^T . P(t)^T
with the reference point m fixed by the first tile's row max (no rescale inside the loop: the caller checks l for
overflow afterwards and falls back to a loop that tracks the max).  S(0) is computed by the caller.

Timeline.  One MFMA "slot" = one v_mfma_f32_16x16x32_f16 (16 cycles of the matrix pipe).  Tile t owns T slots:
  slots T t + [0,32)    S(t+1) = K(t+1).Q^T      (4 K-steps x 4 key blocks x 2 query blocks)
  then per key half ps  O += V(t).P(t)           (8 d blocks x 2 query blocks), followed, with ROWSUM = "mfma", by
                        l += 1.P(t)              (2 query blocks)
The vector work of softmax(t+1) is spread evenly over one tile period starting at slot VALU_START of tile t's
period: it starts when P(t)'s first half has been consumed (its registers are reused) and ends before P(t+1)'s second
half is needed.  A super-step = two tiles = one s_barrier.  K and V tiles live in rings of four 16 KB LDS slots (tile
t in slot t % 4); super-step J (tiles 2J, 2J+1) issues the global->LDS copies of K tiles 2J+3, 2J+4 and V tiles
2J+2, 2J+3 into the slots that the previous super-step read.  The barrier of a super-step sits HOLD MFMAs before its
end: those MFMAs have their operands in registers already and cover the LDS latency of the next super-step's first K
fragments, which may only be read after the barrier.

Registers (VGPRs, fixed; the generated file holds the whole asm statement with its constraints):
  v[192:255] O^T accumulators   o[db][qb]  at 192 + 4 (2 db + qb)
  v[128:159] S set A            s[kb][qb]  at base + 4 (2 kb + qb)     (even tiles)
  v[160:191] S set B                                                    (odd tiles)
  v[96:127]  Q                  q[qb][s]   at 96 + 4 (4 qb + s)
  v[80:95]   P                  p[qb][ps]  at 80 + 4 (2 qb + ps)
  v[48:79]   operand ring, 8 fragments of 4 registers (a K fragment = one ds_read_b128, a V fragment = two
             ds_read_b64_tr_b16); each fragment feeds two MFMAs (query blocks 0 and 1)
  v[24:27] K read addresses per K-step, v[28:35] V read addresses per d block, v[36:37] / v[38:39] lane offsets of
  the K / V copies; the softmax reference point m per query block and the row-sum registers depend on ROWSUM (below)
SGPRs: s[40:41] / s[42:43] global address of the next K / V tile to copy; the rest are compiler-chosen operands.
"""
import json
import os
import sys

# ---- shape --------------------------------------------------------------------------------------------------------
SHAPE = "d128"
QB, NSLOT = 2, 4
K_ST0 = 0                               # LDS map: K slots, then V slots (the read addresses include these bases)

# ---- how the row sum l is taken ----------------------------------------------------------------------------------
#   "mfma": l += 1 . P on the matrix pipe (sums P as rounded to fp16, the weights the second GEMM applies)
#   "add":  v_add_f32 over the fp32 weights before the cast (online_softmax.h:173-206), two chains per query block
#   "dot":  v_dot2c_f32_f16 over the rounded weights, summed per tile in the order of fmha_fwd_kernel16.h's loop
ROWSUM = "add"
# FOLD: Q arrives multiplied by the softmax scale c and S = K.Q^T starts from -m (the C operand of the first K-step is
# a register quad that holds -m) instead of from zero: the scores leave the matrix pipe as c S - m and the softmax has
# no multiply-add per score.  The caller subtracts m from S(0) itself.  (Not with ROWSUM = "dot".)
FOLD = True
RING = 8
LOOKAHEAD = 7      # fragments requested ahead of use
HOLD = 4           # MFMAs of a super-step issued behind its barrier
VALU_START = None  # slot (within the previous tile's period) where softmax(t) starts; None: per ROWSUM
VALU_RATE = None   # issue slots (4 cycles; v_exp_f32 counts two) per MFMA slot; None: even over one tile period
# Ablation switches for timing experiments (the results are then wrong); never set in the committed include.
ABLATE = set(os.environ.get("LOOP16_ABLATE", "").split(",")) - {""}


def configure():
    """derived constants; call again after changing SHAPE, ROWSUM or a parameter"""
    g = globals()
    if SHAPE == "d128":
        g.update(D=128, BN=64, NWAVES=8, O_ACC=False, O0=192, SA0=128, SB0=160, Q0=96, P0=80, RING0=48, KRD0=24, VRD0=28, GOK0=36, GOV0=38)
    elif SHAPE == "d128w4":   # the same loop for 128 query rows: 4 waves, one per SIMD, four copies per wave and tile, O in a[0:63]
        assert ROWSUM == "add" and FOLD
        g.update(D=128, BN=64, NWAVES=4, O_ACC=True, O0=0, SA0=128, SB0=160, Q0=96, P0=80, RING0=48, KRD0=24, VRD0=28, GOK0=192, GOV0=196)
    elif SHAPE == "d64":
        assert ROWSUM == "mfma"
        g.update(D=64, BN=64, NWAVES=8, O_ACC=False, O0=224, SA0=160, SB0=192, Q0=144, P0=128, RING0=96, KRD0=82, VRD0=78, GOK0=77, GOV0=76)
    elif SHAPE == "d64w4":    # ... and the head-dim-64 loop for 128 query rows: 4 waves, two copies per wave and tile, O in a[0:31]
        assert ROWSUM == "mfma" and FOLD
        g.update(D=64, BN=64, NWAVES=4, O_ACC=True, O0=0, SA0=160, SB0=192, Q0=144, P0=128, RING0=96, KRD0=82, VRD0=78, GOK0=224, GOV0=226)
    else:
        assert ROWSUM == "add"
        g.update(D=256, BN=32, NWAVES=4, O_ACC=True, O0=0, SA0=224, SB0=240, Q0=160, P0=144, RING0=112, KRD0=96, VRD0=80, GOK0=72, GOV0=76)
    g.update(KB=BN // 16, KS=D // 32, DB=D // 16, PS=BN // 32, K_PITCH=2 * D, V_PITCH=2 * D)
    g.update(K_TILE=BN * K_PITCH, V_TILE=BN * V_PITCH, V_ST0=NSLOT * BN * K_PITCH)
    g["IPW"] = K_TILE // 1024 // NWAVES     # copies per wave and tile (K and V alike)
    g["QKS"] = KS * KB * QB                 # MFMA slots of S = K.Q^T
    g["FOLDED"] = FOLD and ROWSUM != "dot"
    if SHAPE == "d256":
        g.update(M0R=70, MN0=104, LA0=64, QOFF0=68, LOW=64, L_OUT=(64, 66), T=64, L_TOTAL=False)
        start = 36   # S(t+1) is complete at slot 32; P(t+1) has to be before slot 32 of the next period
    elif SHAPE in ("d64", "d64w4"):
        g.update(M0R=74, MN0=64, ONES0=92, LACC0=84, QOFF0=72, LOW=64 if FOLDED else 72, L_OUT=(84, 88), T=36, L_TOTAL=True)
        start = 23   # P(t)'s first half is consumed by slot 26; P(t+1)'s second half is needed at slot 26 of the next period
    elif ROWSUM == "mfma" and FOLDED:
        g.update(MN0=12, ONES0=20, LACC0=40, QOFF0=10, LOW=10, L_OUT=(40, 44), T=68, L_TOTAL=True)
        start = 46
    elif ROWSUM == "mfma":
        g.update(M0R=18, ONES0=20, LACC0=40, QOFF0=16, LOW=16, L_OUT=(40, 44), T=68, L_TOTAL=True)
        start = 46
    elif ROWSUM == "add" and FOLDED:   # (d128 and d128w4)
        g.update(MN0=40, LA0=18, QOFF0=22, LOW=18, L_OUT=(18, 20), T=64, L_TOTAL=False)
        start = 44
    elif ROWSUM == "add":
        g.update(M0R=40, LA0=42, QOFF0=22, LOW=22, L_OUT=(42, 44), T=64, L_TOTAL=False)
        start = 44
    else:
        g.update(M0R=40, L0=42, RS0=44, RS20=46, QOFF0=22, LOW=22, L_OUT=(42, 43), T=64, L_TOTAL=False)
        start = 44
    g["PV0"] = [QKS + ps * (DB * QB + (2 if ROWSUM == "mfma" else 0)) for ps in range(PS)]   # first slot of each key half's P.V
    g["V_START"] = start if VALU_START is None else VALU_START
    span = T if PS == 2 else T - 6   # one key half per tile: the whole of P is needed at once, by the first P.V slot
    g["V_RATE"] = sum(c for _, c in softmax_ops(0)) / float(span) if VALU_RATE is None else VALU_RATE


def o_reg(db, qb): return O0 + 4 * (2 * db + qb)
def o_txt(db, qb): return ("a[%d:%d]" if O_ACC else "v[%d:%d]") % (o_reg(db, qb), o_reg(db, qb) + 3)
def s_reg(t, kb, qb): return (SA0 if t % 2 == 0 else SB0) + 4 * (2 * kb + qb)
def q_reg(qb, s): return Q0 + 4 * (KS * qb + s)
def p_reg(t, qb, ps):
    # one key half per tile (d256): P is double-buffered by tile parity, its softmax runs beside the other set's P.V
    return P0 + (8 * (t % 2) + 4 * qb if PS == 1 else 4 * (2 * qb + ps))
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
            c0 = vr(MN0 + 4 * qb) if FOLDED else "0"
            return "v_mfma_f32_16x16x32_f16 %s, %s, %s, %s" % (vr(d), vr(self.reg), vr(q_reg(qb, self.a)), c0 if self.a == 0 else vr(d))
        d = o_txt(self.b, qb)
        return "v_mfma_f32_16x16x32_f16 %s, %s, %s, %s" % (d, vr(self.reg), vr(p_reg(self.t, qb, self.a)), d)


def sum_mfma(t, ps, qb):
    d = LACC0 + 4 * qb
    return "v_mfma_f32_16x16x32_f16 %s, %s, %s, %s" % (vr(d), vr(ONES0), vr(p_reg(t, qb, ps)), vr(d))


def softmax_ops(t):
    """vector instructions of softmax(t) in issue order: (text, issue slots)"""
    ops = []
    for kb in range(KB):
        for qb in range(QB):
            s = s_reg(t, kb, qb)
            p = p_reg(t, qb, kb // 2) + 2 * (kb % 2)
            if not FOLDED:
                for i in range(4): ops.append(("v_fma_f32 v%d, v%d, %%[c], -v%d" % (s + i, s + i, M0R + qb), 1))
            for i in range(4): ops.append(("v_exp_f32 v%d, v%d" % (s + i, s + i), 2))
            if ROWSUM == "add" and "rowsum" not in ABLATE:
                for i in range(4): ops.append(("v_add_f32 v%d, v%d, v%d" % (LA0 + 2 * qb + i % 2, LA0 + 2 * qb + i % 2, s + i), 1))
            ops.append(("v_cvt_pk_f16_f32 v%d, v%d, v%d" % (p, s, s + 1), 1))
            ops.append(("v_cvt_pk_f16_f32 v%d, v%d, v%d" % (p + 1, s + 2, s + 3), 1))
            if ROWSUM == "dot":
                if kb == 0:  # the tile's partial sums start from zero
                    ops.append(("v_dot2_f32_f16 v%d, %%[ones], v%d, 0" % (RS0 + qb, p), 1))
                    ops.append(("v_dot2_f32_f16 v%d, %%[ones], v%d, 0" % (RS20 + qb, p + 1), 1))
                else:
                    ops.append(("v_dot2c_f32_f16 v%d, %%[ones], v%d" % (RS0 + qb, p), 1))
                    ops.append(("v_dot2c_f32_f16 v%d, %%[ones], v%d" % (RS20 + qb, p + 1), 1))
    return ops


def tile_sum_ops():
    """ROWSUM = "dot": l += (rs + rs2) per query block; issued a few instructions after the tile's last v_dot2c"""
    ops = []
    if ROWSUM != "dot": return ops
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
                    "global_load_lds_dwordx4 v%d, s[%d:%d]%s" % (go + i, sp, sp + 1, os.environ.get("LOOP16_COPYMOD", ""))])
    ops[-1] += ["s_add_u32 s%d, s%d, %%[stride]" % (sp, sp), "s_addc_u32 s%d, s%d, 0" % (sp + 1, sp + 1)]
    return ops


def schedule(n_tiles):
    """straight-line program for n_tiles key tiles (a multiple of 4, at least 8), as a list of segments, one per
    super-step; a segment ends with its barrier (the last one has none)"""
    assert n_tiles % 4 == 0 and n_tiles >= 8
    n_slots = T * n_tiles
    n_steps = n_tiles // 2
    SS = 2 * T   # slots per super-step
    # ---- MFMA slots: slot -> (fragment, qb) or ("L", ps, qb)
    slot_item = [None] * n_slots
    frags = []
    for t in range(n_tiles):
        base = T * t
        if t + 1 < n_tiles:
            for s in range(KS):
                for kb in range(KB):
                    f = Frag('K', t + 1, s, kb, base + 2 * (s * KB + kb), len(frags)); frags.append(f)
                    for qb in range(QB): slot_item[f.slot0 + qb] = (f, qb)
        for ps in range(PS):
            for db in range(DB):
                f = Frag('V', t, ps, db, base + PV0[ps] + 2 * db, len(frags)); frags.append(f)
                for qb in range(QB): slot_item[f.slot0 + qb] = (f, qb)
            if ROWSUM == "mfma":
                for qb in range(QB): slot_item[base + PV0[ps] + 2 * DB + qb] = ("L", t, ps, qb)
    # ---- vector work: slot -> [text]; positions before slot 0 are issued ahead of it
    valu_at = {}
    for t in range(n_tiles):
        start = T * (t - 1) + V_START
        cum = 0.0
        for txt, cost in softmax_ops(t):
            valu_at.setdefault(max(int(start + cum / V_RATE), -1), []).append(txt)
            cum += cost
        # the tile's sums join l a few instructions into the next tile's softmax (or right after, for the last tile)
        for txt, cost in tile_sum_ops():
            valu_at.setdefault(max(int(start + cum / V_RATE) + 2, -1), []).append(txt)
    # ---- copies: super-step J, one copy instruction group every fourth slot from its second slot on
    copies_at = {}
    for J in range(n_steps):
        todo = [('K', 2 * J + 3), ('K', 2 * J + 4), ('V', 2 * J + 2), ('V', 2 * J + 3)]
        groups = []
        for kind, t in todo:
            if t < n_tiles: groups += copy_ops(kind, t % NSLOT)
        for i, grp in enumerate(groups): copies_at[SS * J + 1 + 4 * i] = grp
    # ---- the workgroup's next work item (persistent workgroups): in the last super-step, whose K slots 0-2 and V slots
    # 0-1 are free, copy that item's first three K and two V tiles into them and, once the last S = K.Q^T has been
    # issued, load its Q into the Q registers; both are waited for at the end of the statement
    Z = SS * (n_steps - 1)
    copies_at.setdefault(Z, [])
    copies_at[Z] = ["s_mov_b64 s[40:41], %[kn]", "s_mov_b64 s[42:43], %[vn]"]
    groups = []
    for kind, slot in (('K', 0), ('K', 1), ('K', 2), ('V', 0), ('V', 1)): groups += copy_ops(kind, slot)
    for i, grp in enumerate(groups): copies_at[Z + 1 + 4 * i] = grp
    for i in range(QB * KS):
        qb, ks = i // KS, i % KS
        copies_at.setdefault(Z + QKS + 1 + 3 * i, []).append("global_load_dwordx4 %s, v%d, %%[qn] offset:%d" % (vr(q_reg(qb, ks)), QOFF0 + qb, 64 * ks))
    # ---- emission
    segs, cur = [], []
    nread = 0             # LDS read instructions issued so far
    done_reads = 0        # ... known complete (by the last wait)
    read_end = {}         # frag idx -> nread after its last read
    next_frag = 0         # next fragment to request

    def barrier_passed_for(f, slot):
        # a K fragment of tile t >= 2 (first read in super-step (t-1)/2) needs the barrier of the super-step before
        if f.kind != 'K' or f.t < 2: return True
        J = (f.t - 1) // 2
        return slot > SS * J - HOLD   # `slot` is the slot after the MFMA just issued
    def request(slot, limit):
        nonlocal next_frag, nread
        n = 0
        while next_frag < len(frags) and n < limit:
            f = frags[next_frag]
            # ring entry free: the fragment RING places earlier has been consumed (both MFMAs issued)
            if next_frag >= RING and frags[next_frag - RING].slot0 + 1 >= slot: break
            if f.slot0 > slot + 2 * LOOKAHEAD: break
            if not barrier_passed_for(f, slot): break
            for r in f.reads():
                if "reads" not in ABLATE: cur.append(r); nread += 1
            read_end[f.idx] = nread
            next_frag += 1; n += 1
    # ahead of slot 0: first operand requests, then the vector work that precedes the timeline
    cur.append("s_waitcnt lgkmcnt(0)")
    cur.append("s_nop 7"); cur.append("s_nop 7")   # MFMA results of the caller's S(0) are read by vector instructions
    for r in range(O0, O0 + 4 * DB * QB): cur.append(("v_accvgpr_write_b32 a%d, 0" if O_ACC else "v_mov_b32 v%d, 0") % r)
    if ROWSUM == "mfma":
        for r in range(ONES0, ONES0 + 4): cur.append("v_mov_b32 v%d, 0x3c003c00" % r)
        for r in range(LACC0, LACC0 + 8): cur.append("v_mov_b32 v%d, 0" % r)
    elif ROWSUM == "add":
        for r in range(LA0, LA0 + 4): cur.append("v_mov_b32 v%d, 0" % r)
    else:
        for qb in range(QB): cur.append("v_mov_b32 v%d, 0" % (L0 + qb))
    if FOLDED:   # -m of a query block, in the four registers of an MFMA's C operand (the caller fills the first)
        for qb in range(QB):
            for i in range(1, 4): cur.append("v_mov_b32 v%d, v%d" % (MN0 + 4 * qb + i, MN0 + 4 * qb))
    if "reads" in ABLATE:
        for r in range(RING0, RING0 + 4 * RING): cur.append("v_mov_b32 v%d, 0" % r)
    request(0, LOOKAHEAD)
    for txt in valu_at.get(-1, []): cur.append(txt)
    for slot in range(n_slots):
        J = slot // SS
        if slot % SS == SS - HOLD and J < n_steps - 1:
            cur.append("s_waitcnt lgkmcnt(0)" if "vmwait" in ABLATE else "s_waitcnt vmcnt(0) lgkmcnt(0)")
            if "barrier" not in ABLATE: cur.append("s_barrier")
            done_reads = nread
            segs.append(cur); cur = []
        it = slot_item[slot]
        if it is not None and "mfma" not in ABLATE:
            if it[0] == "L":
                cur.append(sum_mfma(it[1], it[2], it[3]))
            else:
                f, qb = it
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
    if ROWSUM == "add":
        for qb in range(QB): cur.append("v_add_f32 v%d, v%d, v%d" % (LA0 + 2 * qb, LA0 + 2 * qb, LA0 + 2 * qb + 1))
    cur.append("s_waitcnt vmcnt(0)")               # the next item's Q (registers) and first tiles (LDS) have arrived
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
    """the C++ text of the include: a flag the caller needs, then the complete asm statement.  It expects these names
    in scope: bool sum_is_complete (out: the flag), f32x16 o0, o1, .. (out: the O accumulators, 16 registers each, in register order), sa0, .. (in, clobbered:
    S(0)), q0, .. (in: this item's Q; out: the next item's); float l0, l1 (out); uint64_t kptr, vptr (in: this item's K
    tile 3 / V tile 2; out: the same of the next item), kn, vn, qn (the next item's K, V and this wave's Q rows);
    uint32_t nloop, k_rd[KS], v_rd[DB], goff_k[IPW], goff_v[IPW], qoff[2], lds_wave, tile_stride; float m_ref[2], c_log2
    (FOLD: float m_neg[2] instead of those two); constexpr bool kFold."""
    head, body, tail = folded()
    L = []
    L.append("// GENERATED by gen_fmha_loop16.py -- do not edit.  The hand-scheduled main loop of fmha_fwd_kernel16p (FmhaCfg::ASM: head")
    L.append("// dim %d, %d x %d): %d + %d (loop) + %d instructions, row sum by \"%s\"." % (D, 32 * NWAVES, 2 * BN, len(head), len(body), len(tail), ROWSUM))
    L.append("// l0 / l1 hold the complete row sum of the lane's query in every lane (true) or the lane's share of it (false)")
    L.append("sum_is_complete = %s;" % ("true" if L_TOTAL else "false"))
    L.append("// Q is expected multiplied by the softmax scale, S(0) with the reference point taken off, m_neg[] = minus that point (true);")
    L.append("// or Q and S(0) as they are, m_ref[] = the reference point (false)")
    L.append("static_assert(kFold == %s, \"the caller prepares Q, S(0) and the reference point in the form this loop takes\");" % ("true" if FOLDED else "false"))
    L.append("asm volatile(")
    def emit(ins): L.append('    "%s\\n"' % ins)
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
    def vec16(base, name, n, kind="v", mode="="):
        return ['"%s{%s[%d:%d]}"(%s%d)' % (mode, kind, base + 16 * i, base + 16 * i + 15, name, i) for i in range(n)]
    n_o, n_s, n_q = 4 * DB * QB // 16, 4 * KB * QB // 16, 4 * KS * QB // 16
    outs = vec16(O0, "o", n_o, "a" if O_ACC else "v") + ['"={v%d}"(l0)' % L_OUT[0], '"={v%d}"(l1)' % L_OUT[1]]
    inouts = vec16(SA0, "sa", n_s, mode="+") + vec16(Q0, "q", n_q, mode="+") + ['"+{s[40:41]}"(kptr)', '"+{s[42:43]}"(vptr)', '[nloop] "+s"(nloop)']
    L.append("    : " + ", ".join(outs) + ",")
    L.append("      " + ", ".join(inouts))
    ins = ['"{v%d}"(qoff[%d])' % (QOFF0 + i, i) for i in range(QB)] + ['[kn] "s"(kn)', '[vn] "s"(vn)', '[qn] "s"(qn)']
    ins += ['"{v%d}"(k_rd[%d])' % (KRD0 + i, i) for i in range(KS)] + ['"{v%d}"(v_rd[%d])' % (VRD0 + i, i) for i in range(DB)]
    ins += ['"{v%d}"(goff_k[%d])' % (GOK0 + i, i) for i in range(IPW)] + ['"{v%d}"(goff_v[%d])' % (GOV0 + i, i) for i in range(IPW)]
    if FOLDED:
        ins += ['"{v%d}"(m_neg[%d])' % (MN0 + 4 * i, i) for i in range(QB)]
        ins += ['[ldsw] "s"(lds_wave)', '[stride] "s"(tile_stride)']
    else:
        ins += ['"{v%d}"(m_ref[%d])' % (M0R + i, i) for i in range(QB)]
        ins += ['[c] "s"(c_log2)', '[ldsw] "s"(lds_wave)', '[stride] "s"(tile_stride)']
    if ROWSUM == "dot": ins.append('[ones] "s"(0x3c003c00u)')
    L.append("    : " + ", ".join(ins))
    used = set(range(SA0, SA0 + 16 * n_s)) | set(range(Q0, Q0 + 16 * n_q)) | set(range(KRD0, KRD0 + KS)) | set(range(VRD0, VRD0 + DB))
    used |= set(range(GOK0, GOK0 + IPW)) | set(range(GOV0, GOV0 + IPW)) | {QOFF0, QOFF0 + 1} | set(L_OUT)
    used |= {MN0, MN0 + 4} if FOLDED else {M0R, M0R + 1}
    if not O_ACC: used |= set(range(O0, O0 + 16 * n_o))
    # (vector registers the loop never names stay the compiler's: values it keeps across the statement need not be spilled)
    import re
    named = set()
    for ins in head + body + tail:
        for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", ins):
            named |= set(range(int(m.group(1)), int(m.group(2)) + 1)) if m.group(1) else {int(m.group(3))}
    clob = ['"memory"', '"scc"', '"m0"'] + ['"v%d"' % r for r in range(LOW, 256) if r not in used and r in named]
    L.append("    : " + ", ".join(clob) + ");")
    return "\n".join(L) + "\n"


configure()
if __name__ == "__main__":
    overrides = json.loads(os.environ.get("LOOP16_SET", "{}"))
    stale = False
    defaults = {k: globals()[k] for k in overrides}
    for shape, rowsum in (("d128", "add"), ("d128w4", "add"), ("d256", "add"), ("d64", "mfma"), ("d64w4", "mfma")):
        SHAPE, ROWSUM = shape, rowsum
        for k, v in overrides.items():
            if isinstance(v, dict): v = v.get(shape, rowsum if k == "ROWSUM" else defaults[k])   # {"ROWSUM": {"d128": "mfma"}}: one shape only
            globals()[k] = v
        configure()
        out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fmha_fwd_loop16_%s.inc" % shape)
        txt = render()
        if "--check" in sys.argv:
            stale = stale or not (os.path.exists(out) and open(out).read() == txt)
        else:
            open(out, "w").write(txt)
            print("wrote", out, len(txt.splitlines()), "lines")
    sys.exit(1 if stale else 0)
