#!/usr/bin/env python3
"""Generator of the hand-scheduled main loop of the e4m3 FMHA forward kernel (fmha_fwd_kernel8p.h): head dim 128, 256
query rows per workgroup (8 waves x 32 rows, two waves per SIMD), 64-key tiles, V in [B,S,H,D]; and the same loop for
128 query rows (NWAVES = 4, one wave per SIMD, two copies per wave and tile: problems with too few 256-row work items).

    python3 gen_fmha_loop8.py            # rewrites fmha_fwd_loop8_d128{,w4}{,_direct}.inc beside this file
    python3 gen_fmha_loop8.py --check    # exit status 1 if those files are not what the generator produces

Why: this kernel is bound by instruction issue, not by the matrix pipe.  Measured with register-only loops (two waves per
SIMD, cycles of the SIMD per v_mfma_f32_32x32x64_f8f6f4, 64.0 with nothing else): twelve ordinary vector instructions or
six v_exp_f32 per MFMA are free (64.8 / 65.5), fourteen / seven are not (73.9 / 69.8) -- the MFMA holds the issue port
for about 16 cycles, an ordinary vector instruction for 4, v_exp_f32 for 8 -- and v_cvt_pk_fp8_f32 (like its
v_cvt_scalef32 forms) costs 8 as well; an LDS read beside them adds about 4.  The softmax of a 64-key tile is 32
multiply-adds, 32 exponentials and 16 converts per wave beside 9 MFMAs and 24 LDS reads: about 740 issue cycles against
544 cycles of the matrix pipe.  So the job of the schedule is a dense, stall-free instruction stream in each wave: every
MFMA is followed by its share of the softmax and by the operand reads of the MFMA LOOKAHEAD places ahead, every wait
is for something requested long before, and the two waves of a SIMD fill each other's MFMA shadows.

What the loop computes (same mathematics, LDS tile formats and register layouts as fmha_fwd_kernel.h with e4m3 operands;
reference: src/fmha-pipeline/fmha_consumer.h:8-73, online_softmax.h:87-207, fmha_pipe_ws.h:245-296):
  for key tile t (64 keys):  S(t)^T = K(t) . Q^T ;  P(t) = e4m3(exp2(c S(t) - m)) ;  l += rowsum P(t) ;
                             O^T += V(t)^T . P(t)^T
with the reference point m fixed by the first tile's row max (the weights then reach up to 1 on that tile and
have 8.8 binades left before v_cvt_pk_fp8_f32 turns them into NaN); the caller looks for a non-finite row sum afterwards
and falls back to a loop that tracks the max.  S(0) is computed by the caller.

Timeline.  A tile owns T = 9 MFMA places:
  0-3  S(t+1) = K(t+1).Q^T    32-key block kb = 0, K-steps 0, 1; then kb = 1
  4-7  O += V(t).P(t)         32-row blocks of d
  8    l += 1.P(t)            one v_mfma_f32_16x16x128_f8f6f4 against a 0/1 operand (every lane gets its query's sum)
The vector work of softmax(t+1) is spread evenly over one tile period that starts VALU_START places into tile t (its
first half needs S(t+1)'s block 0, complete after place 1; P is double-buffered).  A super-step = two tiles = one
s_barrier; K and V tiles live in rings of four 8 KB LDS slots (tile t in slot t % 4); super-step J (tiles 2J, 2J+1)
issues the global->LDS copies of K tiles 2J+3, 2J+4 and V tiles 2J+2, 2J+3 into the slots that the previous super-step
read.  The barrier sits HOLD MFMAs before the super-step's end: those have their operands in registers already.

Registers (VGPRs; the generated file holds the whole asm statement with its constraints):
  v[192:255] O^T accumulators   o[db]      at 192 + 16 db
  v[128:159] S set A            s[kb]      at base + 16 kb     (even tiles)      v[160:191] S set B (odd tiles)
  v[112:127] Q                  q[s]       at 112 + 8 s
  v[96:111]  P, two sets of 8   p(t)       at 96 + 8 (t % 2)
  v[48:79]   operand ring, 4 fragments of 8 registers (K: two ds_read_b128; V: four ds_read_b64_tr_b8)
  v[44:47] row-sum accumulator, v[36:43] the 0/1 operand, v[24:27] K read addresses [s][half], v[28:31] V read addresses
  per d block, v32 / v33 lane offsets of the K / V copy, v34 the reference point m, v35 lane offset of the Q rows
SGPRs: s[40:41] / s[42:43] global address of the next K / V tile to copy; the rest are compiler-chosen operands.
"""
import json
import os
import sys

D, BN = 128, 64
NWAVES = 8                               # 8: 256 query rows, two waves per SIMD; 4: 128 query rows, one wave per SIMD (two copies per wave and tile)
KB, KS, DB = BN // 32, D // 64, D // 32
K_PITCH = V_PITCH = D
K_TILE = V_TILE = BN * K_PITCH          # 8192
NSLOT = 4
K_ST0, V_ST0 = 0, NSLOT * K_TILE        # LDS map: K slots, then V slots (the read addresses include these bases)
T = 9                                    # MFMA places per tile

O0, SA0, SB0, Q0, P0, RING0 = 192, 128, 160, 112, 96, 48
LACC0, ONES0, KRD0, VRD0, MREF, QOFF = 44, 36, 24, 28, 34, 35
GOK, GOV = (32, 82), (33, 83)            # lane offsets of the wave's K / V copies (the second ones: 4 waves only)
FLAGS = 80         # DIRECT: OR of all P registers of the item (a byte with bit 7 set is a weight beyond the e4m3 range)
LOW = 24
RING = 4
LOOKAHEAD = 3      # fragments requested ahead of use
HOLD = 2           # MFMAs of a super-step issued behind its barrier
VALU_START = 3.0   # place (within tile t's period) where softmax(t+1) starts
MIN_MFMA_TO_VALU = 20   # instructions between an MFMA and the first vector instruction that reads its result
# DIRECT: the e4m3 codes of the weights are built without an exponential.  The code of a positive e4m3 number, read as
# an integer, is 8 (log2 of the number + 7) with the mantissa interpolated linearly (exact at the powers of two), so
# P = sat_u8(rne(8 (c S - m) + 56 - 0.46)) is exp2(c S - m) rounded to e4m3 up to that interpolation (0.46: its mean, so
# that the codes are unbiased; a fifth of them differ from the correctly rounded code, by one step).  The caller passes
# c_loop = 8 c and m_loop = 8 m - 55.54 (otherwise c and m); per score one multiply-add and one v_cvt_pk_u8_f32 (4 issue cycles
# each, measured) replace multiply-add, v_exp_f32 (8) and half a v_cvt_pk_fp8_f32 (8).  The conversion saturates at 255:
# code 0x7F is NaN and reaches the row sum through the MFMA, codes from 0x80 on (negative numbers) are caught by the
# OR of all P registers in v[FLAGS].  Both forms are generated; the kernel takes this one for callers that set
# CFK_OPT_FAST_E4M3_WEIGHTS (a fifth of the weights one code off is a price the default does not pay).
DIRECT = False
ABLATE = set(os.environ.get("LOOP8_ABLATE", "").split(",")) - {""}


def o_reg(db): return O0 + 16 * db
def s_reg(t, kb): return (SA0 if t % 2 == 0 else SB0) + 16 * kb
def q_reg(s): return Q0 + 8 * s
def p_reg(t): return P0 + 8 * (t % 2)
def vr(r, n): return "v[%d:%d]" % (r, r + n - 1)


class Frag:
    """one MFMA operand fragment: 8 registers of the ring, consumed by the MFMA at place `slot`"""
    def __init__(self, kind, t, a, b, slot, idx):
        self.kind, self.t, self.a, self.b, self.slot, self.idx = kind, t, a, b, slot, idx
        self.reg = RING0 + 8 * (idx % RING)

    def reads(self):
        ring_slot = self.t % NSLOT
        if self.kind == 'K':   # K-step a, key block b
            off = ring_slot * K_TILE + self.b * 32 * K_PITCH
            return ["ds_read_b128 %s, v%d offset:%d" % (vr(self.reg + 4 * h, 4), KRD0 + 2 * self.a + h, off) for h in range(2)]
        off = ring_slot * V_TILE   # d block b
        return ["ds_read_b64_tr_b8 %s, v%d offset:%d" % (vr(self.reg + 2 * u, 2), VRD0 + self.b, off + 16 * u * V_PITCH) for u in range(4)]

    def mfma(self):
        if self.kind == 'K':
            d = s_reg(self.t, self.b)
            return "v_mfma_f32_32x32x64_f8f6f4 %s, %s, %s, %s" % (vr(d, 16), vr(self.reg, 8), vr(q_reg(self.a), 8), "0" if self.a == 0 else vr(d, 16))
        d = o_reg(self.b)
        return "v_mfma_f32_32x32x64_f8f6f4 %s, %s, %s, %s" % (vr(d, 16), vr(self.reg, 8), vr(p_reg(self.t), 8), vr(d, 16))


def sum_mfma(t):
    return "v_mfma_f32_16x16x128_f8f6f4 %s, %s, %s, %s" % (vr(LACC0, 4), vr(ONES0, 8), vr(p_reg(t), 8), vr(LACC0, 4))


def softmax_ops(t):
    """vector instructions of softmax(t) in issue order: (text, issue cost in units of 4 cycles).  Accumulator element
    4 w + j of block kb becomes byte j of P register 4 kb + w (fmha_fwd_kernel.h: softmax_exp)."""
    ops = []
    for kb in range(KB):
        for w in range(4):
            s = s_reg(t, kb) + 4 * w
            p = p_reg(t) + 4 * kb + w
            for i in range(4): ops.append(("v_fma_f32 v%d, v%d, %%[c], -v%d" % (s + i, s + i, MREF), 1))
            if DIRECT:
                for i in range(4): ops.append(("v_cvt_pk_u8_f32 v%d, v%d, %d, %s" % (p, s + i, i, "v%d" % p if i else "0"), 1))
                if w % 2: ops.append(("v_or3_b32 v%d, v%d, v%d, v%d" % (FLAGS, FLAGS, p - 1, p), 1))
                continue
            for i in range(4): ops.append(("v_exp_f32 v%d, v%d" % (s + i, s + i), 2))
            ops.append(("v_cvt_pk_fp8_f32 v%d, v%d, v%d" % (p, s, s + 1), 2))
            ops.append(("v_cvt_pk_fp8_f32 v%d, v%d, v%d op_sel:[0,0,1]" % (p, s + 2, s + 3), 2))
    return ops


def ipw(): return K_TILE // 1024 // NWAVES   # copies per wave and tile (K and V alike)


def copy_ops(kind, ring_slot):
    """the wave's global->LDS copies of its share of one tile into ring slot `ring_slot` (1 KB each, NWAVES KB apart), then
    the pointer moves on one tile"""
    base = (K_ST0 if kind == 'K' else V_ST0) + ring_slot * K_TILE
    go, sp = (GOK, 40) if kind == 'K' else (GOV, 42)
    ops = [["s_add_u32 m0, %%[ldsw], %d" % (base + i * NWAVES * 1024), "s_nop 0", "global_load_lds_dwordx4 v%d, s[%d:%d]" % (go[i], sp, sp + 1)]
           for i in range(ipw())]
    ops[-1] += ["s_add_u32 s%d, s%d, %%[stride]" % (sp, sp), "s_addc_u32 s%d, s%d, 0" % (sp + 1, sp + 1)]
    return ops


def schedule(n_tiles):
    """straight-line program for n_tiles key tiles (a multiple of 4, at least 8), as a list of segments, one per
    super-step; a segment ends with its barrier (the last one has none)"""
    assert n_tiles % 4 == 0 and n_tiles >= 8
    n_slots = T * n_tiles
    n_steps = n_tiles // 2
    SS = 2 * T
    slot_item = [None] * n_slots
    frags = []
    for t in range(n_tiles):
        base = T * t
        if t + 1 < n_tiles:
            for kb in range(KB):
                for s in range(KS):
                    f = Frag('K', t + 1, s, kb, base + kb * KS + s, len(frags)); frags.append(f)
                    slot_item[f.slot] = f
        for db in range(DB):
            f = Frag('V', t, 0, db, base + 4 + db, len(frags)); frags.append(f)
            slot_item[f.slot] = f
        slot_item[base + 8] = ("L", t)
    # ---- vector work: place -> [text]; positions before place 0 are issued ahead of it
    valu_at = {}
    rate = sum(c for _, c in softmax_ops(0)) / float(T)
    for t in range(n_tiles):
        start = T * (t - 1) + VALU_START
        cum = 0.0
        for txt, cost in softmax_ops(t):
            valu_at.setdefault(max(int(start + cum / rate), -1), []).append(txt)
            cum += cost
    # ---- copies: super-step J, one copy every fourth place from its second place on
    copies_at = {}
    for J in range(n_steps):
        groups = []
        for kind, t in (('K', 2 * J + 3), ('K', 2 * J + 4), ('V', 2 * J + 2), ('V', 2 * J + 3)):
            if t < n_tiles: groups += copy_ops(kind, t % NSLOT)
        for i, grp in enumerate(groups): copies_at[SS * J + 1 + (4 // ipw()) * i] = grp
    # ---- the workgroup's next work item (persistent workgroups): in the last super-step, whose K slots 0-2 and V slots
    # 0-1 are free, copy that item's first three K and two V tiles into them and, once the last S = K.Q^T has been
    # issued, load its Q into the Q registers; both are waited for at the end of the statement
    Z = SS * (n_steps - 1)
    copies_at[Z] = ["s_mov_b64 s[40:41], %[kn]", "s_mov_b64 s[42:43], %[vn]"]
    groups = []
    for kind, ring_slot in (('K', 0), ('K', 1), ('K', 2), ('V', 0), ('V', 1)): groups += copy_ops(kind, ring_slot)
    for i, grp in enumerate(groups): copies_at[Z + 1 + (3 * i if ipw() == 1 else i)] = grp
    for i in range(2 * KS):
        copies_at.setdefault(Z + 5 + i, []).append("global_load_dwordx4 %s, v%d, %%[qn] offset:%d" % (vr(q_reg(i // 2) + 4 * (i % 2), 4), QOFF, 64 * (i // 2) + 16 * (i % 2)))
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
        return slot > SS * J - HOLD   # `slot` is the place after the MFMA just issued
    def request(slot, limit):
        nonlocal next_frag, nread
        n = 0
        while next_frag < len(frags) and n < limit:
            f = frags[next_frag]
            # ring entry free: the fragment RING places earlier has been consumed (its MFMA issued)
            if next_frag >= RING and frags[next_frag - RING].slot >= slot: break
            if f.slot > slot + LOOKAHEAD: break
            if not barrier_passed_for(f, slot): break
            for r in f.reads():
                if "reads" not in ABLATE: cur.append(r); nread += 1
            read_end[f.idx] = nread
            next_frag += 1; n += 1
    cur.append("s_waitcnt lgkmcnt(0)")
    cur.append("s_nop 7"); cur.append("s_nop 7"); cur.append("s_nop 7")   # MFMA results of the caller's S(0) are read by vector instructions
    for r in range(O0, O0 + 64): cur.append("v_mov_b32 v%d, 0" % r)
    for r in range(LACC0, LACC0 + 4): cur.append("v_mov_b32 v%d, 0" % r)
    if DIRECT: cur.append("v_mov_b32 v%d, 0" % FLAGS)
    if "reads" in ABLATE:
        for r in range(RING0, RING0 + 8 * RING): cur.append("v_mov_b32 v%d, 0" % r)
    request(0, LOOKAHEAD)
    for txt in valu_at.get(-1, []): cur.append(txt)
    for slot in range(n_slots):
        J = slot // SS
        if slot % SS == SS - HOLD and J < n_steps - 1:
            cur.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
            if "barrier" not in ABLATE: cur.append("s_barrier")
            done_reads = nread
            segs.append(cur); cur = []
        it = slot_item[slot]
        if it is not None and "mfma" not in ABLATE:
            if isinstance(it, tuple):
                cur.append(sum_mfma(it[1]))
            else:
                if read_end[it.idx] > done_reads:
                    out = nread - read_end[it.idx]
                    assert out <= 15
                    if "reads" not in ABLATE: cur.append("s_waitcnt lgkmcnt(%d)" % out)
                    done_reads = read_end[it.idx]
                cur.append(it.mfma())
        request(slot + 1, 1)
        if "valu" not in ABLATE:
            for txt in valu_at.get(slot, []): cur.append(txt)
        if "copies" not in ABLATE:
            for txt in copies_at.get(slot, []): cur.append(txt)
    assert next_frag == len(frags)
    cur.append("s_waitcnt vmcnt(0)")               # the next item's Q (registers) and first tiles (LDS) have arrived
    cur.append("s_nop 7"); cur.append("s_nop 7"); cur.append("s_nop 7")   # the accumulators are read by the caller's vector instructions
    segs.append(cur)
    assert len(segs) == n_steps
    return segs


def folded():
    """(head, loop body, tail): head = super-steps 0,1; body = 2,3 (repeated); tail = the last two"""
    segs = schedule(16)
    assert segs[2] + segs[3] == segs[4] + segs[5], "the schedule is not periodic"
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
    """the C++ text of the include: the complete asm statement.  It expects these names in scope: f32x16 o0..o3 (out), sa0,
    sa1 (in, clobbered: S(0) of key blocks 0, 1), qv (in: this item's Q; out: the next item's); f32x4 lacc (out: the row
    sum, complete in every lane); int8v ones (the 0/1 operand); uint64_t kptr, vptr (in: this item's K tile 3 / V tile
    2; out: the same of the next item), kn, vn, qn (the next item's K, V and this wave's Q rows); uint32_t nloop,
    k_rd[4], v_rd[4], goff_k[], goff_v[] (one per copy of the wave and tile), qoff, lds_wave, tile_stride; float m_loop, c_loop; with DIRECT also uint32_t p_flags
    (out) and constexpr bool kDirect."""
    head, body, tail = folded()
    L = []
    L.append("// GENERATED by gen_fmha_loop8.py -- do not edit.  The hand-scheduled main loop of fmha_fwd_kernel8p (e4m3, head dim")
    L.append("// 128, %d x 128): %d + %d (loop) + %d instructions." % (32 * NWAVES, len(head), len(body), len(tail)))
    L.append("// The weights are built as e4m3 codes without an exponential: c_loop = 8 c, m_loop = 8 m - 55.54, p_flags = OR of all P (true);")
    L.append("// or with v_exp_f32 and v_cvt_pk_fp8_f32: c_loop = c, m_loop = m (false)")
    L.append("static_assert(kDirect == %s, \"the caller passes the scale and the reference point in the form this loop takes\");" % ("true" if DIRECT else "false"))
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
    L.append('    : "={v[192:207]}"(o0), "={v[208:223]}"(o1), "={v[224:239]}"(o2), "={v[240:255]}"(o3), "={v[44:47]}"(lacc),%s' % (' "={v%d}"(p_flags),' % FLAGS if DIRECT else ""))
    L.append('      "+{v[128:143]}"(sa0), "+{v[144:159]}"(sa1), "+{v[112:127]}"(qv), "+{s[40:41]}"(kptr), "+{s[42:43]}"(vptr), [nloop] "+s"(nloop)')
    ins = ['"{v[36:43]}"(ones)', '"{v%d}"(qoff)' % QOFF, '[kn] "s"(kn)', '[vn] "s"(vn)', '[qn] "s"(qn)']
    ins += ['"{v%d}"(k_rd[%d])' % (KRD0 + i, i) for i in range(4)] + ['"{v%d}"(v_rd[%d])' % (VRD0 + i, i) for i in range(DB)]
    ins += ['"{v%d}"(goff_k[%d])' % (GOK[i], i) for i in range(ipw())] + ['"{v%d}"(goff_v[%d])' % (GOV[i], i) for i in range(ipw())]
    ins += ['"{v%d}"(m_loop)' % MREF]
    ins += ['[c] "s"(c_loop)', '[ldsw] "s"(lds_wave)', '[stride] "s"(tile_stride)']
    L.append("    : " + ", ".join(ins))
    used = set(range(O0, O0 + 64)) | set(range(SA0, SA0 + 32)) | set(range(Q0, Q0 + 16)) | set(range(LOW, LACC0 + 4))
    if DIRECT: used.add(FLAGS)
    used |= set(GOK[:ipw()]) | set(GOV[:ipw()])
    # (registers the loop never names stay the compiler's: values it keeps across the statement need not be spilled)
    import re
    named = set()
    for ins in head + body + tail:
        for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", ins):
            named |= set(range(int(m.group(1)), int(m.group(2)) + 1)) if m.group(1) else {int(m.group(3))}
    clob = ['"memory"', '"scc"', '"m0"'] + ['"v%d"' % r for r in range(LOW, 256) if r not in used and r in named]
    L.append("    : " + ", ".join(clob) + ");")
    return "\n".join(L) + "\n"


if __name__ == "__main__":
    for k, v in json.loads(os.environ.get("LOOP8_SET", "{}")).items(): globals()[k] = v
    stale = False
    for NWAVES, DIRECT, name in ((8, False, "fmha_fwd_loop8_d128.inc"), (8, True, "fmha_fwd_loop8_d128_direct.inc"),
                                 (4, False, "fmha_fwd_loop8_d128w4.inc"), (4, True, "fmha_fwd_loop8_d128w4_direct.inc")):
        out = os.path.join(os.path.dirname(os.path.abspath(__file__)), name)
        txt = render()
        if "--check" in sys.argv:
            stale = stale or not (os.path.exists(out) and open(out).read() == txt)
        else:
            open(out, "w").write(txt)
            print("wrote", out, len(txt.splitlines()), "lines")
    sys.exit(1 if stale else 0)
