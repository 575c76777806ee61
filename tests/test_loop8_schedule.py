"""Symbolic check of the hand-scheduled main loop of the e4m3 kernel (cutlass-kernels_amd/csrc/gen_fmha_loop8.py).

Like test_loop16_schedule.py for the fp16 loop: the instruction text a wave executes (loop unrolled for several key
lengths) is walked with symbolic register contents, and instruction by instruction the test checks that
  * every MFMA multiplies the operands the algorithm wants (K fragment x Q of the same K-step into the right score
    block; V fragment x P of the same tile into the right output block; the 0/1 operand x P into the row sum),
    accumulations happen in order and exactly once;
  * every LDS read hits a ring slot that holds the expected tile, completed by a barrier, and no copy overwrites a slot
    that any wave may still read in the same barrier interval; LDS data is waited for (lgkmcnt) before it is used;
  * register reuse: a value is overwritten only after all of its uses;
  * the software-visible hazards: MFMA result -> vector read distance, transcendental result -> use, vector write ->
    MFMA operand, M0 write -> LDS-DMA;
  * the next work item's first tiles and Q are requested in the last super-step and waited for;
  * the committed .inc file is what the generator produces.
No GPU involved.
"""
import importlib.util
import os
import re
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cutlass-kernels_amd", "csrc")
FOREVER = 10 ** 9


def _gen():
    spec = importlib.util.spec_from_file_location("gen_fmha_loop8", os.path.join(CSRC, "gen_fmha_loop8.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


class Val:
    """a symbolic register value with a use counter"""
    __slots__ = ("tag", "need", "uses", "widx", "wkind", "pend")

    def __init__(self, tag, need, widx, wkind, pend=None):
        self.tag, self.need, self.uses, self.widx, self.wkind, self.pend = tag, need, 0, widx, wkind, pend


class Checker:
    def __init__(self, g, n_tiles):
        self.g, self.n = g, n_tiles
        self.v = {}
        self.idx = 0          # instruction distance counter (s_nop n counts n+1)
        self.nread = self.complete = 0
        self.m0 = None
        self.m0_idx = -10
        self.kptr, self.vptr = 3, 2
        self.next_item = {"s40": False, "s42": False}   # the pointer walks the next work item's tiles
        self.vm_pending = False                          # a load with a register destination is in flight
        self.copied = {"s40": set(), "s42": set()}       # the parts of a tile copied since the pointer last moved
        self.kslot = {0: 0, 1: 1, 2: 2, 3: None}
        self.vslot = {0: 0, 1: 1, 2: None, 3: None}
        self.inflight = []    # copies issued since the last barrier: (kind, slot, tile)
        self.seg_reads = set()
        self.waited_all = False
        self.n_mfma = self.n_qk = self.n_flagged = 0
        for s in range(g.KS):
            for i in range(8): self.put(g.q_reg(s) + i, ("Q", s, i), FOREVER, "init")
        self.put(g.MREF, ("m",), FOREVER, "init")
        self.put(g.QOFF, ("qoff",), FOREVER, "init")
        for kb in range(g.KB):
            for i in range(16): self.put(g.s_reg(0, kb) + i, ("S", 0, kb, g.KS - 1, i), 1, "init")
        for s in range(g.KS):
            for h in range(2): self.put(g.KRD0 + 2 * s + h, ("krd", s, h), FOREVER, "init")
        for db in range(g.DB): self.put(g.VRD0 + db, ("vrd", db), FOREVER, "init")
        for i in range(8): self.put(g.ONES0 + i, ("ones", i), FOREVER, "init")
        for i in range(g.ipw()):
            self.put(g.GOK[i], ("gok", i), FOREVER, "init")
            self.put(g.GOV[i], ("gov", i), FOREVER, "init")

    # ---- register file
    def put(self, r, tag, need, kind, pend=None):
        old = self.v.get(r)
        if old is not None and old.need < FOREVER:
            assert old.uses == old.need, "v%d overwritten with %r while %r has %d of %d uses (%s)" % (r, tag, old.tag, old.uses, old.need, self.cur)
        self.v[r] = Val(tag, need, self.idx, kind, pend)

    def get(self, r, reader):
        val = self.v.get(r)
        assert val is not None, "v%d read undefined (%s)" % (r, self.cur)
        if val.pend is not None:
            assert val.pend <= self.complete, "v%d read before its LDS data was waited for (%s)" % (r, self.cur)
        dist = self.idx - val.widx - 1   # instructions between the write and this read
        if val.wkind == "mfma" and reader == "valu":
            assert dist >= self.g.MIN_MFMA_TO_VALU, "MFMA result v%d read by a vector instruction after %d instructions (%s)" % (r, dist, self.cur)
        if val.wkind == "mfma" and reader == "mfma_c":
            assert dist >= 2, "dependent MFMAs %d apart (%s)" % (dist, self.cur)
        if val.wkind == "trans" and reader in ("valu", "mfma"):
            assert dist >= 1, "transcendental result v%d used by the next instruction (%s)" % (r, self.cur)
        if val.wkind == "valu" and reader == "mfma":
            assert dist >= 2, "vector result v%d is an MFMA operand %d instructions later (%s)" % (r, dist, self.cur)
        val.uses += 1
        return val.tag

    # ---- instructions
    def run(self, prog):
        g = self.g
        R = lambda s: [int(x) for x in re.match(r"v\[(\d+):(\d+)\]", s).groups()]
        for ins in prog:
            self.cur = ins
            op, _, rest = ins.partition(" ")
            a = [x.strip() for x in rest.split(",")] if rest else []
            if op == "s_nop":
                self.idx += int(a[0]) + 1
                continue
            if op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", rest)
                n = int(m.group(1)) if m else None
                if n is not None:
                    assert n <= 15
                    self.complete = max(self.complete, self.nread - n)
                if "vmcnt(0)" in rest: self.vm_pending = False
                self.waited_all = "vmcnt(0)" in rest and n == 0
            elif op == "s_barrier":
                assert self.waited_all, "barrier without a full wait in front"
                for kind, slot, t in self.inflight:
                    assert (kind, slot) not in self.seg_reads, "%s slot %d copied and read in one barrier interval" % (kind, slot)
                    (self.kslot if kind == "K" else self.vslot)[slot] = t
                self.inflight, self.seg_reads = [], set()
            elif op == "v_mov_b32":
                assert a[1] == "0"
                self.put(int(a[0][1:]), ("zero",), FOREVER, "valu")
            elif op == "ds_read_b128":
                lo, hi = R(a[0])
                assert hi == lo + 3 and lo % 4 == 0
                addr, off = a[1].split(" offset:")
                tag = self.get(int(addr[1:]), "lds")
                off = int(off)
                assert tag[0] == "krd" and off % 4096 == 0 and off < g.NSLOT * g.K_TILE
                slot, kb = off // g.K_TILE, (off % g.K_TILE) // 4096
                t = self.kslot[slot]
                assert t is not None and ("K", slot) not in [(k, s) for k, s, _ in self.inflight], "K slot %d not readable (%s)" % (slot, ins)
                self.seg_reads.add(("K", slot))
                self.nread += 1
                for i in range(4): self.put(lo + i, ("Kf", t, tag[1], kb, 4 * tag[2] + i), 1, "lds", self.nread)
            elif op == "ds_read_b64_tr_b8":
                lo, hi = R(a[0])
                assert hi == lo + 1 and lo % 2 == 0
                addr, off = a[1].split(" offset:")
                tag = self.get(int(addr[1:]), "lds")
                off = int(off)
                assert tag[0] == "vrd" and off % 2048 == 0 and off < g.NSLOT * g.V_TILE
                slot, u = off // g.V_TILE, (off % g.V_TILE) // 2048
                t = self.vslot[slot]
                assert t is not None and ("V", slot) not in [(k, s) for k, s, _ in self.inflight], "V slot %d not readable (%s)" % (slot, ins)
                self.seg_reads.add(("V", slot))
                self.nread += 1
                for i in range(2): self.put(lo + i, ("Vf", t, tag[1], 2 * u + i), 1, "lds", self.nread)
            elif op == "v_mfma_f32_32x32x64_f8f6f4":
                self.mfma(R(a[0]), R(a[1]), R(a[2]), None if a[3] == "0" else R(a[3]))
            elif op == "v_mfma_f32_16x16x128_f8f6f4":
                self.sum_mfma(R(a[0]), R(a[1]), R(a[2]), R(a[3]))
            elif op == "v_fma_f32":
                d, s_ = int(a[0][1:]), int(a[1][1:])
                assert d == s_ and a[2] == "%[c]" and a[3] == "-v%d" % g.MREF
                tag = self.get(s_, "valu")
                assert self.get(g.MREF, "valu") == ("m",)
                assert tag[0] == "S" and tag[3] == g.KS - 1 and d == g.s_reg(tag[1], tag[2]) + tag[4], ins
                self.put(d, ("X", tag[1], tag[2], tag[4]), 1, "valu")
            elif op == "v_exp_f32":
                d, s_ = int(a[0][1:]), int(a[1][1:])
                tag = self.get(s_, "valu")
                assert not g.DIRECT and d == s_ and tag[0] == "X", ins
                self.put(d, ("E",) + tag[1:], 1, "trans")
            elif op == "v_cvt_pk_u8_f32":   # byte `byte` of a P register: the e4m3 code of one weight, straight from X
                d, s_, byte, src2 = int(a[0][1:]), int(a[1][1:]), int(a[2]), a[3]
                tag = self.get(s_, "valu")
                assert g.DIRECT and tag[0] == "X", ins
                t, kb, e = tag[1], tag[2], tag[3]
                w = e // 4
                assert e % 4 == byte and d == g.p_reg(t) + 4 * kb + w, ins
                if byte == 0: assert src2 == "0", ins
                else: assert src2 == "v%d" % d and self.get(d, "valu") == ("Pb", t, kb, w, byte - 1), ins
                if byte < 3: self.put(d, ("Pb", t, kb, w, byte), 1, "valu")
                else: self.put(d, ("P", t, kb, w), g.DB + 2, "valu")   # four P.V MFMAs, the row sum, the flags
            elif op == "v_or3_b32":         # every P register goes into the overflow flags exactly once
                d = int(a[0][1:])
                assert g.DIRECT and d == g.FLAGS and a[1] == "v%d" % d, ins
                assert self.get(d, "valu")[0] in ("zero", "flags")
                ta, tb = self.get(int(a[2][1:]), "valu"), self.get(int(a[3][1:]), "valu")
                assert ta[0] == "P" and tb[0] == "P" and ta[1:3] == tb[1:3] and ta[3] % 2 == 0 and tb[3] == ta[3] + 1, ins
                self.n_flagged += 2
                self.put(d, ("flags",), FOREVER, "valu")
            elif op == "v_cvt_pk_fp8_f32":
                high = a[-1].endswith("op_sel:[0") or "op_sel" in rest
                d = int(a[0][1:])
                ta, tb = self.get(int(a[1][1:]), "valu"), self.get(int(a[2].split()[0][1:]), "valu")
                assert ta[0] == "E" and tb[0] == "E" and ta[1:3] == tb[1:3] and tb[3] == ta[3] + 1, ins
                t, kb, e = ta[1], ta[2], ta[3]
                w = e // 4
                assert e % 4 == (2 if high else 0) and d == g.p_reg(t) + 4 * kb + w, ins
                if high:
                    assert "op_sel:[0,0,1]" in rest.replace(" ", "")
                    assert self.get(d, "valu") == ("Plo", t, kb, w), ins
                    self.put(d, ("P", t, kb, w), g.DB + 1, "valu")
                else:
                    self.put(d, ("Plo", t, kb, w), 1, "valu")
            elif op == "s_add_u32" and a[0] == "m0":
                assert a[1] == "%[ldsw]"
                self.m0, self.m0_idx = int(a[2]), self.idx
            elif op == "global_load_lds_dwordx4":
                assert self.idx - self.m0_idx >= 2, "M0 written right in front of the copy"
                gt = self.get(int(a[0][1:]), "vmem")
                kind = "K" if self.m0 < g.V_ST0 else "V"
                rel = self.m0 - (g.K_ST0 if kind == "K" else g.V_ST0)
                slot, part = rel // g.K_TILE, (rel % g.K_TILE) // (g.NWAVES * 1024)
                sp = "s40" if kind == "K" else "s42"
                assert rel % (g.NWAVES * 1024) == 0 and part < g.ipw() and slot < g.NSLOT and gt == ("gok" if kind == "K" else "gov", part), ins
                assert a[1] == ("s[40:41]" if kind == "K" else "s[42:43]")
                t = self.kptr if kind == "K" else self.vptr
                if self.next_item[sp]:
                    assert t < (3 if kind == "K" else 2) and slot == t, "next item: copy of tile %d into slot %d (%s)" % (t, slot, ins)
                    t = ("next", t)   # no MFMA of this program may read it
                else:
                    assert t < self.n and slot == t % g.NSLOT, "copy of tile %d into slot %d (%s)" % (t, slot, ins)
                assert (kind, slot) not in self.seg_reads, "%s slot %d read and then copied into in one barrier interval" % (kind, slot)
                assert part not in self.copied[sp], "two copies of one part of a tile"
                self.copied[sp].add(part)
                if part == 0: self.inflight.append((kind, slot, t))
                (self.kslot if kind == "K" else self.vslot)[slot] = None
            elif op == "s_add_u32":
                sp = a[0]
                assert sp == a[1] and a[2] == "%[stride]" and sp in ("s40", "s42")
                assert self.copied[sp] == set(range(g.ipw())), "pointer moved before all copies of the tile"
                self.copied[sp] = set()
                if sp == "s40": self.kptr += 1
                else: self.vptr += 1
            elif op == "s_mov_b64":
                sp = {"s[40:41]": "s40", "s[42:43]": "s42"}[a[0]]
                assert a[1] == ("%[kn]" if sp == "s40" else "%[vn]")
                assert (self.kptr if sp == "s40" else self.vptr) == self.n, "pointer handed to the next item before this item's copies are out"
                assert not self.copied[sp]
                self.next_item[sp] = True
                if sp == "s40": self.kptr = 0
                else: self.vptr = 0
            elif op == "global_load_dwordx4":
                lo, hi = R(a[0])
                addr, off = a[2].split(" offset:")
                off = int(off)
                assert self.get(int(a[1][1:]), "vmem") == ("qoff",)
                s, h = off // 64, (off % 64) // 16
                assert addr == "%[qn]" and hi == lo + 3 and off % 16 == 0 and h < 2 and s < g.KS and lo == g.q_reg(s) + 4 * h, ins
                assert self.n_qk == g.KB * g.KS * (self.n - 1), "Q overwritten before the last S = K.Q^T was issued"
                for i in range(4): self.put(lo + i, ("Qnext", s, 4 * h + i), FOREVER, "vmem")
                self.vm_pending = True
            elif op == "s_addc_u32":
                assert a[0] == a[1] and a[2] == "0" and a[0] in ("s41", "s43")
            else:
                raise AssertionError("unknown instruction: " + ins)
            self.idx += 1

    def mfma(self, d, a, b, c):
        g = self.g
        assert d[1] == d[0] + 15 and a[1] == a[0] + 7 and b[1] == b[0] + 7 and (c is None or c == d), self.cur
        d, a, b = d[0], a[0], b[0]
        self.n_mfma += 1
        ta = [self.get(a + i, "mfma") for i in range(8)]
        tb = [self.get(b + i, "mfma") for i in range(8)]
        if ta[0][0] == "Kf":
            _, t, s, kb, _ = ta[0]
            assert ta == [("Kf", t, s, kb, i) for i in range(8)], self.cur
            assert tb == [("Q", s, i) for i in range(8)] and b == g.q_reg(s), self.cur
            assert d == g.s_reg(t, kb), self.cur
            self.n_qk += 1
            if s == 0:
                assert c is None, self.cur
                for i in range(16):   # the block's previous content (an odd/even tile before) has been consumed
                    old = self.v.get(d + i)
                    assert old is None or old.uses == old.need, "S block overwritten before the softmax read it (%s)" % self.cur
            else:
                assert c is not None
                tc = [self.get(d + i, "mfma_c") for i in range(16)]
                assert tc == [("S", t, kb, s - 1, i) for i in range(16)], self.cur
            for i in range(16): self.put(d + i, ("S", t, kb, s, i), 1, "mfma")
        else:
            _, t, db, _ = ta[0]
            assert ta == [("Vf", t, db, i) for i in range(8)], self.cur
            assert tb == [("P", t, kb, w) for kb in range(g.KB) for w in range(4)] and b == g.p_reg(t), self.cur
            assert d == g.o_reg(db) and c is not None, self.cur
            tc = [self.get(d + i, "mfma_c") for i in range(16)]
            n_prev = 0 if tc[0] == ("zero",) else tc[0][2]
            assert all(x == ("zero",) for x in tc) or tc == [("O", db, n_prev, i) for i in range(16)], self.cur
            assert n_prev == t, "O[%d] accumulates tile %d as its %d-th term" % (db, t, n_prev)
            for i in range(16): self.put(d + i, ("O", db, n_prev + 1, i), 1, "mfma")

    def sum_mfma(self, d, a, b, c):
        g = self.g
        assert d == [g.LACC0, g.LACC0 + 3] and c == d and a == [g.ONES0, g.ONES0 + 7] and b[1] == b[0] + 7, self.cur
        self.n_mfma += 1
        assert [self.get(a[0] + i, "mfma") for i in range(8)] == [("ones", i) for i in range(8)]
        tb = [self.get(b[0] + i, "mfma") for i in range(8)]
        t = tb[0][1]
        assert tb == [("P", t, kb, w) for kb in range(g.KB) for w in range(4)] and b[0] == g.p_reg(t), self.cur
        tc = [self.get(d[0] + i, "mfma_c") for i in range(4)]
        n_prev = 0 if tc[0] == ("zero",) else tc[0][1]
        assert all(x == ("zero",) for x in tc) or tc == [("lacc", n_prev, i) for i in range(4)], self.cur
        assert n_prev == t, "row sum takes tile %d as its %d-th term" % (t, n_prev)
        for i in range(4): self.put(d[0] + i, ("lacc", n_prev + 1, i), 1, "mfma")

    def finish(self):
        g, n = self.g, self.n
        for db in range(g.DB):
            for i in range(16): assert self.v[g.o_reg(db) + i].tag == ("O", db, n, i)
        for i in range(4): assert self.v[g.LACC0 + i].tag == ("lacc", n, i)
        if g.DIRECT: assert self.n_flagged == 4 * g.KB * n and self.v[g.FLAGS].tag == ("flags",)
        assert self.n_mfma == g.KB * g.KS * (n - 1) + (g.DB + 1) * n
        # the next work item: its first three K and two V tiles are on their way into slots 0-2 / 0-1, its Q is in the Q
        # registers, and everything has been waited for
        assert self.next_item == {"s40": True, "s42": True} and self.kptr == 3 and self.vptr == 2 and not any(self.copied.values())
        assert sorted((k, s, t) for k, s, t in self.inflight) == [("K", i, ("next", i)) for i in range(3)] + [("V", i, ("next", i)) for i in range(2)]
        assert not self.vm_pending
        for s in range(g.KS):
            for i in range(8): assert self.v[g.q_reg(s) + i].tag == ("Qnext", s, i)
        # the accumulators are read by the caller right after the statement
        last_mfma = max(v.widx for v in self.v.values() if v.wkind == "mfma")
        assert self.idx - last_mfma > g.MIN_MFMA_TO_VALU


@pytest.mark.parametrize("nwaves", [8, 4])
@pytest.mark.parametrize("direct", [True, False])
@pytest.mark.parametrize("n_tiles", [8, 12, 16, 32, 64, 128])
def test_loop_is_correct_symbolically(n_tiles, direct, nwaves):
    g = _gen()
    g.DIRECT, g.NWAVES = direct, nwaves
    c = Checker(g, n_tiles)
    c.run(g.program(n_tiles))
    c.finish()


def test_checker_catches_a_broken_schedule():
    g = _gen()
    prog = g.program(8)
    # drop one LDS wait: some MFMA then reads a fragment that was not waited for
    k = next(i for i, ins in enumerate(prog) if ins.startswith("s_waitcnt lgkmcnt(") and i > 200)
    bad = prog[:k] + prog[k + 1:]
    with pytest.raises(AssertionError):
        c = Checker(g, 8)
        c.run(bad)
        c.finish()
    # move a fragment read to the neighbouring key block
    k = next(i for i, ins in enumerate(prog) if ins.startswith("ds_read_b128") and i > 300)
    bad = list(prog)
    bad[k] = re.sub(r"offset:(\d+)", lambda m: "offset:%d" % ((int(m.group(1)) + 4096) % 32768), bad[k])
    with pytest.raises(AssertionError):
        c = Checker(g, 8)
        c.run(bad)
        c.finish()
    # start the softmax of a tile too close behind the MFMAs that produce its scores
    k = next(i for i, ins in enumerate(prog) if ins.startswith("v_fma_f32") and i > 400)
    reg = int(prog[k].split()[1][1:-1])
    block = reg - (reg - g.SA0) % 16
    j = max(i for i in range(k) if prog[i].startswith("v_mfma_f32_32x32x64") and prog[i].split()[1].startswith("v[%d:" % block))
    bad = prog[:j + 1] + [prog[k]] + prog[j + 1:k] + prog[k + 1:]
    with pytest.raises(AssertionError):
        c = Checker(g, 8)
        c.run(bad)
        c.finish()


def test_committed_include_is_the_generators_output():
    r = subprocess.run([sys.executable, os.path.join(CSRC, "gen_fmha_loop8.py"), "--check"])
    assert r.returncode == 0, "fmha_fwd_loop8_d128*.inc are stale: run gen_fmha_loop8.py"
