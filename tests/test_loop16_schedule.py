"""Symbolic check of the hand-scheduled main loops of the fp16 kernel (cutlass-kernels_amd/csrc/gen_fmha_loop16.py), in
its five shapes (head dim 128: 8 waves, 64-key tiles; head dim
256: 4 waves, 32-key tiles, O in accumulation registers;
head dim 64: 8 waves, 64-key tiles of 8 KB, row sum on the matrix pipe; head dims 128 and 64 again for 4 waves with O
in accumulation registers).

A loop is ~2800 hand-allocated instructions inside one asm statement, where neither the compiler's register
allocator nor its hazard recognizer helps.  This test walks the instruction text a wave executes (loop unrolled for
several key lengths) with symbolic register contents and checks, instruction by instruction:
  * every MFMA multiplies the operands the algorithm wants (K fragment x Q of the same K-step into the right score
    block; V fragment x P of the same tile, key half and query block into the right output block), accumulations happen
    in order and exactly once;
  * every LDS read hits a ring slot that holds the expected tile, completed by a barrier, and no copy overwrites a slot
    that any wave may still read in the same barrier interval; LDS data is waited for (lgkmcnt) before it is used;
  * register reuse: a value is overwritten only after all of its uses;
  * the hardware's software-visible hazards: MFMA result -> vector read distance, transcendental result -> use,
    dot-product result -> other vector instruction, M0 write -> LDS-DMA;
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


def _gen():
    spec = importlib.util.spec_from_file_location("gen_fmha_loop16", os.path.join(CSRC, "gen_fmha_loop16.py"))
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
        self.kparts, self.vparts = set(), set()
        self.kslot = {0: 0, 1: 1, 2: 2, 3: None}
        self.vslot = {0: 0, 1: 1, 2: None, 3: None}
        self.inflight = []    # copies issued since the last barrier: (kind, slot, tile)
        self.seg_reads = set()
        self.waited_all = False
        self.n_mfma = self.n_qk = 0
        for qb in range(g.QB):
            for s in range(g.KS):
                for i in range(4): self.put(g.q_reg(qb, s) + i, ("Q", qb, s, i), 10 ** 9, "init")
            if g.FOLDED: self.put(g.MN0 + 4 * qb, ("mneg", qb), 10 ** 9, "init")
            else: self.put(g.M0R + qb, ("m", qb), 10 ** 9, "init")
            self.put(g.QOFF0 + qb, ("qoff", qb), 10 ** 9, "init")
        self.e_need = 2 if g.ROWSUM == "add" else 1                 # uses of an exponential: the convert (+ the add)
        self.p_need = g.DB + (0 if g.ROWSUM == "add" else 1)        # uses of a packed weight: 8 MFMAs (+ the row sum)
        for kb in range(g.KB):
            for qb in range(g.QB):
                for i in range(4): self.put(g.s_reg(0, kb, qb) + i, ("S", 0, kb, qb, g.KS - 1, i), 1, "init")
        for s in range(g.KS): self.put(g.KRD0 + s, ("krd", s), 10 ** 9, "init")
        for db in range(g.DB): self.put(g.VRD0 + db, ("vrd", db), 10 ** 9, "init")
        for i in range(g.IPW):
            self.put(g.GOK0 + i, ("gok", i), 10 ** 9, "init")
            self.put(g.GOV0 + i, ("gov", i), 10 ** 9, "init")

    # ---- register file
    def put(self, r, tag, need, kind, pend=None):
        old = self.v.get(r)
        if old is not None and old.need < 10 ** 9:
            assert old.uses == old.need, "v%d overwritten with %r while %r has %d of %d uses (%s)" % (r, tag, old.tag, old.uses, old.need, self.cur)
        self.v[r] = Val(tag, need, self.idx, kind, pend)

    def get(self, r, reader):
        val = self.v.get(r)
        assert val is not None, "v%d read undefined (%s)" % (r, self.cur)
        if val.pend is not None:
            assert val.pend <= self.complete, "v%d read before its LDS data was waited for (%s)" % (r, self.cur)
        dist = self.idx - val.widx - 1   # instructions between the write and this read
        if val.wkind == "mfma" and reader == "valu":
            assert dist >= 8, "MFMA result v%d read by a vector instruction after %d instructions (%s)" % (r, dist, self.cur)
        if val.wkind == "mfma" and reader == "mfma_c":
            assert dist >= 2, "dependent MFMAs %d apart (%s)" % (dist, self.cur)
        if val.wkind == "trans" and reader in ("valu", "mfma"):
            assert dist >= 1, "transcendental result v%d used by the next instruction (%s)" % (r, self.cur)
        if val.wkind == "dot" and reader == "valu":
            assert dist >= 3, "dot result v%d read by another vector instruction after %d (%s)" % (r, dist, self.cur)
        val.uses += 1
        return val.tag

    # ---- instructions
    def run(self, prog):
        g = self.g
        def R(s):   # register range -> [first, last]; accumulation registers a[n] are numbered 1000 + n
            m = re.match(r"([va])\[(\d+):(\d+)\]", s)
            base = 1000 if m.group(1) == "a" else 0
            return [base + int(m.group(2)), base + int(m.group(3))]
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
            elif op == "v_mov_b32" and a[1].startswith("v"):
                tag = self.get(int(a[1][1:]), "valu")
                assert g.FOLDED and tag[0] == "mneg" and 0 < int(a[0][1:]) - (g.MN0 + 4 * tag[1]) < 4, ins
                self.put(int(a[0][1:]), tag, 10 ** 9, "valu")
            elif op == "v_mov_b32":
                assert a[1] in ("0", "0x3c003c00")
                self.put(int(a[0][1:]), ("zero",) if a[1] == "0" else ("one",), 10 ** 9, "valu")
            elif op == "v_accvgpr_write_b32":
                assert a[1] == "0" and a[0][0] == "a"
                self.put(1000 + int(a[0][1:]), ("zero",), 10 ** 9, "valu")
            elif op == "ds_read_b128":
                lo, hi = R(a[0])
                assert hi == lo + 3 and lo % 4 == 0
                addr, off = a[1].split(" offset:")
                tag = self.get(int(addr[1:]), "lds")
                off = int(off)
                assert tag[0] == "krd" and off % (16 * g.K_PITCH) == 0 and off < 65536
                slot, kb = off // g.K_TILE, (off % g.K_TILE) // (16 * g.K_PITCH)
                t = self.kslot[slot]
                assert t is not None and ("K", slot) not in [(k, s) for k, s, _ in self.inflight], "K slot %d not readable (%s)" % (slot, ins)
                self.seg_reads.add(("K", slot))
                self.nread += 1
                for i in range(4): self.put(lo + i, ("Kf", t, tag[1], kb, i), 2, "lds", self.nread)
            elif op == "ds_read_b64_tr_b16":
                lo, hi = R(a[0])
                assert hi == lo + 1 and lo % 2 == 0
                addr, off = a[1].split(" offset:")
                tag = self.get(int(addr[1:]), "lds")
                off = int(off)
                assert tag[0] == "vrd" and off % (16 * g.V_PITCH) == 0 and off < 65536
                slot, rem = off // g.V_TILE, off % g.V_TILE
                ps, half = rem // (32 * g.V_PITCH), (rem % (32 * g.V_PITCH)) // (16 * g.V_PITCH)
                t = self.vslot[slot]
                assert t is not None and ("V", slot) not in [(k, s) for k, s, _ in self.inflight], "V slot %d not readable (%s)" % (slot, ins)
                self.seg_reads.add(("V", slot))
                self.nread += 1
                for i in range(2): self.put(lo + i, ("Vf", t, ps, tag[1], half, i), 2, "lds", self.nread)
            elif op == "v_mfma_f32_16x16x32_f16":
                self.mfma(R(a[0])[0], R(a[1])[0], R(a[2])[0], None if a[3] == "0" else R(a[3])[0])
            elif op == "v_fma_f32":
                d, s_ = int(a[0][1:]), int(a[1][1:])
                assert not g.FOLDED and d == s_ and a[2] == "%[c]" and a[3].startswith("-v")
                tag = self.get(s_, "valu")
                mt = self.get(int(a[3][2:]), "valu")
                assert tag[0] == "S" and tag[4] == g.KS - 1 and d == g.s_reg(tag[1], tag[2], tag[3]) + tag[5] and mt == ("m", tag[3]), ins
                self.put(d, ("X",) + tag[1:4] + (tag[5],), 1, "valu")
            elif op == "v_exp_f32":
                d, s_ = int(a[0][1:]), int(a[1][1:])
                tag = self.get(s_, "valu")
                if g.FOLDED:   # the score comes off the matrix pipe scaled and with the reference point taken off
                    assert tag[0] == "S" and tag[4] == g.KS - 1 and d == g.s_reg(tag[1], tag[2], tag[3]) + tag[5], ins
                    tag = ("X",) + tag[1:4] + (tag[5],)
                assert d == s_ and tag[0] == "X", ins
                self.put(d, ("E",) + tag[1:], self.e_need, "trans")
            elif op == "v_cvt_pk_f16_f32":
                d = int(a[0][1:])
                ta, tb = self.get(int(a[1][1:]), "valu"), self.get(int(a[2][1:]), "valu")
                assert ta[0] == "E" and tb[0] == "E" and ta[1:4] == tb[1:4] and ta[4] % 2 == 0 and tb[4] == ta[4] + 1, ins
                t, kb, qb, j = ta[1], ta[2], ta[3], ta[4] // 2
                assert d == g.p_reg(t, qb, kb // 2) + 2 * (kb % 2) + j, ins
                self.put(d, ("Ph", t, qb, kb, j), self.p_need, "valu")
            elif op in ("v_dot2_f32_f16", "v_dot2c_f32_f16"):
                d = int(a[0][1:])
                assert a[1] == "%[ones]"
                pt = self.get(int(a[2][1:]), "valu")
                assert pt[0] == "Ph"
                t, qb, kb, j = pt[1:]
                assert d == (g.RS0 if j == 0 else g.RS20) + qb, ins
                if op == "v_dot2_f32_f16":
                    assert a[3] == "0" and kb == 0, ins
                    done = ()
                else:
                    old = self.v[d]
                    assert old.tag[0] == "rs" and old.tag[1:4] == (t, qb, j) and old.tag[4] == tuple(range(kb)), ins
                    old.uses = old.need = 0
                    done = old.tag[4]
                self.put(d, ("rs", t, qb, j, done + (kb,)), 1, "dot")
            elif op == "v_add_f32":
                d, x, y = (int(s[1:]) for s in a)
                assert d == x
                tx, ty = self.get(x, "valu"), self.get(y, "valu")
                if g.ROWSUM == "add":
                    if ty[0] == "E":      # l chain j of query block qb takes elements j, j+2 of every block, in order
                        t, kb, qb, i = ty[1:]
                        assert d == g.LA0 + 2 * qb + i % 2, ins
                        cnt = 0 if tx == ("zero",) else tx[3]
                        assert tx == ("zero",) or tx[:3] == ("la", qb, i % 2)
                        assert cnt == (t * g.KB + kb) * 2 + i // 2, "weights summed out of order (%s)" % ins
                        self.put(d, ("la", qb, i % 2, cnt + 1), 10 ** 9, "valu")
                    else:                 # the two chains of a query block meet after the last tile
                        full = self.n * g.KB * 2
                        assert tx[0] == "la" and ty[0] == "la" and tx[1] == ty[1] and (tx[2], ty[2]) == (0, 1) and tx[3] == full and ty[3] == full, ins
                        self.put(d, ("l", tx[1], self.n), 10 ** 9, "valu")
                elif tx[0] == "rs":
                    full = tuple(range(g.KB))
                    assert ty[0] == "rs" and tx[1:3] == ty[1:3] and (tx[3], ty[3]) == (0, 1) and tx[4] == full and ty[4] == full, ins
                    self.put(d, ("rsum", tx[1], tx[2]), 1, "valu")
                else:
                    assert ty[0] == "rsum" and d == g.L0 + ty[2], ins
                    n_prev = 0 if tx == ("zero",) else tx[2]
                    assert tx == ("zero",) or tx[:2] == ("l", ty[2])
                    assert n_prev == ty[1], "row sums joined out of order (%s)" % ins
                    self.put(d, ("l", ty[2], n_prev + 1), 10 ** 9, "valu")
            elif op == "s_add_u32" and a[0] == "m0":
                assert a[1] == "%[ldsw]"
                self.m0, self.m0_idx = int(a[2]), self.idx
            elif op == "global_load_lds_dwordx4":
                assert self.idx - self.m0_idx >= 2, "M0 written right in front of the copy"
                gt = self.get(int(a[0][1:]), "vmem")
                kind = "K" if self.m0 < g.V_ST0 else "V"
                rel = self.m0 - (g.K_ST0 if kind == "K" else g.V_ST0)
                slot, part = rel // g.K_TILE, (rel % g.K_TILE) // (g.NWAVES * 1024)
                assert rel % (g.NWAVES * 1024) == 0 and part < g.IPW and gt == ("gok" if kind == "K" else "gov", part), ins
                assert a[1] == ("s[40:41]" if kind == "K" else "s[42:43]")
                t = self.kptr if kind == "K" else self.vptr
                if self.next_item["s40" if kind == "K" else "s42"]:
                    assert t < (3 if kind == "K" else 2) and slot == t, "next item: copy of tile %d into slot %d (%s)" % (t, slot, ins)
                    t = ("next", t)   # no MFMA of this program may read it
                else:
                    assert t < self.n and slot == t % g.NSLOT, "copy of tile %d into slot %d (%s)" % (t, slot, ins)
                assert (kind, slot) not in self.seg_reads, "%s slot %d read and then copied into in one barrier interval" % (kind, slot)
                parts = self.kparts if kind == "K" else self.vparts
                assert part not in parts
                parts.add(part)
                if part == 0: self.inflight.append((kind, slot, t))
                (self.kslot if kind == "K" else self.vslot)[slot] = None
            elif op == "s_add_u32":
                sp = a[0]
                assert sp == a[1] and a[2] == "%[stride]" and sp in ("s40", "s42")
                parts = self.kparts if sp == "s40" else self.vparts
                assert parts == set(range(g.IPW)), "pointer moved before all copies of the tile"
                parts.clear()
                if sp == "s40": self.kptr += 1
                else: self.vptr += 1
            elif op == "s_mov_b64":
                sp = {"s[40:41]": "s40", "s[42:43]": "s42"}[a[0]]
                assert a[1] == ("%[kn]" if sp == "s40" else "%[vn]")
                assert (self.kptr if sp == "s40" else self.vptr) == self.n, "pointer handed to the next item before this item's copies are out"
                assert not (self.kparts if sp == "s40" else self.vparts)
                self.next_item[sp] = True
                if sp == "s40": self.kptr = 0
                else: self.vptr = 0
            elif op == "global_load_dwordx4":
                lo, hi = R(a[0])
                addr, off = a[2].split(" offset:")
                qt = self.get(int(a[1][1:]), "vmem")
                assert addr == "%[qn]" and qt[0] == "qoff" and hi == lo + 3 and lo == g.q_reg(qt[1], int(off) // 64) and int(off) % 64 == 0, ins
                assert self.n_qk == g.QKS * (self.n - 1), "Q overwritten before the last S = K.Q^T was issued"
                for i in range(4): self.put(lo + i, ("Qnext", qt[1], int(off) // 64, i), 10 ** 9, "vmem")
                self.vm_pending = True
            elif op == "s_addc_u32":
                assert a[0] == a[1] and a[2] == "0" and a[0] in ("s41", "s43")
            else:
                raise AssertionError("unknown instruction: " + ins)
            self.idx += 1

    def mfma(self, d, a, b, c):
        g = self.g
        self.n_mfma += 1
        ta = [self.get(a + i, "mfma") for i in range(4)]
        tb = [self.get(b + i, "mfma") for i in range(4)]
        if ta[0] == ("one",):
            assert ta == [("one",)] * 4 and a == g.ONES0, self.cur
            _, t, qb, kb0, _ = tb[0]
            ps = kb0 // 2
            assert tb == [("Ph", t, qb, 2 * ps + j // 2, j % 2) for j in range(4)] and b == g.p_reg(t, qb, ps), self.cur
            assert d == g.LACC0 + 4 * qb and c == d, self.cur
            tc = [self.get(d + i, "mfma_c") for i in range(4)]
            n_prev = 0 if tc[0] == ("zero",) else tc[0][2]
            assert all(x == ("zero",) for x in tc) or tc == [("lacc", qb, n_prev, i) for i in range(4)], self.cur
            assert n_prev == 2 * t + ps, "row sum takes tile %d half %d as its %d-th term" % (t, ps, n_prev)
            for i in range(4): self.put(d + i, ("lacc", qb, n_prev + 1, i), 1, "mfma")
        elif ta[0][0] == "Kf":
            _, t, s, kb, _ = ta[0]
            assert ta == [("Kf", t, s, kb, i) for i in range(4)], self.cur
            qb = tb[0][1]
            assert tb == [("Q", qb, s, i) for i in range(4)] and b == g.q_reg(qb, s), self.cur
            assert d == g.s_reg(t, kb, qb), self.cur
            self.n_qk += 1
            if s == 0 and g.FOLDED:
                assert c == g.MN0 + 4 * qb and [self.get(c + i, "mfma_c") for i in range(4)] == [("mneg", qb)] * 4, self.cur
            elif s == 0:
                assert c is None, self.cur
            else:
                assert c == d
                tc = [self.get(d + i, "mfma_c") for i in range(4)]
                assert tc == [("S", t, kb, qb, s - 1, i) for i in range(4)], self.cur
            for i in range(4): self.put(d + i, ("S", t, kb, qb, s, i), 1, "mfma")
        else:
            _, t, ps, db, _, _ = ta[0]
            assert ta == [("Vf", t, ps, db, h, i) for h in range(2) for i in range(2)], self.cur
            qb = tb[0][2]
            assert tb == [("Ph", t, qb, 2 * ps + j // 2, j % 2) for j in range(4)] and b == g.p_reg(t, qb, ps), self.cur
            assert d == self.o_id(db, qb) and c == d, self.cur
            tc = [self.get(d + i, "mfma_c") for i in range(4)]
            n_prev = 0 if tc[0] == ("zero",) else tc[0][3]
            assert all(x == ("zero",) for x in tc) or tc == [("O", db, qb, n_prev, i) for i in range(4)], self.cur
            assert n_prev == g.PS * t + ps, "O[%d][%d] accumulates tile %d half %d as its %d-th term" % (db, qb, t, ps, n_prev)
            for i in range(4): self.put(d + i, ("O", db, qb, n_prev + 1, i), 1, "mfma")

    def o_id(self, db, qb):
        return (1000 if self.g.O_ACC else 0) + self.g.o_reg(db, qb)

    def finish(self):
        g, n = self.g, self.n
        for db in range(g.DB):
            for qb in range(g.QB):
                for i in range(4): assert self.v[self.o_id(db, qb) + i].tag == ("O", db, qb, g.PS * n, i)
        for qb in range(g.QB):
            if g.ROWSUM == "mfma": assert self.v[g.L_OUT[qb]].tag == ("lacc", qb, 2 * n, 0)
            else: assert self.v[g.L_OUT[qb]].tag == ("l", qb, n)
        assert self.n_mfma == g.QKS * (n - 1) + (g.T - g.QKS) * n
        # the next work item: its first three K and two V tiles are on their way into slots 0-2 / 0-1, its Q is in the Q
        # registers, and everything has been waited for
        assert self.next_item == {"s40": True, "s42": True} and self.kptr == 3 and self.vptr == 2 and not self.kparts and not self.vparts
        assert sorted((k, s, t) for k, s, t in self.inflight) == [("K", i, ("next", i)) for i in range(3)] + [("V", i, ("next", i)) for i in range(2)]
        assert not self.vm_pending
        for qb in range(g.QB):
            for ks in range(g.KS):
                for i in range(4): assert self.v[g.q_reg(qb, ks) + i].tag == ("Qnext", qb, ks, i)
        # the accumulators are read by the caller right after the statement
        last_mfma = max(v.widx for v in self.v.values() if v.wkind == "mfma")
        assert self.idx - last_mfma > 8


@pytest.mark.parametrize("shape,rowsum,fold", [("d128", "mfma", False), ("d128", "mfma", True), ("d128", "add", True), ("d128w4", "add", True), ("d128", "add", False), ("d128", "dot", False),
                                               ("d256", "add", True), ("d256", "add", False), ("d64", "mfma", True), ("d64", "mfma", False), ("d64w4", "mfma", True)])
@pytest.mark.parametrize("n_tiles", [8, 12, 16, 32, 64])
def test_loop_is_correct_symbolically(n_tiles, shape, rowsum, fold):
    g = _gen()
    g.SHAPE, g.ROWSUM, g.FOLD = shape, rowsum, fold
    g.configure()
    assert g.FOLDED == fold
    c = Checker(g, n_tiles)
    c.run(g.program(n_tiles))
    c.finish()


@pytest.mark.parametrize("shape", ["d128", "d128w4", "d256", "d64", "d64w4"])
def test_checker_catches_a_broken_schedule(shape):
    g = _gen()
    g.SHAPE, g.ROWSUM = shape, ("mfma" if shape.startswith("d64") else "add")
    g.configure()
    prog = g.program(8)
    # drop one LDS wait: some MFMA then reads a fragment that was not waited for
    k = next(i for i, ins in enumerate(prog) if ins.startswith("s_waitcnt lgkmcnt(") and i > 200)
    bad = prog[:k] + prog[k + 1:]
    with pytest.raises(AssertionError):
        c = Checker(g, 8)
        c.run(bad)
        c.finish()
    # swap the operands of two neighbouring fragment reads
    k = next(i for i, ins in enumerate(prog) if ins.startswith("ds_read_b128") and i > 300)
    bad = list(prog)
    bad[k] = re.sub(r"offset:(\d+)", lambda m: "offset:%d" % ((int(m.group(1)) + 16 * g.K_PITCH) % 65536), bad[k])
    with pytest.raises(AssertionError):
        c = Checker(g, 8)
        c.run(bad)
        c.finish()


def test_committed_include_is_the_generators_output():
    r = subprocess.run([sys.executable, os.path.join(CSRC, "gen_fmha_loop16.py"), "--check"])
    assert r.returncode == 0, "fmha_fwd_loop16_{d128,d128w4,d256,d64,d64w4}.inc are stale: run gen_fmha_loop16.py"
