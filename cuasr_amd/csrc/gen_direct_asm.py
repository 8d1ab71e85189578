#!/usr/bin/env python3
"""Generates the hand-scheduled main loops of the 4-wave direct-to-LDS SRGEMM tiles
(direct_tile.h for 4-byte, direct64_tile.h for 8-byte element types) as inline-asm text:
one k-tile (16 k) of the register tile per asm statement, for each pair of panel forms.

Why generated asm and not C++: on gfx950 a SIMD issues about one instruction every 2.1 cycles
whatever its kind (a satisfied s_waitcnt, an s_nop or a scalar add costs as much as a v_add_f32),
and an LDS read costs about 5.5 cycles whatever its width.  The compiler's version of the 4-byte
loop spends 1536 vector instructions per k-tile plus 96 LDS reads, 89 waits and 76 nops; this
schedule spends the same 1536 plus 64 LDS reads (16-byte reads only), about 20 waits and no nops.
For 8-byte types (4.5 cycles per fp64 instruction, the other instructions hide beneath them) the
gain is the register count: accumulators, ONE set of fragments refilled in place and four
temporaries fit 128 registers, i.e. 4 waves per SIMD, where the compiled loop needs 136.

Register plan (128 VGPRs, 4 waves per SIMD):
    v0   .. v63    accumulators: 4-byte acc[i][j] = v(8 i + j), 8 x 8; 8-byte acc[i][j] = v[8 i + 2 j : +1], 8 x 4
    v64  .. v111   fragments of the operand called Q, then of the operand called P
    v112 .. v115   temporaries
  A fragment register group is refilled for its next use right after its last use, so that every
  LDS read is issued half a k-pair or more before its data is consumed.
  4-byte types: P is an x-contiguous panel ([k][X] in LDS, one 16-byte read = 4 x at one k): 16
    registers hold one k-pair, refilled half by half (4 x, both k).  Q is either k-contiguous
    ([k/4][X][4], one read = 4 k of one x): 32 registers hold a k-quad, each x refilled after its
    last use in the quad's second k-pair; or x-contiguous like P.
  8-byte types: Q = A (8 x), P = B (4 x), each holding one k-pair: x-contiguous ([k][X], one read =
    2 x at one k) or k-contiguous ([k/2][X][2], one read = both k of one x).
  A k-pair is worked in two phases, one per half of P; within a phase the x of Q in order.

LDS reads complete in order, so "s_waitcnt lgkmcnt(N)" leaves the N youngest in flight.  The
generator keeps the queue of reads in flight, emits a wait only where a fragment is consumed
whose read the queue still holds, lets each wait also cover every read old enough to have landed,
and checks for every vector instruction that the registers it reads hold the operand, x and k
it means.  A statement ends with everything drained, so no read is in flight while compiler
code runs.

Output: string-literal fragments for `asm volatile(` to include.  The arithmetic is a macro the
including code defines for its semiring (register names as string literals):
    4-byte: CUASR_TERM2(acc, t0, t1, q0, p0, q1, p1)   acc <- add(acc, mult(q0, p0), mult(q1, p1))
    8-byte: CUASR_TERM1(acc, t, q, p)                  acc <- add(acc, mult(q, p))
everything else is literal text.
"""
import os
import sys

BK = 16
ACC0, FRAG0, TEMP0 = 0, 64, 112
WAIT_AGE = 20   # a wait also covers reads issued at least this many groups of 3-4 instructions ago


class Panel:
    """Fragment registers and LDS reads of one operand.
    esize 4 or 8; nx = x per thread; xt = threads along x (the panel is nx * xt wide)."""

    def __init__(self, name, kc, esize, nx, xt, reg0, addr):
        self.name, self.kc, self.esize, self.nx, self.xt, self.reg0, self.addr = name, kc, esize, nx, xt, reg0, addr
        self.er = esize // 4                                   # registers per element
        self.period = 4 if (kc and esize == 4) else 2          # k a fill of one unit covers
        self.nregs = nx * self.period * self.er
        self.X = nx * xt

    # a unit = what one refill replaces: one x of a k-contiguous panel, 4 (2) x of an x-contiguous one
    def units(self):
        return range(self.nx) if self.kc else range(self.nx * self.esize // 16)

    def unit_of(self, x):
        return x if self.kc else x // (16 // self.esize)

    def reg(self, x, k):
        if self.kc:
            return self.reg0 + (x * self.period + k % self.period) * self.er
        per = 16 // self.esize                                  # x per read
        return self.reg0 + ((k & 1) * (self.nx // per) + x // per) * 4 + (x % per) * self.er

    def reads_for(self, unit, k_first):
        """[(asm text, {register: (operand, x, k)})] filling `unit` with the period starting at the
        tile-relative k_first (>= 16: the next tile, read through the already advanced address)."""
        out = []
        k = k_first % BK
        if self.kc:
            r = self.reg(unit, k_first)
            off = ((k // self.period) * self.X + unit * self.xt) * 16
            fills = {}
            for e in range(self.period):
                for w in range(self.er):
                    fills[r + e * self.er + w] = (self.name, unit, k_first + e)
            out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{self.addr}] offset:{off}", fills))
        else:
            per = 16 // self.esize
            for s in range(2):
                r = self.reg(unit * per, k_first + s)
                off = ((k + s) * self.X + unit * per * self.xt) * self.esize
                fills = {}
                for e in range(per):
                    for w in range(self.er):
                        fills[r + e * self.er + w] = (self.name, unit * per + e, k_first + s)
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{self.addr}] offset:{off}", fills))
        return out


class Body:
    def __init__(self, esize, a_kc, b_kc):
        self.esize = esize
        if esize == 4:
            assert not (a_kc and b_kc), "two k-quad operands do not fit 128 registers"
            ty, tx = 32, 16
            q_is_a = a_kc or not b_kc          # Q = the operand held per k-quad if there is one, else A
            nq = np_ = 8
        else:
            ty, tx = 16, 32
            q_is_a = True
            nq, np_ = 8, 4
        self.q_is_a = q_is_a
        qa, pa = ("a_addr", "b_addr") if q_is_a else ("b_addr", "a_addr")
        self.Q = Panel("A" if q_is_a else "B", a_kc if q_is_a else b_kc, esize, nq, ty if q_is_a else tx, FRAG0, qa)
        self.P = Panel("B" if q_is_a else "A", b_kc if q_is_a else a_kc, esize, np_, tx if q_is_a else ty,
                       FRAG0 + self.Q.nregs, pa)
        assert self.P.period == 2 and self.P.reg0 + self.P.nregs <= TEMP0
        self.a_kc, self.b_kc = a_kc, b_kc
        self.lines = []
        self.content = {}     # register -> (operand, x, k) it holds or is being filled with
        self.inflight = []    # [(registers, group count at issue)] oldest first
        self.groups = 0       # groups emitted so far (the clock of WAIT_AGE)
        self.tcount = 0
        self.stats = {"groups": 0, "lds": 0, "waits": 0, "other": 0}

    # ---- emission
    def emit(self, text, kind="other"):
        self.lines.append(text)
        self.stats[kind] += 1

    def issue(self, panel, unit, k_first):
        for text, fills in panel.reads_for(unit, k_first):
            self.emit(text, "lds")
            self.content.update(fills)
            self.inflight.append((set(fills), self.groups))

    def require(self, regs):
        """Make sure no read into `regs` is still in flight (wait if the queue holds one)."""
        last = max((i for i, (rs, _) in enumerate(self.inflight) if rs & regs), default=None)
        if last is None:
            return
        # also cover everything old enough to have landed, so that the next uses need no wait
        for i, (_, born) in enumerate(self.inflight):
            if self.groups - born >= WAIT_AGE:
                last = max(last, i)
        left = len(self.inflight) - 1 - last
        assert left <= 15
        self.emit(f"s_waitcnt lgkmcnt({left})", "waits")
        self.inflight = self.inflight[last + 1:]

    def drain(self, text="s_waitcnt lgkmcnt(0)"):
        self.emit(text, "waits")
        self.inflight = []

    def vname(self, r):
        return f"v{r}" if self.esize == 4 else f"v[{r}:{r + 1}]"

    def operands(self, i, j, k):
        qx, px = (i, j) if self.q_is_a else (j, i)
        rq, rp = self.Q.reg(qx, k), self.P.reg(px, k)
        for w in range(self.Q.er):
            assert self.content.get(rq + w) == (self.Q.name, qx, k), (rq, self.content.get(rq + w), qx, k)
            assert self.content.get(rp + w) == (self.P.name, px, k), (rp, self.content.get(rp + w), px, k)
        return rq, rp

    def term(self, i, j, k0):
        """4-byte: acc[i][j] <- add(acc, mult(a[i][k0], b[k0][j]), mult(a[i][k0 + 1], b[k0 + 1][j]))
        8-byte: the two terms one after the other."""
        if self.esize == 4:
            q0, p0 = self.operands(i, j, k0)
            q1, p1 = self.operands(i, j, k0 + 1)
            self.require({q0, p0, q1, p1})
            t0 = TEMP0 + self.tcount % 4
            t1 = TEMP0 + (self.tcount + 1) % 4
            self.tcount += 2
            acc = ACC0 + i * 8 + j
            self.lines.append(f'CUASR_TERM2("v{acc}", "v{t0}", "v{t1}", "v{q0}", "v{p0}", "v{q1}", "v{p1}")')
        else:
            acc = ACC0 + (i * 4 + j) * 2
            for k in (k0, k0 + 1):
                q, p = self.operands(i, j, k)
                self.require({q, q + 1, p, p + 1})
                t = TEMP0 + (self.tcount % 2) * 2
                self.tcount += 1
                self.lines.append(f'CUASR_TERM1("{self.vname(acc)}", "{self.vname(t)}", "{self.vname(q)}", "{self.vname(p)}")')
        self.groups += 1
        self.stats["groups"] += 1

    # ---- global -> LDS: this wave's pieces (1 KiB each) of the tile two ahead
    def fetch(self):
        e = self.emit
        e("s_cmp_lt_i32 %[fetch], 1")
        e("s_cbranch_scc1 .Lcuasr_nofetch_%=")
        e("s_mov_b32 %[m0_save], m0")   # M0 is the compiler's own for its LDS-bound loads: hand it back unchanged
        if self.esize == 4:
            # two pieces of the A panel, one of the B panel; lane offsets come ready-made
            e("s_mov_b32 m0, %[m0_a]")
            e("s_nop 0")
            e("global_load_lds_dwordx4 %[off_a0], %[base_a]")
            e("s_add_u32 m0, m0, 0x400")
            e("s_nop 0")
            e("global_load_lds_dwordx4 %[off_a1], %[base_a]")
            e("s_mov_b32 m0, %[m0_b]")
            e("s_nop 0")
            e("global_load_lds_dwordx4 %[off_b0], %[base_b]")
        else:
            # two pieces of each panel (128 x 16 doubles = 16 KiB = 2 pieces for each of 8 waves).
            # Piece q of a wave is LDS positions (2 wave + q) * 64 + lane (16 bytes each):
            #   x-contiguous (64 positions per k): the same x, k = 2 wave + q -> the base moves on by one k
            #   k-contiguous (128 positions per k-pair): x = 64 q + lane, same k-pair -> a second lane offset
            for name, kc in (("a", self.a_kc), ("b", self.b_kc)):
                e(f"s_mov_b32 m0, %[m0_{name}]")
                e("s_nop 0")
                e(f"global_load_lds_dwordx4 %[off_{name}0], %[base_{name}]")
                e("s_add_u32 m0, m0, 0x400")
                e("s_nop 0")
                e(f"global_load_lds_dwordx4 %[off_{name}1], %[base_{name}]")
        e("s_mov_b32 m0, %[m0_save]")
        e(".Lcuasr_nofetch_%=:")

    # ---- the bodies
    def resident_after_prime(self):
        for unit in self.Q.units():
            for _, fills in self.Q.reads_for(unit, 0):
                self.content.update(fills)
        for unit in self.P.units():
            for _, fills in self.P.reads_for(unit, 0):
                self.content.update(fills)

    def prime(self):
        """Fragments of the first k-quad / k-pair of the first tile."""
        for unit in self.Q.units():
            self.issue(self.Q, unit, 0)
        for unit in self.P.units():
            self.issue(self.P, unit, 0)
        self.drain()
        return self.lines

    def tile(self):
        # state on entry = state after prime() or after a previous tile(): everything resident, nothing in flight
        self.resident_after_prime()
        entry = dict(self.content)
        three_stages = self.esize == 4
        if three_stages:
            # three LDS stages: the stage of the tile two ahead was handed back by the previous tile's barrier
            self.fetch()
        nkp = BK // 2
        P, Q = self.P, self.Q
        p_units = list(P.units())
        for kp in range(nkp):
            k0 = 2 * kp
            last = kp == nkp - 1
            nk0 = k0 + 2                    # the next k-pair (>= 16: in the next tile)
            q_ends = (k0 + 2) % Q.period == 0       # Q's residency ends with this k-pair
            for half in range(2):
                if half == 1 and last:
                    # every read of this stage has returned and this wave's part of the next tile
                    # has landed; after the barrier that holds for the whole workgroup, and the
                    # stage is free to be overwritten.  The refills from here on read the next stage.
                    self.drain("s_waitcnt vmcnt(0) lgkmcnt(0)")
                    self.emit("s_barrier")
                    self.emit("v_add_u32 %[a_addr], %[a_step], %[a_addr]")
                    self.emit("v_add_u32 %[b_addr], %[b_step], %[b_addr]")
                    if not three_stages:
                        self.fetch()         # two stages: the one just handed back takes the tile two ahead
                if half == 1:
                    for u in p_units[:len(p_units) // 2]:
                        self.issue(P, u, nk0)       # half 0 of P is free: refill it for the next k-pair
                for qx in range(Q.nx):
                    for px in range(P.nx // 2 * half, P.nx // 2 * (half + 1)):
                        i, j = (qx, px) if self.q_is_a else (px, qx)
                        self.term(i, j, k0)
                    if half == 1 and q_ends:
                        u = Q.unit_of(qx)
                        if qx == max(x for x in range(Q.nx) if Q.unit_of(x) == u):   # the unit's last x is done
                            self.issue(Q, u, k0 + 2)
            for u in p_units[len(p_units) // 2:]:
                self.issue(P, u, nk0)
        self.drain()
        # the registers now hold the next tile's first fragments: same state as on entry
        shifted = {r: (o, x, k - BK) for r, (o, x, k) in self.content.items()}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines

    def text(self, lines):
        out = []
        for ln in lines:
            out.append(ln if ln.startswith("CUASR_TERM") else '"' + ln + '\\n"')
        return "\n".join(out) + "\n"


# name -> (element size, A k-contiguous, B k-contiguous)
VARIANTS = {"kx": (4, True, False), "xx": (4, False, False), "xk": (4, False, True),
            "d_kx": (8, True, False), "d_xx": (8, False, False), "d_xk": (8, False, True), "d_kk": (8, True, True)}


def generate(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    report = []
    for name, (esize, a_kc, b_kc) in VARIANTS.items():
        b = Body(esize, a_kc, b_kc)
        with open(os.path.join(out_dir, f"direct_asm_{name}_prime.inc"), "w") as f:
            f.write(b.text(b.prime()))
        b = Body(esize, a_kc, b_kc)
        with open(os.path.join(out_dir, f"direct_asm_{name}_tile.inc"), "w") as f:
            f.write(b.text(b.tile()))
        report.append((name, dict(b.stats)))
    return report


# ---------------------------------------------------------------------------------------------
# plus-times on the matrix cores (mfma_direct_f32.hip): v_mfma_f32_32x32x2_f32, direct-to-LDS panels
#
#   workgroup 256 threads = 4 waves (2 x 2), output tile 128 x 256, wave tile 64 x 128 = 2 x 4 blocks of 32 x 32
#   v0   .. v127   accumulators, block (bm, bn) in v[16 (4 bm + bn) : +15]
#   v128 .. v143   A fragments: buffer u, block bm, four registers = the four steps of a period of 8 k
#   v144 .. v175   B fragments: buffer u, block bn, four registers
# The instruction takes k from lanes 0..31 and another k from lanes 32..63; WHICH two k a step multiplies is
# free as long as A and B agree, so a period of 8 k is walked as (k, k + 4) for k = 0..3: lanes 0..31 hold the
# first k-quad of the period, lanes 32..63 the second.  A k-contiguous panel ([k/4][X][4] in LDS) then delivers a
# block's four steps with ONE 16-byte read per lane and no bank conflict; an x-contiguous panel ([k][X]) with
# four 4-byte reads of 32 + 32 consecutive floats.  Fragments are double-buffered by period; the reads for the
# next period are issued after the first eight matrix instructions of this one, so a register is overwritten
# 500 cycles and more after the last instruction that read it was issued.
class MfmaBody(Body):
    def __init__(self, a_kc, b_kc, nbn=4):
        self.a_kc, self.b_kc = a_kc, b_kc
        self.nbn = nbn   # 32-column blocks per wave: 4 (output tile 128 x 256) or 2 (128 x 128, accumulators v0 .. v63)
        self.lines, self.inflight, self.groups = [], [], 0
        self.stats = {"groups": 0, "lds": 0, "waits": 0, "other": 0}
        self.content = {}

    def frag(self, operand, u, blk, s):
        return (128 + (u * 2 + blk) * 4 + s) if operand == "A" else (144 + (u * self.nbn + blk) * 4 + s)

    def reads(self, period):
        """[(asm text, {register: content})]: LDS reads of the fragments of absolute period `period` (0, 1 of this
        tile; 2 = the next tile's first, through the already advanced addresses) into buffer period % 2."""
        u, P, out = period % 2, period % 2, []
        for operand, kc, X, nblk, addr in (("A", self.a_kc, 128, 2, "a_addr"), ("B", self.b_kc, 64 * self.nbn, self.nbn, "b_addr")):
            for blk in range(nblk):
                r = self.frag(operand, u, blk, 0)
                if kc:
                    out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}] offset:{(2 * P * X + blk * 32) * 16}",
                                {r + s: (operand, blk, period, s) for s in range(4)}))
                else:
                    for s in range(4):
                        out.append((f"ds_read_b32 v{r + s}, %[{addr}] offset:{((8 * P + s) * X + blk * 32) * 4}",
                                    {r + s: (operand, blk, period, s)}))
        return out

    def read(self, item):
        text, fills = item
        self.emit(text, "lds")
        self.content.update(fills)
        self.inflight.append((set(fills), self.groups))

    def mfma(self, period, s, bm, bn):
        u = period % 2
        ra, rb = self.frag("A", u, bm, s), self.frag("B", u, bn, s)
        assert self.content.get(ra) == ("A", bm, period, s) and self.content.get(rb) == ("B", bn, period, s)
        self.require_exact({ra, rb})
        acc = 16 * (self.nbn * bm + bn)
        self.lines.append(f'"v_mfma_f32_32x32x2_f32 v[{acc}:{acc + 15}], v{ra}, v{rb}, v[{acc}:{acc + 15}]\\n"')
        self.groups += 1
        self.stats["groups"] += 1

    def require_exact(self, regs):
        last = max((i for i, (rs, _) in enumerate(self.inflight) if rs & regs), default=None)
        if last is None:
            return
        left = len(self.inflight) - 1 - last
        assert left <= 15
        self.emit(f"s_waitcnt lgkmcnt({left})", "waits")
        self.inflight = self.inflight[last + 1:]

    def period(self, period, aux, first, last):
        """The 32 matrix instructions of a period of 8 k, with the callables of `aux` spread evenly behind
        instructions first .. last of them (counted from 0)."""
        order = [(s, bm, bn) for s in range(4) for bn in range(self.nbn) for bm in range(2)]
        behind = {}
        for i, item in enumerate(aux):
            slot = first + (i * (last - first + 1)) // len(aux)
            behind.setdefault(slot, []).append(item)
        for i, (s, bm, bn) in enumerate(order):
            self.mfma(period, s, bm, bn)
            for item in behind.get(i, []):
                item()

    def prime(self):
        for item in self.reads(0):
            self.read(item)
        self.drain()
        return self.lines

    def dma_chunk(self, index):
        """One 1 KiB piece of the tile two ahead, global -> LDS (skipped when there is no such tile): pieces 0, 1
        of the A panel, 2..5 of the B panel.  M0 holds the LDS address of the piece."""
        e = self.emit
        name, base, m0, h = ("a", "base_a", "m0_a", index) if index < 2 else ("b", "base_b", "m0_b", index - 2)
        e("s_cmp_lt_i32 %[fetch], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_%=")
        e(f"s_add_u32 m0, %[{m0}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[{base}]")
        e(f".Lcuasr_nofetch{index}_%=:")

    def tile(self):
        e = self.emit
        for operand, nblk in (("A", 2), ("B", self.nbn)):
            for blk in range(nblk):
                for s in range(4):
                    self.content[self.frag(operand, 0, blk, s)] = (operand, blk, 0, s)
        entry = dict(self.content)
        e("s_mov_b32 %[m0_save], m0")
        # period 0 (buffer 0).  Behind its matrix instructions, a few at a time: the six loads of the tile two
        # ahead and the LDS reads of period 1 (same stage) -- everything but the matrix instructions is spread so
        # that the matrix pipe never waits for a run of other instructions, and the last eight matrix instructions
        # (500 cycles) cover the latency of the last read
        nld = 2 + self.nbn                       # this wave's loads per k-tile
        last = 8 * self.nbn - 9                  # the last eight matrix instructions of a period cover the latency
        aux = [(lambda i=i: self.dma_chunk(i)) for i in range(nld)]
        rd = [(lambda it=it: self.read(it)) for it in self.reads(1)]
        # interleave the two kinds
        mixed, q = [], 0
        for i, r in enumerate(rd):
            while q < nld and q * len(rd) <= i * nld:
                mixed.append(aux[q])
                q += 1
            mixed.append(r)
        mixed += aux[q:]
        self.period(0, mixed, 1, last)
        e("s_mov_b32 m0, %[m0_save]")
        # every read of this stage has returned; this wave's part of the next tile has landed (its six loads are
        # older than the six of the tile two ahead, if those were issued); after the barrier both hold for the
        # workgroup, and the reads from here on go to the next stage
        e("s_cmp_lt_i32 %[fetch], 1")
        e("s_cbranch_scc1 .Lcuasr_all_%=")
        e(f"s_waitcnt vmcnt({nld}) lgkmcnt(0)")
        e("s_branch .Lcuasr_join_%=")
        e(".Lcuasr_all_%=:")
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e(".Lcuasr_join_%=:")
        self.inflight = []
        e("s_barrier")
        e("v_add_u32 %[a_addr], %[a_step], %[a_addr]")
        e("v_add_u32 %[b_addr], %[b_step], %[b_addr]")
        self.period(1, [(lambda it=it: self.read(it)) for it in self.reads(2)], 1, last)
        self.drain()
        shifted = {r: (o, b, p - 2, s) for r, (o, b, p, s) in self.content.items() if p >= 2}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines

    def text(self, lines):
        return "\n".join(ln if ln.startswith('"v_mfma') else '"' + ln + '\\n"' for ln in lines) + "\n"


MFMA_VARIANTS = {"m_kx": (True, False, 4), "m_xx": (False, False, 4), "m_xk": (False, True, 4), "m_kk": (True, True, 4),
                 "m2_kx": (True, False, 2), "m2_xx": (False, False, 2), "m2_xk": (False, True, 2), "m2_kk": (True, True, 2)}


def generate_mfma(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    report = []
    for name, (a_kc, b_kc, nbn) in MFMA_VARIANTS.items():
        b = MfmaBody(a_kc, b_kc, nbn)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_prime.inc"), "w") as f:
            f.write(b.text(b.prime()))
        b = MfmaBody(a_kc, b_kc, nbn)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_tile.inc"), "w") as f:
            f.write(b.text(b.tile()))
        report.append((name, dict(b.stats)))
    return report


# ---------------------------------------------------------------------------------------------
# plus-times for double on the matrix cores (mfma_direct_f64.hip): v_mfma_f64_16x16x4_f64
#
#   workgroup 256 threads = 4 waves (2 x 2), output tile 128 x 128, wave tile 64 x 64 = 4 x 4 blocks of 16 x 16
#   v0   .. v127   accumulators, block (bm, bn) in v[8 (4 bm + bn) : +7] (four doubles per lane)
#   v128 .. v159   A fragments: buffer u, block bm, two doubles = the two steps of a period of 8 k
#   v160 .. v191   B fragments: buffer u, block bn
# The instruction takes four k, one from each group of 16 lanes; a period of 8 k is walked as the k-pairs
# (2 g, 2 g + 1) of lane group g: step s multiplies k = 2 g + s.  A k-contiguous panel ([k/2][X][2] in LDS) then
# delivers a block's two steps with one 16-byte read per lane, an x-contiguous one ([k][X]) with two 8-byte reads.
# Two LDS stages: the loads of the tile two ahead are issued after the barrier in the middle of a tile, which
# is where the stage they go to has been read for the last time.
class Mfma64Body(MfmaBody):
    @staticmethod
    def frag(operand, u, blk, s):
        return (128 if operand == "A" else 160) + (u * 4 + blk) * 4 + 2 * s

    def reads(self, period):
        u, P, out = period % 2, period % 2, []
        for operand, kc, addr in (("A", self.a_kc, "a_addr"), ("B", self.b_kc, "b_addr")):
            X = 128
            for blk in range(4):
                r = self.frag(operand, u, blk, 0)
                if kc:
                    fills = {}
                    for s in range(2):
                        fills[r + 2 * s] = fills[r + 2 * s + 1] = (operand, blk, period, s)
                    out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}] offset:{(4 * P * X + blk * 16) * 16}", fills))
                else:
                    for s in range(2):
                        out.append((f"ds_read_b64 v[{r + 2 * s}:{r + 2 * s + 1}], %[{addr}] offset:{((8 * P + s) * X + blk * 16) * 8}",
                                    {r + 2 * s: (operand, blk, period, s), r + 2 * s + 1: (operand, blk, period, s)}))
        return out

    def mfma(self, period, s, bm, bn):
        u = period % 2
        ra, rb = self.frag("A", u, bm, s), self.frag("B", u, bn, s)
        for r, want in ((ra, ("A", bm, period, s)), (rb, ("B", bn, period, s))):
            assert self.content.get(r) == want and self.content.get(r + 1) == want
        self.require_exact({ra, ra + 1, rb, rb + 1})
        acc = 8 * (4 * bm + bn)
        self.lines.append(f'"v_mfma_f64_16x16x4_f64 v[{acc}:{acc + 7}], v[{ra}:{ra + 1}], v[{rb}:{rb + 1}], v[{acc}:{acc + 7}]\\n"')
        self.groups += 1
        self.stats["groups"] += 1

    def period(self, period, aux, first, last):
        order = [(s, bm, bn) for s in range(2) for bn in range(4) for bm in range(4)]
        behind = {}
        for i, item in enumerate(aux):
            slot = first + (i * (last - first + 1)) // len(aux)
            behind.setdefault(slot, []).append(item)
        for i, (s, bm, bn) in enumerate(order):
            self.mfma(period, s, bm, bn)
            for item in behind.get(i, []):
                item()

    def dma_chunk(self, index):
        """One 1 KiB piece of the tile two ahead: pieces 0..3 of the A panel, 4..7 of the B panel."""
        e = self.emit
        name, base, m0, h = ("a", "base_a", "m0_a", index) if index < 4 else ("b", "base_b", "m0_b", index - 4)
        e("s_cmp_lt_i32 %[fetch], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_%=")
        e(f"s_add_u32 m0, %[{m0}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[{base}]")
        e(f".Lcuasr_nofetch{index}_%=:")

    def tile(self):
        e = self.emit
        for operand in ("A", "B"):
            for blk in range(4):
                for s in range(2):
                    r = self.frag(operand, 0, blk, s)
                    self.content[r] = self.content[r + 1] = (operand, blk, 0, s)
        entry = dict(self.content)
        # period 0 (buffer 0), the LDS reads of period 1 (same stage) behind its matrix instructions
        self.period(0, [(lambda it=it: self.read(it)) for it in self.reads(1)], 1, 22)
        # every read of this stage has returned and this wave's part of the next tile has landed (no younger load
        # is in flight: those of the tile two ahead are issued below); after the barrier both hold for the workgroup
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        self.inflight = []
        e("s_barrier")
        e("v_add_u32 %[a_addr], %[a_step], %[a_addr]")
        e("v_add_u32 %[b_addr], %[b_step], %[b_addr]")
        e("s_mov_b32 %[m0_save], m0")
        # period 1 (buffer 1): the next tile's first fragments and the eight loads of the tile two ahead, into the
        # stage this tile has just left
        rd = [(lambda it=it: self.read(it)) for it in self.reads(2)]
        aux = [(lambda i=i: self.dma_chunk(i)) for i in range(8)]
        mixed, q = [], 0
        for i, r in enumerate(rd):
            while q < 8 and q * len(rd) <= i * 8:
                mixed.append(aux[q])
                q += 1
            mixed.append(r)
        mixed += aux[q:]
        self.period(1, mixed, 0, 22)
        e("s_mov_b32 m0, %[m0_save]")
        self.drain()
        shifted = {r: (o, b, p - 2, s) for r, (o, b, p, s) in self.content.items() if p >= 2}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines


MFMA64_VARIANTS = {"md_kx": (True, False), "md_xx": (False, False), "md_xk": (False, True), "md_kk": (True, True)}


def generate_mfma64(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    report = []
    for name, (a_kc, b_kc) in MFMA64_VARIANTS.items():
        b = Mfma64Body(a_kc, b_kc)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_prime.inc"), "w") as f:
            f.write(b.text(b.prime()))
        b = Mfma64Body(a_kc, b_kc)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_tile.inc"), "w") as f:
            f.write(b.text(b.tile()))
        report.append((name, dict(b.stats)))
    return report



# ---------------------------------------------------------------------------------------------
# plus-times on the matrix cores for the narrow element types (mfma_direct_narrow.hip): int8 operands with
# v_mfma_i32_32x32x32_i8, binary16 operands with v_mfma_f32_32x32x16_f16, both operands k-contiguous.
#
# Either instruction multiplies 32 rows by 32 columns over 32 BYTES of k per row, every lane supplying 16
# consecutive bytes of one row (column): lanes 0..31 the first 16 bytes of the step, lanes 32..63 the second.  So
# in bytes the two types are the same kernel:
#   workgroup 256 threads = 4 waves (2 x 2), one wave per SIMD; output tile 256 x 256, wave tile 128 x 128 =
#   4 x 4 blocks of 32 x 32
#   a0 .. a255   accumulators, block (bm, bn) in a[16 (4 bm + bn) : +15]
#   v0 .. v31    fragments, buffer 0: A blocks 0..3 (four registers = 16 bytes of k each), then B blocks 0..3
#   v32 .. v63   fragments, buffer 1
# A stage of the LDS ring holds 64 bytes of k of both panels = two steps of the instruction, in the image the
# direct-to-LDS loads produce -- lane i of a load writes 16-byte slot i of its KiB -- with the lanes dealt to memory
# so that four neighbouring lanes fetch the four 16-byte chunks of ONE row's 64 bytes (16 cache lines per load
# instruction; with one row per lane it was 64, and the tag lookups, not the bytes, bounded the kernel), and so
# that fragment reads stay free of bank conflicts: row r's chunk c sits in slot 4 r + (c ^ ((r >> 2) & 3)), which
# spreads the 16 rows a quarter-wave reads at one chunk over all 16 slot positions of the banks.  A lane reads
# chunk (2 step + half) of its row, so its address for step 1 is that for step 0 with the chunk's bit 1
# flipped: two address registers per panel.  Four stages: a body works on stage t, fetches stage t + 3 behind the
# matrix instructions of its second step (into the ring slot that stage t - 1 has left) and passes ONE barrier,
# in its middle: before it every read of this stage has been issued and has returned, and this wave's loads of
# stage t + 1 have landed; after it the reads of stage t + 1's first step are issued, under the second step's
# matrix instructions.
class NarrowMfmaBody(MfmaBody):
    def __init__(self, instruction):
        self.instruction = instruction
        self.lines, self.inflight, self.groups = [], [], 0
        self.stats = {"groups": 0, "lds": 0, "waits": 0, "other": 0}
        self.content = {}

    @staticmethod
    def frag(operand, u, blk):
        return u * 32 + (0 if operand == "A" else 16) + blk * 4

    def reads(self, step):
        """LDS reads of the fragments of absolute step `step` (0, 1 of this stage; 2 = the next stage's first,
        through the already advanced addresses) into buffer step % 2."""
        u, out = step % 2, []
        for operand, addr in (("A", "a_addr"), ("B", "b_addr")):
            for blk in range(4):
                r = self.frag(operand, u, blk)
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}{step % 2}] offset:{blk * 32 * 64}",
                            {r + i: (operand, blk, step) for i in range(4)}))
        return out

    def mfma(self, step, bm, bn):
        u = step % 2
        ra, rb = self.frag("A", u, bm), self.frag("B", u, bn)
        for i in range(4):
            assert self.content.get(ra + i) == ("A", bm, step) and self.content.get(rb + i) == ("B", bn, step)
        self.require_exact({ra + i for i in range(4)} | {rb + i for i in range(4)})
        acc = 16 * (4 * bm + bn)
        self.lines.append(f'"{self.instruction} a[{acc}:{acc + 15}], v[{ra}:{ra + 3}], v[{rb}:{rb + 3}], a[{acc}:{acc + 15}]\\n"')
        self.groups += 1
        self.stats["groups"] += 1

    def step(self, step, aux, first, last):
        """The 16 matrix instructions of one step, the callables of `aux` spread behind instructions first .. last."""
        order = [(bm, bn) for bn in range(4) for bm in range(4)]
        behind = {}
        for i, item in enumerate(aux):
            slot = first + (i * (last - first + 1)) // len(aux)
            behind.setdefault(slot, []).append(item)
        for i, (bm, bn) in enumerate(order):
            self.mfma(step, bm, bn)
            for item in behind.get(i, []):
                item()

    def prime(self):
        for item in self.reads(0):
            self.read(item)
        self.drain()
        return self.lines

    def dma_chunk(self, index):
        """One 1 KiB piece of the stage three ahead (skipped when there is no such stage): 16 rows x 64 bytes of
        this wave's 64 rows of the A panel (pieces 0..3) or of the B panel (4..7); consecutive pieces are
        consecutive KiB of the ring slot (M0) and 16 rows apart in memory (a lane offset of their own each)."""
        e = self.emit
        name, h = ("a", index) if index < 4 else ("b", index - 4)
        e("s_cmp_lt_i32 %[fetch], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_%=")
        e(f"s_add_u32 m0, %[m0_{name}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[base_{name}]")
        e(f".Lcuasr_nofetch{index}_%=:")

    def tile(self):
        e = self.emit
        for operand in ("A", "B"):
            for blk in range(4):
                for i in range(4):
                    self.content[self.frag(operand, 0, blk) + i] = (operand, blk, 0)
        entry = dict(self.content)
        # step 0 (buffer 0); the reads of step 1 (same stage) behind its first matrix instructions, so that the
        # last eight (256 cycles) cover the latency of the last read
        self.step(0, [(lambda it=it: self.read(it)) for it in self.reads(1)], 0, 7)
        # every read of this stage has returned; this wave's part of stage t + 1 has landed (the eight loads of
        # stage t + 2 are younger and stay in flight, if there is such a stage); after the barrier both hold for
        # the workgroup: stage t + 1 may be read, and the slot of stage t - 1 refilled
        e("s_cmp_lt_i32 %[fetch], 0")
        e("s_cbranch_scc1 .Lcuasr_all_%=")
        e("s_waitcnt vmcnt(8) lgkmcnt(0)")
        e("s_branch .Lcuasr_join_%=")
        e(".Lcuasr_all_%=:")
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e(".Lcuasr_join_%=:")
        self.inflight = []
        e("s_barrier")
        for name in ("a_addr0", "a_addr1", "b_addr0", "b_addr1"):
            e(f"v_add_u32 %[{name}], %[step], %[{name}]")
        e("s_mov_b32 %[m0_save], m0")
        # step 1 (buffer 1): the next stage's first fragments behind the first eight matrix instructions, the
        # eight loads of the stage three ahead behind the last eight
        rd = [(lambda it=it: self.read(it)) for it in self.reads(2)]
        aux = [(lambda i=i: self.dma_chunk(i)) for i in range(8)]
        self.step(1, rd + aux, 0, 15)
        e("s_mov_b32 m0, %[m0_save]")
        self.drain()
        shifted = {r: (o, b, t - 2) for r, (o, b, t) in self.content.items() if t >= 2}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines


class Narrow16Body(NarrowMfmaBody):
    """binary16 on v_mfma_f32_16x16x32_f16 (the shape that delivers more per watt on this chip for binary16; int8
    is better served by 32 x 32): the instruction takes 64 bytes of k per row, so a stage of the ring is ONE step,
    64 matrix instructions on the wave's 8 x 8 blocks of 16 x 16.  Accumulators a[4 (8 bm + bn) : +3]; two fragment
    buffers of 64 registers (A block b in v[64 u + 4 b : +3], B block b in v[64 u + 32 + 4 b : +3]), stage t in
    buffer t % 2, so the body exists in two forms (`parity` = which buffer holds the stage it computes) that the
    kernel alternates.  One statement: the counted wait and the barrier (the next stage has landed for everyone),
    then the 64 matrix instructions with the 16 fragment reads of the next stage behind the first 32 and the 8 loads
    of the stage three ahead behind the rest."""

    def __init__(self, parity, suffix=""):
        super().__init__("v_mfma_f32_16x16x32_f16")
        self.parity = parity
        self.suffix = suffix   # of the per-stage operands and the labels: two stages may share one statement

    def dma_chunk(self, index):
        e, x = self.emit, self.suffix
        name, h = ("a", index) if index < 4 else ("b", index - 4)
        e(f"s_cmp_lt_i32 %[fetch{x}], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_{x}_%=")
        e(f"s_add_u32 m0, %[m0_{name}{x}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[base_{name}{x}]")
        e(f".Lcuasr_nofetch{index}_{x}_%=:")

    @staticmethod
    def frag(operand, u, blk):
        return 64 * u + (0 if operand == "A" else 32) + 4 * blk

    def reads(self, stage):
        """LDS reads of the fragments of stage `stage` (relative to the body: 0 = the one it computes, 1 = the next,
        through the already advanced addresses) into buffer (parity + stage) % 2."""
        u, out = (self.parity + stage) % 2, []
        for operand, addr in (("A", "a_addr"), ("B", "b_addr")):
            for blk in range(8):
                r = self.frag(operand, u, blk)
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}] offset:{blk * 16 * 64}",
                            {r + i: (operand, blk, stage) for i in range(4)}))
        return out

    def mfma(self, stage, bm, bn):
        u = (self.parity + stage) % 2
        ra, rb = self.frag("A", u, bm), self.frag("B", u, bn)
        for i in range(4):
            assert self.content.get(ra + i) == ("A", bm, stage) and self.content.get(rb + i) == ("B", bn, stage)
        self.require_exact({ra + i for i in range(4)} | {rb + i for i in range(4)})
        acc = 4 * (8 * bm + bn)
        self.lines.append(f'"{self.instruction} a[{acc}:{acc + 3}], v[{ra}:{ra + 3}], v[{rb}:{rb + 3}], a[{acc}:{acc + 3}]\\n"')
        self.groups += 1
        self.stats["groups"] += 1

    def prime(self):
        assert self.parity == 0
        for item in self.reads(0):
            self.read(item)
        self.drain()
        return self.lines

    def tile(self):
        e = self.emit
        for operand in ("A", "B"):
            for blk in range(8):
                for i in range(4):
                    self.content[self.frag(operand, self.parity, blk) + i] = (operand, blk, 0)
        # this wave's part of the next stage has landed (the eight loads of the stage after it are younger and stay
        # in flight, if there is such a stage); after the barrier that holds for the workgroup, and every wave has
        # its fragments of this stage in registers: the next stage may be read, the slot of the stage before this
        # one refilled
        x = self.suffix
        order = [(bm, bn) for bn in range(8) for bm in range(8)]
        # matrix instructions ahead of the barrier, and where the reads end and the loads begin: (0, 32), (0, 40),
        # (8, 44), (16, 48) and (0, 48) are within 1 % of one another at 4096^3 and 8192^3, (0, 32) ahead
        HEAD, RD_END = 0, 32
        for bm, bn in order[:HEAD]:
            self.mfma(0, bm, bn)
        e(f"s_cmp_lt_i32 %[fetch{x}], 0")
        e(f"s_cbranch_scc1 .Lcuasr_all_{x}_%=")
        e("s_waitcnt vmcnt(8)")
        e(f"s_branch .Lcuasr_join_{x}_%=")
        e(f".Lcuasr_all_{x}_%=:")
        e("s_waitcnt vmcnt(0)")
        e(f".Lcuasr_join_{x}_%=:")
        e("s_barrier")
        e(f"v_add_u32 %[a_addr], %[step{x}], %[a_addr]")
        e(f"v_add_u32 %[b_addr], %[step{x}], %[b_addr]")
        e("s_mov_b32 %[m0_save], m0")
        rd = [(lambda it=it: self.read(it)) for it in self.reads(1)]
        aux = [(lambda i=i: self.dma_chunk(i)) for i in range(8)]
        behind = {}
        for i, item in enumerate(rd):
            behind.setdefault(HEAD + (i * (RD_END - HEAD)) // len(rd), []).append(item)
        for i, item in enumerate(aux):
            behind.setdefault(RD_END + (i * (64 - RD_END)) // len(aux), []).append(item)
        for i, (bm, bn) in enumerate(order):
            if i >= HEAD:
                self.mfma(0, bm, bn)
            for item in behind.get(i, []):
                item()
        e("s_mov_b32 m0, %[m0_save]")
        self.drain()
        # what the other form expects on entry: its stage 0 = this form's stage 1, in the other buffer
        other = {}
        for operand in ("A", "B"):
            for blk in range(8):
                for i in range(4):
                    other[self.frag(operand, 1 - self.parity, blk) + i] = (operand, blk, 1)
        assert all(self.content.get(r) == v for r, v in other.items()), "tile body does not leave the other form's entry state"
        return self.lines


class NarrowLine16Body(NarrowMfmaBody):
    """binary16 on v_mfma_f32_16x16x32_f16 with panels fetched 128 bytes of k per row (whole cache lines: half the
    requests to L2 per byte): a stage is 128 bytes of k = TWO steps of 64 matrix instructions, the LDS ring holds
    five units of one operand's 256 rows x 128 bytes (this stage's A and B, the next stage's, and the A after
    that).  Fragment buffers as in Narrow16Body (step s of a stage in buffer s), addresses per operand and step.
    One statement per stage: step 0 with the reads of step 1 behind its first half; the counted wait and the
    barrier (the next stage has landed for everyone, and everyone holds this stage's fragments: its two units may
    be refilled); step 1 with the reads of the next stage's step 0 behind its first half and the sixteen loads of
    the two units to refill (the B panel two stages ahead, the A panel three ahead) behind the second."""

    def __init__(self):
        super().__init__("v_mfma_f32_16x16x32_f16")

    @staticmethod
    def frag(operand, u, blk):
        return 64 * u + (0 if operand == "A" else 32) + 4 * blk

    def reads(self, step):
        u, out = step % 2, []
        for operand, addr in (("A", f"a_addr{step % 2}"), ("B", f"b_addr{step % 2}")):
            for blk in range(8):
                r = self.frag(operand, u, blk)
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}] offset:{blk * 16 * 128}",
                            {r + i: (operand, blk, step) for i in range(4)}))
        return out

    def mfma(self, step, bm, bn):
        u = step % 2
        ra, rb = self.frag("A", u, bm), self.frag("B", u, bn)
        for i in range(4):
            assert self.content.get(ra + i) == ("A", bm, step) and self.content.get(rb + i) == ("B", bn, step)
        self.require_exact({ra + i for i in range(4)} | {rb + i for i in range(4)})
        acc = 4 * (8 * bm + bn)
        self.lines.append(f'"{self.instruction} a[{acc}:{acc + 3}], v[{ra}:{ra + 3}], v[{rb}:{rb + 3}], a[{acc}:{acc + 3}]\\n"')
        self.groups += 1
        self.stats["groups"] += 1

    def dma_chunk(self, index):
        """One 1 KiB piece (8 rows x 128 bytes) of this wave's 64 rows of a unit: pieces 0..7 of unit x (a B panel),
        8..15 of unit y (an A panel); a unit that does not exist any more is skipped."""
        e = self.emit
        name, unit, h = ("b", "x", index) if index < 8 else ("a", "y", index - 8)
        e(f"s_cmp_lt_i32 %[fetch_{unit}], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_%=")
        e(f"s_add_u32 m0, %[m0_{unit}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[base_{unit}]")
        e(f".Lcuasr_nofetch{index}_%=:")

    def spread(self, step, first_half, second_half):
        order = [(bm, bn) for bn in range(8) for bm in range(8)]
        behind = {}
        for i, item in enumerate(first_half):
            behind.setdefault((i * 32) // len(first_half), []).append(item)
        for i, item in enumerate(second_half):
            behind.setdefault(32 + (i * 32) // len(second_half), []).append(item)
        for i, (bm, bn) in enumerate(order):
            self.mfma(step, bm, bn)
            for item in behind.get(i, []):
                item()

    def prime(self):
        for item in self.reads(0):
            self.read(item)
        self.drain()
        return self.lines

    def tile(self):
        e = self.emit
        for operand in ("A", "B"):
            for blk in range(8):
                for i in range(4):
                    self.content[self.frag(operand, 0, blk) + i] = (operand, blk, 0)
        entry = dict(self.content)
        self.spread(0, [(lambda it=it: self.read(it)) for it in self.reads(1)], [])
        # every read of this stage has returned; this wave's part of the next stage has landed (the eight loads of
        # the A panel after it are younger and stay in flight, if there is such a panel)
        e("s_cmp_lt_i32 %[fetch_x], 1")
        e("s_cbranch_scc1 .Lcuasr_all_%=")
        e("s_waitcnt vmcnt(8) lgkmcnt(0)")
        e("s_branch .Lcuasr_join_%=")
        e(".Lcuasr_all_%=:")
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e(".Lcuasr_join_%=:")
        self.inflight = []
        e("s_barrier")
        for name, step in (("a_addr0", "a_step"), ("a_addr1", "a_step"), ("b_addr0", "b_step"), ("b_addr1", "b_step")):
            e(f"v_add_u32 %[{name}], %[{step}], %[{name}]")
        e("s_mov_b32 %[m0_save], m0")
        self.spread(1, [(lambda it=it: self.read(it)) for it in self.reads(2)], [(lambda i=i: self.dma_chunk(i)) for i in range(16)])
        e("s_mov_b32 m0, %[m0_save]")
        self.drain()
        shifted = {r: (o, b, t - 2) for r, (o, b, t) in self.content.items() if t >= 2}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines


class NarrowLineI8Body(NarrowMfmaBody):
    """int8 on v_mfma_i32_32x32x32_i8 with panels fetched 128 bytes of k per row (see NarrowLine16Body: the same ring of
    five one-operand units): a stage is FOUR steps of 16 matrix instructions, fragments double-buffered by step as
    in NarrowMfmaBody, one fragment address per operand and step.  One statement per stage: steps 0 .. 2 with the reads
    of the step after behind their first eight matrix instructions; then the counted wait and the barrier (every
    read of this stage has returned, the next stage has landed for everyone); step 3 with the reads of the next stage's
    step 0 and the sixteen loads of the two units to refill behind its matrix instructions."""

    def __init__(self):
        super().__init__("v_mfma_i32_32x32x32_i8")

    def reads(self, step):
        u, out = step % 2, []
        for operand, addr in (("A", f"a_addr{step % 4}"), ("B", f"b_addr{step % 4}")):
            for blk in range(4):
                r = self.frag(operand, u, blk)
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{addr}] offset:{blk * 32 * 128}",
                            {r + i: (operand, blk, step) for i in range(4)}))
        return out

    def dma_chunk(self, index):
        e = self.emit
        name, unit, h = ("b", "x", index) if index < 8 else ("a", "y", index - 8)
        e(f"s_cmp_lt_i32 %[fetch_{unit}], 1")
        e(f"s_cbranch_scc1 .Lcuasr_nofetch{index}_%=")
        e(f"s_add_u32 m0, %[m0_{unit}], {hex(0x400 * h)}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 %[off_{name}{h}], %[base_{unit}]")
        e(f".Lcuasr_nofetch{index}_%=:")

    def tile(self):
        e = self.emit
        for operand in ("A", "B"):
            for blk in range(4):
                for i in range(4):
                    self.content[self.frag(operand, 0, blk) + i] = (operand, blk, 0)
        entry = dict(self.content)
        for step in range(3):
            self.step(step, [(lambda it=it: self.read(it)) for it in self.reads(step + 1)], 0, 7)
        e("s_cmp_lt_i32 %[fetch_x], 1")
        e("s_cbranch_scc1 .Lcuasr_all_%=")
        e("s_waitcnt vmcnt(8) lgkmcnt(0)")
        e("s_branch .Lcuasr_join_%=")
        e(".Lcuasr_all_%=:")
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e(".Lcuasr_join_%=:")
        self.inflight = []
        e("s_barrier")
        for op in ("a", "b"):
            for st in range(4):
                e(f"v_add_u32 %[{op}_addr{st}], %[{op}_step], %[{op}_addr{st}]")
        e("s_mov_b32 %[m0_save], m0")
        rd = [(lambda it=it: self.read(it)) for it in self.reads(4)]
        aux = [(lambda i=i: self.dma_chunk(i)) for i in range(16)]
        # the reads first (their latency wants the rest of the step), a load behind every matrix instruction
        self.step(3, rd[:4] + [aux[0]] + rd[4:] + aux[1:], 0, 15)
        e("s_mov_b32 m0, %[m0_save]")
        self.drain()
        shifted = {r: (o, b, t - 4) for r, (o, b, t) in self.content.items() if t >= 4}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines


NARROW_VARIANTS = {"n_i8": "v_mfma_i32_32x32x32_i8"}


def generate_narrow(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    report = []
    for name, instruction in NARROW_VARIANTS.items():
        b = NarrowMfmaBody(instruction)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_prime.inc"), "w") as f:
            f.write(b.text(b.prime()))
        b = NarrowMfmaBody(instruction)
        with open(os.path.join(out_dir, f"mfma_asm_{name}_tile.inc"), "w") as f:
            f.write(b.text(b.tile()))
        report.append((name, dict(b.stats)))
    b = Narrow16Body(0)
    with open(os.path.join(out_dir, "mfma_asm_n16_f16_prime.inc"), "w") as f:
        f.write(b.text(b.prime()))
    # two stages in one statement (the kernel's loop: 384 pinned registers pass from one statement to the next
    # without copies only when the loop holds a single statement), and the first form alone for an odd last stage
    b0, b1 = Narrow16Body(0, "0"), Narrow16Body(1, "1")
    with open(os.path.join(out_dir, "mfma_asm_n16_f16_pair.inc"), "w") as f:
        f.write(b0.text(b0.tile()) + b1.text(b1.tile()))
    report += [("n16_f16_0", dict(b0.stats)), ("n16_f16_1", dict(b1.stats))]
    b = Narrow16Body(0, "0")
    with open(os.path.join(out_dir, "mfma_asm_n16_f16_tile0.inc"), "w") as f:
        f.write(b.text(b.tile()))
    b = NarrowLine16Body()
    with open(os.path.join(out_dir, "mfma_asm_n16l_f16_prime.inc"), "w") as f:
        f.write(b.text(b.prime()))
    b = NarrowLine16Body()
    with open(os.path.join(out_dir, "mfma_asm_n16l_f16_tile.inc"), "w") as f:
        f.write(b.text(b.tile()))
    report.append(("n16l_f16", dict(b.stats)))
    b = NarrowLineI8Body()
    with open(os.path.join(out_dir, "mfma_asm_nl_i8_prime.inc"), "w") as f:
        f.write(b.text(b.prime()))
    b = NarrowLineI8Body()
    with open(os.path.join(out_dir, "mfma_asm_nl_i8_tile.inc"), "w") as f:
        f.write(b.text(b.tile()))
    report.append(("nl_i8", dict(b.stats)))
    return report


# ---------------------------------------------------------------------------------------------
# The bookkeeping of the predecessor-tracking product on the direct tile (fwgemm.hip, fwgemm_direct_kernel):
# after a chunk of k the loop's 64 accumulators (v0 .. v63) are compared with their values before it
# (v128 .. v191); where one is lower, the chunk's index goes into that element's 16 bits of v192 .. v223 and
# the copy is brought up to date.  First a cheap test whether ANY of the wave's elements changed at all -- one
# three-input bit operation per element, diff |= now ^ before -- because once the distances have settled
# almost no chunk changes anything.  Fixed registers throughout, so the compiler has nothing to allocate
# around the loop's statements (as C++, the rare path's temporaries pushed the loop's fragments out to
# scratch memory at every check).
def generate_fwgemm_merge(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    lines = ["v_mov_b32 v224, 0"]
    for e in range(64):
        lines.append(f"v_bitop3_b32 v224, v{e}, v{128 + e}, v224 bitop3:0xbe")
    lines += ["v_cmp_ne_u32 vcc, 0, v224", "s_cbranch_vccz .Lcuasr_same_%="]
    # (the wait between a comparison and its select is deliberate: with the copy of the element before in its place
    # the product ran 4 % slower over a shortest-path job; and the two halves of a chunk word are written four
    # instructions apart, more than the one wait state a write of part of a register wants before it is read again)
    for e in range(64):
        w, half = 192 + e // 2, e & 1
        lines += [f"v_cmp_lt_f32 vcc, v{e}, v{128 + e}",
                  "s_nop 1",
                  f"v_cndmask_b32_sdwa v{w}, v{w}, %[chunk], vcc dst_sel:WORD_{half} dst_unused:UNUSED_PRESERVE "
                  f"src0_sel:WORD_{half} src1_sel:WORD_0",
                  f"v_mov_b32 v{128 + e}, v{e}"]
    lines.append(".Lcuasr_same_%=:")
    with open(os.path.join(out_dir, "fwgemm_merge.inc"), "w") as f:
        f.write("\n".join('"' + ln + '\\n"' for ln in lines) + "\n")
    return [("fwgemm_merge", {"lines": len(lines)})]


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "gen")
    for name, stats in generate(out) + generate_mfma(out) + generate_mfma64(out) + generate_fwgemm_merge(out):
        print(name, stats)
