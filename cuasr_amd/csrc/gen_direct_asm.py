#!/usr/bin/env python3
"""Generates the hand-scheduled main loop of the 4-wave direct-to-LDS SRGEMM tile
(direct_tile.h) as inline-asm text: one k-tile (16 k) of the 8 x 8 register tile per asm
statement, for each pair of panel forms.

Why generated asm and not C++: on gfx950 a SIMD issues about one instruction every 2.1 cycles
whatever its kind (a satisfied s_waitcnt, an s_nop or a scalar add costs as much as a v_add_f32),
and an LDS read costs about 5.5 cycles whatever its width.  The compiler's version of this loop
spends 1536 vector instructions per k-tile plus 96 LDS reads, 89 waits and 76 nops; this schedule
spends the same 1536 plus 64 LDS reads (16-byte reads only), about 20 waits and no nops.

Register plan (128 VGPRs, 4 waves per SIMD):
    v0   .. v63    accumulators, acc[i][j] = v(8 i + j)      (i: A index, j: B index)
    v64  .. v111   fragments of the operand called Q, then of the operand called P
    v112 .. v115   temporaries
  P is an x-contiguous panel ([k][X] in LDS, one 16-byte read = 4 x at one k): 16 registers hold
    one k-pair, refilled half by half (4 x, both k) as soon as a half's last use is over.
  Q is either k-contiguous ([k/4][X][4] in LDS, one 16-byte read = 4 k of one x): 32 registers
    hold a k-quad, each x refilled right after its last use in the quad's second k-pair,
    or x-contiguous like P: 16 registers, refilled by halves.
  A k-pair is worked in two phases, one per half of P; within a phase the 8 x of Q in order.

LDS reads complete in order, so "s_waitcnt lgkmcnt(N)" leaves the N youngest in flight.  The
generator keeps the queue of reads in flight, emits a wait only where a fragment is consumed
whose read the queue still holds, lets each wait also cover every read old enough to have landed,
and checks for every vector instruction that the registers it reads hold the operand, x and k
it means.  A statement ends with everything drained, so no read is in flight while compiler
code runs.

Output: string-literal fragments for `asm volatile(` to include; the arithmetic of two terms
is the macro CUASR_TERM2(acc, t0, t1, q0, p0, q1, p1) that the including code defines for its
semiring (register names as string literals), everything else is literal text.
"""
import os
import sys

TY, TX, BK = 32, 16, 16
ACC0 = 0
FRAG0 = 64
TEMP0 = 112  # four temporaries, v112 .. v115
WAIT_AGE = 20   # a wait also covers reads issued at least this many two-term groups ago


class Panel:
    """Fragment registers and LDS reads of one operand; xt = threads along its x (8 * xt wide)."""

    def __init__(self, name, kc, xt, reg0, addr):
        self.name, self.kc, self.xt, self.reg0, self.addr = name, kc, xt, reg0, addr
        self.nregs = 32 if kc else 16

    def reg(self, x, k):
        if self.kc:
            return self.reg0 + x * 4 + (k & 3)
        return self.reg0 + ((k & 1) * 2 + (x >> 2)) * 4 + (x & 3)

    def reads_for(self, unit, k_first):
        """LDS reads that fill `unit` with the data starting at tile-relative k_first (< 32: the
        next tile's k is 16 + k, read through the already advanced address, i.e. offset k - 16).
        unit: x (0..7) of a k-contiguous panel -> one read of 4 k; half (0, 1) of an x-contiguous
        one -> two reads (k_first, k_first + 1) of 4 x."""
        out = []
        if self.kc:
            k = k_first % BK
            off = ((k >> 2) * 8 * self.xt + unit * self.xt) * 16
            r = self.reg0 + unit * 4
            out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{self.addr}] offset:{off}",
                        {r + e: (self.name, unit, k_first + e) for e in range(4)}))
        else:
            for s in range(2):
                k = (k_first + s) % BK
                off = (k * 8 * self.xt + unit * 4 * self.xt) * 4
                r = self.reg0 + (((k_first + s) & 1) * 2 + unit) * 4
                out.append((f"ds_read_b128 v[{r}:{r + 3}], %[{self.addr}] offset:{off}",
                            {r + e: (self.name, unit * 4 + e, k_first + s) for e in range(4)}))
        return out


class Body:
    def __init__(self, a_kc, b_kc):
        assert not (a_kc and b_kc), "two k-quad operands do not fit 128 registers"
        # Q = the operand held per k-quad if there is one, else A; P = the other
        q_is_a = a_kc or not b_kc
        qa, pa = ("a_addr", "b_addr") if q_is_a else ("b_addr", "a_addr")
        self.Q = Panel("A" if q_is_a else "B", a_kc if q_is_a else b_kc, TY if q_is_a else TX, FRAG0, qa)
        self.P = Panel("B" if q_is_a else "A", False, TX if q_is_a else TY, FRAG0 + self.Q.nregs, pa)
        self.q_is_a = q_is_a
        self.temp0 = TEMP0
        assert self.P.reg0 + self.P.nregs <= TEMP0
        self.ntemps = 4
        self.lines = []
        self.content = {}     # register -> (operand, x, k) it holds or is being filled with
        self.inflight = []    # [(registers, group count at issue)] oldest first
        self.groups = 0       # two-term groups emitted so far (the clock of WAIT_AGE)
        self.tcount = 0
        self.stats = {"valu_groups": 0, "lds": 0, "waits": 0, "other": 0}

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

    def term2(self, i, j, k0):
        """acc[i][j] <- add(acc, mult(a[i][k0], b[k0][j]), mult(a[i][k0 + 1], b[k0 + 1][j]))"""
        qx, px = (i, j) if self.q_is_a else (j, i)
        regs = []
        for k in (k0, k0 + 1):
            rq, rp = self.Q.reg(qx, k), self.P.reg(px, k)
            assert self.content.get(rq) == (self.Q.name, qx, k), (rq, self.content.get(rq), qx, k)
            assert self.content.get(rp) == (self.P.name, px, k), (rp, self.content.get(rp), px, k)
            regs += [rq, rp]
        self.require(set(regs))
        t0 = self.temp0 + self.tcount % self.ntemps
        t1 = self.temp0 + (self.tcount + 1) % self.ntemps
        self.tcount += 2
        acc = ACC0 + i * 8 + j
        self.lines.append(f'CUASR_TERM2("v{acc}", "v{t0}", "v{t1}", "v{regs[0]}", "v{regs[1]}", "v{regs[2]}", "v{regs[3]}")')
        self.groups += 1
        self.stats["valu_groups"] += 1

    # ---- the bodies
    def prime(self):
        """Fragments of the first k-quad / k-pair of the first tile."""
        for unit in range(8 if self.Q.kc else 2):
            self.issue(self.Q, unit, 0)
        for half in range(2):
            self.issue(self.P, half, 0)
        self.drain()
        return self.lines

    def tile(self):
        # state on entry = state after prime() or after a previous tile(): everything resident, nothing in flight
        for unit in range(8 if self.Q.kc else 2):
            for fills in [f for _, f in self.Q.reads_for(unit, 0)]:
                self.content.update(fills)
        for half in range(2):
            for fills in [f for _, f in self.P.reads_for(half, 0)]:
                self.content.update(fills)
        entry = dict(self.content)

        # global -> LDS for the tile two ahead (skipped when there is none): each wave moves two
        # 1 KiB pieces of the A panel and one of the B panel; M0 = LDS address of the wave's piece
        self.emit("s_cmp_lt_i32 %[fetch], 1")
        self.emit("s_cbranch_scc1 .Lcuasr_nofetch_%=")
        self.emit("s_mov_b32 %[m0_save], m0")   # M0 is the compiler's own for its LDS-bound loads: hand it back unchanged
        self.emit("s_mov_b32 m0, %[m0_a]")
        self.emit("s_nop 0")
        self.emit("global_load_lds_dwordx4 %[off_a0], %[base_a]")
        self.emit("s_add_u32 m0, m0, 0x400")
        self.emit("s_nop 0")
        self.emit("global_load_lds_dwordx4 %[off_a1], %[base_a]")
        self.emit("s_mov_b32 m0, %[m0_b]")
        self.emit("s_nop 0")
        self.emit("global_load_lds_dwordx4 %[off_b0], %[base_b]")
        self.emit("s_mov_b32 m0, %[m0_save]")
        self.emit(".Lcuasr_nofetch_%=:")

        nkp = BK // 2
        for kp in range(nkp):
            k0 = 2 * kp
            second = (kp & 1) == 1          # second k-pair of its k-quad
            last = kp == nkp - 1
            nk0 = k0 + 2                    # the next k-pair (>= 16: in the next tile)
            for half in range(2):
                if half == 1 and last:
                    # every read of this stage has returned and this wave's part of the next tile
                    # has landed; after the barrier that holds for the whole workgroup, and the
                    # stage two ahead may be overwritten.  The refills from here on read the next stage.
                    self.drain("s_waitcnt vmcnt(0) lgkmcnt(0)")
                    self.emit("s_barrier")
                    self.emit("v_add_u32 %[a_addr], %[a_step], %[a_addr]")
                    self.emit("v_add_u32 %[b_addr], %[b_step], %[b_addr]")
                if half == 1:
                    self.issue(self.P, 0, nk0)   # half 0 of P is free: refill it for the next k-pair
                for qx in range(8):
                    for px in range(4 * half, 4 * half + 4):
                        i, j = (qx, px) if self.q_is_a else (px, qx)
                        self.term2(i, j, k0)
                    if half == 1:
                        if self.Q.kc:
                            if second:
                                self.issue(self.Q, qx, (k0 + 2))   # next k-quad of this x
                        elif qx & 3 == 3:
                            self.issue(self.Q, qx >> 2, nk0)
            self.issue(self.P, 1, nk0)
        self.drain()
        # the registers now hold the next tile's first fragments: same state as on entry
        shifted = {r: (o, x, k - BK) for r, (o, x, k) in self.content.items()}
        assert shifted == entry, "tile body does not reproduce its entry state"
        return self.lines

    def text(self, lines):
        out = []
        for ln in lines:
            out.append(ln if ln.startswith("CUASR_TERM2") else '"' + ln + '\\n"')
        return "\n".join(out) + "\n"


VARIANTS = {"kx": (True, False), "xx": (False, False), "xk": (False, True)}


def generate(out_dir):
    os.makedirs(out_dir, exist_ok=True)
    report = []
    for name, (a_kc, b_kc) in VARIANTS.items():
        b = Body(a_kc, b_kc)
        with open(os.path.join(out_dir, f"direct_asm_{name}_prime.inc"), "w") as f:
            f.write(b.text(b.prime()))
        b = Body(a_kc, b_kc)
        with open(os.path.join(out_dir, f"direct_asm_{name}_tile.inc"), "w") as f:
            f.write(b.text(b.tile()))
        report.append((name, dict(b.stats)))
    return report


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for name, stats in generate(sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "gen")):
        print(name, stats)
