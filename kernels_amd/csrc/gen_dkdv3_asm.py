#!/usr/bin/env python3
"""Generator of the main-loop assembly of dkdv3_kernel (sa_bwd3.h) -> sa_dkdv3_asm.inc.

The loop body of the dK/dV kernel is a fixed schedule of "slots": each slot issues one
v_mfma_f32_32x32x16, the LDS read that a slot 15 places later consumes, and a share of the vector
work of the previous 32-query block.  The compiler's register allocator does not cope with the
~400 live registers of that loop (it keeps copying whole accumulators between the two register
files), so the loop is emitted here with every register chosen by hand, every s_waitcnt counted,
and the hazards the hardware leaves to software spaced out by construction.

Register map (the kernel is built for D = 128):
  a[0:63]    dV^T blocks (16 registers per 32 columns of D)     a[64:127]  dK^T blocks
  a[128:159] K fragments (4 registers per 16 columns of D)      a[160:191] V fragments (negated)
  v[0:31]    lse - score accumulators of the even / odd block   v[32:63]   delta - dP accumulators
  v[64:79]   probabilities, then -dS, of the current block      v[80:95]   free
  v[96:103]  P rounded (two B operands)                         v[104:111] -dS rounded
  v[112:143] fragment ring, entries 0..7 of 4 registers; a[192:223] entries 8..15
  v[144:151] row-fragment addresses, tile of the B side         v[152:159] same, next tile
  v[160:167] transposing-read addresses, tile of the B side     v168, v169 lse/delta addresses (this / next tile)
  v[176:183] row-fragment offsets inside a stage                v[184:191] transposing-read offsets
  v192 lse/delta offset   v193, v194 query window [lo, hi) of this lane's key   v195 4*(lane/32)
  v[196:207] temporaries
  v[208:239] wave-uniform inputs, copied to s40... at entry (see SCALARS below)
  v240, v241 buffer offsets of this lane for the Q / dO tile loads    v[242:243] lse (lanes 0-15) or delta
  (lanes 16-31) row pointer    v244 row of the next tile this lane fetches lse / delta for    v[245:247] temporaries
  s40 free  s41 one past the last query tile  s42 query tile of the B side  s43 64*s42  s44 first row of
  the block being masked  s45..s47 LDS address of the stages of tiles s42, s42+1, s42+2  s48 wave offset inside a
  tile for the asynchronous loads  s49 same for lse/delta  s50 last valid row  s[52:55], s[56:59] buffer resources
  of Q and dO  s60, s61 their running byte offsets  s62, s63 bytes between a wave's load instructions
  s64, s65 bytes between tiles  s66..s68 temporaries  s51, s69: a 32-query block inside [s51, s69) lies inside the
  window of every key of this wave

Run:  python3 gen_dkdv3_asm.py > sa_dkdv3_asm.inc   (the Makefile does this)
"""

TQ = 64
RPW = 16
import os

# 16 entries let a read be issued up to 15 slots ahead, which is also the most the 4-bit LDS counter of s_waitcnt
# can keep apart (a transposed fragment is two reads).  8 entries (v[112:143] only) measured 3-5 % slower.
RING = int(os.environ.get("SA_DKDV3_RING", "16"))
PF = RING - 1


class Gen:
    def __init__(self, D, dt):
        self.D, self.dt = D, dt
        self.NF, self.DB = D // 16, D // 32
        self.ROWB = D * 2
        self.TILE_B = TQ * self.ROWB
        self.NA, self.NB = 2 * self.NF, 2 * self.DB
        self.NS = self.NA + 2 * self.NB
        assert self.NS % RING == 0 and 16 % self.NA == 0 and 16 % self.NB == 0 and 8 % self.NB == 0
        self.mfma = "v_mfma_f32_32x32x16_" + dt
        self.cvt = "v_cvt_pk_bf16_f32" if dt == "bf16" else "v_cvt_pk_f16_f32"
        self.issued = []      # tags of LDS reads in issue order
        self.done = -1        # index of the youngest read known to have returned
        self.out = []

    # ---- registers -------------------------------------------------------------------------
    @staticmethod
    def vr(lo, n=1):
        return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"

    @staticmethod
    def ar(lo, n=1):
        return f"a{lo}" if n == 1 else f"a[{lo}:{lo + n - 1}]"

    def S(self, p, i=None):
        return self.vr(16 * p, 16) if i is None else self.vr(16 * p + i)

    def DP(self, p, i=None):
        return self.vr(32 + 16 * p, 16) if i is None else self.vr(32 + 16 * p + i)

    def PR(self, i):
        return self.vr(64 + i)

    def PB(self, half, w=None):
        return self.vr(96 + 4 * half, 4) if w is None else self.vr(96 + 4 * half + w)

    def DSB(self, half, w=None):
        return self.vr(104 + 4 * half, 4) if w is None else self.vr(104 + 4 * half + w)

    def RG(self, r, lo=0, n=4):
        # the second half of the ring lives in accumulation registers: LDS reads can land there and MFMAs can
        # take their A operand from there
        if r < 8:
            return self.vr(112 + 4 * r + lo, n)
        return self.ar(192 + 4 * (r - 8) + lo, n)

    AROW_CUR, AROW_NXT, ATR_CUR, ALD_CUR, ALD_NXT = 144, 152, 160, 168, 169
    AROW_BASE, ATR_BASE, ALD_BASE, QLO, QHI, H4, TMP = 176, 184, 192, 193, 194, 195, 196

    def DV(self, m):
        return self.ar(16 * m, 16)

    def DK(self, m):
        return self.ar(64 + 16 * m, 16)

    def KF(self, g):
        return self.ar(128 + 4 * g, 4)

    def VF(self, g):
        return self.ar(160 + 4 * g, 4)

    # ---- emission ---------------------------------------------------------------------------
    def emit(self, s):
        self.out.append(s)

    def lds(self, tag, text):
        self.issued.append(tag)
        self.emit(text)

    def need(self, tag):
        """Wait until the LDS read `tag` has returned (reads return in issue order)."""
        if tag not in self.issued:      # only in the warm-up round of the steady-state simulation
            return
        idx = len(self.issued) - 1 - self.issued[::-1].index(tag)
        if idx <= self.done:
            return
        n = len(self.issued) - 1 - idx
        self.emit(f"s_waitcnt lgkmcnt({min(n, 15)})")
        self.done = idx if n <= 15 else len(self.issued) - 16

    # ---- LDS reads ----------------------------------------------------------------------------
    def fetch(self, gslot, j, par, nxt_body):
        """Read the fragment slot j of a block step consumes into its ring entry.
        par: parity of the step that consumes it; nxt_body: issued by the step before."""
        r = gslot % RING
        tag = ("ring", gslot)
        qbB, qbA = par, par ^ 1
        if j < self.NA:
            g, w = j >> 1, j & 1
            # A side of an odd step is block 0 of the next tile; of an even step block 1 of this tile.
            # Seen from the step before (which issues slots 0..PF-1), "this tile" of an even step is
            # that step's "next tile" until it rotates its address registers, which an odd step does
            # before these reads.
            base = (self.AROW_NXT if par == 1 else self.AROW_CUR) + g
            off = w * self.TILE_B + qbA * 32 * self.ROWB
            self.lds(tag, f"ds_read_b128 {self.RG(r)}, v{base} offset:{off}")
        else:
            idx, isdk = (j - self.NA) % self.NB, (j - self.NA) // self.NB
            half, m = idx // self.DB, idx % self.DB
            off = (0 if isdk else self.TILE_B) + qbB * 32 * self.ROWB + half * 16 * self.ROWB
            self.lds(("ringlo", gslot), f"ds_read_b64_tr_b16 {self.RG(r, 0, 2)}, v{self.ATR_CUR + m} offset:{off}")
            self.lds(tag, f"ds_read_b64_tr_b16 {self.RG(r, 2, 2)}, v{self.ATR_CUR + 4 + m} offset:{off}")

    def row_off(self, qb, which, g4):
        r = qb * 32 + 8 * g4
        return ((r // RPW) * 2 * RPW + (r % RPW) + which * RPW) * 4

    # ---- vector work ---------------------------------------------------------------------------
    def v1_ops(self, par):
        """Probabilities of the block whose accumulator S[par] holds lse - score*scale*log2(e):
        P = exp2(-S), rounded per pair.  Returns one list of instructions per element step; a v_exp
        result is never consumed by the very next instruction (transcendental forwarding needs one
        instruction in between), so a pair is rounded after the exponential of the next element."""
        def cvt(i):     # pair (i - 1, i)
            return f"{self.cvt} {self.PB(i >> 3, (i & 7) >> 1)}, {self.PR(i - 1)}, {self.PR(i)}"
        steps = []
        for i in range(16):
            ops = [f"v_exp_f32 {self.PR(i)}, -{self.S(par, i)}"]
            if i >= 2 and (i & 1) == 0:
                ops.append(cvt(i - 1))
            if i == 15:
                ops += ["s_nop 0", cvt(15)]
            steps.append(ops)
        return steps

    def v2_ops(self, par):
        steps = []
        for i in range(0, 16, 2):
            steps.append([f"v_mul_f32 {self.PR(i)}, {self.PR(i)}, {self.DP(par, i)}",
                          f"v_mul_f32 {self.PR(i + 1)}, {self.PR(i + 1)}, {self.DP(par, i + 1)}",
                          f"{self.cvt} {self.DSB(i >> 3, (i & 7) >> 1)}, {self.PR(i)}, {self.PR(i + 1)}"])
        return steps

    def mask_ops(self, par):
        """S[par] keeps its value (the lse of the row) where (row, this lane's key) is inside the
        key's window and becomes +inf elsewhere, for the block whose first row is s44."""
        t = self.TMP
        ops = ["s_mov_b32 s67, 0x7f800000",
               f"v_subrev_u32 v{t}, s44, v{self.QLO}",
               f"v_subrev_u32 v{t + 1}, s44, v{self.QHI}",
               f"v_med3_i32 v{t}, v{t}, 0, 32",
               f"v_med3_i32 v{t + 1}, v{t + 1}, 0, 32",
               f"v_lshlrev_b64 v[{t + 2}:{t + 3}], v{t}, 1",
               f"v_lshlrev_b64 v[{t + 4}:{t + 5}], v{t + 1}, 1",
               f"v_add_u32 v{t + 2}, -1, v{t + 2}",
               f"v_add_u32 v{t + 4}, -1, v{t + 4}",
               f"v_not_b32 v{t + 2}, v{t + 2}",
               f"v_and_b32 v{t + 4}, v{t + 4}, v{t + 2}",
               f"v_lshrrev_b32 v{t + 4}, v{self.H4}, v{t + 4}"]
        # bit -> all-ones / zero with v_bfe_i32 into one of four temporaries; the select that uses it
        # is issued three elements later, before that temporary is written again
        def sel(k):
            return f"v_bitop3_b32 {self.S(par, k)}, {self.S(par, k)}, s67, v{t + 7 + (k & 3)} bitop3:0xe4"
        for i in range(16):
            pos = 8 * (i >> 2) + (i & 3)
            ops.append(f"v_bfe_i32 v{t + 7 + (i & 3)}, v{t + 4}, {pos}, 1")
            if i >= 3:
                ops.append(sel(i - 3))
        for k in range(13, 16):
            ops.append(sel(k))
        return ops

    # ---- one block step ---------------------------------------------------------------------
    def body(self, k, par, split_at=None, label=""):
        """Step k (global counter): B side block k, A side block k + 1.  Returns the list of
        instruction lists per part (two parts when split_at is given)."""
        NA, NB, NS, DB = self.NA, self.NB, self.NS, self.DB
        parts, self.out = [], []
        v1 = self.v1_ops(par)
        v2 = self.v2_ops(par)
        mask = self.mask_ops(par)
        # address work of an odd step: this tile <- next tile, next tile and B side recomputed
        movs = [f"v_mov_b32 v{self.AROW_CUR + g}, v{self.AROW_NXT + g}" for g in range(self.NF)]
        adds = [f"v_add_u32 v{self.AROW_NXT + g}, s47, v{self.AROW_BASE + g}" for g in range(self.NF)]
        adds += [f"v_add_u32 v{self.ATR_CUR + x}, s46, v{self.ATR_BASE + x}"
                 for x in list(range(DB)) + list(range(4, 4 + DB))]
        tail = [f"v_mov_b32 v{self.ALD_CUR}, v{self.ALD_NXT}",
                f"v_add_u32 v{self.ALD_NXT}, s47, v{self.ALD_BASE}"]
        eps, epv = 16 // NA, 16 // NB
        for j in range(NS):
            if split_at is not None and j == split_at:
                parts.append(self.out)
                self.out = []
            gs = k * NS + j
            # the read that slot j + PF consumes
            jn = j + PF
            if jn < NS:
                self.fetch(gs + PF, jn, par, False)
            else:
                self.fetch(gs + PF, jn - NS, par ^ 1, True)
            r = gs % RING
            self.need(("ring", gs))
            if j < NA:
                g = j >> 1
                if j & 1:
                    if j == 1:
                        self.need(("delta", k + 1, 3))
                    self.emit(f"{self.mfma} {self.DP(par ^ 1)}, {self.RG(r)}, {self.VF(g)}, {self.DP(par ^ 1)}")
                else:
                    if j == 0:
                        self.need(("lse", k + 1, 3))
                    self.emit(f"{self.mfma} {self.S(par ^ 1)}, {self.RG(r)}, {self.KF(g)}, {self.S(par ^ 1)}")
                for e in range(j * eps, (j + 1) * eps):
                    for op in v1[e]:
                        self.emit(op)
            elif j < NA + NB:
                idx = j - NA
                half, m = idx // DB, idx % DB
                self.emit(f"{self.mfma} {self.DV(m)}, {self.RG(r)}, {self.PB(half)}, {self.DV(m)}")
                for e in range(idx * epv // 2, (idx + 1) * epv // 2):
                    for op in v2[e]:
                        self.emit(op)
                if par == 1 and idx < len(movs):
                    self.emit(movs[idx])
            else:
                idx = j - NA - NB
                half, m = idx // DB, idx % DB
                self.emit(f"{self.mfma} {self.DK(m)}, {self.RG(r)}, {self.DSB(half)}, {self.DK(m)}")
                # row statistics of block k + 2, which has this step's parity (block `par` of the next
                # tile; for an odd step: of the tile that becomes "this tile" when it rotates its
                # addresses): its lse starts the score accumulator, its delta the dP accumulator.
                # They read the next tile, so they come after the point where an even step waits for
                # it, two per slot, lse first: the next step's first MFMA reads it.
                i0 = max(0, (NS - PF) - (NA + NB))
                assert NB - i0 >= 4
                if i0 <= idx < i0 + 4:
                    for rr in range(2 * (idx - i0), 2 * (idx - i0) + 2):
                        if rr < 4:
                            self.lds(("lse", k + 2, rr),
                                     f"ds_read_b128 {self.vr(16 * par + 4 * rr, 4)}, v{self.ALD_NXT} "
                                     f"offset:{self.row_off(par, 0, rr)}")
                        else:
                            self.lds(("delta", k + 2, rr - 4),
                                     f"ds_read_b128 {self.vr(32 + 16 * par + 4 * (rr - 4), 4)}, v{self.ALD_NXT} "
                                     f"offset:{self.row_off(par, 1, rr - 4)}")
                if par == 1:
                    n_add = -(-len(adds) // max(NB - 1, 1))
                    if idx >= 1:
                        for op in adds[(idx - 1) * n_add: idx * n_add]:
                            self.emit(op)
                    if idx == NB - 1:
                        for op in tail:
                            self.emit(op)
        # a block that is not inside the window of every key of this wave gets its mask now
        self.out += [f"s_cmp_lt_i32 s44, s51",
                     f"s_cbranch_scc1 Lmask_{label}",
                     f"s_add_i32 s66, s44, 32",
                     f"s_cmp_le_i32 s66, s69",
                     f"s_cbranch_scc1 Lnomask_{label}",
                     f"Lmask_{label}:"]
        # (the lse of that block has to be there; the other path does not wait and the static count
        # of returned reads stays that of the other path)
        if ("lse", k + 2, 3) in self.issued:
            idx = len(self.issued) - 1 - self.issued[::-1].index(("lse", k + 2, 3))
            if idx > self.done:
                self.out.append(f"s_waitcnt lgkmcnt({min(len(self.issued) - 1 - idx, 15)})")
        self.out += mask
        self.out.append(f"Lnomask_{label}:")
        parts.append(self.out)
        self.out = []
        return parts

    def prologue(self):
        self.out = []
        for g in range(self.NF):
            self.emit(f"v_add_u32 v{self.AROW_NXT + g}, s46, v{self.AROW_BASE + g}")
            self.emit(f"v_mov_b32 v{self.AROW_CUR + g}, v{self.AROW_NXT + g}")
        for x in list(range(self.DB)) + list(range(4, 4 + self.DB)):
            self.emit(f"v_add_u32 v{self.ATR_CUR + x}, s46, v{self.ATR_BASE + x}")
        self.emit(f"v_add_u32 v{self.ALD_NXT}, s46, v{self.ALD_BASE}")
        self.emit(f"v_mov_b32 v{self.ALD_CUR}, v{self.ALD_NXT}")
        return self.out


SCALARS = ["spare", "qt1", "t", "q64", "n32", "st0", "st1", "st2", "wave_tile", "wave_rows", "last_row", "qlo_max",
           "rq0", "rq1", "rq2", "rq3", "rg0", "rg1", "rg2", "rg3", "soff_q", "soff_g", "istep_q", "istep_g",
           "tstep_q", "tstep_g", "tmp0", "tmp1", "tmp2", "qhi_min"]          # v208 + i  ->  s40 + i


def issue_tile(g):
    """Asynchronous loads of the tile NST - 1 = 2 ahead into the stage at s47: this wave's share of the
    Q and dO tiles (global -> LDS, 16 bytes per lane) and of their lse / delta rows."""
    NW = 4
    rpi = 1024 // g.ROWB                  # rows per load instruction
    per_wave = (TQ // rpi) // NW
    out = ["s_add_u32 s68, s47, s48"]
    for tensor, (rs, soff, istep, tstep, voff) in enumerate(((52, 60, 62, 64, 240), (56, 61, 63, 65, 241))):
        out.append(f"s_mov_b32 s66, s{soff}")
        for i in range(per_wave):
            out += [f"s_add_u32 m0, s68, {tensor * g.TILE_B + i * NW * rpi * g.ROWB}",
                    "s_nop 0",
                    f"buffer_load_dwordx4 v{voff}, s[{rs}:{rs + 3}], s66 offen lds"]
            if i + 1 < per_wave:
                out.append(f"s_add_u32 s66, s66, s{istep}")
        out.append(f"s_add_u32 s{soff}, s{soff}, s{tstep}")
    out += ["v_min_i32 v245, s50, v244",
            "v_lshlrev_b32 v245, 2, v245",
            "v_add_co_u32 v246, vcc, v242, v245",
            "v_addc_co_u32 v247, vcc, 0, v243, vcc",
            "s_add_u32 m0, s47, s49",
            "s_mov_b32 exec_hi, 0",
            "global_load_lds_dword v[246:247], off",
            "s_mov_b32 exec_hi, -1",
            "v_add_u32 v244, 64, v244"]
    return out, 2 * per_wave + 1


def generate(D, dt):
    g = Gen(D, dt)
    NS = g.NS
    split = NS - PF
    # steady state: simulate odd, even, odd, even steps and keep the last pair
    texts = {}
    k = 1   # an odd step first, as in the kernel
    for rnd in range(3):
        b1 = g.body(k, 1, label=f"o_{D}_{dt}_%=")
        b0 = g.body(k + 1, 0, split_at=split, label=f"e_{D}_{dt}_%=")
        texts = {"B1": b1[0], "B0A": b0[0], "B0B": b0[1]}
        k += 2
    # prologue: addresses of the first tile, ring entries of the first step's slots 0..PF-1, the first
    # block's accumulator starts; everything has returned when it ends
    p = Gen(D, dt)
    pro = [f"v_readfirstlane_b32 s{40 + i}, v{208 + i}" for i in range(len(SCALARS))]
    p.out = pro + p.prologue()
    for j in range(PF):
        p.fetch(NS + j, j, 1, True)   # same ring positions as any step's slots 0..PF-1 (NS % RING == 0)
    for rr in range(4):
        p.lds(("lse", 0, rr), f"ds_read_b128 {p.vr(4 * rr, 4)}, v{p.ALD_NXT} offset:{p.row_off(0, 0, rr)}")
    for rr in range(4):
        p.lds(("delta", 0, rr), f"ds_read_b128 {p.vr(32 + 4 * rr, 4)}, v{p.ALD_NXT} offset:{p.row_off(0, 1, rr)}")
    p.emit("s_waitcnt lgkmcnt(0)")
    p.emit("s_add_i32 s44, s43, 64")     # first row of block 0 of tile s42 + 1
    for op in p.mask_ops(0):
        p.emit(op)
    # the phantom block: every probability exp2(-inf) = 0
    for i in range(16):
        p.emit(f"v_mov_b32 {p.S(1, i)}, 0x7f800000")
        p.emit(f"v_mov_b32 {p.DP(1, i)}, 0")
    issue, lpt = issue_tile(g)
    L = lambda name: f"{name}_{D}_{dt}_%="
    text = p.out
    text += [L("Lloop") + ":",
             "s_add_i32 s44, s43, 96"]          # odd step masks block 1 of tile s42 + 1
    text += texts["B1"]
    text += ["s_add_i32 s42, s42, 1",
             "s_add_i32 s43, s43, 64",
             "s_mov_b32 s66, s45", "s_mov_b32 s45, s46", "s_mov_b32 s46, s47", "s_mov_b32 s47, s66",
             "s_cmp_ge_i32 s42, s41",
             "s_cbranch_scc1 " + L("Lend")]
    text += texts["B0A"]
    # Block 0 of tile s42 + 1 is read from here on: its loads must have landed in every wave's share.
    # The stage of tile s42 - 1 (now s47), which no wave reads any more, takes tile s42 + 2.
    text += ["s_add_i32 s66, s42, 1",
             "s_cmp_ge_i32 s66, s41",
             "s_cbranch_scc1 " + L("Lskip"),
             "s_waitcnt vmcnt(0)",
             "s_barrier",
             "s_add_i32 s66, s42, 2",
             "s_cmp_ge_i32 s66, s41",
             "s_cbranch_scc1 " + L("Lskip")]
    text += issue
    text += [L("Lskip") + ":",
             "s_add_i32 s44, s43, 64"]          # even step masks block 0 of tile s42 + 1
    text += texts["B0B"]
    text += ["s_branch " + L("Lloop"),
             L("Lend") + ":",
             "s_nop 15", "s_nop 15"]            # the accumulators are read by vector instructions next
    name = f"SA_DKDV3_{D}_{dt.upper()}"
    return f"#define {name} \\\n" + " \\\n".join('    "' + ln + '\\n"' for ln in text) + "\n"


def main():
    print("// Generated by gen_dkdv3_asm.py -- do not edit.  Prologue and main loop of dkdv3_kernel.")
    print("#define SA_DKDV3_RING %d" % RING)
    print("#define SA_DKDV3_NUM_SCALARS %d" % len(SCALARS))
    for i, nm in enumerate(SCALARS):
        print(f"#define SA_DKDV3_SC_{nm.upper()} {i}")
    for D in (128,):
        for dt in ("bf16", "f16"):
            print(generate(D, dt))


if __name__ == "__main__":
    main()
