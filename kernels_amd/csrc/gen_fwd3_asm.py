#!/usr/bin/env python3
"""Generator of the main-loop assembly of fwd3_kernel (sa_fwd3.h) -> sa_fwd3_asm.inc.

One wave per SIMD owns 64 queries (two blocks of 32) and walks the 32-key blocks j of its
workgroup's window.  Iteration j issues 32 MFMAs - S(j+1) = K Q^T for both query blocks, then
O += V^T P(j-1) - and, in the gaps between them, the softmax arithmetic of block j.  Scores and
rounded probabilities are double-buffered, so nothing in an iteration waits for anything else in it,
and every K and V fragment read from LDS feeds two MFMAs (one per query block).

A single wave issues at most one instruction per four cycles, whatever its kind, so the loop is
bound by its instruction count; the common path is therefore kept to the arithmetic that every score
needs (multiply-add, exp2, an addition for the row sum, half a conversion):

  * the probabilities of a block are formed against the reference maximum as it stands.  Only when
    a lane's half-row sum of the block exceeds its limit (a score more than 8 above the reference,
    or no reference yet) does the wave leave through `Lfull`, which looks for the block maximum,
    moves the reference of the lanes that need it, rescales their row sums, recomputes the block's
    probabilities from the scores (which the common path leaves intact) and flags the accumulators
    for rescaling at the end of the iteration (`Lscale`);
  * -reference (0 while there is none) and the limit (256, or -1 while there is none, which sends
    the lane through `Lfull`) are kept per lane and only change inside `Lfull`;
  * blocks that are not inside the window of every query of the wave first take the masking detour
    `Lmask`, which sets the scores outside a lane's window to -inf.

Register map (D = 128):
  a[0:127]   O^T accumulators, 16 registers per (query block, 32 columns of D)
  a[128:191] Q fragments, 4 registers per (query block, 16 columns of D)
  v[0:31]    scores of even blocks (16 per query block)      v[32:63]  scores of odd blocks
  v[64:79]   rounded probabilities of even blocks             v[80:95]  of odd blocks
  a[192:223] fragment ring, 8 entries of 4 registers           v[96:127] free
  v[128:135] K row-fragment addresses (tile being read)      v[136:143] temporaries of the rare paths
  v[144:151] K row-fragment offsets inside a stage            v[152:159] V transposing-read offsets
  v[160:167] V transposing-read addresses (tile being read)
  v168, v169 reference maximum per query block (log2 units)   v170, v171 running row sums
  v[172:175] row sums of the block (two chains per query block)
  v176..v179 key window [lo, hi) of this lane's query, per query block        v180 4*(lane/32)
  v181, v182 rescale factors    v183, v184 -reference (0 while it is -inf)    v185, v186 sum limits
  v187, v188 block maximum      v189, v190 block sums    v[191:198] exp2 temporaries    v[199:207] temporaries
  v[208:239] wave-uniform inputs, copied to s40... at entry (see SCALARS)
  v240, v241 buffer offsets of this lane for the K / V tile loads
  s40 |scale*log2e|  s41 one past the last key tile of the workgroup  s42 key tile of even block j  s43 first key of block j
  s44..s47 LDS address of the stages of tiles s42-1, s42, s42+1, s42+2  s48 wave offset inside a tile for the
  asynchronous loads  s49 -inf  s50, s51: a block inside [s50, s51) lies inside the window of every query of
  this wave  s[52:55], s[56:59] buffer resources of K and V  s60, s61 their running byte offsets  s62, s63 bytes
  between a wave's load instructions  s64, s65 bytes between tiles  s66..s69 temporaries  s[70:75] lane masks
  s76 set when the accumulators must be rescaled at the end of the iteration
  s77, s78 first key tile of this wave's own window and one past its last

Run:  python3 gen_fwd3_asm.py > sa_fwd3_asm.inc   (the Makefile does this)
"""

RING = 8
PF = RING - 1          # fragments between a read and its use
NFRAG = 16             # fragments per iteration: 8 of K, 8 of V
NSLOT = 32
ROWB = 256
TILE_B = 64 * ROWB
BLK_B = 32 * ROWB


def vr(lo, n=1):
    return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"


def ar(lo, n=1):
    return f"a{lo}" if n == 1 else f"a[{lo}:{lo + n - 1}]"


def O(qb, m):
    return ar(64 * qb + 16 * m, 16)


def QF(qb, g):
    return ar(128 + 32 * qb + 4 * g, 4)


def S(buf, qb, i=None):
    return vr(32 * buf + 16 * qb, 16) if i is None else vr(32 * buf + 16 * qb + i)


def PB(buf, qb, half, w=None):
    base = 64 + 16 * buf + 8 * qb + 4 * half
    return vr(base, 4) if w is None else vr(base + w)


def RG(r, lo=0, n=4):
    """Ring entry r.  The ring lives in accumulation registers: LDS reads can land there and MFMAs can take
    their A operand from there, which leaves v[96:127] to the vector arithmetic."""
    return ar(192 + 4 * r + lo, n)


AK, RT, AROW_BASE, ATR_BASE, AV = 128, 136, 144, 152, 160
M, LRUN, BS, QLO, QHI, H4 = 168, 170, 172, 176, 177, 180
ALPHA, NEGM, LIMIT, MX, BSUM, TMP, TD = 181, 183, 185, 187, 189, 191, 199


class Gen:
    def __init__(self, dt):
        self.dt = dt
        self.mfma = "v_mfma_f32_32x32x16_" + dt
        self.cvt = "v_cvt_pk_bf16_f32" if dt == "bf16" else "v_cvt_pk_f16_f32"
        self.issued, self.done, self.out = [], -1, []
        self.tails = []      # out-of-line blocks

    def emit(self, s):
        self.out.append(s)

    def lds(self, tag, text):
        self.issued.append(tag)
        self.emit(text)

    def need(self, tag):
        """Wait until the LDS read `tag` has returned (reads return in issue order)."""
        if tag not in self.issued:
            return
        idx = len(self.issued) - 1 - self.issued[::-1].index(tag)
        if idx <= self.done:
            return
        n = len(self.issued) - 1 - idx
        self.emit(f"s_waitcnt lgkmcnt({min(n, 15)})")
        self.done = idx if n <= 15 else len(self.issued) - 16

    # ---- LDS reads -----------------------------------------------------------------------
    def fetch(self, gf, f, par):
        """Fragment f of an iteration of parity par into ring entry gf % RING."""
        r = gf % RING
        if f < 8:
            # K fragment g of block j + 1: parity par ^ 1 of the tile the K addresses point at
            off = (par ^ 1) * BLK_B
            self.lds(("ring", gf), f"ds_read_b128 {RG(r)}, v{AK + f} offset:{off}")
        else:
            # V fragment of block j - 1 (parity par ^ 1): rows half*16 + r_lo (+8), columns of block m
            x = f - 8
            half, m = x // 4, x % 4
            off = TILE_B + (par ^ 1) * BLK_B + half * 16 * ROWB
            self.lds(("ringlo", gf), f"ds_read_b64_tr_b16 {RG(r, 0, 2)}, v{AV + m} offset:{off}")
            self.lds(("ring", gf), f"ds_read_b64_tr_b16 {RG(r, 2, 2)}, v{AV + 4 + m} offset:{off}")

    # ---- probabilities of one query block from its scores, rounded, with the block's row sums ------
    def prob_ops(self, par, qb):
        """P = exp2(S c - reference) through rotating temporaries (the scores stay), rounded per pair
        into the B fragments of the second product, and added up in float32 in two chains (plain
        additions: dot-product instructions stall against the MFMAs in flight).  A v_exp result is never
        consumed by the very next instruction."""
        ops = []
        t = lambda i: vr(TMP + (i % 8))

        def fma(i):
            return f"v_fma_f32 {t(i)}, {S(par, qb, i)}, s40, {vr(NEGM + qb)}"

        def pbw(k):     # the packed word that holds elements k - 1, k (k odd)
            return PB(par, qb, k >> 3, (k & 7) >> 1)

        def add(k):     # element k joins chain k & 1; elements 0 and 1 enter with elements 2 and 3
            acc = vr(BS + 2 * qb + (k & 1))
            if k < 2:
                return None
            return f"v_add_f32 {acc}, {t(k - 2) if k < 4 else acc}, {t(k)}"

        ops += [fma(0), fma(1)]
        for i in range(16):
            ops.append(f"v_exp_f32 {t(i)}, {t(i)}")
            if i + 2 < 16:
                ops.append(fma(i + 2))
            if i >= 1 and add(i - 1):
                ops.append(add(i - 1))
            if i & 1:
                ops.append(f"{self.cvt} {pbw(i)}, {t(i - 1)}, {t(i)}")
        ops.append(add(15))
        return ops

    def block_sum(self, qb):
        return f"v_add_f32 {vr(BSUM + qb)}, {vr(BS + 2 * qb)}, {vr(BS + 2 * qb + 1)}"

    def prob_both(self, par):
        """Probabilities and block sums of both query blocks."""
        return self.prob_ops(par, 0) + [self.block_sum(0)] + self.prob_ops(par, 1) + [self.block_sum(1)]

    # ---- vector work of block j (scores in buffer par) ----------------------------------------
    def softmax_ops(self, par, lab):
        ops = []
        # blocks that are not inside every query's window take the masking detour first
        # (a detour and the label it returns to are one entry, so that no MFMA lands between them)
        ops += [("s_cmp_lt_i32 s43, s50",
                 f"s_cbranch_scc1 Lmask_{lab}",
                 "s_add_i32 s66, s43, 32",
                 "s_cmp_gt_i32 s66, s51",
                 f"s_cbranch_scc1 Lmask_{lab}",
                 f"Lmaskback_{lab}:")]
        ops += self.prob_both(par)
        for qb in range(2):
            ops.append(f"v_cmp_nle_f32 s[{70 + 2 * qb}:{71 + 2 * qb}], {vr(BSUM + qb)}, {vr(LIMIT + qb)}")
        ops += [("s_or_b64 s[74:75], s[70:71], s[72:73]",
                 f"s_cbranch_scc1 Lfull_{lab}",
                 f"Lfullback_{lab}:")]
        for qb in range(2):
            ops.append(f"v_add_f32 {vr(LRUN + qb)}, {vr(LRUN + qb)}, {vr(BSUM + qb)}")
        return ops

    def mask_block(self, par, lab):
        """Scores of block j outside this lane's [lo, hi) become -inf."""
        t = RT
        ops = [f"Lmask_{lab}:"]
        for qb in range(2):
            ops += [f"v_subrev_u32 v{t}, s43, {vr(QLO + 2 * qb)}",
                    f"v_subrev_u32 v{t + 1}, s43, {vr(QHI + 2 * qb)}",
                    f"v_med3_i32 v{t}, v{t}, 0, 32",
                    f"v_med3_i32 v{t + 1}, v{t + 1}, 0, 32",
                    f"v_lshlrev_b64 v[{t + 2}:{t + 3}], v{t}, 1",
                    f"v_lshlrev_b64 v[{t + 4}:{t + 5}], v{t + 1}, 1",
                    f"v_add_u32 v{t + 2}, -1, v{t + 2}",
                    f"v_add_u32 v{t + 4}, -1, v{t + 4}",
                    f"v_not_b32 v{t + 2}, v{t + 2}",
                    f"v_and_b32 v{t + 4}, v{t + 4}, v{t + 2}",
                    f"v_lshrrev_b32 v{t + 4}, {vr(H4)}, v{t + 4}"]
            for i in range(16):
                pos = 8 * (i >> 2) + (i & 3)
                ops.append(f"v_bfe_i32 v{t + 6 + (i & 1)}, v{t + 4}, {pos}, 1")
                if i >= 1:
                    k = i - 1
                    ops.append(f"v_bitop3_b32 {S(par, qb, k)}, {S(par, qb, k)}, s49, v{t + 6 + (k & 1)} bitop3:0xe4")
            ops.append(f"v_bitop3_b32 {S(par, qb, 15)}, {S(par, qb, 15)}, s49, v{t + 7} bitop3:0xe4")
        ops.append(f"s_branch Lmaskback_{lab}")
        return ops

    def full_block(self, par, lab):
        """Some lane's block sum is over its limit: find the block maximum, move the reference of the lanes
        whose maximum exceeds it by more than 8 (or that had none), and form the block's probabilities again."""
        ops = [f"Lfull_{lab}:"]
        # block maximum: two chains per query block, the four chains interleaved
        c = [[TD + 0, TD + 1], [TD + 2, TD + 3]]
        seq0 = [(None, 0, 1, 2), (0, 6, 7), (0, 10, 11), (0, 14, 15)]
        seq1 = [(None, 3, 4, 5), (1, 8, 9), (1, 12, 13)]
        for step in range(4):
            for qb in range(2):
                for ch, seq in ((0, seq0), (1, seq1)):
                    if step >= len(seq):
                        continue
                    e = seq[step]
                    dst = vr(c[qb][ch])
                    if e[0] is None:
                        ops.append(f"v_max3_f32 {dst}, {S(par, qb, e[1])}, {S(par, qb, e[2])}, {S(par, qb, e[3])}")
                    else:
                        ops.append(f"v_max3_f32 {dst}, {dst}, {S(par, qb, e[1])}, {S(par, qb, e[2])}")
        for qb in range(2):
            ops.append(f"v_max_f32 {vr(c[qb][0])}, {vr(c[qb][0])}, {vr(c[qb][1])}")
        # the other half of the key rows sits in lane ^ 32
        for qb in range(2):
            ops.append(f"v_mov_b32 {vr(c[qb][1])}, {vr(c[qb][0])}")
        ops.append("s_nop 1")
        for qb in range(2):
            ops.append(f"v_permlane32_swap_b32 {vr(c[qb][0])}, {vr(c[qb][1])}")
        ops.append("s_nop 1")
        for qb in range(2):
            ops.append(f"v_max_f32 {vr(MX + qb)}, {vr(c[qb][0])}, {vr(c[qb][1])}")
        for qb in range(2):
            ops.append(f"v_add_f32 {vr(TD + 4 + qb)}, 0x41000000, {vr(M + qb)}")
        for qb in range(2):
            ops.append(f"v_mul_f32 {vr(MX + qb)}, s40, {vr(MX + qb)}")
        ops.append(f"v_cmp_gt_f32 s[70:71], {vr(MX)}, {vr(TD + 4)}")
        ops.append(f"v_cmp_gt_f32 s[72:73], {vr(MX + 1)}, {vr(TD + 5)}")
        for qb in range(2):
            ops.append(f"v_sub_f32 v{TD + 6 + qb}, {vr(M + qb)}, {vr(MX + qb)}")
        for qb in range(2):
            ops.append(f"v_exp_f32 v{TD + 6 + qb}, v{TD + 6 + qb}")
        ops.append("s_nop 0")
        for qb in range(2):
            mask = f"s[{70 + 2 * qb}:{71 + 2 * qb}]"
            ops.append(f"v_cndmask_b32 {vr(ALPHA + qb)}, 1.0, v{TD + 6 + qb}, {mask}")
            ops.append(f"v_cndmask_b32 {vr(M + qb)}, {vr(M + qb)}, {vr(MX + qb)}, {mask}")
        for qb in range(2):
            ops.append(f"v_mul_f32 {vr(LRUN + qb)}, {vr(LRUN + qb)}, {vr(ALPHA + qb)}")
        # -reference and the sum limit of the lanes, from the reference as it now stands
        ops.append(f"v_mov_b32 v{TD + 8}, 0x43800000")
        for qb in range(2):
            ops.append(f"v_cmp_neq_f32 vcc, s49, {vr(M + qb)}")
            ops.append(f"v_cndmask_b32 {vr(NEGM + qb)}, 0, -{vr(M + qb)}, vcc")
            ops.append(f"v_cndmask_b32 {vr(LIMIT + qb)}, -1.0, v{TD + 8}, vcc")
        ops.append("s_mov_b32 s76, 1")
        ops += self.prob_both(par)
        ops.append(f"s_branch Lfullback_{lab}")
        return ops

    def scale_block(self, lab):
        """O *= alpha for both query blocks, after the iteration's last MFMA has retired."""
        ops = [f"Lscale_{lab}:", "s_nop 15", "s_nop 15", "s_nop 15", "s_nop 15"]
        for qb in range(2):
            for r0 in range(0, 64, 8):
                for r in range(r0, r0 + 8):
                    ops.append(f"v_accvgpr_read_b32 v{RT + r - r0}, a{64 * qb + r}")
                ops.append("s_nop 0")
                for r in range(r0, r0 + 8):
                    ops.append(f"v_mul_f32 v{RT + r - r0}, v{RT + r - r0}, {vr(ALPHA + qb)}")
                ops.append("s_nop 0")
                for r in range(r0, r0 + 8):
                    ops.append(f"v_accvgpr_write_b32 a{64 * qb + r}, v{RT + r - r0}")
        ops += ["s_nop 1", "s_mov_b32 s76, 0", f"s_branch Lscaleback_{lab}"]
        return ops

    # ---- one iteration ---------------------------------------------------------------------
    def body(self, k, par, lab, with_pv=True, mid=None):
        """Iteration k (global counter, parity par).  The instructions that are not MFMAs are spread over
        the 32 gaps between the MFMAs so that every gap carries about the same issue time.  `mid` (even
        iterations: the tile hand-over) goes into gap 10."""
        self.out = []
        vops = self.softmax_ops(par, lab)

        def cost(op):
            if isinstance(op, tuple):
                return sum(0 if ln.endswith(":") else 1 for ln in op)
            return 2 if op.startswith("v_exp") else 1

        # fixed content of the gaps: LDS reads and waits (before the MFMA), address moves, hand-over
        fixed = [[] for _ in range(NSLOT)]
        if par == 0:
            # K addresses move to the next tile after this iteration's own last K read (slot 0 issues
            # it) and before slot 18 reads the next iteration's first fragments; V addresses move to
            # this tile after the last V read (slot 16)
            for g in range(8):
                fixed[2 + g].append(f"v_add_u32 v{AK + g}, s46, v{AROW_BASE + g}")
                fixed[18 + g].append(f"v_add_u32 v{AV + g}, s45, v{ATR_BASE + g}")
        if mid is not None:
            fixed[10] += mid
        lds_cost = [0] * NSLOT
        for s in range(0, NSLOT, 2):
            f = s // 2
            lds_cost[s] = 2 if (f + PF) % NFRAG < 8 else 3
        total = sum(cost(op) for op in vops) + sum(len(x) for x in fixed) + sum(lds_cost)
        vi, cum = 0, 0.0
        for s in range(NSLOT):
            f = s // 2
            gf = k * NFRAG + f
            if s % 2 == 0:
                fn = f + PF
                if fn < NFRAG:
                    self.fetch(gf + PF, fn, par)
                else:
                    self.fetch(gf + PF, fn - NFRAG, par ^ 1)
                self.need(("ring", gf))
            r = gf % RING
            qb = s % 2
            if f < 8:
                nb = par ^ 1
                c = "0" if f == 0 else S(nb, qb)
                self.emit(f"{self.mfma} {S(nb, qb)}, {RG(r)}, {QF(qb, f)}, {c}")
            elif with_pv:
                x = f - 8
                half, m = x // 4, x % 4
                self.emit(f"{self.mfma} {O(qb, m)}, {RG(r)}, {PB(par ^ 1, qb, half)}, {O(qb, m)}")
            cum += lds_cost[s] + len(fixed[s])
            target = total * (s + 1) / NSLOT
            while vi < len(vops) and (s == NSLOT - 1 or cum + cost(vops[vi]) / 2 <= target):
                op = vops[vi]
                for line in (op if isinstance(op, tuple) else (op,)):
                    self.emit(line)
                cum += cost(op)
                vi += 1
            for line in fixed[s]:
                self.emit(line)
        assert vi >= len(vops)
        self.out += ["s_cmp_eq_u32 s76, 0",
                     f"s_cbranch_scc0 Lscale_{lab}",
                     f"Lscaleback_{lab}:"]
        self.tails += self.mask_block(par, lab) + self.full_block(par, lab) + self.scale_block(lab)
        return self.out


SCALARS = ["sl2e", "kt1", "t", "kb", "st0", "st1", "st2", "st3", "wave_tile", "ninf", "lo_max", "hi_min",
           "rk0", "rk1", "rk2", "rk3", "rv0", "rv1", "rv2", "rv3", "soff_k", "soff_v", "istep_k", "istep_v",
           "tstep_k", "tstep_v", "wfirst", "wend"]   # v208 + i -> s40 + i; the last two -> s77, s78 (s66..s76 are taken)
SREG = {i: 40 + i for i in range(26)}
SREG.update({26: 77, 27: 78})


def issue_tile():
    """Asynchronous loads of tile s42 + 2 into the stage at s47: this wave's share of the K and V tiles."""
    NW, rpi = 4, 1024 // ROWB
    per_wave = (64 // rpi) // NW
    out = ["s_add_u32 s68, s47, s48"]
    for tensor, (rs, soff, istep, tstep, voff) in enumerate(((52, 60, 62, 64, 240), (56, 61, 63, 65, 241))):
        out.append(f"s_mov_b32 s66, s{soff}")
        for i in range(per_wave):
            out += [f"s_add_u32 m0, s68, {tensor * TILE_B + i * NW * rpi * ROWB}",
                    "s_nop 0",
                    f"buffer_load_dwordx4 v{voff}, s[{rs}:{rs + 3}], s66 offen lds"]
            if i + 1 < per_wave:
                out.append(f"s_add_u32 s66, s66, s{istep}")
        out.append(f"s_add_u32 s{soff}, s{soff}, s{tstep}")
    return out


def generate(dt):
    L = lambda name: f"{name}_{dt}_%="
    g = Gen(dt)
    # tile hand-over of an even iteration: tile s42 + 1 must have landed in every wave's share before its K
    # is read (slot 18 on); the stage of tile s42 - 2 (s47), which nobody reads any more, takes tile s42 + 2
    def mid(lab):
        return ["s_add_i32 s66, s42, 1",
                "s_cmp_ge_i32 s66, s41",
                f"s_cbranch_scc1 Lskip_{lab}",
                "s_waitcnt vmcnt(0)",
                "s_barrier",
                "s_add_i32 s66, s42, 2",
                "s_cmp_ge_i32 s66, s41",
                f"s_cbranch_scc1 Lskip_{lab}"] + issue_tile() + [f"Lskip_{lab}:"]
    rotate = ["s_mov_b32 s66, s44", "s_mov_b32 s44, s45", "s_mov_b32 s45, s46", "s_mov_b32 s46, s47", "s_mov_b32 s47, s66"]
    # ---- prologue: scalars, per-lane state, addresses, scores of block 0, ring entries of the first iteration
    pro = [f"v_readfirstlane_b32 s{SREG[i]}, v{208 + i}" for i in range(len(SCALARS))]
    # Tiles of the workgroup's window that lie before this wave's own window (s77 = its first tile): no arithmetic,
    # only the wave's part in the hand-over of every tile (its share of the loads, the barrier).  The same after
    # the wave's last tile (s78 = one past it).
    pro += [L("Lin") + ":",
            "s_cmp_ge_i32 s42, s77",
            "s_cbranch_scc1 " + L("Lin_done")] + mid(L("i")) + [
            "s_add_i32 s42, s42, 1"] + rotate + [
            "s_branch " + L("Lin"),
            L("Lin_done") + ":",
            "s_lshl_b32 s43, s42, 6"]
    pro += ["s_mov_b32 s76, 0"]
    for qb in range(2):
        pro += [f"v_mov_b32 {vr(M + qb)}, s49", f"v_mov_b32 {vr(LRUN + qb)}, 0",
                f"v_mov_b32 {vr(NEGM + qb)}, 0", f"v_mov_b32 {vr(LIMIT + qb)}, -1.0",
                f"v_mov_b32 {vr(ALPHA + qb)}, 1.0"]
    pro += [f"v_add_u32 v{AK + x}, s45, v{AROW_BASE + x}" for x in range(8)]
    pro += [f"v_add_u32 v{AV + x}, s44, v{ATR_BASE + x}" for x in range(8)]
    g.out = pro
    for f in range(8):
        g.lds(("pro", f), f"ds_read_b128 {RG(f)}, v{AK + f} offset:0")
    for f in range(8):
        g.need(("pro", f))
        for qb in range(2):
            c = "0" if f == 0 else S(0, qb)
            g.emit(f"{g.mfma} {S(0, qb)}, {RG(f)}, {QF(qb, f)}, {c}")
    g.emit("s_nop 7")
    g.emit("s_nop 7")
    # ring entries of fragments 0..6 of iteration 0 (same ring positions as in any iteration)
    for f in range(PF):
        g.fetch(NFRAG + f, f, 0)
    text = g.out

    k = 1
    first = g.body(k, 0, L("f"), with_pv=False, mid=mid(L("f")))
    k += 1
    for rnd in range(3):
        save = len(g.tails)
        b1 = g.body(k, 1, L("o"))
        b0 = g.body(k + 1, 0, L("e"), mid=mid(L("e")))
        if rnd < 2:
            del g.tails[save:]
        k += 2
    text += first
    text += [L("Lloop") + ":",
             "s_add_i32 s43, s43, 32"]
    text += b1
    text += ["s_add_i32 s42, s42, 1",
             "s_add_i32 s43, s43, 32",
             *rotate,
             "s_cmp_ge_i32 s42, s78",
             "s_cbranch_scc1 " + L("Lend")]
    text += b0
    text += ["s_branch " + L("Lloop"),
             L("Lend") + ":"]
    # ---- drain: O += V^T P of the last block (odd parity: block 1 of the tile the V addresses point at) ----
    text.append("s_waitcnt lgkmcnt(0)")
    for x in range(8):
        half, m = x // 4, x % 4
        off = TILE_B + BLK_B + half * 16 * ROWB
        text.append(f"ds_read_b64_tr_b16 {RG(x, 0, 2)}, v{AV + m} offset:{off}")
        text.append(f"ds_read_b64_tr_b16 {RG(x, 2, 2)}, v{AV + 4 + m} offset:{off}")
    for x in range(8):
        half, m = x // 4, x % 4
        n = 2 * (7 - x)
        text.append(f"s_waitcnt lgkmcnt({min(n, 15)})")
        for qb in range(2):
            text.append(f"{g.mfma} {O(qb, m)}, {RG(x)}, {PB(1, qb, half)}, {O(qb, m)}")
    text += ["s_nop 15", "s_nop 15", "s_nop 15", "s_nop 15"]
    # tiles of the workgroup's window after this wave's last one
    text += [L("Lfin") + ":",
             "s_cmp_ge_i32 s42, s41",
             "s_cbranch_scc1 " + L("Lout")] + mid(L("x")) + [
             "s_add_i32 s42, s42, 1"] + rotate + [
             "s_branch " + L("Lfin")]
    text += g.tails
    text.append(L("Lout") + ":")
    name = f"SA_FWD3_128_{dt.upper()}"
    return f"#define {name} \\\n" + " \\\n".join('    "' + ln + '\\n"' for ln in text) + "\n"


def main():
    print("// Generated by gen_fwd3_asm.py -- do not edit.  Prologue, main loop and drain of fwd3_kernel.")
    print("#define SA_FWD3_NUM_SCALARS %d" % len(SCALARS))
    for i, nm in enumerate(SCALARS):
        print(f"#define SA_FWD3_SC_{nm.upper()} {i}")
    for dt in ("bf16", "f16"):
        print(generate(dt))


if __name__ == "__main__":
    main()
