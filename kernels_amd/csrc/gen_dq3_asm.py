#!/usr/bin/env python3
"""Generator of the main-loop assembly of dq3_kernel (sa_bwd4.h) -> sa_dq3_asm.inc.

One wave per SIMD owns 64 queries (two blocks of 32) with their Q and dO fragments and both dQ
accumulators in registers, and walks the 32-key blocks j of its workgroup's window.  Iteration j
issues 48 MFMAs - S(j+1) = K Q^T and delta - dP(j+1) = delta - V dO^T for both query blocks (K and V
row fragments alternate, so four accumulator chains interleave), then dQ^T -= K^T (-dS(j-1)) - and,
between them, the arithmetic of block j: P = exp2(S c - lse), -dS = P (delta - dP), rounding.  Scores,
dP and the rounded -dS are double-buffered, so nothing in an iteration waits for anything else in
it; every fragment read from LDS feeds two MFMAs (one per query block).  There is no running
maximum and no row sum in the backward pass, which is why this loop (2.3 vector instructions per
MFMA) is bound by the matrix pipe where the forward loop is not.

dO enters negated and the dP accumulators start at delta (a block of 16 registers per query block
that holds the lane's delta in every register serves as the first MFMA's addend), so delta - dP
comes out of the matrix pipe; the sign is put back by the scale of the final store.

Register map (D = 128):
  a[0:127]   -dQ^T accumulators, 16 registers per (query block, 32 columns of D)
  a[128:191] Q fragments, a[192:255] -dO fragments, 4 registers per (query block, 16 columns of D)
  v[0:31]    scores of even blocks (16 per query block)          v[32:63]   scores of odd blocks
  v[64:95]   delta - dP of even blocks                            v[96:127]  of odd blocks
  v[128:143] rounded -dS of even blocks                           v[144:159] of odd blocks
  v[160:191] fragment ring, 8 entries of 4 registers (at entry: the wave-uniform inputs, copied to s40...)
  v[192:199] row-fragment addresses of the K tile being read (V: + one tile)
  v[200:207] transposing-read addresses of the K tile being read
  v[208:239] delta of this lane's two queries, 16 copies each
  v240, v241 -lse per query block     v242..v245 key window [lo, hi) per query block     v246 4*(lane/32)
  v247, v248 buffer offsets of this lane for the K / V tile loads     v[250:255] temporaries of the masking detour
  s40 |scale*log2e|  s41 one past the last key tile  s42 key tile of even block j  s43 first key of block j
  s44..s47 LDS address of the stages of tiles s42-1, s42, s42+1, s42+2  s48 wave offset inside a tile for the
  asynchronous loads  s49 -inf  s50, s51: a block inside [s50, s51) lies inside the window of every query of
  this wave  s[52:55], s[56:59] buffer resources of K and V  s60, s61 their running byte offsets  s62, s63 bytes
  between a wave's load instructions  s64, s65 bytes between tiles  s66..s69 temporaries
  s70, s71 first key tile of this wave's own window and one past its last (s41: of the workgroup's window)

Run:  python3 gen_dq3_asm.py > sa_dq3_asm.inc   (the Makefile does this)
"""

RING = 8
PF = RING - 1          # fragments between a read and its use
NFRAG = 24             # fragments per iteration: 8 K rows, 8 V rows (alternating), 8 K transposed
NSLOT = 48
ROWB = 256
TILE_B = 64 * ROWB
BLK_B = 32 * ROWB


def vr(lo, n=1):
    return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"


def ar(lo, n=1):
    return f"a{lo}" if n == 1 else f"a[{lo}:{lo + n - 1}]"


def DQ(qb, m):
    return ar(64 * qb + 16 * m, 16)


def QF(qb, g):
    return ar(128 + 32 * qb + 4 * g, 4)


def GF(qb, g):
    return ar(192 + 32 * qb + 4 * g, 4)


def S(buf, qb, i=None):
    return vr(32 * buf + 16 * qb, 16) if i is None else vr(32 * buf + 16 * qb + i)


def DP(buf, qb, i=None):
    return vr(64 + 32 * buf + 16 * qb, 16) if i is None else vr(64 + 32 * buf + 16 * qb + i)


def DSB(buf, qb, half, w=None):
    base = 128 + 16 * buf + 8 * qb + 4 * half
    return vr(base, 4) if w is None else vr(base + w)


def RG(r, lo=0, n=4):
    return vr(160 + 4 * r + lo, n)


def DINIT(qb):
    return vr(208 + 16 * qb, 16)


AK, ATR, NLSE, QLO, QHI, H4, RT = 192, 200, 240, 242, 243, 246, 250   # RT even: it heads 64-bit pairs


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
        if f < 16:
            # row fragment g of block j + 1 (parity par ^ 1 of the tile the row addresses point at):
            # even f from the K tile, odd f from the V tile behind it
            g, isv = f >> 1, f & 1
            off = isv * TILE_B + (par ^ 1) * BLK_B
            self.lds(("ring", gf), f"ds_read_b128 {RG(r)}, v{AK + g} offset:{off}")
        else:
            # K^T fragment of block j - 1 (parity par ^ 1): rows half*16 + r_lo (+8), columns of block m
            x = f - 16
            half, m = x // 4, x % 4
            off = (par ^ 1) * BLK_B + half * 16 * ROWB
            self.lds(("ringlo", gf), f"ds_read_b64_tr_b16 {RG(r, 0, 2)}, v{ATR + m} offset:{off}")
            self.lds(("ring", gf), f"ds_read_b64_tr_b16 {RG(r, 2, 2)}, v{ATR + 4 + m} offset:{off}")

    # ---- vector work of block j (scores and delta - dP in buffer par) ------------------------------
    def vector_ops(self, par, lab):
        ops = []
        # blocks that are not inside every query's window take the masking detour first
        # (a detour and the label it returns to are one entry, so that no MFMA lands between them)
        ops += [("s_cmp_lt_i32 s43, s50",
                 f"s_cbranch_scc1 Lmask_{lab}",
                 "s_add_i32 s66, s43, 32",
                 "s_cmp_gt_i32 s66, s51",
                 f"s_cbranch_scc1 Lmask_{lab}",
                 f"Lmaskback_{lab}:")]
        # P in place of the scores, -dS in place of P, rounded per pair; a v_exp result is never
        # consumed by the very next instruction
        for qb in range(2):
            def fma(i):
                return f"v_fma_f32 {S(par, qb, i)}, {S(par, qb, i)}, s40, {vr(NLSE + qb)}"
            def mul(i):
                return f"v_mul_f32 {S(par, qb, i)}, {S(par, qb, i)}, {DP(par, qb, i)}"
            for i in range(16):
                if i == 0:
                    ops += [fma(0), fma(1)]
                ops.append(f"v_exp_f32 {S(par, qb, i)}, {S(par, qb, i)}")
                if i + 2 < 16:
                    ops.append(fma(i + 2))
                if i >= 1:
                    ops.append(mul(i - 1))
                if i >= 2 and (i & 1) == 0:
                    k = i - 1     # pair (k - 1, k) is complete
                    ops.append(f"{self.cvt} {DSB(par, qb, k >> 3, (k & 7) >> 1)}, {S(par, qb, k - 1)}, {S(par, qb, k)}")
            ops.append("s_nop 0")
            ops.append(mul(15))
            ops.append(f"{self.cvt} {DSB(par, qb, 1, 3)}, {S(par, qb, 14)}, {S(par, qb, 15)}")
        return ops

    def mask_block(self, par, lab):
        """Scores of block j outside this lane's [lo, hi) become -inf (their P, and so their dS, 0)."""
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
                ops.append(f"v_bfe_i32 v{t + (i & 1)}, v{t + 4}, {pos}, 1")
                if i >= 1:
                    k = i - 1
                    ops.append(f"v_bitop3_b32 {S(par, qb, k)}, {S(par, qb, k)}, s49, v{t + (k & 1)} bitop3:0xe4")
            ops.append(f"v_bitop3_b32 {S(par, qb, 15)}, {S(par, qb, 15)}, s49, v{t + 1} bitop3:0xe4")
        ops.append(f"s_branch Lmaskback_{lab}")
        return ops

    # ---- one iteration ---------------------------------------------------------------------
    def body(self, k, par, lab, with_dq=True, mid=None):
        """Iteration k (global counter, parity par).  `mid` is inserted after slot 20 (even
        iterations: the tile hand-over)."""
        self.out = []
        vops = self.vector_ops(par, lab)
        if par == 0:
            # row addresses move to the next tile after this iteration's own last row read (slot 16
            # issues it) and after the hand-over, before slot 34 reads the next iteration's first
            # fragments; K^T addresses move to this tile after the last K^T read (slot 32)
            addr_k = ["s_sub_u32 s67, s46, s45"] + [f"v_add_u32 v{AK + g}, s67, v{AK + g}" for g in range(8)]
            addr_t = ["s_sub_u32 s67, s45, s44"] + [f"v_add_u32 v{ATR + x}, s67, v{ATR + x}" for x in range(8)]
        else:
            addr_k, addr_t = [], []
        per = -(-len(vops) // NSLOT)
        vi = 0
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
            nb = par ^ 1
            if f < 16:
                g, isv = f >> 1, f & 1
                if isv:
                    c = DINIT(qb) if g == 0 else DP(nb, qb)
                    self.emit(f"{self.mfma} {DP(nb, qb)}, {RG(r)}, {GF(qb, g)}, {c}")
                else:
                    c = "0" if g == 0 else S(nb, qb)
                    self.emit(f"{self.mfma} {S(nb, qb)}, {RG(r)}, {QF(qb, g)}, {c}")
            elif with_dq:
                x = f - 16
                half, m = x // 4, x % 4
                self.emit(f"{self.mfma} {DQ(qb, m)}, {RG(r)}, {DSB(nb, qb, half)}, {DQ(qb, m)}")
            for op in vops[vi:vi + per]:
                for line in (op if isinstance(op, tuple) else (op,)):
                    self.emit(line)
            vi += per
            if par == 0:
                if mid is not None and s == 20:
                    for op in mid:
                        self.emit(op)
                if 22 <= s < 22 + len(addr_k):
                    self.emit(addr_k[s - 22])
                if 36 <= s < 36 + len(addr_t):
                    self.emit(addr_t[s - 36])
        assert vi >= len(vops)
        self.tails += self.mask_block(par, lab)
        return self.out


SCALARS = ["sl2e", "kt1", "t", "kb", "st0", "st1", "st2", "st3", "wave_tile", "ninf", "lo_max", "hi_min",
           "rk0", "rk1", "rk2", "rk3", "rv0", "rv1", "rv2", "rv3", "soff_k", "soff_v", "istep_k", "istep_v",
           "tstep_k", "tstep_v", "wfirst", "wend"]          # v160 + i  ->  s40 + i


def issue_tile():
    """Asynchronous loads of tile s42 + 2 into the stage at s47: this wave's share of the K and V tiles."""
    NW, rpi = 4, 1024 // ROWB
    per_wave = (64 // rpi) // NW
    out = ["s_add_u32 s68, s47, s48"]
    for tensor, (rs, soff, istep, tstep, voff) in enumerate(((52, 60, 62, 64, 247), (56, 61, 63, 65, 248))):
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
    # tile hand-over of an even iteration: tile s42 + 1 must have landed in every wave's share before its
    # rows are read (slot 34 on); the stage of tile s42 - 2 (s47), which nobody reads any more, takes tile s42 + 2
    def mid(lab):
        return ["s_add_i32 s66, s42, 1",
                "s_cmp_ge_i32 s66, s41",
                f"s_cbranch_scc1 Lskip_{lab}",
                "s_waitcnt vmcnt(0)",
                "s_barrier",
                "s_add_i32 s66, s42, 2",
                "s_cmp_ge_i32 s66, s41",
                f"s_cbranch_scc1 Lskip_{lab}"] + issue_tile() + [f"Lskip_{lab}:"]
    # ---- prologue: scalars, scores and delta - dP of block 0, ring entries of the first iteration -------
    sreg = lambda i: 40 + i if i < 26 else 70 + (i - 26)     # s66..s69 are temporaries
    pro = [f"v_readfirstlane_b32 s{sreg(i)}, v{160 + i}" for i in range(len(SCALARS))]
    rotate = ["s_mov_b32 s66, s44", "s_mov_b32 s44, s45", "s_mov_b32 s45, s46", "s_mov_b32 s46, s47", "s_mov_b32 s47, s66"]
    # Tiles of the workgroup's window that lie before this wave's own window (s70 = its first tile): no arithmetic,
    # only the wave's part in the hand-over of every tile (its share of the loads, the barrier).  The same after
    # the wave's last tile (s71 = one past it).
    pro += [L("Lin") + ":",
            "s_cmp_ge_i32 s42, s70",
            "s_cbranch_scc1 " + L("Lin_done")] + mid(L("i")) + [
            "s_add_i32 s42, s42, 1"] + rotate + [
            "s_branch " + L("Lin"),
            L("Lin_done") + ":",
            "s_lshl_b32 s43, s42, 6"]
    g.out = pro
    for half in range(2):          # row fragments 4*half .. 4*half+3 of K and V: 8 ring entries at a time
        for x in range(8):
            gi, isv = 4 * half + (x >> 1), x & 1
            g.lds(("pro", half, x), f"ds_read_b128 {RG(x)}, v{AK + gi} offset:{isv * TILE_B}")
        for x in range(8):
            gi, isv = 4 * half + (x >> 1), x & 1
            g.need(("pro", half, x))
            for qb in range(2):
                if isv:
                    c = DINIT(qb) if gi == 0 else DP(0, qb)
                    g.emit(f"{g.mfma} {DP(0, qb)}, {RG(x)}, {GF(qb, gi)}, {c}")
                else:
                    c = "0" if gi == 0 else S(0, qb)
                    g.emit(f"{g.mfma} {S(0, qb)}, {RG(x)}, {QF(qb, gi)}, {c}")
        g.emit("s_nop 7")
    # ring entries of fragments 0..6 of iteration 0 (same ring positions as in any iteration)
    for f in range(PF):
        g.fetch(NFRAG + f, f, 0)
    text = g.out
    k = 1
    first = g.body(k, 0, L("f"), with_dq=False, mid=mid(L("f")))
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
             "s_cmp_ge_i32 s42, s71",
             "s_cbranch_scc1 " + L("Lend")]
    text += b0
    text += ["s_branch " + L("Lloop"),
             L("Lend") + ":"]
    # ---- drain: dQ^T -= K^T (-dS) of the last block (odd parity: block 1 of the tile the K^T addresses point at)
    text.append("s_waitcnt lgkmcnt(0)")
    for x in range(8):
        half, m = x // 4, x % 4
        off = BLK_B + half * 16 * ROWB
        text.append(f"ds_read_b64_tr_b16 {RG(x, 0, 2)}, v{ATR + m} offset:{off}")
        text.append(f"ds_read_b64_tr_b16 {RG(x, 2, 2)}, v{ATR + 4 + m} offset:{off}")
    for x in range(8):
        half, m = x // 4, x % 4
        n = 2 * (7 - x)
        text.append(f"s_waitcnt lgkmcnt({min(n, 15)})")
        for qb in range(2):
            text.append(f"{g.mfma} {DQ(qb, m)}, {RG(x)}, {DSB(1, qb, half)}, {DQ(qb, m)}")
    text += ["s_nop 15", "s_nop 15", "s_nop 15", "s_nop 15"]
    # tiles of the workgroup's window after this wave's last one
    text += [L("Lfin") + ":",
             "s_cmp_ge_i32 s42, s41",
             "s_cbranch_scc1 " + L("Lout")] + mid(L("x")) + [
             "s_add_i32 s42, s42, 1"] + rotate + [
             "s_branch " + L("Lfin")]
    text += g.tails
    text.append(L("Lout") + ":")
    name = f"SA_DQ3_128_{dt.upper()}"
    return f"#define {name} \\\n" + " \\\n".join('    "' + ln + '\\n"' for ln in text) + "\n"


def main():
    print("// Generated by gen_dq3_asm.py -- do not edit.  Prologue, main loop and drain of dq3_kernel.")
    print("#define SA_DQ3_NUM_SCALARS %d" % len(SCALARS))
    for i, nm in enumerate(SCALARS):
        print(f"#define SA_DQ3_SC_{nm.upper()} {i}")
    for dt in ("bf16", "f16"):
        print(generate(dt))


if __name__ == "__main__":
    main()
