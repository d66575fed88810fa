// Forward kernel: O = softmax_window(scale * Q K^T) V and the base-2 log-sum-exp.
//
// Replaces the reference's Triton kernel `_streaming_attn_fwd`
// (src/streaming_attention/kernel.py:196-430).  One workgroup owns TQ = 32*NW queries of
// one (batch, head); each wave owns 32 of them and each lane one query column, so the
// running max / sum and the [lo, hi) key window of a query are per-lane scalars.
// The workgroup visits only the key tiles that intersect the window of its queries
// (kernel.py:282-291); tiles that lie wholly inside every lane's window skip the mask.
#pragma once
#include "sa_common.h"

namespace sa {

template <typename T, int D, int NW, int TK>
__global__ __launch_bounds__(NW * 64) void fwd_kernel(const FwdParams p) {
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  constexpr int TQ = NW * 32, NT = NW * 64, KBN = TK / 32;
  constexpr int PITCH = G::PITCH, NF = G::NF, DB = G::DB;
  constexpr int TILE = TK * PITCH;  // elements per staged K or V tile
  constexpr float kRescaleGap = 8.0f;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);  // [stage][K|V][TK][PITCH]

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bh, qt;
  tile_coords(blockIdx.x, gridDim.x, p.n_tiles, bh, qt);
  const int hd = bh % p.H, b = bh / p.H;
  const int T_ = p.T, C = p.C, R = p.R;
  auto cdiv = [&](int x) { return div_by(x, p.cdiv); };   // x / C

  int L = T_;
  if (p.lens) {
    L = p.lens[(int64_t)b * p.lens_stride];
    L = L < 0 ? 0 : (L > T_ ? T_ : L);
  }
  const int q0 = qt * TQ;
  T* o_base = reinterpret_cast<T*>(p.o) + (int64_t)bh * T_ * D;
  float* lse_base = p.lse ? p.lse + (int64_t)bh * T_ : nullptr;
  const int q_end = q0 + TQ < T_ ? q0 + TQ : T_;

  if (q0 >= L) {  // whole tile is padding: the outputs there are defined as zero
    zero_rows<T, D, NT>(o_base, q0, q_end, tid);
    if (lse_base)
      for (int r = q0 + tid; r < q_end; r += NT) lse_base[r] = 0.0f;
    return;
  }

  // ---- per-lane query and its key window ------------------------------------------
  const int qrow = q0 + wave * 32 + c;
  const int qe = qrow < L ? qrow : L - 1;  // rows past L mimic the last valid row
  const int qchunk = cdiv(qe);
  const int lo = (qchunk > R ? qchunk - R : 0) * C;
  const int hi = (qchunk + 1) * C < L ? (qchunk + 1) * C : L;
  // the tightest window over the wave decides whether a tile needs masking at all
  const int wq_first = q0 + wave * 32 < L ? q0 + wave * 32 : L - 1;
  const int wq_last = q0 + wave * 32 + 31 < L ? q0 + wave * 32 + 31 : L - 1;
  const int hi_min = (cdiv(wq_first) + 1) * C < L ? (cdiv(wq_first) + 1) * C : L;
  const int lo_max = (cdiv(wq_last) > R ? cdiv(wq_last) - R : 0) * C;
  // union over the workgroup decides which tiles are visited
  const int gq_last = q0 + TQ - 1 < L ? q0 + TQ - 1 : L - 1;
  const int lo_wg = (cdiv(q0) > R ? cdiv(q0) - R : 0) * C;
  const int hi_wg = (cdiv(gq_last) + 1) * C < L ? (cdiv(gq_last) + 1) * C : L;
  const int kt0 = lo_wg / TK, kt1 = (hi_wg + TK - 1) / TK;

  const float sl2e = fabsf(p.scale_log2e);
  const bool neg = p.scale_log2e < 0.0f;

  // ---- Q fragments stay in registers for the whole key loop -------------------------
  Frag qf[NF];
  {
    const int qr = qrow < L ? qrow : L - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh +
                  (int64_t)qr * p.q_st;
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      qf[g] = *reinterpret_cast<const Frag*>(qp + (g * 2 + h) * E::VEC);
      if (neg) qf[g] = negate<T>(qf[g]);
    }
  }

  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh;

  f32x16 oacc[DB];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[m][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  Stager<T, D, TK, NT> sk, sv;
  sk.load(kbase, p.k_st, kt0 * TK, L - 1, tid);
  sv.load(vbase, p.v_st, kt0 * TK, L - 1, tid);
  sk.store(smem, tid);
  sv.store(smem + TILE, tid);
  wait_all_loads();
  __syncthreads();

  for (int t = kt0; t < kt1; ++t) {
    const int cur = (t - kt0) & 1;
    const T* Kt = smem + cur * 2 * TILE;
    const T* Vt = Kt + TILE;
    const bool more = t + 1 < kt1;
    if (more) {
      sk.load(kbase, p.k_st, (t + 1) * TK, L - 1, tid);
      sv.load(vbase, p.v_st, (t + 1) * TK, L - 1, tid);
    }
    const int k0 = t * TK;

    // S^T[key][q] = K Q^T
    f32x16 s[KBN];
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kb][i] = 0.0f;
    mma_rows<T, D>(s, Kt, 0, qf, lane);

    // Online softmax in base 2 on the raw scores: p = exp2(s*sl2e - m).  The two halves of
    // the wave hold disjoint keys of the same query, so only the max crosses lanes inside
    // the loop.  The reference point m moves only when the tile's max exceeds it by more
    // than kRescaleGap (p then stays below 2^kRescaleGap, harmless in fp32 and in the 16-bit
    // operand of the next product); most tiles therefore skip the rescale of O entirely.
    const bool interior = (k0 >= lo_max) && (k0 + TK <= hi_min);
    float mx = -INFINITY;
    if (interior) {
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
    } else {
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = k0 + kb * 32 + crow(i, h);
          mx = (key >= lo && key < hi) ? fmaxf(mx, s[kb][i]) : mx;
        }
    }
    mx = half_max(mx) * sl2e;                 // -inf when no key of this tile is visible
    const bool move = mx > m_run + kRescaleGap;   // false for mx = -inf or NaN
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float m_new = move ? mx : m_run;
      // m_run = -inf gives alpha = 0 (the accumulators are 0 then); lanes that stay put get 1
      const float alpha = move ? fast_exp2(m_run - mx) : 1.0f;
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int m = 0; m < DB; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[m][i] *= alpha;
    }
    // a query that has seen no key yet keeps m_run = -inf; use 0 there so that exp2 gets a
    // finite argument (its keys in this tile are all masked, so p is forced to 0 below)
    const float m_use = m_run == -INFINITY ? 0.0f : m_run;
    float rs = 0.0f;
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = fast_exp2(__builtin_fmaf(s[kb][i], sl2e, -m_use));
        s[kb][i] = e;
      }
    if (!interior) {
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = k0 + kb * 32 + crow(i, h);
          s[kb][i] = (key >= lo && key < hi) ? s[kb][i] : 0.0f;
        }
    }
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) rs += s[kb][i];
    l_run += rs;

    // O^T[d][q] += V^T P^T
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb) mma_tr<T, D>(oacc, Vt, kb, s[kb], lane);

    if (more) {
      T* nxt = smem + (cur ^ 1) * 2 * TILE;
      sk.store(nxt, tid);
      sv.store(nxt + TILE, tid);
    }
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------------
  const float l_tot = half_sum(l_run);
  const bool valid = qrow < L;
  if (qrow < T_) {
    const float inv = valid ? 1.0f / l_tot : 0.0f;
    if (!valid) {
#pragma unroll
      for (int m = 0; m < DB; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[m][i] = 0.0f;
    }
    store_acc_T<T, D, DB>(o_base + (int64_t)qrow * D, oacc, inv, h);
    if (lse_base && h == 0) lse_base[qrow] = valid ? m_run + __builtin_amdgcn_logf(l_tot) : 0.0f;
  }
}

// Forward kernel for 16-bit elements with swizzled tiles (D = 64, 128 or 256; at 256 only with 4 waves, one per SIMD, which then has all 512 registers).
//
// Same algorithm as fwd_kernel, different resource balance: each wave owns QB blocks of 32
// queries, so every K / V fragment fetched from LDS feeds QB MFMAs (the transposing V reads
// are 8-byte LDS reads and would otherwise cap the second product well below the MFMA
// rate); K and V tiles are brought in by asynchronous global->LDS copies into a ring of NST
// stages, NST-1 tiles ahead of the compute, with one barrier per key tile.
// SHORT selects the form for short windows (a handful of key tiles per workgroup): work is skipped
// and masks are decided per 32-key block instead of per tile, and a wave's first tile goes straight
// to the search for its maximum.  Long windows run the plain form, whose loop is a few per cent
// tighter (fewer registers, no per-block tests).
template <typename T, int D, int QB, int NW, int TK, int NST, bool SHORT>
__global__ __launch_bounds__(NW * 64) void fwd2_kernel(const FwdParams p) {
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(G::SWZ && NST >= 2 && (NST - 2) * 2 * AsyncTile<T, D, TK, NW>::PER_WAVE < 64, "swizzled 16-bit tiles; the loads of NST-2 tiles fit the load counter");
  constexpr int WQ = QB * 32, TQ = NW * WQ, NT = NW * 64, KBN = TK / 32;
  constexpr int NF = G::NF, DB = G::DB;
  constexpr int TILE = TK * D;            // elements per K or V tile
  constexpr int STAGE = 2 * TILE;
  constexpr float kRescaleGap = 8.0f;
  constexpr float kSumLimit = 256.0f;
  using Loader = AsyncTile<T, D, TK, NW>;
  constexpr int LPT = 2 * Loader::PER_WAVE;   // async loads per wave per stage (K and V)

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);  // [stage][K|V][TK][D]

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bh, qt;
  tile_coords(blockIdx.x, gridDim.x, p.n_tiles, bh, qt, SHORT ? growing_tiles(p.C, p.R, p.T, NW * QB * 32) : 0);
  const int hd = bh % p.H, b = bh / p.H;
  const int T_ = p.T, C = p.C, R = p.R;
  auto cdiv = [&](int x) { return div_by(x, p.cdiv); };   // x / C

  int L = T_;
  if (p.lens) {
    L = p.lens[(int64_t)b * p.lens_stride];
    L = L < 0 ? 0 : (L > T_ ? T_ : L);
  }
  const int q0 = qt * TQ;
  T* o_base = reinterpret_cast<T*>(p.o) + (int64_t)bh * T_ * D;
  float* lse_base = p.lse ? p.lse + (int64_t)bh * T_ : nullptr;
  const int q_end = q0 + TQ < T_ ? q0 + TQ : T_;
  if (q0 >= L) {
    zero_rows<T, D, NT>(o_base, q0, q_end, tid);
    if (lse_base)
      for (int r = q0 + tid; r < q_end; r += NT) lse_base[r] = 0.0f;
    return;
  }

  // ---- per-lane queries (one per owned block) and their key windows -----------------
  int qrow[QB], lo[QB], hi[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    qrow[qb] = q0 + wave * WQ + qb * 32 + c;
    const int qe = qrow[qb] < L ? qrow[qb] : L - 1;
    const int qchunk = cdiv(qe);
    lo[qb] = (qchunk > R ? qchunk - R : 0) * C;
    hi[qb] = (qchunk + 1) * C < L ? (qchunk + 1) * C : L;
  }
  const int wq_first = q0 + wave * WQ < L ? q0 + wave * WQ : L - 1;
  const int wq_last = q0 + wave * WQ + WQ - 1 < L ? q0 + wave * WQ + WQ - 1 : L - 1;
  const int hi_min = (cdiv(wq_first) + 1) * C < L ? (cdiv(wq_first) + 1) * C : L;
  const int lo_max = (cdiv(wq_last) > R ? cdiv(wq_last) - R : 0) * C;
  // keys any query of this wave can see; a wave whose queries are all padding sees none
  const bool wave_live = q0 + wave * WQ < L;
  const int lo_min = (cdiv(wq_first) > R ? cdiv(wq_first) - R : 0) * C;
  const int hi_max = !wave_live ? 0 : ((cdiv(wq_last) + 1) * C < L ? (cdiv(wq_last) + 1) * C : L);
  const int gq_last = q0 + TQ - 1 < L ? q0 + TQ - 1 : L - 1;
  const int lo_wg = (cdiv(q0) > R ? cdiv(q0) - R : 0) * C;
  const int hi_wg = (cdiv(gq_last) + 1) * C < L ? (cdiv(gq_last) + 1) * C : L;
  const int kt0 = lo_wg / TK, kt1 = (hi_wg + TK - 1) / TK;

  // never exactly 0, so that a masked score of -inf stays -inf after scaling
  const float sl2e = fmaxf(fabsf(p.scale_log2e), 1e-30f);
  const bool neg = p.scale_log2e < 0.0f;

  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh;
  Loader ldk, ldv;
  ldk.init(kbase, p.k_st, kt0 * TK, L - 1, wave, lane);
  ldv.init(vbase, p.v_st, kt0 * TK, L - 1, wave, lane);
  auto issue_tile = [&](int t) {   // tiles are issued in ascending order
    T* st = smem + ((t - kt0) % NST) * STAGE;
    ldk.issue(st, wave);
    ldv.issue(st + TILE, wave);
    ldk.advance();
    ldv.advance();
  };
  // prologue: NST-1 tiles in flight
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (kt0 + i < kt1) issue_tile(kt0 + i);

  Frag qf[QB][NF];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int qr = qrow[qb] < L ? qrow[qb] : L - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh +
                  (int64_t)qr * p.q_st;
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      qf[qb][g] = *reinterpret_cast<const Frag*>(qp + (g * 2 + h) * E::VEC);
      if (neg) qf[qb][g] = negate<T>(qf[qb][g]);
    }
  }

  f32x16 oacc[QB][DB];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.0f;
#pragma unroll
    for (int m = 0; m < DB; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[qb][m][i] = 0.0f;
  }
  wait_all_loads();   // Q fragments (and, as loads complete in order, the first tiles)

  for (int t = kt0; t < kt1; ++t) {
    // tile t has landed once at most the loads of the younger tiles are outstanding: NST-2 of them, fewer
    // near the end of the window
    wait_tiles<LPT, NST - 2>(kt1 - 1 - t);
    __syncthreads();   // every wave's share is visible; stage (t-1) % NST is free again
    if (t + NST - 1 < kt1) issue_tile(t + NST - 1);

    const T* Kt = smem + ((t - kt0) % NST) * STAGE;
    const T* Vt = Kt + TILE;
    const int k0 = t * TK;
    // the workgroup's key range is the union over its waves; skip what this wave cannot see
    if (k0 + TK <= lo_min || k0 >= hi_max) continue;

    // S^T[key][q] = K Q^T for the QB query blocks
    f32x16 s[QB][KBN];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[qb][kb][i] = 0.0f;
    // Short windows end inside a tile: a 32-key block that no query of this wave can see is left
    // out of both products and of the arithmetic, one that every query sees in full needs no mask.
    bool live[KBN], inside[KBN], all_live = true;
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb) {
      const int kb0 = SHORT ? k0 + kb * 32 : k0, kbn = SHORT ? 32 : TK;   // the block, or the whole tile
      live[kb] = !SHORT || (kb0 + kbn > lo_min && kb0 < hi_max);
      inside[kb] = kb0 >= lo_max && kb0 + kbn <= hi_min;
      all_live = all_live && live[kb];
    }
    if (all_live) {
      mma_rows_n<T, D>(s, Kt, 0, qf, lane);
    } else {
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb) {
        if (live[kb]) {
          f32x16 one[QB][1];
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) one[qb][0] = s[qb][kb];
          mma_rows_n<T, D>(one, Kt, kb * 32, qf, lane);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) s[qb][kb] = one[qb][0];
        } else {
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[qb][kb][i] = -INFINITY;
        }
      }
    }

    Frag pb[QB][KBN][2];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      // keys outside [lo, hi) score -inf (whatever the product gave, NaN from padding included)
#pragma unroll
      for (int kb = 0; kb < KBN; ++kb) {
        if (live[kb] && !inside[kb]) {
          const uint32_t rm = row_mask(lo[qb] - (k0 + kb * 32), hi[qb] - (k0 + kb * 32), h);
#pragma unroll
          for (int i = 0; i < 16; ++i) s[qb][kb][i] = keep_or_neg_inf(s[qb][kb][i], keep_bits(rm, i));
        }
      }
      // Probabilities relative to the running maximum as it stands.  The maximum is only looked
      // for when they show that it has been left behind: a tile whose probabilities of one half
      // row add up to at most kSumLimit holds no score more than log2(kSumLimit) above it, which
      // is harmless in fp32 and in the 16-bit operand (the result does not depend on which
      // maximum is subtracted).  Lanes without a maximum yet always look for one.
      float rs[2];
      auto probabilities = [&](float m_use) {
        rs[0] = rs[1] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < KBN; ++kb) {
          if (!live[kb]) continue;   // never multiplied
          f32x16 pr;
#pragma unroll
          for (int i = 0; i < 16; ++i) pr[i] = fast_exp2(__builtin_fmaf(s[qb][kb][i], sl2e, -m_use));
          pack_c<T>(pb[qb][kb], pr);
#ifdef SA_FWD2_DOT_SUMS
          rs[0] = sum_frag(pb[qb][kb][0], rs[0]);
          rs[1] = sum_frag(pb[qb][kb][1], rs[1]);
#else
          // plain float32 additions in two chains: the two-element dot products that could add up the rounded
          // values at half the instruction count stall against the MFMAs in flight
#pragma unroll
          for (int i = 0; i < 16; i += 2) rs[0] += pr[i], rs[1] += pr[i + 1];
#endif
        }
      };
      // A wave none of whose lanes has a maximum yet (its first visible tile) goes straight to the
      // search: the speculative pass would be thrown away, and short windows are all first tiles.
      const bool fresh = SHORT && __builtin_amdgcn_ballot_w64(m_run[qb] != -INFINITY) == 0;
      bool search = fresh;
      if (!fresh) {
        probabilities(m_run[qb] == -INFINITY ? 0.0f : m_run[qb]);
        const bool behind = !(rs[0] + rs[1] <= kSumLimit) || m_run[qb] == -INFINITY;   // true for NaN too
        search = __builtin_amdgcn_ballot_w64(behind) != 0;
      }
      if (search) {
        float mx = -INFINITY;
        {
          float mk[KBN];   // one chain per key block, so that consecutive instructions are independent
#pragma unroll
          for (int kb = 0; kb < KBN; ++kb) mk[kb] = -INFINITY;
#pragma unroll
          for (int i = 0; i < 16; i += 2)
#pragma unroll
            for (int kb = 0; kb < KBN; ++kb) mk[kb] = fast_max3(mk[kb], s[qb][kb][i], s[qb][kb][i + 1]);
#pragma unroll
          for (int kb = 0; kb < KBN; ++kb) mx = fast_max(mx, mk[kb]);
        }
        mx = half_max(mx) * sl2e;
        const bool move = mx > m_run[qb] + kRescaleGap;   // false for mx = -inf or NaN
        if (fresh || __builtin_amdgcn_ballot_w64(move) != 0) {
          const float alpha = move ? fast_exp2(m_run[qb] - mx) : 1.0f;
          m_run[qb] = move ? mx : m_run[qb];
          l_run[qb] *= alpha;
          if (!fresh) {   // a fresh wave has accumulated nothing yet
#pragma unroll
            for (int m = 0; m < DB; ++m)
#pragma unroll
              for (int i = 0; i < 16; ++i) oacc[qb][m][i] *= alpha;
          }
          probabilities(m_run[qb] == -INFINITY ? 0.0f : m_run[qb]);
        }
      }
      l_run[qb] += rs[0] + rs[1];
    }

    // O^T[d][q] += V^T P^T
#pragma unroll
    for (int kb = 0; kb < KBN; ++kb) {
      if (!live[kb]) continue;
      Frag bq[QB][2];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) bq[qb][0] = pb[qb][kb][0], bq[qb][1] = pb[qb][kb][1];
      mma_tr_n<T, D>(oacc, Vt, kb, bq, lane);
    }
  }

  // ---- epilogue --------------------------------------------------------------------
  __syncthreads();   // the row patches lie over the tile stages
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = half_sum(l_run[qb]);
    const bool valid = qrow[qb] < L;
    const float inv = valid ? 1.0f / l_tot : 0.0f;
    if (!valid) {
#pragma unroll
      for (int m = 0; m < DB; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[qb][m][i] = 0.0f;
    }
    T* patch = smem + wave * RowPatch<T, D>::ELEMS;
    const int row0 = q0 + wave * WQ + qb * 32;
    store_rows_coalesced<T, D, DB>(patch, o_base + (int64_t)row0 * D, T_ - row0, oacc[qb], inv, lane);
    if (lse_base && h == 0 && qrow[qb] < T_)
      lse_base[qrow[qb]] = valid ? m_run[qb] + __builtin_amdgcn_logf(l_tot) : 0.0f;
  }
}

}  // namespace sa
