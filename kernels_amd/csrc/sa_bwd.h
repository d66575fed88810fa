// Backward kernels.
//
//   delta_kernel  delta[b,h,t] = sum_d O*dO      replaces `_streaming_attn_bwd_precompute`
//                                                (src/streaming_attention/kernel.py:433-514)
//   dq_kernel     dQ = scale * dS K              replaces `_streaming_attn_bwd_dq(_inner)`
//                                                (kernel.py:638-773, 940-1023)
//   dkdv_kernel   dV = P^T dO, dK = scale dS^T Q replaces `_streaming_attn_bwd_dkdv(_inner)`
//                                                (kernel.py:776-937, 1026-1129)
// with P = exp2(scale*log2e * Q K^T - LSE), dP = dO V^T, dS = P o (dP - delta).
//
// dq_kernel mirrors the forward: a lane owns a query column, so LSE, delta and the key
// window are per-lane scalars.  dkdv_kernel is its transpose: a workgroup owns 32*NW keys,
// a lane owns one key column with its query window [qlo, qhi), and the loop runs over the
// query tiles that can see those keys (kernel.py:1046-1054).  Both kernels write every
// element of their outputs, zeros included, so the caller does not pre-clear them.
#pragma once
#include <type_traits>
#include "sa_common.h"

namespace sa {

template <typename T, int D>
__global__ __launch_bounds__(256) void delta_kernel(const DeltaParams p) {
  using E = Elem<T>;
  using Frag = typename E::Frag;
  constexpr int LPR = D / E::VEC;      // lanes per row, a power of two <= 64
  constexpr int RPB = 256 / LPR;       // rows per block
  const int tid = threadIdx.x;
  const int sub = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + tid / LPR;   // flattened (b,h,t)
  const int64_t total = (int64_t)p.B * p.H * p.T;
  float acc = 0.0f;
  if (row < total) {
    const int t = (int)(row % p.T);
    const int64_t bh = row / p.T;
    const int hd = (int)(bh % p.H);
    const int64_t b = bh / p.H;
    const T* op = reinterpret_cast<const T*>(p.o) + b * p.o_sb + hd * p.o_sh + (int64_t)t * p.o_st;
    const T* gp = reinterpret_cast<const T*>(p.d_o) + b * p.do_sb + hd * p.do_sh + (int64_t)t * p.do_st;
    const Frag a = *reinterpret_cast<const Frag*>(op + sub * E::VEC);
    const Frag g = *reinterpret_cast<const Frag*>(gp + sub * E::VEC);
#pragma unroll
    for (int e = 0; e < E::VEC; ++e) acc += (float)a[e] * (float)g[e];
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (row < total && sub == 0) p.delta[row] = acc;
}

template <typename T, int D, int NW, int TK>
__global__ __launch_bounds__(NW * 64) void dq_kernel(const BwdParams p) {
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  constexpr int TQ = NW * 32, NT = NW * 64, KBN = TK / 32;
  constexpr int PITCH = G::PITCH, NF = G::NF, DB = G::DB;
  constexpr int TILE = TK * PITCH;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);

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
  T* dq_base = reinterpret_cast<T*>(p.dq) + (int64_t)bh * T_ * D;
  const int q_end = q0 + TQ < T_ ? q0 + TQ : T_;
  if (q0 >= L) {
    zero_rows<T, D, NT>(dq_base, q0, q_end, tid);
    return;
  }

  const int qrow = q0 + wave * 32 + c;
  const int qe = qrow < L ? qrow : L - 1;
  const int qchunk = cdiv(qe);
  const int lo = (qchunk > R ? qchunk - R : 0) * C;
  const int hi = (qchunk + 1) * C < L ? (qchunk + 1) * C : L;
  const int wq_first = q0 + wave * 32 < L ? q0 + wave * 32 : L - 1;
  const int wq_last = q0 + wave * 32 + 31 < L ? q0 + wave * 32 + 31 : L - 1;
  const int hi_min = (cdiv(wq_first) + 1) * C < L ? (cdiv(wq_first) + 1) * C : L;
  const int lo_max = (cdiv(wq_last) > R ? cdiv(wq_last) - R : 0) * C;
  const int gq_last = q0 + TQ - 1 < L ? q0 + TQ - 1 : L - 1;
  const int lo_wg = (cdiv(q0) > R ? cdiv(q0) - R : 0) * C;
  const int hi_wg = (cdiv(gq_last) + 1) * C < L ? (cdiv(gq_last) + 1) * C : L;
  const int kt0 = lo_wg / TK, kt1 = (hi_wg + TK - 1) / TK;

  const float sl2e = fabsf(p.scale_log2e);
  const bool neg = p.scale_log2e < 0.0f;

  Frag qf[NF], gf[NF];
  float lse_q, delta_q;
  {
    const int qr = qrow < L ? qrow : L - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh +
                  (int64_t)qr * p.q_st;
    const T* gp = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.do_sb + (int64_t)hd * p.do_sh +
                  (int64_t)qr * p.do_st;
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      qf[g] = *reinterpret_cast<const Frag*>(qp + (g * 2 + h) * E::VEC);
      if (neg) qf[g] = negate<T>(qf[g]);
      gf[g] = *reinterpret_cast<const Frag*>(gp + (g * 2 + h) * E::VEC);
    }
    // rows past L get P = exp2(-inf) = 0
    lse_q = qrow < L ? p.lse[(int64_t)bh * T_ + qr] : INFINITY;
    delta_q = p.delta[(int64_t)bh * T_ + qr];
  }

  const T* kbase = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh;
  const T* vbase = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh;

  f32x16 acc[DB];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;

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
    const bool interior = (k0 >= lo_max) && (k0 + TK <= hi_min);

#pragma unroll
    for (int kb = 0; kb < KBN; ++kb) {
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.0f, dp[i] = 0.0f;
      {
        f32x16 (&s1)[1] = reinterpret_cast<f32x16(&)[1]>(s);
        f32x16 (&dp1)[1] = reinterpret_cast<f32x16(&)[1]>(dp);
        mma_rows<T, D>(s1, Kt, kb * 32, qf, lane);
        mma_rows<T, D>(dp1, Vt, kb * 32, gf, lane);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pr = fast_exp2(s[i] * sl2e - lse_q);
        s[i] = pr * (dp[i] - delta_q);
      }
      if (!interior) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = k0 + kb * 32 + crow(i, h);
          s[i] = (key < lo || key >= hi) ? 0.0f : s[i];
        }
      }
      // dQ^T[d][q] += K^T dS^T
      mma_tr<T, D>(acc, Kt, kb, s, lane);
    }

    if (more) {
      T* nxt = smem + (cur ^ 1) * 2 * TILE;
      sk.store(nxt, tid);
      sv.store(nxt + TILE, tid);
    }
    __syncthreads();
  }

  if (qrow < T_) {
    if (qrow >= L) {
#pragma unroll
      for (int m = 0; m < DB; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
    }
    store_acc_T<T, D, DB>(dq_base + (int64_t)qrow * D, acc, p.scale, h);
  }
}

// PASS selects what one launch produces: 0 both gradients, 1 dV only, 2 dK only.  Two float32 accumulators of 32 x 256
// and the resident K and V rows are 512 registers per lane before any operand, so float32 at head dimension 256 runs
// as two launches: the dV pass needs neither V nor dP and fits without spills; the dK pass has one accumulator and
// stages the next tile in two steps (Q while the first products run, dO during the rest).  It still spills some values
// around the products; the form that staged both tensors at once was miscompiled (the spill code of the first tile
// dropped a register copy), which the head-dimension parity tests catch.
template <typename T, int D, int NW, int TQ, int PASS = 0>
__global__ __launch_bounds__(NW * 64) void dkdv_kernel(const BwdParams p) {
  constexpr bool WITH_DV = PASS != 2, WITH_DK = PASS != 1;
  constexpr bool HALVES = PASS == 2;   // stage Q and dO one after the other
  static_assert(!HALVES || TQ == 32, "the two staging halves bracket a single 32-query block");
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  constexpr int TKB = NW * 32, NT = NW * 64, QBN = TQ / 32;
  constexpr int PITCH = G::PITCH, NF = G::NF, DB = G::DB;
  constexpr int TILE = TQ * PITCH;
  // stage layout: [Q tile][dO tile][lse TQ floats][delta TQ floats]
  constexpr int STAGE_BYTES = 2 * TILE * (int)sizeof(T) + 2 * TQ * (int)sizeof(float);

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bh, kt;
  tile_coords(blockIdx.x, gridDim.x, p.n_tiles, bh, kt);
  const int hd = bh % p.H, b = bh / p.H;
  const int T_ = p.T, C = p.C, R = p.R;
  auto cdiv = [&](int x) { return div_by(x, p.cdiv); };   // x / C

  int L = T_;
  if (p.lens) {
    L = p.lens[(int64_t)b * p.lens_stride];
    L = L < 0 ? 0 : (L > T_ ? T_ : L);
  }
  const int k0 = kt * TKB;
  T* dk_base = reinterpret_cast<T*>(p.dk) + (int64_t)bh * T_ * D;
  T* dv_base = reinterpret_cast<T*>(p.dv) + (int64_t)bh * T_ * D;
  const int k_end = k0 + TKB < T_ ? k0 + TKB : T_;
  if (k0 >= L) {
    if constexpr (WITH_DK) zero_rows<T, D, NT>(dk_base, k0, k_end, tid);
    if constexpr (WITH_DV) zero_rows<T, D, NT>(dv_base, k0, k_end, tid);
    return;
  }

  // query window [qlo, qhi) of a key: its own chunk and the R chunks after it, below L
  auto win_lo = [&](int key) { return (cdiv(key)) * C; };
  auto win_hi = [&](int key) {
    const int64_t e = ((int64_t)(cdiv(key)) + R + 1) * (int64_t)C;
    return e < (int64_t)L ? (int)e : L;
  };
  const int krow = k0 + wave * 32 + c;
  const int ke = krow < L ? krow : L - 1;  // keys past L mimic the last valid key
  const int qlo = win_lo(ke), qhi = win_hi(ke);
  const int wk_first = k0 + wave * 32 < L ? k0 + wave * 32 : L - 1;
  const int wk_last = k0 + wave * 32 + 31 < L ? k0 + wave * 32 + 31 : L - 1;
  const int qhi_min = win_hi(wk_first), qlo_max = win_lo(wk_last);
  const int gk_last = k0 + TKB - 1 < L ? k0 + TKB - 1 : L - 1;
  const int qt0 = win_lo(k0) / TQ, qt1 = (win_hi(gk_last) + TQ - 1) / TQ;

  const float sl2e = fabsf(p.scale_log2e);
  const bool neg = p.scale_log2e < 0.0f;

  Frag kf[NF], vf[WITH_DK ? NF : 1];
  {
    const int kr = krow < L ? krow : L - 1;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh +
                  (int64_t)kr * p.k_st;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh +
                  (int64_t)kr * p.v_st;
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      kf[g] = *reinterpret_cast<const Frag*>(kp + (g * 2 + h) * E::VEC);
      if (neg) kf[g] = negate<T>(kf[g]);
      if constexpr (WITH_DK) vf[g] = *reinterpret_cast<const Frag*>(vp + (g * 2 + h) * E::VEC);
    }
  }

  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh;
  const T* gbase = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.do_sb + (int64_t)hd * p.do_sh;
  const float* lse_base = p.lse + (int64_t)bh * T_;
  const float* delta_base = p.delta + (int64_t)bh * T_;

  f32x16 dk[WITH_DK ? DB : 1], dv[WITH_DV ? DB : 1];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if constexpr (WITH_DK) dk[m][i] = 0.0f;
      if constexpr (WITH_DV) dv[m][i] = 0.0f;
    }

  Stager<T, D, TQ, NT> sq, sg;
  float r_lse = 0.0f, r_delta = 0.0f;   // thread tid < TQ stages row tid of the tile
  auto load_rows = [&](int row0) {
    if (tid < TQ) {
      int r = row0 + tid;
      r = r < L ? r : L - 1;
      r_lse = lse_base[r];
      r_delta = delta_base[r];
    }
  };
  auto stage_ptr = [&](int s) { return smem_raw + s * STAGE_BYTES; };
  auto store_stage = [&](int s) {
    T* qd = reinterpret_cast<T*>(stage_ptr(s));
    if constexpr (!HALVES) sq.store(qd, tid);
    sg.store(qd + TILE, tid);
    if (tid < TQ) {
      float* f = reinterpret_cast<float*>(stage_ptr(s) + 2 * TILE * sizeof(T));
      f[tid] = r_lse;
      f[TQ + tid] = r_delta;
    }
  };
  static_assert(TQ <= NW * 64, "one thread per staged row");

  sq.load(qbase, p.q_st, qt0 * TQ, L - 1, tid);
  if constexpr (HALVES) sq.store(reinterpret_cast<T*>(stage_ptr(0)), tid);
  sg.load(gbase, p.do_st, qt0 * TQ, L - 1, tid);
  load_rows(qt0 * TQ);
  store_stage(0);
  wait_all_loads();
  __syncthreads();

  for (int t = qt0; t < qt1; ++t) {
    const int cur = (t - qt0) & 1;
    const T* Qt = reinterpret_cast<const T*>(stage_ptr(cur));
    const T* Gt = Qt + TILE;
    const float* lse_t = reinterpret_cast<const float*>(stage_ptr(cur) + 2 * TILE * sizeof(T));
    const float* delta_t = lse_t + TQ;
    const bool more = t + 1 < qt1;
    if (more) {
      sq.load(qbase, p.q_st, (t + 1) * TQ, L - 1, tid);
      if constexpr (!HALVES) sg.load(gbase, p.do_st, (t + 1) * TQ, L - 1, tid);
      load_rows((t + 1) * TQ);
    }
    const int qs = t * TQ;
    const bool interior = (qs >= qlo_max) && (qs + TQ <= qhi_min);

#pragma unroll
    for (int qb = 0; qb < QBN; ++qb) {
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.0f, dp[i] = 0.0f;
      // S[q][key] = Q K^T, dP[q][key] = dO V^T
      {
        f32x16 (&s1)[1] = reinterpret_cast<f32x16(&)[1]>(s);
        f32x16 (&dp1)[1] = reinterpret_cast<f32x16(&)[1]>(dp);
        mma_rows<T, D>(s1, Qt, qb * 32, kf, lane);
        if constexpr (WITH_DK) mma_rows<T, D>(dp1, Gt, qb * 32, vf, lane);
      }
      if constexpr (HALVES) {
        // the other stage has had no reader since the last barrier: Q goes there now, dO takes over the registers
        sched_fence();   // the loads below must not be moved up into the products
        if (more) {
          sq.store(reinterpret_cast<T*>(stage_ptr(cur ^ 1)), tid);
          sg.load(gbase, p.do_st, (t + 1) * TQ, L - 1, tid);
        }
        sched_fence();
      }
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_t + qb * 32 + 8 * g4 + 4 * h);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_t + qb * 32 + 8 * g4 + 4 * h);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * g4 + e;
          const float pr = fast_exp2(s[i] * sl2e - l4[e]);
          s[i] = pr;
          dp[i] = pr * (dp[i] - d4[e]);
        }
      }
      if (!interior) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int qr = qs + qb * 32 + crow(i, h);
          const bool ok = qr >= qlo && qr < qhi;
          s[i] = ok ? s[i] : 0.0f;
          dp[i] = ok ? dp[i] : 0.0f;
        }
      }
      // dV^T[d][key] += dO^T P,  dK^T[d][key] += Q^T dS
      if constexpr (WITH_DV) mma_tr<T, D>(dv, Gt, qb, s, lane);
      if constexpr (WITH_DK) mma_tr<T, D>(dk, Qt, qb, dp, lane);
    }

    if (more) store_stage(cur ^ 1);
    __syncthreads();
  }

  if (krow < T_) {
    if (krow >= L) {
#pragma unroll
      for (int m = 0; m < DB; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if constexpr (WITH_DK) dk[m][i] = 0.0f;
          if constexpr (WITH_DV) dv[m][i] = 0.0f;
        }
    }
    if constexpr (WITH_DK) store_acc_T<T, D, DB>(dk_base + (int64_t)krow * D, dk, p.scale, h);
    if constexpr (WITH_DV) store_acc_T<T, D, DB>(dv_base + (int64_t)krow * D, dv, 1.0f, h);
  }
}

// ---------------------------------------------------------------------------------------
// Variants for 16-bit elements with swizzled tiles (D = 64, 128 or 256): tiles arrive by
// asynchronous global->LDS copies into a ring of NST stages, one barrier per tile.
// ---------------------------------------------------------------------------------------

template <typename T, int D, int NW, int TK, int NST>
__global__ __launch_bounds__(NW * 64) void dq2_kernel(const BwdParams p) {
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(G::SWZ && (NST == 2 || NST == 3), "swizzled 16-bit tiles, 2 or 3 stages");
  constexpr int TQ = NW * 32, NT = NW * 64, KBN = TK / 32;
  constexpr int NF = G::NF, DB = G::DB;
  constexpr int TILE = TK * D, STAGE = 2 * TILE;
  using Loader = AsyncTile<T, D, TK, NW>;
  constexpr int LPT = 2 * Loader::PER_WAVE;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bh, qt;
  tile_coords(blockIdx.x, gridDim.x, p.n_tiles, bh, qt, growing_tiles(p.C, p.R, p.T, NW * 32));
  const int hd = bh % p.H, b = bh / p.H;
  const int T_ = p.T, C = p.C, R = p.R;
  auto cdiv = [&](int x) { return div_by(x, p.cdiv); };   // x / C

  int L = T_;
  if (p.lens) {
    L = p.lens[(int64_t)b * p.lens_stride];
    L = L < 0 ? 0 : (L > T_ ? T_ : L);
  }
  const int q0 = qt * TQ;
  T* dq_base = reinterpret_cast<T*>(p.dq) + (int64_t)bh * T_ * D;
  const int q_end = q0 + TQ < T_ ? q0 + TQ : T_;
  if (q0 >= L) {
    zero_rows<T, D, NT>(dq_base, q0, q_end, tid);
    if (p.delta_out)
      for (int r = q0 + tid; r < q_end; r += NT) p.delta_out[(int64_t)bh * T_ + r] = 0.0f;
    return;
  }

  const int qrow = q0 + wave * 32 + c;
  const int qe = qrow < L ? qrow : L - 1;
  const int qchunk = cdiv(qe);
  const int lo = (qchunk > R ? qchunk - R : 0) * C;
  const int hi = (qchunk + 1) * C < L ? (qchunk + 1) * C : L;
  const int wq_first = q0 + wave * 32 < L ? q0 + wave * 32 : L - 1;
  const int wq_last = q0 + wave * 32 + 31 < L ? q0 + wave * 32 + 31 : L - 1;
  const int hi_min = (cdiv(wq_first) + 1) * C < L ? (cdiv(wq_first) + 1) * C : L;
  const int lo_max = (cdiv(wq_last) > R ? cdiv(wq_last) - R : 0) * C;
  // keys any query of this wave can see; a wave whose queries are all padding sees none
  const bool wave_live = q0 + wave * 32 < L;
  const int lo_min = (cdiv(wq_first) > R ? cdiv(wq_first) - R : 0) * C;
  const int hi_max = !wave_live ? 0 : ((cdiv(wq_last) + 1) * C < L ? (cdiv(wq_last) + 1) * C : L);
  const int gq_last = q0 + TQ - 1 < L ? q0 + TQ - 1 : L - 1;
  const int lo_wg = (cdiv(q0) > R ? cdiv(q0) - R : 0) * C;
  const int hi_wg = (cdiv(gq_last) + 1) * C < L ? (cdiv(gq_last) + 1) * C : L;
  const int kt0 = lo_wg / TK, kt1 = (hi_wg + TK - 1) / TK;

  const float sl2e = fabsf(p.scale_log2e);
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
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (kt0 + i < kt1) issue_tile(kt0 + i);

  Frag qf[NF], gf[NF];
  float lse_q, delta_q;
  {
    const int qr = qrow < L ? qrow : L - 1;
    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh +
                  (int64_t)qr * p.q_st;
    const T* gp = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.do_sb + (int64_t)hd * p.do_sh +
                  (int64_t)qr * p.do_st;
    // delta = rowsum(O * dO) is formed here when the caller has not run the delta kernel: this lane holds half
    // of its query's dO row, so the forward output is fetched in the same pattern, in flight together with the
    // other rows, and the two halves are added across lanes
    // (no branch around the loads: a value defined on one side only is copied where the sides join, and the copy
    // waits for the load; without a row of O to read, the dO row is read twice)
    Frag of[NF];
    const T* op = p.delta_out ? reinterpret_cast<const T*>(p.o) + (int64_t)b * p.o_sb + (int64_t)hd * p.o_sh +
                                    (int64_t)qr * p.o_st
                              : gp;
#pragma unroll
    for (int g = 0; g < NF; ++g) of[g] = *reinterpret_cast<const Frag*>(op + (g * 2 + h) * E::VEC);
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      qf[g] = *reinterpret_cast<const Frag*>(qp + (g * 2 + h) * E::VEC);
      if (neg) qf[g] = negate<T>(qf[g]);
      // dO enters negated: the dP accumulator starts at delta and ends at delta - dP, which
      // saves the subtraction per element; the sign is put back by the scale of the store
      gf[g] = negate<T>(*reinterpret_cast<const Frag*>(gp + (g * 2 + h) * E::VEC));
    }
    lse_q = qrow < L ? p.lse[(int64_t)bh * T_ + qr] : INFINITY;   // rows past L: P = exp2(-inf) = 0
    float osum = 0.0f;
#pragma unroll
    for (int g = 0; g < NF; ++g) osum = dot_frag(of[g], gf[g], osum);
    delta_q = -half_sum(osum);
    if (p.delta_out) {
      if (h == 0 && qrow < T_) p.delta_out[(int64_t)bh * T_ + qrow] = qrow < L ? delta_q : 0.0f;
    } else {
      delta_q = p.delta[(int64_t)bh * T_ + qr];
    }
  }
  f32x16 dinit;
#pragma unroll
  for (int i = 0; i < 16; ++i) dinit[i] = delta_q;

  f32x16 acc[DB];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  wait_all_loads();

  for (int t = kt0; t < kt1; ++t) {
    if (NST == 3 && t + 1 < kt1) wait_loads<LPT>();
    else wait_loads<0>();
    __syncthreads();
    if (t + NST - 1 < kt1) issue_tile(t + NST - 1);

    const T* Kt = smem + ((t - kt0) % NST) * STAGE;
    const T* Vt = Kt + TILE;
    const int k0 = t * TK;
    if (k0 + TK <= lo_min || k0 >= hi_max) continue;   // outside this wave's windows

#pragma unroll
    for (int kb = 0; kb < KBN; ++kb) {
      // the same two tests per 32-key block: short windows end inside a tile
      const int kb0 = k0 + kb * 32;
      if (kb0 + 32 <= lo_min || kb0 >= hi_max) continue;
      const bool interior = (kb0 >= lo_max) && (kb0 + 32 <= hi_min);
      f32x16 s[1], dp[1];
#pragma unroll
      for (int i = 0; i < 16; ++i) s[0][i] = 0.0f;
      dp[0] = dinit;
      mma_rows_pair<T, D>(s[0], dp[0], Kt, Vt, kb * 32, qf, gf, lane);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float pr = fast_exp2(__builtin_fmaf(s[0][i], sl2e, -lse_q));
        s[0][i] = pr * dp[0][i];   // = -dS
      }
      if (!interior) {
        const uint32_t rm = row_mask(lo - (k0 + kb * 32), hi - (k0 + kb * 32), h);
#pragma unroll
        for (int i = 0; i < 16; ++i) s[0][i] = keep_or_zero(s[0][i], keep_bits(rm, i));
      }
      mma_tr<T, D>(acc, Kt, kb, s[0], lane);   // -dQ^T[d][q] += K^T (-dS^T)
    }
  }

  if (qrow >= L) {
#pragma unroll
    for (int m = 0; m < DB; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  }
  __syncthreads();   // the row patches lie over the tile stages
  {
    T* patch = smem + wave * RowPatch<T, D>::ELEMS;
    const int row0 = q0 + wave * 32;
    store_rows_coalesced<T, D, DB>(patch, dq_base + (int64_t)row0 * D, T_ - row0, acc, -p.scale, lane);
  }
}

template <typename T, int D, int NW, int TQ, int NST>
// At head dimension 64 the kernel needs 174 registers, six more than three waves per SIMD may have; held to 168 it
// reloads a few values per tile and runs 5 % faster with three workgroups per CU instead of two (measured at B=8,
// H=16, T=4096).  At 128 the same step (290 -> 256 registers) spills inside the products and is 40 % slower.
__global__ __launch_bounds__(NW * 64, (D == 64 ? 3 : 1)) void dkdv2_kernel(const BwdParams p) {
  using E = Elem<T>;
  // fragments fetched ahead of the MFMAs, per group: two at head dimension 64, where the smaller groups let the kernel
  // fit the 168 registers of three waves per SIMD with one reloaded value instead of six (another 5 % faster)
  constexpr int PG = D == 64 ? 2 : 4;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(G::SWZ && (NST == 2 || NST == 3), "swizzled 16-bit tiles, 2 or 3 stages");
  constexpr int TKB = NW * 32, NT = NW * 64, QBN = TQ / 32;
  constexpr int NF = G::NF, DB = G::DB;
  constexpr int TILE = TQ * D;
  constexpr int RPW = TQ / NW;   // rows of lse / delta each wave stages
  static_assert(TQ % NW == 0 && RPW % 4 == 0 && 2 * RPW <= 64, "lse/delta staging: one instruction per wave");
  // stage layout: [Q tile][dO tile][NW chunks of {lse[RPW], delta[RPW]}]
  constexpr int STAGE_BYTES = 2 * TILE * (int)sizeof(T) + 2 * TQ * (int)sizeof(float);
  using Loader = AsyncTile<T, D, TQ, NW>;
  constexpr int LPT = 2 * Loader::PER_WAVE + 1;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int bh, kt, L;
  key_tile_coords(blockIdx.x, gridDim.x, p.n_tiles, growing_tiles(p.C, p.R, p.T, TKB), TKB, p.H, p.T, p.lens,
                  p.lens_stride, bh, kt, L);
  const int hd = bh % p.H, b = bh / p.H;
  const int T_ = p.T, C = p.C, R = p.R;
  auto cdiv = [&](int x) { return div_by(x, p.cdiv); };   // x / C
  const int k0 = kt * TKB;
  T* dk_base = reinterpret_cast<T*>(p.dk) + (int64_t)bh * T_ * D;
  T* dv_base = reinterpret_cast<T*>(p.dv) + (int64_t)bh * T_ * D;
  const int k_end = k0 + TKB < T_ ? k0 + TKB : T_;
  if (k0 >= L) {
    zero_rows<T, D, NT>(dk_base, k0, k_end, tid);
    zero_rows<T, D, NT>(dv_base, k0, k_end, tid);
    return;
  }

  auto win_lo = [&](int key) { return (cdiv(key)) * C; };
  auto win_hi = [&](int key) {
    const int64_t e = ((int64_t)(cdiv(key)) + R + 1) * (int64_t)C;
    return e < (int64_t)L ? (int)e : L;
  };
  const int krow = k0 + wave * 32 + c;
  const int ke = krow < L ? krow : L - 1;
  const int qlo = win_lo(ke), qhi = win_hi(ke);
  const int wk_first = k0 + wave * 32 < L ? k0 + wave * 32 : L - 1;
  const int wk_last = k0 + wave * 32 + 31 < L ? k0 + wave * 32 + 31 : L - 1;
  const int qhi_min = win_hi(wk_first), qlo_max = win_lo(wk_last);
  // queries that can see any key of this wave; a wave whose keys are all padding has none
  const bool wave_live = k0 + wave * 32 < L;
  const int qlo_min = win_lo(wk_first), qhi_max = wave_live ? win_hi(wk_last) : 0;
  const int gk_last = k0 + TKB - 1 < L ? k0 + TKB - 1 : L - 1;
  const int qt0 = win_lo(k0) / TQ, qt1 = (win_hi(gk_last) + TQ - 1) / TQ;

  const float kmul = -p.scale_log2e;

  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh;
  const T* gbase = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.do_sb + (int64_t)hd * p.do_sh;
  const float* lse_base = p.lse + (int64_t)bh * T_;
  const float* delta_base = p.delta + (int64_t)bh * T_;
  auto stage_ptr = [&](int t) { return smem_raw + ((t - qt0) % NST) * STAGE_BYTES; };
  Loader ldq, ldg;
  ldq.init(qbase, p.q_st, qt0 * TQ, L - 1, wave, lane);
  ldg.init(gbase, p.do_st, qt0 * TQ, L - 1, wave, lane);
  auto issue_tile = [&](int t) {   // tiles are issued in ascending order
    T* st = reinterpret_cast<T*>(stage_ptr(t));
    // lanes [0, RPW) fetch lse, lanes [RPW, 2*RPW) fetch delta of this wave's RPW rows
    if (lane < 2 * RPW) {
      int r = t * TQ + wave * RPW + (lane % RPW);
      r = r < L ? r : L - 1;
      const float* src = (lane < RPW ? lse_base : delta_base) + r;
      float* dst = reinterpret_cast<float*>(stage_ptr(t) + 2 * TILE * sizeof(T)) + wave * 2 * RPW;
      async_copy_f32(src, dst);
    }
    ldq.issue(st, wave);
    ldg.issue(st + TILE, wave);
    ldq.advance();
    ldg.advance();
  };
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (qt0 + i < qt1) issue_tile(qt0 + i);

  Frag kf[NF], vf[NF];
  {
    const int kr = krow < L ? krow : L - 1;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh +
                  (int64_t)kr * p.k_st;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh +
                  (int64_t)kr * p.v_st;
#pragma unroll
    for (int g = 0; g < NF; ++g) {
      // K enters multiplied by -scale*log2(e), rounded to the element type: the score accumulator
      // starts at lse and ends at lse - score*scale*log2(e), whose negated exp2 is the probability
      kf[g] = *reinterpret_cast<const Frag*>(kp + (g * 2 + h) * E::VEC);
#pragma unroll
      for (int e = 0; e < E::VEC; ++e) kf[g][e] = (T)((float)kf[g][e] * kmul);
      // V enters negated: the dP accumulator starts at delta and ends at delta - dP
      vf[g] = negate<T>(*reinterpret_cast<const Frag*>(vp + (g * 2 + h) * E::VEC));
    }
  }

  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) dk[m][i] = 0.0f, dv[m][i] = 0.0f;
  wait_all_loads();

  for (int t = qt0; t < qt1; ++t) {
    if (NST == 3 && t + 1 < qt1) wait_loads<LPT>();
    else wait_loads<0>();
    __syncthreads();
    if (t + NST - 1 < qt1) issue_tile(t + NST - 1);

    const T* Qt = reinterpret_cast<const T*>(stage_ptr(t));
    const T* Gt = Qt + TILE;
    const float* ld_t = reinterpret_cast<const float*>(stage_ptr(t) + 2 * TILE * sizeof(T));
    const int qs = t * TQ;
    if (qs + TQ <= qlo_min || qs >= qhi_max) continue;   // outside this wave's windows

#pragma unroll
    for (int qb = 0; qb < QBN; ++qb) {
      // the same two tests per 32-query block: short windows end inside a tile
      const int qb0 = qs + qb * 32;
      if (qb0 + 32 <= qlo_min || qb0 >= qhi_max) continue;
      const bool interior = (qb0 >= qlo_max) && (qb0 + 32 <= qhi_min);
      f32x16 s[1], dp[1];
      // lse / delta of the 16 rows this lane holds, fetched ahead of the products and read
      // straight into the score and dP accumulators
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int r = qb * 32 + 8 * g4 + 4 * h;     // tile row of 4 consecutive C-fragment rows
        const float* chunk = ld_t + (r / RPW) * 2 * RPW + (r % RPW);
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(chunk);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(chunk + RPW);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[0][4 * g4 + e] = l4[e], dp[0][4 * g4 + e] = d4[e];
      }
      // S[q][key] = Q K^T and dP[q][key] = dO V^T
      mma_rows_pair<T, D, NF, PG>(s[0], dp[0], Qt, Gt, qb * 32, kf, vf, lane);
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * g4 + e;
          const float pr = fast_exp2(-s[0][i]);
          s[0][i] = pr;
          dp[0][i] = pr * dp[0][i];   // = -dS
        }
      }
      if (!interior) {
        const uint32_t rm = row_mask(qlo - (qs + qb * 32), qhi - (qs + qb * 32), h);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t keep = keep_bits(rm, i);
          s[0][i] = keep_or_zero(s[0][i], keep);
          dp[0][i] = keep_or_zero(dp[0][i], keep);
        }
      }
      // dV^T[d][key] += dO^T P and -dK^T[d][key] += Q^T (-dS)
      mma_tr_pair<T, D, DB, PG>(dv, dk, Gt, Qt, qb, s[0], dp[0], lane);
    }
  }

  if (krow >= L) {
#pragma unroll
    for (int m = 0; m < DB; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) dk[m][i] = 0.0f, dv[m][i] = 0.0f;
  }
  // the row patches lie over the tile stages: wait until no wave reads the last tile any more
  __syncthreads();
  {
    T* patch = reinterpret_cast<T*>(smem_raw) + wave * RowPatch<T, D>::ELEMS;
    const int row0 = k0 + wave * 32;
    store_rows_coalesced<T, D, DB>(patch, dk_base + (int64_t)row0 * D, T_ - row0, dk, -p.scale, lane);
    store_rows_coalesced<T, D, DB>(patch, dv_base + (int64_t)row0 * D, T_ - row0, dv, 1.0f, lane);
  }
}

}  // namespace sa
