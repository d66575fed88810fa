// dK/dV kernel whose four matrix products are split between two waves, for 16-bit elements with
// swizzled tiles (D = 64 or 128).
//
// dkdv2_kernel and dkdv3_kernel give one wave 32 keys and all four products of a block step
// (S, dP, dV, dK): two 32 x D accumulators and the K and V fragments make more than 256
// registers per lane at D = 128, so one wave per SIMD is resident and nothing but that wave's own
// instruction order can overlap matrix, vector and LDS work.  Here the same 32 keys belong to a
// PAIR of waves that sit on the same SIMD:
//     wave A ("score" role):  S = Q K^T,  P = exp2(-(lse - S)),  dV^T += dO^T P        holds K, dV
//     wave B ("grad" role):   delta - dP = delta - dO V^T,  -dS = P o (delta - dP),
//                             -dK^T += Q^T (-dS)                                        holds V, dK
// Each wave needs one accumulator and one set of resident fragments (about 170 registers), two
// waves per SIMD are resident, and while one of them waits for its MFMA results or its LDS
// fragments the other one issues.  The only value that crosses is P, rounded to the element type
// exactly as the dV product consumes it: wave A writes its two packed fragments (32 bytes per
// lane, same lane layout) into a double-buffered LDS slot of the pair, and wave B picks them up
// one block step later, after the barrier that every step has anyway.  So B runs one 32-query
// block behind A: in step g it forms delta - dP of block g and finishes dS and dK of block g-1.
//
// A workgroup is 4 pairs = 8 waves = 128 keys; query tiles of 64 rows (two block steps) arrive
// by asynchronous global->LDS copies in a ring of three stages.  A tile is read during three
// steps (B's lagging dK product reads the previous tile in the first step of a tile), so the
// copy that reuses its stage is issued at the second step of the following tile.
#pragma once
#include "sa_common.h"

namespace sa {

template <typename T, int D, int NST>
__global__ __launch_bounds__(512) void dkdv_split_kernel(const BwdParams p) {
  using E = Elem<T>;
  using G = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(G::SWZ && NST == 3, "swizzled 16-bit tiles, three stages");
  constexpr int NP = 4, NW = 2 * NP, TQ = 64, TKB = NP * 32, NT = NW * 64;
  constexpr int NF = G::NF, DB = G::DB;
  constexpr int TILE = TQ * D;
  constexpr int RPW = TQ / NW;   // rows of lse / delta each wave stages
  static_assert(RPW % 4 == 0 && 2 * RPW <= 64, "lse/delta staging: one instruction per wave");
  // stage layout: [Q tile][dO tile][NW chunks of {lse[RPW], delta[RPW]}]
  constexpr int STAGE_BYTES = 2 * TILE * (int)sizeof(T) + 2 * TQ * (int)sizeof(float);
  constexpr int XSLOT = 64 * 2 * 16;             // bytes of one exchange slot: two fragments per lane
  constexpr int XBUF_OFF = NST * STAGE_BYTES;    // exchange slots follow the stages: [pair][2][XSLOT]
  using Loader = AsyncTile<T, D, TQ, NW, true>;   // copies as assembly: three stages, see AsyncTile
  constexpr int LPT = 2 * Loader::PER_WAVE + 1;  // asynchronous loads per wave per tile
  // LDS fragments requested ahead of the MFMAs that consume them: with two waves per SIMD a depth of
  // 2 measured the same as 4 and 8 and leaves the most registers
  constexpr int GRP = 2;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, c = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // waves w and w + 4 run on the same SIMD: they form a pair
  const int pair = wave & (NP - 1);
  const bool grad_role = wave >= NP;

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
  const int krow = k0 + pair * 32 + c;
  const int ke = krow < L ? krow : L - 1;
  const int qlo = win_lo(ke), qhi = win_hi(ke);
  const int wk_first = k0 + pair * 32 < L ? k0 + pair * 32 : L - 1;
  const int wk_last = k0 + pair * 32 + 31 < L ? k0 + pair * 32 + 31 : L - 1;
  const int qhi_min = win_hi(wk_first), qlo_max = win_lo(wk_last);
  // queries that can see any key of this pair; a pair whose keys are all padding has none
  const bool pair_live = k0 + pair * 32 < L;
  const int qlo_min = win_lo(wk_first), qhi_max = pair_live ? win_hi(wk_last) : 0;
  const int gk_last = k0 + TKB - 1 < L ? k0 + TKB - 1 : L - 1;
  const int qt0 = win_lo(k0) / TQ, qt1 = (win_hi(gk_last) + TQ - 1) / TQ;
  // 32-query block g: both waves of a pair take the same decisions
  auto blk_live = [&](int g) { return g * 32 + 32 > qlo_min && g * 32 < qhi_max; };
  auto blk_interior = [&](int g) { return g * 32 >= qlo_max && g * 32 + 32 <= qhi_min; };

  const T* qbase = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)hd * p.q_sh;
  const T* gbase = reinterpret_cast<const T*>(p.d_o) + (int64_t)b * p.do_sb + (int64_t)hd * p.do_sh;
  const float* lse_base = p.lse + (int64_t)bh * T_;
  const float* delta_base = p.delta + (int64_t)bh * T_;
  Loader ldq, ldg;
  ldq.init(qbase, p.q_st, qt0 * TQ, L - 1, wave, lane);
  ldg.init(gbase, p.do_st, qt0 * TQ, L - 1, wave, lane);
  auto issue_tile = [&](int t, int stage_off) {   // tiles are issued in ascending order
    T* st = reinterpret_cast<T*>(smem_raw + stage_off);
    // lanes [0, RPW) fetch lse, lanes [RPW, 2*RPW) fetch delta of this wave's RPW rows
    if (lane < 2 * RPW) {
      int r = t * TQ + wave * RPW + (lane % RPW);
      r = r < L ? r : L - 1;
      const float* src = (lane < RPW ? lse_base : delta_base) + r;
      float* dst = reinterpret_cast<float*>(smem_raw + stage_off + 2 * TILE * sizeof(T)) + wave * 2 * RPW;
      async_copy_f32<true>(src, dst);
    }
    ldq.issue(st, wave);
    ldg.issue(st + TILE, wave);
    ldq.advance();
    ldg.advance();
  };
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (qt0 + i < qt1) issue_tile(qt0 + i, i * STAGE_BYTES);

  // resident fragments: K for the score role, V for the grad role
  Frag rf[NF];
  {
    const int kr = krow < L ? krow : L - 1;
    const float kmul = -p.scale_log2e;
    if (!grad_role) {
      const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)hd * p.k_sh +
                    (int64_t)kr * p.k_st;
#pragma unroll
      for (int g = 0; g < NF; ++g) {
        // K enters multiplied by -scale*log2(e), rounded to the element type: the score accumulator
        // starts at lse and ends at lse - score*scale*log2(e), whose negated exp2 is the probability
        rf[g] = *reinterpret_cast<const Frag*>(kp + (g * 2 + h) * E::VEC);
#pragma unroll
        for (int e = 0; e < E::VEC; ++e) rf[g][e] = (T)((float)rf[g][e] * kmul);
      }
    } else {
      const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)hd * p.v_sh +
                    (int64_t)kr * p.v_st;
      // V enters negated: the dP accumulator starts at delta and ends at delta - dP
#pragma unroll
      for (int g = 0; g < NF; ++g) rf[g] = negate<T>(*reinterpret_cast<const Frag*>(vp + (g * 2 + h) * E::VEC));
    }
  }

  // dV^T[d][key] (score role) or -dK^T[d][key] (grad role)
  f32x16 acc[1][DB];
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[0][m][i] = 0.0f;
  // delta - dP of the block the grad role formed in the previous step
  f32x16 dp[1];
#pragma unroll
  for (int i = 0; i < 16; ++i) dp[0][i] = 0.0f;

  char* const xbuf = smem_raw + XBUF_OFF + pair * 2 * XSLOT + lane * 16;

  // Byte offsets of this lane's fragments inside a tile, block 0: row-major fragment g of row c, and the two
  // transposing reads (rows r_lo and r_lo + 8 of the first 16) of column block m.  The swizzle of a row depends
  // on its low four bits only, so every other block of a tile is a compile-time distance away and an LDS read
  // costs one address addition; left to itself the compiler rebuilds the swizzled address for every read.
  uint32_t row_off[NF], tr_off[2][DB];
  {
    const int g16 = lane >> 4, j = lane & 15;
    const int r_lo = 4 * (g16 >> 1) + (j >> 2), col = (g16 & 1) * 16 + 4 * (j & 3);
#pragma unroll
    for (int g = 0; g < NF; ++g) row_off[g] = (uint32_t)G::off(c, (g * 2 + h) * E::VEC) * (uint32_t)sizeof(T);
#pragma unroll
    for (int m = 0; m < DB; ++m) {
      tr_off[0][m] = (uint32_t)G::off(r_lo, m * 32 + col) * (uint32_t)sizeof(T);
      tr_off[1][m] = (uint32_t)G::off(r_lo + 8, m * 32 + col) * (uint32_t)sizeof(T);
    }
  }
  constexpr int BLOCK_BYTES = 32 * G::PITCH * (int)sizeof(T);   // 32 rows of a tile
  // accS += rows [32 qb, 32 qb + 32) of the tile at byte offset `tile` of the LDS allocation, times rf
  auto rows_product = [&](f32x16& accS, int tile, int qb) {
    const char* base = smem_raw + tile + qb * BLOCK_BYTES;
    pipeline<NF, GRP>([&](int g) { return *reinterpret_cast<const Frag*>(base + row_off[g]); },
                      [&](int g, const Frag& a) { mma(accS, a, rf[g]); });
  };
  // accD[m] += (rows [32 qb, 32 qb + 32) of that tile)^T times the packed block b
  auto tr_product = [&](f32x16 (&accD)[DB], int tile, int qb, const Frag (&b)[2]) {
    const char* base = smem_raw + tile + qb * BLOCK_BYTES;
    pipeline<2 * DB, GRP>(
        [&](int it) {
          const char* p = base + (it / DB) * (BLOCK_BYTES / 2);
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p + tr_off[0][it % DB]));
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p + tr_off[1][it % DB]));
          return __builtin_bit_cast(Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        },
        [&](int it, const Frag& a) { mma(accD[it % DB], a, b[it / DB]); });
  };
  wait_all_loads();

  // lse (WHICH = 0) or delta (WHICH = 1) of the 16 rows of block qb this lane holds in a C fragment
  auto rows16 = [&](const float* ld_t, int qb, int which, f32x16& out) {
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int r = qb * 32 + 8 * g4 + 4 * h;     // tile row of 4 consecutive C-fragment rows
      const float* chunk = ld_t + (r / RPW) * 2 * RPW + (r % RPW) + which * RPW;
      const f32x4 v4 = *reinterpret_cast<const f32x4*>(chunk);
#pragma unroll
      for (int e = 0; e < 4; ++e) out[4 * g4 + e] = v4[e];
    }
  };

  // Byte offsets of the stages that hold tile t (cur) and tile t - 1 (prev); the third stage is the
  // one being filled.  They are carried from tile to tile instead of being derived from t, so that a
  // lane's LDS addresses are one add away from its loop-invariant offsets.
  int st_cur = 0, st_prev = 2 * STAGE_BYTES;
  auto wait_tile = [&](int t) {
    if (t + 1 < qt1) wait_loads<LPT>();
    else wait_loads<0>();
  };
  auto next_tile = [&]() {
    const int st_next = 3 * STAGE_BYTES - st_cur - st_prev;
    st_prev = st_cur;
    st_cur = st_next;
  };

  if (!grad_role) {
    // ---- score role: block g = 2 t + qb ------------------------------------------------------
    auto step = [&](int t, int qb) {
      const int g = 2 * t + qb;
      if (!blk_live(g)) return;
      const float* ld_t = reinterpret_cast<const float*>(smem_raw + st_cur + 2 * TILE * sizeof(T));
      f32x16 s[1];
      rows16(ld_t, qb, 0, s[0]);
      rows_product(s[0], st_cur, qb);                              // lse - S[q][key]
#pragma unroll
      for (int i = 0; i < 16; ++i) s[0][i] = fast_exp2(-s[0][i]);
      if (!blk_interior(g)) {
        asm volatile("");   // a real branch: as straight-line selects the mask would cost every block 3 instructions per score
        const uint32_t rm = row_mask(qlo - g * 32, qhi - g * 32, h);
#pragma unroll
        for (int i = 0; i < 16; ++i) s[0][i] = keep_or_zero(s[0][i], keep_bits(rm, i));
      }
      Frag pf[1][2];
      pack_c<T>(pf[0], s[0]);
      char* slot = xbuf + (g & 1) * XSLOT;
      *reinterpret_cast<Frag*>(slot) = pf[0][0];
      *reinterpret_cast<Frag*>(slot + 1024) = pf[0][1];
      tr_product(acc[0], st_cur + TILE * (int)sizeof(T), qb, pf[0]);   // dV^T[d][key] += dO^T P
    };
    for (int t = qt0; t < qt1; ++t) {
      wait_tile(t);
      __syncthreads();
      step(t, 0);
      __syncthreads();
      // every wave has left the step that read tile t - 1 for the last time
      if (t + 2 < qt1) issue_tile(t + 2, st_prev);
      step(t, 1);
      next_tile();
    }
    __syncthreads();   // the grad role's last block
  } else {
    // ---- grad role: delta - dP of block g, then dS and dK of block g - 1 -------------------------
    // (tile t, block 0 when qb = 1; tile t - 1, block 1 when qb = 0)
    auto step = [&](int t, int qb) {
      const int g = 2 * t + qb;
      const bool cur = t < qt1 && blk_live(g);
      const bool prev = g > 2 * qt0 && blk_live(g - 1);
      const float* ld_t = reinterpret_cast<const float*>(smem_raw + st_cur + 2 * TILE * sizeof(T));
      // dS of the previous block first: its delta - dP leaves the registers that the next product fills
      Frag df[1][2];
      if (prev) {
        const char* slot = xbuf + ((g - 1) & 1) * XSLOT;
        const Frag pf0 = *reinterpret_cast<const Frag*>(slot);
        const Frag pf1 = *reinterpret_cast<const Frag*>(slot + 1024);
        f32x16 ds;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          ds[e] = (float)pf0[e] * dp[0][e];           // = -dS
          ds[8 + e] = (float)pf1[e] * dp[0][8 + e];
        }
        pack_c<T>(df[0], ds);
      }
      if (cur) {
        rows16(ld_t, qb, 1, dp[0]);
        rows_product(dp[0], st_cur + TILE * (int)sizeof(T), qb);   // delta - dP[q][key]
      }
      if (prev) {
        tr_product(acc[0], qb ? st_cur : st_prev, qb ? 0 : 1, df[0]);   // -dK^T[d][key] += Q^T (-dS)
      }
    };
    for (int t = qt0; t < qt1; ++t) {
      wait_tile(t);
      __syncthreads();
      step(t, 0);
      __syncthreads();
      if (t + 2 < qt1) issue_tile(t + 2, st_prev);
      step(t, 1);
      next_tile();
    }
    __syncthreads();
    step(qt1, 0);
  }

  if (krow >= L) {
#pragma unroll
    for (int m = 0; m < DB; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[0][m][i] = 0.0f;
  }
  // the row patches lie over the tile stages: wait until no wave reads the last tiles any more
  __syncthreads();
  {
    T* patch = reinterpret_cast<T*>(smem_raw) + wave * RowPatch<T, D>::ELEMS;
    const int row0 = k0 + pair * 32;
    if (!grad_role) store_rows_coalesced<T, D, DB>(patch, dv_base + (int64_t)row0 * D, T_ - row0, acc[0], 1.0f, lane);
    else store_rows_coalesced<T, D, DB>(patch, dk_base + (int64_t)row0 * D, T_ - row0, acc[0], -p.scale, lane);
  }
}

}  // namespace sa
