// Shared device-side building blocks for the streaming-attention kernels (gfx950 / CDNA4).
//
// Conventions used by every kernel in this directory
// --------------------------------------------------
// A wavefront has 64 lanes; lane l is split as c = l & 31 ("owner" index) and h = l >> 5.
// All matrix products are 32x32 MFMA tiles, D = A*B + C:
//   * A fragment: lane supplies A[row c][contraction slots of half h]
//   * B fragment: lane supplies B[contraction slots of half h][col c]
//   * C fragment: 16 floats per lane, acc[i] is C[row 8*(i/4) + 4*h + (i%4)][col c]
// Only the pairing of A and B slots matters for correctness, so every fragment that
// is loaded straight from memory uses the same rule: fragment g of a row covers the
// contraction indices [g*2*VEC + h*VEC, g*2*VEC + h*VEC + VEC), one 16-byte vector.
// For 16-bit types VEC = 8 and a fragment feeds one v_mfma_f32_32x32x16_{bf16,f16};
// for fp32 VEC = 4 and a fragment feeds four v_mfma_f32_32x32x2_f32.
//
// The second product of each attention step contracts over the ROW index of a C
// fragment that was just computed (keys for P*V, queries for P^T*dO ...).  The lane
// that owns column c of that C fragment already holds exactly the values a B operand
// needs, so the probabilities never leave registers; the matching A operand is the
// transpose of a row-major LDS tile, fetched with ds_read_b64_tr_b16 (16-bit) or with
// scalar LDS reads (fp32).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sa {

#define SA_DEV __device__ __forceinline__
#define SA_LDS __attribute__((address_space(3)))

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  static constexpr int VEC = 8;
  static constexpr bool HALF = true;
  using Frag = bf16x8;
  using Quad = bf16x4;
  static constexpr uint32_t SIGN = 0x80008000u;
};
template <> struct Elem<_Float16> {
  static constexpr int VEC = 8;
  static constexpr bool HALF = true;
  using Frag = f16x8;
  using Quad = f16x4;
  static constexpr uint32_t SIGN = 0x80008000u;
};
template <> struct Elem<float> {
  static constexpr int VEC = 4;
  static constexpr bool HALF = false;
  using Frag = f32x4;
  using Quad = f32x4;
  static constexpr uint32_t SIGN = 0x80000000u;
};

// LDS tile geometry.  Two layouts:
//  * swizzled (16-bit types, D >= 32): rows are stored unpadded and the 16-byte chunk index
//    inside a row is XOR-ed with a permutation of the low row bits, chosen so that both access
//    patterns of the kernels spread over all 64 banks: 16 lanes reading the same chunk of 16
//    consecutive rows (row-major fragments), and 32 lanes reading a 4-row x 64-byte patch
//    (transposing reads).
//  * padded (everything else): the head dimension (at least one 32-wide block, so that
//    transposed reads of a D=16 tile stay inside the row) plus one 16-byte pad.
#ifndef SA_PAD_VECS
#define SA_PAD_VECS 1
#endif
#ifndef SA_SWIZZLE
#define SA_SWIZZLE 1
#endif
template <typename T, int D> struct TileGeom {
  static constexpr int VEC = Elem<T>::VEC;
  static constexpr int DP = D < 32 ? 32 : D;
  static constexpr bool SWZ = SA_SWIZZLE && Elem<T>::HALF && D >= 32;
  static constexpr int PITCH = SWZ ? D : DP + SA_PAD_VECS * VEC;
  static constexpr int NF = D / (2 * VEC);   // row fragments per lane
  static constexpr int DB = DP / 32;         // 32-wide blocks along D
  static constexpr int CPR = D / VEC;        // 16-byte chunks per row

  // XOR mask (in chunks) for a row; depends on row & 15 only
  SA_DEV static int swz(int row) {
    if constexpr (!SWZ) return 0;
    else if constexpr (CPR >= 16) return ((row & 3) << 2) | ((row >> 2) & 3);
    else if constexpr (CPR == 8) return ((row >> 2) & 1) | (((row >> 3) & 1) << 1) | (((row >> 1) & 1) << 2);
    else return (row >> 2) & 3;   // CPR == 4: four rows fill the 64 banks, rows 4 apart must differ
  }
  // element offset of (row, element col) inside a tile
  SA_DEV static int off(int row, int col) {
    if constexpr (!SWZ) return row * PITCH + col;
    else return row * PITCH + ((((col / VEC) ^ swz(row)) * VEC) | (col % VEC));
  }
};

SA_DEV void mma(f32x16& acc, bf16x8 a, bf16x8 b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
SA_DEV void mma(f32x16& acc, f16x8 a, f16x8 b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
}
SA_DEV void mma(f32x16& acc, f32x4 a, f32x4 b) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
}

// Value held by lane l^32 combined with the lane's own: v_permlane32_swap hands each
// lane both its own value and its partner's (in an order that depends on the half),
// which is all a max or a sum needs.
SA_DEV float half_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
SA_DEV float half_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Block until every outstanding global load of this wave has returned (vmcnt = 0, the other
// counters untouched).  Placed before a main loop so that the waits the compiler must insert
// for loop-invariant operands do not also drain the prefetch loads issued inside the loop.
SA_DEV void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

SA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max(a, b) as median(a, b, +inf): one v_med3_f32, with none of the input canonicalisation
// that fmaxf() costs per operand.
SA_DEV float fast_max(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }

// max(a, b, c) in one instruction.  Written as asm because the three-operand form is only
// selected from fmaxf() chains together with a canonicalising move per operand.
SA_DEV float fast_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// acc + the sum of the eight 16-bit values of a fragment: four dot products with (1, 1), i.e.
// half a vector instruction per element, and the sum is over the rounded values that the
// following matrix product consumes.
SA_DEV float sum_frag(bf16x8 f, float acc) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j)
    acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{f[2 * j], f[2 * j + 1]}, one, acc, false);
  return acc;
}
// acc + the dot product of two fragments, two elements per instruction, products and sums in float32
SA_DEV float dot_frag(bf16x8 a, bf16x8 b, float acc) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int j = 0; j < 4; ++j)
    acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{a[2 * j], a[2 * j + 1]}, bf16x2{b[2 * j], b[2 * j + 1]}, acc, false);
  return acc;
}
SA_DEV float dot_frag(f16x8 a, f16x8 b, float acc) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int j = 0; j < 4; ++j)
    acc = __builtin_amdgcn_fdot2(f16x2{a[2 * j], a[2 * j + 1]}, f16x2{b[2 * j], b[2 * j + 1]}, acc, false);
  return acc;
}
SA_DEV float sum_frag(f16x8 f, float acc) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f16x2 one = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j)
    acc = __builtin_amdgcn_fdot2(f16x2{f[2 * j], f[2 * j + 1]}, one, acc, false);
  return acc;
}

// Masks for the edge of a window.  Rows [a, b) of a 32-row block are allowed; row_mask() packs
// that into one bit per row, pre-shifted for the lane's half so that the bit of accumulator
// register i sits at the compile-time position 8*(i/4) + i%4.  keep_bits() expands one bit
// into all-ones / zero; an element is then kept or cleared with a single bitwise operation
// instead of two compares, a mask merge and a select.
SA_DEV uint32_t row_mask(int a, int b, int h) {
  a = a < 0 ? 0 : a;
  b = b < 0 ? 0 : b;
  const uint32_t below_b = b >= 32 ? 0xFFFFFFFFu : ((1u << b) - 1u);
  const uint32_t below_a = a >= 32 ? 0xFFFFFFFFu : ((1u << a) - 1u);
  return (below_b & ~below_a) >> (4 * h);
}
SA_DEV uint32_t keep_bits(uint32_t m, int i) {
  return (uint32_t)__builtin_amdgcn_sbfe((int)m, 8 * (i >> 2) + (i & 3), 1);
}
SA_DEV float keep_or_zero(float x, uint32_t keep) { return __uint_as_float(__float_as_uint(x) & keep); }
SA_DEV float keep_or_neg_inf(float x, uint32_t keep) {
  return __uint_as_float((__float_as_uint(x) & keep) | (0xFF800000u & ~keep));
}

template <typename T> SA_DEV typename Elem<T>::Frag negate(typename Elem<T>::Frag f) {
  u32x4 u = __builtin_bit_cast(u32x4, f);
  u ^= Elem<T>::SIGN;
  return __builtin_bit_cast(typename Elem<T>::Frag, u);
}

// Row of a C fragment that register i of half h holds.
SA_DEV constexpr int crow(int i, int h) { return 8 * (i >> 2) + 4 * h + (i & 3); }

// The compiler's scheduler, left alone, issues each LDS read right before the MFMA that
// consumes it and so exposes the full LDS latency once per MFMA.  pipeline() forces the
// shape "fetch group n+1, then multiply group n" with scheduling fences between groups:
// N items in groups of G, load(i) returns the fragment of item i, use(i, frag) consumes it.
SA_DEV void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

template <int N, int G, typename LoadF, typename UseF>
SA_DEV void pipeline(LoadF&& load, UseF&& use) {
  static_assert(N % G == 0, "items must fill whole groups");
  using F = decltype(load(0));
  constexpr int NG = N / G;
  F buf[2][G];
#pragma unroll
  for (int j = 0; j < G; ++j) buf[0][j] = load(j);
#pragma unroll
  for (int grp = 0; grp < NG; ++grp) {
    sched_fence();
    if (grp + 1 < NG) {
#pragma unroll
      for (int j = 0; j < G; ++j) buf[(grp + 1) & 1][j] = load((grp + 1) * G + j);
    }
#pragma unroll
    for (int j = 0; j < G; ++j) use(grp * G + j, buf[grp & 1][j]);
  }
  sched_fence();
}

// acc[nb] += A_nb * B for NB row blocks of a row-major LDS tile that share the register
// fragments bf:  acc[nb][row r][col c] += sum_k tile[row0 + nb*32 + r][k] * B[k][c].
template <typename T, int D, int NB, int NF, int GRP = 4>
SA_DEV void mma_rows(f32x16 (&acc)[NB], const T* tile, int row0, const typename Elem<T>::Frag (&bf)[NF],
                     int lane) {
  using G_ = TileGeom<T, D>;
  static_assert(NF == G_::NF, "one register fragment per 2*VEC slice of the head dimension");
  constexpr int PITCH = G_::PITCH, VEC = Elem<T>::VEC;
  const int c = lane & 31, h = lane >> 5;
  constexpr int N = NB * NF, G = N < GRP ? N : GRP;
  // row0 is a multiple of 32, so the swizzle of this lane's rows depends on c alone
  const T* base = tile + (row0 + c) * PITCH;
  const int sw = G_::swz(c);
  pipeline<N, G>(
      [&](int it) {
        const int nb = it / NF, g = it % NF;
        return *reinterpret_cast<const typename Elem<T>::Frag*>(base + nb * 32 * PITCH + (((g * 2 + h) ^ sw) * VEC));
      },
      [&](int it, const typename Elem<T>::Frag& a) { mma(acc[it / NF], a, bf[it % NF]); });
}

// acc[m] += X^T * P for one 32-row block `rb` of a row-major LDS tile X[rows][cols]:
//   acc[m][row x][col c] += sum_r X[rb*32 + r][m*32 + x] * P[r][c]
// where P is a C fragment (its rows are the contraction index).  P is rounded to T
// before the product, as the operand of a 16-bit MFMA must be.
template <typename T, int D, int NM>
SA_DEV void mma_tr(f32x16 (&acc)[NM], const T* X, int rb, const f32x16& P, int lane) {
  using E = Elem<T>;
  using G_ = TileGeom<T, D>;
  static_assert(NM == G_::DB, "one accumulator per 32-wide block of the head dimension");
  constexpr int PITCH = G_::PITCH;
  if constexpr (E::HALF) {
    using Frag = typename E::Frag;
    const int g16 = lane >> 4, j = lane & 15;
    const int h = g16 >> 1, mb = (g16 & 1) * 16;
    // This lane's source address for the transposing read: row (j/4) of a 4-row run, the
    // 4 columns starting at 4*(j%4); the instruction hands lane j column j of the 4x16
    // block, i.e. 4 consecutive rows of one column.  Two runs, 8 rows apart, make the
    // 8 contraction slots of one fragment.
    const int r_lo = 4 * h + (j >> 2);            // row inside a 16-row half, first run
    const int col = mb + 4 * (j & 3);             // element column inside a 32-wide block
    const T* blk = X + rb * 32 * PITCH;
    Frag b[2];
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int e = 0; e < 8; ++e) b[half][e] = (T)P[half * 8 + e];
    constexpr int N = 2 * NM, G = N < 4 ? N : 4;
    pipeline<N, G>(
        [&](int it) {
          const int half = it / NM, m = it % NM;
          const T* p0 = blk + G_::off(half * 16 + r_lo, m * 32 + col);
          const T* p1 = blk + G_::off(half * 16 + 8 + r_lo, m * 32 + col);
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p0));
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p1));
          return __builtin_bit_cast(Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        },
        [&](int it, const Frag& a) { mma(acc[it % NM], a, b[it / NM]); });
  } else {
    const int c = lane & 31, h = lane >> 5;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const T* row = X + (rb * 32 + crow(i, h)) * PITCH + c;
#pragma unroll
      for (int m = 0; m < NM; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(row[m * 32], P[i], acc[m], 0, 0, 0);
    }
  }
}

// Variants of the two products for a wave that owns NQ 32-wide blocks of the "owner" index:
// every fragment fetched from LDS is multiplied against NQ register fragments, which
// divides the LDS traffic per MFMA by NQ.
template <typename T, int D, int NQ, int NB, int NF>
SA_DEV void mma_rows_n(f32x16 (&acc)[NQ][NB], const T* tile, int row0,
                       const typename Elem<T>::Frag (&bf)[NQ][NF], int lane) {
  using G_ = TileGeom<T, D>;
  static_assert(NF == G_::NF, "one register fragment per 2*VEC slice of the head dimension");
  constexpr int PITCH = G_::PITCH, VEC = Elem<T>::VEC;
  const int c = lane & 31, h = lane >> 5;
  constexpr int N = NB * NF, G = N < 4 ? N : 4;
  const T* base = tile + (row0 + c) * PITCH;
  const int sw = G_::swz(c);
  pipeline<N, G>(
      [&](int it) {
        const int nb = it / NF, g = it % NF;
        return *reinterpret_cast<const typename Elem<T>::Frag*>(base + nb * 32 * PITCH + (((g * 2 + h) ^ sw) * VEC));
      },
      [&](int it, const typename Elem<T>::Frag& a) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) mma(acc[q][it / NF], a, bf[q][it % NF]);
      });
}

// Round a C fragment to T and pack it as the two B fragments (16 contraction rows each)
// that mma_tr_n consumes.
template <typename T> SA_DEV void pack_c(typename Elem<T>::Frag (&b)[2], const f32x16& P) {
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int e = 0; e < 8; ++e) b[half][e] = (T)P[half * 8 + e];
}

// Two products that share the pipeline: acc0 += A0 * B0 and acc1 += A1 * B1, where A0 and A1
// are the same 32 rows of two row-major LDS tiles (scores from Q and K, dP from dO and V).
// One fragment stream means one exposed LDS latency instead of two.
template <typename T, int D, int NF, int GRP = 4>
SA_DEV void mma_rows_pair(f32x16& acc0, f32x16& acc1, const T* tile0, const T* tile1, int row0,
                          const typename Elem<T>::Frag (&b0)[NF], const typename Elem<T>::Frag (&b1)[NF],
                          int lane) {
  using G_ = TileGeom<T, D>;
  using Frag = typename Elem<T>::Frag;
  static_assert(NF == G_::NF, "one register fragment per 2*VEC slice of the head dimension");
  constexpr int PITCH = G_::PITCH, VEC = Elem<T>::VEC;
  const int c = lane & 31, h = lane >> 5;
  constexpr int N = 2 * NF, G = N < GRP ? N : GRP;
  const int off = (row0 + c) * PITCH;
  const int sw = G_::swz(c);
  pipeline<N, G>(
      [&](int it) {
        const T* base = (it < NF ? tile0 : tile1) + off;
        return *reinterpret_cast<const Frag*>(base + ((((it % NF) * 2 + h) ^ sw) * VEC));
      },
      [&](int it, const Frag& a) {
        if (it < NF) mma(acc0, a, b0[it]);
        else mma(acc1, a, b1[it - NF]);
      });
}

// Likewise for the transposed products: acc0[m] += X0^T * P0 and acc1[m] += X1^T * P1 over the
// same 32-row block of two tiles (dV from dO and P, dK from Q and dS).  16-bit types only.
template <typename T, int D, int NM, int GRP = 4>
SA_DEV void mma_tr_pair(f32x16 (&acc0)[NM], f32x16 (&acc1)[NM], const T* X0, const T* X1, int rb,
                        const f32x16& P0, const f32x16& P1, int lane) {
  using E = Elem<T>;
  using G_ = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(E::HALF && NM == G_::DB, "transposing reads exist for 16-bit elements only");
  constexpr int PITCH = G_::PITCH;
  const int g16 = lane >> 4, j = lane & 15;
  const int r_lo = 4 * (g16 >> 1) + (j >> 2);
  const int col = (g16 & 1) * 16 + 4 * (j & 3);
  Frag b0[2], b1[2];
  pack_c<T>(b0, P0);
  pack_c<T>(b1, P1);
  constexpr int N = 4 * NM, G = N < GRP ? N : GRP;
  pipeline<N, G>(
      [&](int it) {
        const int k2 = it % (2 * NM), half = k2 / NM, m = k2 % NM;
        const T* blk = (it < 2 * NM ? X0 : X1) + rb * 32 * PITCH;
        const T* p0 = blk + G_::off(half * 16 + r_lo, m * 32 + col);
        const T* p1 = blk + G_::off(half * 16 + 8 + r_lo, m * 32 + col);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p0));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p1));
        return __builtin_bit_cast(Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      },
      [&](int it, const Frag& a) {
        const int k2 = it % (2 * NM), half = k2 / NM, m = k2 % NM;
        if (it < 2 * NM) mma(acc0[m], a, b0[half]);
        else mma(acc1[m], a, b1[half]);
      });
}

// 16-bit only: acc[q][m] += X^T * B[q] for 32-row block rb of tile X, B[q] packed by pack_c.
template <typename T, int D, int NQ, int NM, int GRP = 4>
SA_DEV void mma_tr_n(f32x16 (&acc)[NQ][NM], const T* X, int rb, const typename Elem<T>::Frag (&b)[NQ][2],
                     int lane) {
  using E = Elem<T>;
  using G_ = TileGeom<T, D>;
  using Frag = typename E::Frag;
  static_assert(E::HALF && NM == G_::DB, "transposing reads exist for 16-bit elements only");
  constexpr int PITCH = G_::PITCH;
  const int g16 = lane >> 4, j = lane & 15;
  const int h = g16 >> 1, mb = (g16 & 1) * 16;
  const int r_lo = 4 * h + (j >> 2);
  const int col = mb + 4 * (j & 3);
  const T* blk = X + rb * 32 * PITCH;
  constexpr int N = 2 * NM, G = N < GRP ? N : GRP;
  pipeline<N, G>(
      [&](int it) {
        const int half = it / NM, m = it % NM;
        const T* p0 = blk + G_::off(half * 16 + r_lo, m * 32 + col);
        const T* p1 = blk + G_::off(half * 16 + 8 + r_lo, m * 32 + col);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p0));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((SA_LDS s16x4*)(p1));
        return __builtin_bit_cast(Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      },
      [&](int it, const Frag& a) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) mma(acc[q][it % NM], a, b[q][it / NM]);
      });
}

// Asynchronous copy of [ROWS][D] row-major global tiles into swizzled LDS tiles with
// buffer_load_dwordx4 ... lds: the data never passes through registers.  One instruction moves
// 1 KiB (64 lanes x 16 bytes) to consecutive LDS addresses, i.e. 1024/(2*D) whole rows; lane l
// therefore fetches, for physical chunk l % CPR of its row, the logical chunk that the swizzle
// maps there.  The NW waves of a workgroup interleave instruction by instruction.  Completion
// is tracked by vmcnt; visibility to the other waves needs a barrier after the wait.
//
// Tiles are issued in ascending order.  Offsets are 32-bit byte offsets inside one (batch, head)
// slice: the host checks that T * row_stride * sizeof(T) fits.
template <typename T, int D, int ROWS, int NW, bool ASM_COPIES = false> struct AsyncTile {
  using G_ = TileGeom<T, D>;
  static_assert(G_::SWZ, "asynchronous tiles use the swizzled layout");
  static constexpr int ROW_BYTES = D * (int)sizeof(T);
  static constexpr int RPI = 1024 / ROW_BYTES;             // rows per instruction
  static constexpr int NI = ROWS / RPI;                     // instructions per tile
  static_assert(ROWS % (RPI * NW) == 0, "tile must split evenly over the waves");
  // The swizzle of a lane's row repeats every 16 rows; consecutive instructions of a wave are NW*RPI rows
  // apart, so a lane needs 16 / (NW*RPI) different offsets when that is less than 16 (wide rows, few waves).
  static constexpr int NVO = (RPI * NW) % 16 == 0 ? 1 : 16 / (RPI * NW);
  static_assert((RPI * NW * NVO) % 16 == 0, "the swizzle must repeat after NVO instructions");
  static constexpr int PER_WAVE = NI / NW;                  // instructions per wave per tile

  // Buffer addressing: a resource descriptor for the (batch, head) slice whose extent ends with
  // the last valid row, one per-lane byte offset that never changes, and a scalar byte offset
  // that carries the tile and the instruction.  No vector arithmetic per load, and rows past
  // the last valid one come back as zeros from the hardware's range check.
  // With ASM_COPIES the copies are written as assembly: the compiler cannot tell which LDS reads a
  // copy may overlap, so for copies it knows about it waits for ALL of them (vmcnt 0) before the
  // first transposing LDS read that follows and before every barrier.  A ring of two stages loses
  // nothing by that (measured), a ring of three would lose its point.  Completion is the caller's
  // business either way (wait_loads + barrier).
  u32x4 rsrc;                      // descriptor words for the assembly form
  __amdgpu_buffer_rsrc_t brsrc;    // the same descriptor for the builtin
  uint32_t voff[NVO]; // byte offset of this lane's 16 bytes inside instruction 0 of tile 0 (per swizzle phase)
  uint32_t soff;      // wave-uniform byte offset of the next tile
  uint32_t istep;     // bytes between rows of consecutive instructions of one wave
  uint32_t tstep;     // bytes between consecutive tiles

  SA_DEV void init(const T* gbase, int64_t row_stride, int first_row, int last_row, int wave, int lane) {
    constexpr uint32_t ES = (uint32_t)sizeof(T);
    const int lrow = lane / G_::CPR, pch = lane % G_::CPR;
    const uint32_t rs = (uint32_t)row_stride;
    const uint32_t bytes = ((uint32_t)last_row * rs + (uint32_t)D) * ES;
    const uint64_t addr = reinterpret_cast<uint64_t>(gbase);
    rsrc[0] = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
    rsrc[1] = (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(addr >> 32) & 0xFFFFu));   // stride 0
    rsrc[2] = (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes);
    rsrc[3] = 0x00020000u;
    brsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(gbase), 0, (int)bytes, 0x00020000);
#pragma unroll
    for (int j = 0; j < NVO; ++j)
      voff[j] = ((uint32_t)(wave * RPI + lrow) * rs +
                 (uint32_t)((pch ^ G_::swz((j * NW + wave) * RPI + lrow)) * Elem<T>::VEC)) * ES;
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)first_row * rs * ES));
    istep = (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(NW * RPI) * rs * ES));
    tstep = (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)ROWS * rs * ES));
  }
  // instructions [I0, I1) of this wave's share of the next tile
  template <int I0, int I1> SA_DEV void issue_part(T* tile, int wave) const {
    static_assert(0 <= I0 && I0 <= I1 && I1 <= PER_WAVE, "instruction range");
#pragma unroll
    for (int i = I0; i < I1; ++i) {
      T* dst = tile + (i * NW + wave) * RPI * D;           // wave-uniform
      if constexpr (ASM_COPIES) {
        // both scalars are wave-uniform by construction; readfirstlane makes that known to the compiler
        const uint32_t lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(SA_LDS void*)dst);
        const uint32_t so = (uint32_t)__builtin_amdgcn_readfirstlane((int)(soff + (uint32_t)i * istep));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(lds_addr), "v"(voff[i % NVO]), "s"(rsrc), "s"(so)
                     : "memory", "m0");
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(brsrc, (SA_LDS void*)dst, 16, (int)voff[i % NVO],
                                                 (int)(soff + (uint32_t)i * istep), 0, 0);
      }
    }
  }
  SA_DEV void issue(T* tile, int wave) const { issue_part<0, PER_WAVE>(tile, wave); }
  SA_DEV void advance() { soff += tstep; }
};

// Asynchronous copy of one float per active lane to consecutive LDS words starting at dst
// (wave-uniform); as assembly for the same reason as the tile copies above when ASM_COPIES is set.
template <bool ASM_COPIES = false> SA_DEV void async_copy_f32(const float* src, float* dst) {
  if constexpr (ASM_COPIES) {
    const uint32_t lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(SA_LDS void*)dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :
                 : "s"(lds_addr), "v"(src)
                 : "memory", "m0");
  } else {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src, (SA_LDS void*)dst, 4, 0, 0);
  }
}

// s_waitcnt vmcnt(N), other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
template <int N> SA_DEV void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Waits until at most min(ahead, MAXA) tiles of LPT loads each are outstanding (ahead is wave-uniform).
template <int LPT, int MAXA> SA_DEV void wait_tiles(int ahead) {
  if constexpr (MAXA <= 0) {
    wait_loads<0>();
  } else {
    if (ahead >= MAXA) wait_loads<MAXA * LPT>();
    else wait_tiles<LPT, MAXA - 1>(ahead);
  }
}

// Cooperative copy of a [ROWS][D] row-major global tile into registers and on into an
// LDS tile.  Rows are clamped to `last_row` so that a ragged final tile reads valid
// memory (the values are masked by the caller).
template <typename T, int D, int ROWS, int NT> struct Stager {
  using E = Elem<T>;
  using Frag = typename E::Frag;
  static constexpr int CPR = D / E::VEC;                 // 16-byte chunks per row
  static constexpr int TOTAL = ROWS * CPR;
  static constexpr int N = (TOTAL + NT - 1) / NT;
  static constexpr int PITCH = TileGeom<T, D>::PITCH;
  Frag regs[N];

  SA_DEV void load(const T* base, int64_t row_stride, int row0, int last_row, int tid) {
#pragma unroll
    for (int it = 0; it < N; ++it) {
      const int ch = tid + it * NT;
      if (TOTAL % NT == 0 || ch < TOTAL) {
        const int r = ch / CPR, col = (ch % CPR) * E::VEC;
        int gr = row0 + r;
        gr = gr < last_row ? gr : last_row;
        regs[it] = *reinterpret_cast<const Frag*>(base + (int64_t)gr * row_stride + col);
      }
    }
  }
  SA_DEV void store(T* tile, int tid) const {
#pragma unroll
    for (int it = 0; it < N; ++it) {
      const int ch = tid + it * NT;
      if (TOTAL % NT == 0 || ch < TOTAL) {
        const int r = ch / CPR, col = (ch % CPR) * E::VEC;
        *reinterpret_cast<Frag*>(tile + TileGeom<T, D>::off(r, col)) = regs[it];
      }
    }
  }
};

// Hardware hands workgroup i to XCD i % 8 (each XCD has its own L2).  Map block ids so that
// all tiles of one (batch, head) run on one XCD, in consecutive dispatch slots -- neighbouring
// tiles then share that L2 for the keys and values they have in common -- and so that the
// (batch, head) pairs are dealt round-robin over the XCDs: with ragged sequence lengths every
// XCD then receives a mix of long and short batches instead of a contiguous block of one.
// Tiles are visited from the end of the sequence backwards: the long-window tiles start first.
// The first n_start tiles of a sequence are cheaper than the rest (a query tile whose window is still
// growing).  They are taken out of that order and dispatched last on every XCD, tile by tile over its
// (batch, head) pairs, cheapest at the very end: the last workgroups of a launch, which run while part
// of the chip is already idle, are then the short ones.  Measured on an MI355X: dQ 1.5 % faster at
// B=4, H=16, T=16384, D=128 and 3-4 % on small problems; the long-window forward kernel loses 1 % (tiles
// of one sequence that share keys in L2 no longer run side by side) and passes n_start = 0.  A tail that
// keeps the tiles of a (batch, head) pair together measured slower than either.
SA_DEV void tile_coords(int bid, int n_blocks, int n_tiles, int& bh, int& tile, int n_start = 0) {
  const int nbh = n_blocks / n_tiles;
  int logical;
  if ((nbh & 7) == 0) {
    const int x = bid & 7, idx = bid >> 3;
    const int nb = nbh >> 3;
    const int ns = 2 * n_start <= n_tiles ? n_start : 0;
    const int nl = n_tiles - ns;
    if (idx < nb * nl) {
      bh = (idx / nl) * 8 + x;
      logical = idx % nl;
    } else {
      const int r = idx - nb * nl;
      bh = (r % nb) * 8 + x;
      logical = nl + r / nb;
    }
  } else {
    const int per = n_blocks >> 3, rem = n_blocks & 7;
    const int x = bid & 7, idx = bid >> 3;
    const int l = x * per + (x < rem ? x : rem) + idx;
    bh = l / n_tiles;
    logical = l % n_tiles;
  }
  tile = n_tiles - 1 - logical;
}
// The same for key tiles of ROWS keys.  There the short tiles are the last n_end ones below a sequence's length
// L (the queries that see those keys stop at L), so the order depends on L: tiles below them and the empty
// tiles beyond L come first, then, tile by tile over the XCD's (batch, head) pairs, the n_end tiles that lead up to L.
// Returns the clamped length of the pair's sequence as well.
#ifndef SA_ORDER_KEYS
#define SA_ORDER_KEYS 1
#endif
SA_DEV void key_tile_coords(int bid, int n_blocks, int n_tiles, int n_end, int ROWS, int H, int T,
                            const int32_t* lens, int64_t lens_stride, int& bh, int& tile, int& L) {
  const int nbh = n_blocks / n_tiles;
  const int ns = (SA_ORDER_KEYS && (nbh & 7) == 0 && 2 * n_end <= n_tiles) ? n_end : 0;
  if (ns == 0) {
    tile_coords(bid, n_blocks, n_tiles, bh, tile);
  } else {
    const int x = bid & 7, idx = bid >> 3, nb = nbh >> 3, nl = n_tiles - ns;
    if (idx < nb * nl) {
      bh = (idx / nl) * 8 + x;
      tile = nl - 1 - idx % nl;      // position among the tiles that are not in the tail
    } else {
      const int r = idx - nb * nl;
      bh = (r % nb) * 8 + x;
      tile = -1 - r / nb;            // -1 - j: tail tile j, counted towards L
    }
  }
  L = T;
  if (lens) {
    L = lens[(int64_t)(bh / H) * lens_stride];
    L = L < 0 ? 0 : (L > T ? T : L);
  }
  if (ns != 0) {
    const int live = (L + ROWS - 1) / ROWS < n_tiles ? (L + ROWS - 1) / ROWS : n_tiles;   // tiles with a key below L
    const int a = live > ns ? live - ns : 0;                                               // tiles before the tail
    tile = tile < 0 ? a + (-1 - tile) : (tile < a ? tile : tile + ns);
  }
}

// Number of leading query tiles of ROWS rows whose windows are still growing: rows below back_contexts chunks.
SA_DEV int growing_tiles(int C, int R, int T, int ROWS) {
  const int64_t rows = (int64_t)C * (int64_t)R;
  return rows >= (int64_t)T ? 0x3fffffff : (int)((rows + ROWS - 1) / ROWS);
}

// Write four consecutive fp32 values as four elements of T.
template <typename T> SA_DEV void store4(T* dst, float a, float b, float c, float d) {
  typename Elem<T>::Quad q;
  q[0] = (T)a; q[1] = (T)b; q[2] = (T)c; q[3] = (T)d;
  *reinterpret_cast<typename Elem<T>::Quad*>(dst) = q;
}

// Zero rows [row0, row1) of a contiguous [*, D] matrix with the whole workgroup.
template <typename T, int D, int NT> SA_DEV void zero_rows(T* base, int row0, int row1, int tid) {
  using E = Elem<T>;
  constexpr int CPR = D / E::VEC;
  const int total = (row1 - row0) * CPR;
  typename E::Frag z;
#pragma unroll
  for (int e = 0; e < E::VEC; ++e) z[e] = (T)0.0f;
  for (int ch = tid; ch < total; ch += NT)
    *reinterpret_cast<typename E::Frag*>(base + (int64_t)row0 * D + (int64_t)ch * E::VEC) = z;
}

// Transposed store of DB accumulator blocks holding X^T[d][row] into X[row][d]:
// register group (4 consecutive d) -> one 8- or 16-byte store.
template <typename T, int D, int DB>
SA_DEV void store_acc_T(T* row_ptr, const f32x16 (&acc)[DB], float mul, int h) {
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = m * 32 + 8 * g + 4 * h;
      if (d < D)
        store4<T>(row_ptr + d, acc[m][4 * g] * mul, acc[m][4 * g + 1] * mul, acc[m][4 * g + 2] * mul,
                  acc[m][4 * g + 3] * mul);
    }
}

// The same store through a wave-private LDS patch, so that global memory sees whole rows: the
// accumulators hold X^T (a lane owns one row, four consecutive d per register group), which
// stored directly puts 8 bytes per lane on 32 different rows per instruction.  Here the lane
// writes its row into the patch, and the wave reads it back four rows at a time, 16 lanes x 16
// bytes per row, for 1 KiB stores of contiguous rows.  16-bit types only.
template <typename T, int D> struct RowPatch {
  static constexpr int PITCH = D + 8;              // elements: rows stay 16-byte aligned, 4 banks apart
  static constexpr int ELEMS = 32 * PITCH;         // per wave
  static constexpr int CPR = D / 8;                // 16-byte chunks per row
  static constexpr int RPI = 64 / CPR;             // rows per store instruction
};
template <typename T, int D, int DB>
SA_DEV void store_rows_coalesced(T* patch, T* out_rows, int rows_valid, const f32x16 (&acc)[DB], float mul,
                                 int lane) {
  using P = RowPatch<T, D>;
  static_assert(Elem<T>::HALF && DB * 32 == D, "16-bit types, one accumulator block per 32 columns");
  const int c = lane & 31, h = lane >> 5;
#pragma unroll
  for (int m = 0; m < DB; ++m)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      store4<T>(patch + c * P::PITCH + m * 32 + 8 * g + 4 * h, acc[m][4 * g] * mul, acc[m][4 * g + 1] * mul,
                acc[m][4 * g + 2] * mul, acc[m][4 * g + 3] * mul);
  const int rr = lane / P::CPR, ch = lane % P::CPR;
#pragma unroll
  for (int j = 0; j < 32 / P::RPI; ++j) {
    const int row = j * P::RPI + rr;
    const u32x4 v16 = *reinterpret_cast<const u32x4*>(patch + row * P::PITCH + ch * 8);
    if (row < rows_valid) *reinterpret_cast<u32x4*>(out_rows + (int64_t)row * D + ch * 8) = v16;
  }
}

// Division of a position below 2^31 by the chunk size without the hardware's 30-instruction emulation:
// with l = ceil(log2(d)) and m = ceil(2^(31+l) / d) (m < 2^32), n / d == (n * m) >> (31 + l) for every
// 0 <= n < 2^31 (Granlund and Montgomery, "Division by invariant integers using multiplication", 1994).
struct ChunkDiv {
  uint32_t mul, shift;
};
constexpr ChunkDiv chunk_div(int d) {   // d >= 1
  uint32_t l = 0;
  while ((1ull << l) < (unsigned long long)d) ++l;
  const unsigned long long two = 1ull << (31 + l);
  return ChunkDiv{(uint32_t)((two + (unsigned long long)d - 1) / (unsigned long long)d), 31 + l};
}
constexpr int div_by(int n, ChunkDiv c) { return (int)(((unsigned long long)(uint32_t)n * c.mul) >> c.shift); }
static_assert(div_by(0x7fffffff, chunk_div(1)) == 0x7fffffff && div_by(12345, chunk_div(1)) == 12345, "d = 1");
static_assert(div_by(0x7fffffff, chunk_div(2)) == 0x3fffffff && div_by(0x7ffffffe, chunk_div(0x7fffffff)) == 0 &&
              div_by(0x7fffffff, chunk_div(0x7fffffff)) == 1, "extremes");
static_assert(div_by(2999, chunk_div(10)) == 299 && div_by(3000, chunk_div(10)) == 300 && div_by(95, chunk_div(96)) == 0 &&
              div_by(96, chunk_div(96)) == 1 && div_by(0x7fffffff, chunk_div(10)) == 214748364 &&
              div_by(0x7fffffff, chunk_div(3)) == 715827882 && div_by(0x7fffffff, chunk_div(641)) == 3350208 &&
              div_by(65535, chunk_div(256)) == 255 && div_by(0x7fffffff, chunk_div(10000)) == 214748, "samples");

struct FwdParams {
  const void *q, *k, *v;
  void* o;          // contiguous [B,H,T,D]
  float* lse;       // contiguous [B,H,T] or null
  const int32_t* lens;  // null: every sequence has length T
  int64_t lens_stride;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st;  // element strides
  int B, H, T, C, R;
  float scale_log2e;  // sm_scale * log2(e); sign carried separately
  int n_tiles;        // query tiles per (b,h)
  ChunkDiv cdiv;      // division by C
};

struct BwdParams {
  const void *q, *k, *v, *d_o;
  const float *lse, *delta;   // contiguous [B,H,T]
  void *dq, *dk, *dv;         // contiguous [B,H,T,D]
  const int32_t* lens;
  int64_t lens_stride;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, do_sb, do_sh, do_st;
  int B, H, T, C, R;
  float scale, scale_log2e;
  int n_tiles;
  // Set only for a dQ kernel that forms the row sums itself (delta_out != null): the forward output, its
  // element strides, and where the sums go for the dK/dV kernel that runs after it.  `delta` is then unused.
  const void* o;
  int64_t o_sb, o_sh, o_st;
  float* delta_out;
  ChunkDiv cdiv;      // division by C
};

struct DeltaParams {
  const void *o, *d_o;
  float* delta;
  int64_t o_sb, o_sh, o_st, do_sb, do_sh, do_st;
  int B, H, T;
};

}  // namespace sa
