// Kernel instantiations for one element type and one kernel family.
// Compiled once per (SA_DTYPE_ID, SA_KIND) pair so that the families build in parallel.
//   SA_DTYPE_ID: 0 fp32, 1 fp16, 2 bf16        SA_KIND: 0 forward, 1 delta + dQ, 2 dK/dV
//   SA_DGROUP: 0 head dims 16..128, 1 head dim 256
#include <mutex>
#include "sa_launch.h"
#if SA_KIND == 0
#include "sa_fwd.h"
#ifndef SA_NO_ASM_KERNELS
#include "sa_fwd3.h"
#endif
#else
#include "sa_bwd.h"
#ifndef SA_NO_ASM_KERNELS
#include "sa_bwd3.h"
#include "sa_bwd4.h"
#endif
#include "sa_bwd_split.h"
#endif

namespace sa {

#if SA_DTYPE_ID == 0
using ElemT = float;
#elif SA_DTYPE_ID == 1
using ElemT = _Float16;
#elif SA_DTYPE_ID == 2
using ElemT = __bf16;
#else
#error "SA_DTYPE_ID must be 0, 1 or 2"
#endif

// Kernels whose dynamic LDS exceeds the 64 KiB default need the limit raised once per kernel
// and per device (the attribute belongs to the device that is current when it is set).  The
// outcome of that one call is kept and handed to every caller on that device.
struct PrepareState {
  static constexpr int kMaxDevices = 64;
  std::mutex mu;
  bool done[kMaxDevices] = {};
  int rc[kMaxDevices] = {};
};
template <typename K> static int prepare(K kernel, size_t lds_bytes, PrepareState& state) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= PrepareState::kMaxDevices) {
    return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  }
  std::lock_guard<std::mutex> lock(state.mu);
  if (!state.done[dev]) {
    state.rc[dev] = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    state.done[dev] = true;
  }
  return state.rc[dev];
}

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// SA_DGROUP 0 holds head dimensions 16..128, SA_DGROUP 1 holds 256 (built with different
// compiler options, see the Makefile).
#if SA_DGROUP == 0
#define SA_FOR_EACH_D(X) \
  switch (D) {           \
    case 16: X(16);      \
    case 32: X(32);      \
    case 64: X(64);      \
    case 128: X(128);    \
    default: return SA_ERR_HEAD_DIM; \
  }
#else
#define SA_FOR_EACH_D(X) \
  switch (D) {           \
    case 256: X(256);    \
    default: return SA_ERR_HEAD_DIM; \
  }
#endif

#if SA_KIND == 0
template <int D, int NW, bool SHORT> static int fwd2_launch(FwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  constexpr int TQ = NW * C::FWD2_QB * 32;
  // tile stages; the epilogue's row patches (one per wave) reuse the same memory
  constexpr size_t stages = (size_t)C::FWD2_NST * 2 * C::FWD_TK * D * sizeof(ElemT);
  constexpr size_t patches = (size_t)NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
  constexpr size_t lds = stages > patches ? stages : patches;
  auto kern = fwd2_kernel<ElemT, D, C::FWD2_QB, NW, C::FWD_TK, C::FWD2_NST, SHORT>;
  static PrepareState once;
  if (int rc = prepare(kern, lds, once)) return rc;
  p.n_tiles = (int)ceil_div(p.T, TQ);
  const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
  if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), lds, st, p);
  return (int)hipGetLastError();
}
// hand-scheduled loop, one wave per SIMD, 64 queries per wave (head dimension 128)
template <int D> static int fwd3_launch(FwdParams p, hipStream_t st) {
#ifdef SA_NO_ASM_KERNELS
  (void)p; (void)st;
  return SA_ERR_HEAD_DIM;
#else
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D) && D == 128) {
    constexpr int NW = 4, TQ = NW * 64, NST = 4;
    constexpr size_t stages = (size_t)NST * 2 * 64 * D * sizeof(ElemT);
    constexpr size_t patches = (size_t)NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
    constexpr size_t lds = stages > patches ? stages : patches;
    auto kern = fwd3_kernel<ElemT, D, NST>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TQ);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), lds, st, p);
    return (int)hipGetLastError();
  } else {
    return SA_ERR_HEAD_DIM;
  }
#endif
}
template <int D> static int fwd_d(FwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D)) {
    if constexpr (D == 128) {
      if (launch_choice(D, p.C, p.R).fwd == FWD_PIPELINED) return fwd3_launch<D>(p, st);
    }
    // windows of less than 1024 keys (the table's first two window classes) run the short-window form
    // head dimension 256 exists in the 4-wave shape only: a wave then has all 512 registers of its SIMD lane
    if constexpr (D > 128) {
      if (window_class(p.C, p.R) <= 1) return fwd2_launch<D, C::NARROW_NW, true>(p, st);
      return fwd2_launch<D, C::NARROW_NW, false>(p, st);
    } else {
      if (window_class(p.C, p.R) <= 1) return fwd2_launch<D, C::NARROW_NW, true>(p, st);
      return fwd2_launch<D, C::NARROW_NW, false>(p, st);
    }
  } else {
    constexpr int TQ = C::NW * 32;
    constexpr size_t lds = (size_t)2 * 2 * C::FWD_TK * TileGeom<ElemT, D>::PITCH * sizeof(ElemT);
    auto kern = fwd_kernel<ElemT, D, C::NW, C::FWD_TK>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TQ);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(C::NW * 64), lds, st, p);
    return (int)hipGetLastError();
  }
}
template <> int launch_fwd<ElemT, SA_DGROUP>(const FwdParams& p, int D, hipStream_t st) {
#define X(d) return fwd_d<d>(p, st)
  SA_FOR_EACH_D(X)
#undef X
}
#elif SA_KIND == 1
template <int D> static int delta_d(const DeltaParams& p, hipStream_t st) {
  constexpr int RPB = 256 / (D / Elem<ElemT>::VEC);
  const int64_t rows = (int64_t)p.B * p.H * p.T;
  const int64_t blocks = ceil_div(rows, RPB);
  if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
  hipLaunchKernelGGL((delta_kernel<ElemT, D>), dim3((unsigned)blocks), dim3(256), 0, st, p);
  return (int)hipGetLastError();
}
template <> int launch_delta<ElemT, SA_DGROUP>(const DeltaParams& p, int D, hipStream_t st) {
#define X(d) return delta_d<d>(p, st)
  SA_FOR_EACH_D(X)
#undef X
}
template <int D, int NW> static int dq2_launch(BwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  constexpr int TQ = NW * 32;
  constexpr size_t stages = (size_t)C::DQ2_NST * 2 * C::DQ2_TK * D * sizeof(ElemT);
  constexpr size_t patches = (size_t)NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
  constexpr size_t lds = stages > patches ? stages : patches;
  auto kern = dq2_kernel<ElemT, D, NW, C::DQ2_TK, C::DQ2_NST>;
  static PrepareState once;
  if (int rc = prepare(kern, lds, once)) return rc;
  p.n_tiles = (int)ceil_div(p.T, TQ);
  const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
  if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), lds, st, p);
  return (int)hipGetLastError();
}
// hand-scheduled loop, one wave per SIMD, 64 queries per wave (head dimension 128)
template <int D> static int dq3_launch(BwdParams p, hipStream_t st) {
#ifdef SA_NO_ASM_KERNELS
  (void)p; (void)st;
  return SA_ERR_HEAD_DIM;
#else
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D) && D == 128) {
    constexpr int NW = 4, TQ = NW * 64, NST = 4;
    constexpr size_t stages = (size_t)NST * 2 * 64 * D * sizeof(ElemT);
    constexpr size_t patches = (size_t)NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
    constexpr size_t lds = stages > patches ? stages : patches;
    auto kern = dq3_kernel<ElemT, D, NST>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TQ);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), lds, st, p);
    return (int)hipGetLastError();
  } else {
    return SA_ERR_HEAD_DIM;
  }
#endif
}
template <int D> static int dq_d(BwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D)) {
    if constexpr (D == 128) {
      if (launch_choice(D, p.C, p.R).dq == DQ_PIPELINED) return dq3_launch<D>(p, st);
    }
    return dq2_launch<D, C::NARROW_NW>(p, st);
  } else {
    if (p.delta_out) return SA_ERR_ARG;
    constexpr int TQ = C::NW * 32;
    constexpr size_t lds = (size_t)2 * 2 * C::DQ_TK * TileGeom<ElemT, D>::PITCH * sizeof(ElemT);
    auto kern = dq_kernel<ElemT, D, C::NW, C::DQ_TK>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TQ);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(C::NW * 64), lds, st, p);
    return (int)hipGetLastError();
  }
}
template <> int launch_dq<ElemT, SA_DGROUP>(const BwdParams& p, int D, hipStream_t st) {
#define X(d) return dq_d<d>(p, st)
  SA_FOR_EACH_D(X)
#undef X
}
#else
template <int D> static int dkdv3_launch(BwdParams p, hipStream_t st) {
#ifdef SA_NO_ASM_KERNELS
  (void)p; (void)st;
  return SA_ERR_HEAD_DIM;
#else
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D) && D == 128) {
    constexpr int TKB = 128, TQ = 64;
    // tile stages; the epilogue's row patches (one per wave) reuse the same memory
    constexpr size_t stages = (size_t)C::DKDV3_NST * (2 * TQ * D * sizeof(ElemT) + 2 * TQ * sizeof(float));
    constexpr size_t patches = (size_t)4 * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
    constexpr size_t lds = stages > patches ? stages : patches;
    auto kern = dkdv3_kernel<ElemT, D, C::DKDV3_NST>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TKB);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), lds, st, p);
    return (int)hipGetLastError();
  } else {
    return SA_ERR_HEAD_DIM;
  }
#endif
}
// wave pairs: 8 waves (two per SIMD) own 128 keys
template <int D> static int dkdv_split_launch(BwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D) && D >= 64 && D <= 128) {
    constexpr int TKB = 128, TQ = 64, NST = 3, NW = 8;
    // tile stages followed by the pairs' exchange slots; the epilogue's row patches reuse the stages
    constexpr size_t stages = (size_t)NST * (2 * TQ * D * sizeof(ElemT) + 2 * TQ * sizeof(float));
    constexpr size_t patches = (size_t)NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
    static_assert(patches <= stages, "row patches must not reach the exchange slots");
    constexpr size_t lds = stages + (size_t)4 * 2 * 2048;
    auto kern = dkdv_split_kernel<ElemT, D, NST>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TKB);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), lds, st, p);
    return (int)hipGetLastError();
  } else {
    return SA_ERR_HEAD_DIM;
  }
}
template <int D> static int dkdv_d(BwdParams p, hipStream_t st) {
  using C = Cfg<ElemT>;
  if constexpr (C::fwd2(D)) {
    if constexpr (D >= 64) {   // a 64-byte row splits over four waves' copies, not over eight
      if (launch_choice(D, p.C, p.R).dkdv == DKDV_SPLIT) return dkdv_split_launch<D>(p, st);
    }
    // The pipelined kernel (head dimension 128) makes every wave walk the whole window of its
    // workgroup's 128 keys; that wastes nothing once a chunk holds at least those 128 keys.  Smaller
    // chunks go to the kernel whose waves skip the query tiles outside their own 32 keys' windows.
    if constexpr (D == 128) {
      if (launch_choice(D, p.C, p.R).dkdv == DKDV_PIPELINED) return dkdv3_launch<D>(p, st);
    }
    constexpr int TKB = C::DKDV2_NW * 32;
    constexpr size_t stages =
        (size_t)C::DKDV2_NST * (2 * C::DKDV2_TQ * D * sizeof(ElemT) + 2 * C::DKDV2_TQ * sizeof(float));
    constexpr size_t patches = (size_t)C::DKDV2_NW * RowPatch<ElemT, D>::ELEMS * sizeof(ElemT);
    constexpr size_t lds = stages > patches ? stages : patches;
    auto kern = dkdv2_kernel<ElemT, D, C::DKDV2_NW, C::DKDV2_TQ, C::DKDV2_NST>;
    static PrepareState once;
    if (int rc = prepare(kern, lds, once)) return rc;
    p.n_tiles = (int)ceil_div(p.T, TKB);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(C::DKDV2_NW * 64), lds, st, p);
    return (int)hipGetLastError();
  } else {
    constexpr int TKB = C::NW * 32;
    constexpr size_t lds =
        (size_t)2 * (2 * C::DKDV_TQ * TileGeom<ElemT, D>::PITCH * sizeof(ElemT) + 2 * C::DKDV_TQ * sizeof(float));
    p.n_tiles = (int)ceil_div(p.T, TKB);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_tiles;
    if (blocks > 0x7fffffffLL) return SA_ERR_TOO_LARGE;
    if constexpr (sizeof(ElemT) == 4 && D == 256) {
      // both accumulators and both resident rows do not fit a lane's registers: one launch per gradient
      auto kern_dv = dkdv_kernel<ElemT, D, C::NW, C::DKDV_TQ, 1>;
      auto kern_dk = dkdv_kernel<ElemT, D, C::NW, C::DKDV_TQ, 2>;
      static PrepareState once_dv, once_dk;
      if (int rc = prepare(kern_dv, lds, once_dv)) return rc;
      if (int rc = prepare(kern_dk, lds, once_dk)) return rc;
      hipLaunchKernelGGL(kern_dv, dim3((unsigned)blocks), dim3(C::NW * 64), lds, st, p);
      if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
      hipLaunchKernelGGL(kern_dk, dim3((unsigned)blocks), dim3(C::NW * 64), lds, st, p);
      return (int)hipGetLastError();
    } else {
      auto kern = dkdv_kernel<ElemT, D, C::NW, C::DKDV_TQ>;
      static PrepareState once;
      if (int rc = prepare(kern, lds, once)) return rc;
      hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(C::NW * 64), lds, st, p);
      return (int)hipGetLastError();
    }
  }
}
template <> int launch_dkdv<ElemT, SA_DGROUP>(const BwdParams& p, int D, hipStream_t st) {
#define X(d) return dkdv_d<d>(p, st)
  SA_FOR_EACH_D(X)
#undef X
}
#endif

}  // namespace sa
