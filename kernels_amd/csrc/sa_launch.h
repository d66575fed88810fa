// Host-side launch entry points, one explicit instantiation per element type.
// Each returns 0, a positive hipError_t, or a negative SA_ERR_* code.
#pragma once
#include "../../include/streaming_attention.h"
#include "sa_common.h"

#define SA_OK 0

namespace sa {


template <typename T, int DGROUP> int launch_fwd(const FwdParams& p, int D, hipStream_t st);
template <typename T, int DGROUP> int launch_delta(const DeltaParams& p, int D, hipStream_t st);
template <typename T, int DGROUP> int launch_dq(const BwdParams& p, int D, hipStream_t st);
template <typename T, int DGROUP> int launch_dkdv(const BwdParams& p, int D, hipStream_t st);

// tile sizes, shared between the launchers and sa_query()
#ifndef SA_FWD2_QB
#define SA_FWD2_QB 1
#endif
#ifndef SA_DQ2_TK
#define SA_DQ2_TK 64
#endif
#ifndef SA_DQ2_NST
#define SA_DQ2_NST 2
#endif
#ifndef SA_DKDV2_NW
#define SA_DKDV2_NW 4
#endif
#ifndef SA_DKDV2_TQ
#define SA_DKDV2_TQ 64
#endif
#ifndef SA_DKDV2_NST
#define SA_DKDV2_NST 2
#endif
#ifndef SA_DKDV3_MIN_CHUNK
#define SA_DKDV3_MIN_CHUNK 128
#endif
#ifndef SA_DKDV3_NST
#define SA_DKDV3_NST 3
#endif
#ifndef SA_FWD2_NST
#define SA_FWD2_NST 2
#endif
template <typename T> struct Cfg {
  static constexpr int NW = 4;                                   // waves per workgroup
  // 16-bit, D in {64, 128}: forward kernel with QB query blocks per wave and NST LDS stages
  // The forward and dQ kernels come in two widths, chosen per call from the chunk size:
  // 8 waves (256 queries) share each key tile among more waves, which pays once the
  // workgroup's queries lie in one chunk; with smaller chunks the union of the waves'
  // windows grows and 4 waves (128 queries) waste less of every tile.
  static constexpr int WIDE_NW = 8, NARROW_NW = 4;
  static constexpr int WIDE_CHUNK = 256;
  static constexpr bool wide(int chunk) { return chunk >= WIDE_CHUNK; }
  static constexpr int DQ2_TK = SA_DQ2_TK, DQ2_NST = SA_DQ2_NST;
  static constexpr int DKDV2_NW = SA_DKDV2_NW, DKDV2_TQ = SA_DKDV2_TQ, DKDV2_NST = SA_DKDV2_NST;
  // smallest chunk for which the software-pipelined dK/dV kernel is chosen (0x7fffffff: never)
  static constexpr int DKDV3_MIN_CHUNK = SA_DKDV3_MIN_CHUNK;
  // ... and only at head dimension 128: at 64 a block step has half the MFMAs for the same softmax
  // arithmetic, the loop is bound by its vector work and dkdv2 is faster (0.23 against 0.30 ms at
  // B=8, H=16, T=4096, chunk 128)
  static constexpr bool pipelined_dkdv(int chunk, int D) { return D == 128 && chunk >= DKDV3_MIN_CHUNK; }
  static constexpr int DKDV3_NST = SA_DKDV3_NST;
  static constexpr int FWD2_QB = SA_FWD2_QB;
  static constexpr int FWD2_NST = SA_FWD2_NST;
#ifdef SA_FWD2_DISABLE
  static constexpr bool fwd2(int) { return false; }
#else
  static constexpr bool fwd2(int D) { return sizeof(T) == 2 && (D == 64 || D == 128); }
#endif
#ifdef SA_FWD_TK16
  static constexpr int FWD_TK = sizeof(T) == 4 ? 32 : SA_FWD_TK16;
#else
  static constexpr int FWD_TK = sizeof(T) == 4 ? 32 : 64;        // keys per forward step
#endif
  static constexpr int DQ_TK = 32;                               // keys per dQ step
  static constexpr int DKDV_TQ = 32;                             // queries per dK/dV step
};

}  // namespace sa
