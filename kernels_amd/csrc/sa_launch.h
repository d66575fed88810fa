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
template <typename T> struct Cfg {
  static constexpr int NW = 4;                                   // waves per workgroup
  static constexpr int FWD_TK = sizeof(T) == 4 ? 32 : 64;        // keys per forward step
  static constexpr int DQ_TK = 32;                               // keys per dQ step
  static constexpr int DKDV_TQ = 32;                             // queries per dK/dV step
};

}  // namespace sa
