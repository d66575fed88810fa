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
#ifndef SA_DKDV3_NST
#define SA_DKDV3_NST 3
#endif
#ifndef SA_FWD2_NST
#define SA_FWD2_NST 2
#endif
// ---- launch-configuration table -------------------------------------------------------------------
// The 16-bit kernels for head dimensions 64 and 128 exist in several shapes (256 in one); which one runs is read
// from a table indexed by head dimension, chunk-size class and window-size class.  The entries are
// the fastest variant measured on an MI355X at B=4, H=16, T=16384 (`bench.py --tune-sweep`, turned into
// sa_tune_table.inc by gen_tune_table.py); float16 and bfloat16 measured alike and share the entries.
enum FwdVariant : int { FWD_NARROW = 0,     // 4 waves (128 queries) per workgroup, two workgroups per CU
                        FWD_WIDE = 1,       // 8 waves (256 queries) share every key tile
                        FWD_VARIANTS = 2 };
enum DqVariant : int { DQ_NARROW = 0, DQ_WIDE = 1,
                       DQ_PIPELINED = 2,   // hand-scheduled loop, 4 waves of 64 queries (head dimension 128 only)
                       DQ_VARIANTS = 3 };
enum DkdvVariant : int { DKDV_BLOCKSKIP = 0,   // every wave skips the query tiles outside its own 32 keys' windows
                         DKDV_PIPELINED = 1,   // hand-scheduled loop, head dimension 128 only
                         DKDV_SPLIT = 2,       // wave pairs share 32 keys: one wave forms S and dV, the other dP and dK
                         DKDV_VARIANTS = 3 };
struct LaunchChoice { int fwd, dq, dkdv; };
constexpr int TUNE_CHUNK_CLASSES = 7;    // context_size < 32, < 64, < 128, < 256, < 512, < 1024, >= 1024
constexpr int TUNE_WINDOW_CLASSES = 4;   // context_size * (back_contexts + 1) < 256, < 1024, < 4096, >= 4096
constexpr int chunk_class(int chunk) {
  return chunk < 32 ? 0 : chunk < 64 ? 1 : chunk < 128 ? 2 : chunk < 256 ? 3 : chunk < 512 ? 4 : chunk < 1024 ? 5 : 6;
}
constexpr int window_class(int chunk, int back) {
  const long long w = (long long)chunk * ((long long)back + 1);
  return w < 256 ? 0 : w < 1024 ? 1 : w < 4096 ? 2 : 3;
}
#include "sa_tune_table.inc"
// Variants pinned through sa_tune_override() for measurements; -1 = use the table.
extern int g_tune_override[3];
inline LaunchChoice launch_choice(int D, int chunk, int back) {
  // head dimension 256 has one shape per kernel: anything wider or deeper does not fit registers or LDS
  if (D == 256) return LaunchChoice{FWD_NARROW, DQ_NARROW, DKDV_BLOCKSKIP};
  LaunchChoice c = (D == 128 ? TUNE_D128 : TUNE_D64)[chunk_class(chunk)][window_class(chunk, back)];
  if (g_tune_override[0] >= 0 && g_tune_override[0] < FWD_VARIANTS) c.fwd = g_tune_override[0];
  if (g_tune_override[1] >= 0 && g_tune_override[1] < DQ_VARIANTS) c.dq = g_tune_override[1];
  if (g_tune_override[2] >= 0 && g_tune_override[2] < DKDV_VARIANTS) c.dkdv = g_tune_override[2];
  if (D != 128 && c.dkdv == DKDV_PIPELINED) c.dkdv = DKDV_BLOCKSKIP;
  if (D != 128 && c.dq == DQ_PIPELINED) c.dq = DQ_NARROW;
  return c;
}

template <typename T> struct Cfg {
  static constexpr int NW = 4;                                   // waves per workgroup
  // 16-bit, D in {64, 128, 256}: forward kernel with QB query blocks per wave and NST LDS stages
  // The forward and dQ kernels come in two widths: 8 waves (256 queries) share each key tile among
  // more waves, which pays once the workgroup's queries lie in one chunk; with smaller chunks the
  // union of the waves' windows grows and 4 waves (128 queries) waste less of every tile.
  static constexpr int WIDE_NW = 8, NARROW_NW = 4;
  static constexpr int DQ2_TK = SA_DQ2_TK, DQ2_NST = SA_DQ2_NST;
  static constexpr int DKDV2_NW = SA_DKDV2_NW, DKDV2_TQ = SA_DKDV2_TQ, DKDV2_NST = SA_DKDV2_NST;
  // The software-pipelined dK/dV kernel exists at head dimension 128 only: at 64 a block step has
  // half the MFMAs for the same softmax arithmetic, the loop is bound by its vector work and dkdv2
  // is faster (0.23 against 0.30 ms at B=8, H=16, T=4096, chunk 128).
  static constexpr int DKDV3_NST = SA_DKDV3_NST;
  static constexpr int FWD2_QB = SA_FWD2_QB;
  static constexpr int FWD2_NST = SA_FWD2_NST;
#ifdef SA_FWD2_DISABLE
  static constexpr bool fwd2(int) { return false; }
#else
  static constexpr bool fwd2(int D) { return sizeof(T) == 2 && (D == 64 || D == 128 || D == 256); }
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
