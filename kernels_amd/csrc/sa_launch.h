// Host-side launch entry points, one explicit instantiation per element type.
// Each returns 0, a positive hipError_t, or a negative SA_ERR_* code.
#pragma once
#include <atomic>
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
                        FWD_PIPELINED = 1,  // hand-scheduled loop, 4 waves of 64 queries (head dimension 128 only)
                        FWD_VARIANTS = 2 };
enum DqVariant : int { DQ_NARROW = 0,      // 4 waves (128 queries) per workgroup
                       DQ_PIPELINED = 1,   // hand-scheduled loop, 4 waves of 64 queries (head dimension 128 only)
                       DQ_VARIANTS = 2 };
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
// Variants pinned through sa_tune_override() for measurements and tests; -1 = use the table.  Atomics, so
// that a launch on one thread reads a whole value while another thread pins or releases a variant.
extern std::atomic<int> g_tune_override[3];
// The hand-scheduled kernels are single assembly statements over fixed registers.  A build with
// -DSA_NO_ASM_KERNELS leaves them out (for a compiler that cannot satisfy their register constraints)
// and serves their table cells with the compiler-scheduled kernels.
#ifdef SA_NO_ASM_KERNELS
constexpr bool kAsmKernels = false;
#else
constexpr bool kAsmKernels = true;
#endif
inline LaunchChoice launch_choice(int D, int chunk, int back) {
  // head dimension 256 has one shape per kernel: anything wider or deeper does not fit registers or LDS
  if (D == 256) return LaunchChoice{FWD_NARROW, DQ_NARROW, DKDV_BLOCKSKIP};
  LaunchChoice c = (D == 128 ? TUNE_D128 : TUNE_D64)[chunk_class(chunk)][window_class(chunk, back)];
  const int o0 = g_tune_override[0].load(std::memory_order_relaxed);
  const int o1 = g_tune_override[1].load(std::memory_order_relaxed);
  const int o2 = g_tune_override[2].load(std::memory_order_relaxed);
  if (o0 >= 0 && o0 < FWD_VARIANTS) c.fwd = o0;
  if (o1 >= 0 && o1 < DQ_VARIANTS) c.dq = o1;
  if (o2 >= 0 && o2 < DKDV_VARIANTS) c.dkdv = o2;
  const bool pipelined = kAsmKernels && D == 128;
  if (!pipelined && c.dkdv == DKDV_PIPELINED) c.dkdv = DKDV_BLOCKSKIP;
  if (!pipelined && c.dq == DQ_PIPELINED) c.dq = DQ_NARROW;
  if (!pipelined && c.fwd == FWD_PIPELINED) c.fwd = FWD_NARROW;
  return c;
}

template <typename T> struct Cfg {
  static constexpr int NW = 4;                                   // waves per workgroup
  // 16-bit, D in {64, 128, 256}: forward kernel with QB query blocks per wave and NST LDS stages.
  // The compiler-scheduled forward and dQ kernels run 4 waves (128 queries) per workgroup, two workgroups
  // per CU (an 8-wave shape measured slower or equal in every cell of the tuning sweep and was removed).
  static constexpr int NARROW_NW = 4;
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
  static constexpr bool fwd2(int D) { return sizeof(T) == 2 && (D == 32 || D == 64 || D == 128 || D == 256); }
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
