/* C ABI of libstreaming_attention.so -- hand-written gfx950 (MI355X) kernels for
 * chunk-windowed ("streaming") attention, forward and backward.
 *
 * This is the seam at which the reference launches its Triton kernels; every entry
 * point cites the reference launch it replaces (paths relative to the reference
 * repository).  The reference has no FFI of its own (it is Python + a run-time
 * compiled DSL), so the binding on its side is a ctypes stub.
 *
 * Common rules
 *   - Every pointer is a device pointer owned by the caller.  Nothing is allocated,
 *     freed or synchronised here: each call enqueues kernels on `stream` (a hipStream_t,
 *     NULL = the default stream) and returns.
 *   - q/k/v/dO/o inputs are [B,H,T,D] with element strides given as int64[4]
 *     (batch, head, time, dim).  The dim stride must be 1; base pointers must be
 *     16-byte aligned and the other strides multiples of 16 bytes.  Rows of one
 *     (batch, head) slice are addressed with 32-bit byte offsets: the time stride must
 *     be >= 0 and (T + 1024) * time_stride * element_size < 2^32, else SA_ERR_TOO_LARGE.  Outputs are
 *     written contiguous [B,H,T,D] (lse/delta: contiguous [B,H,T] float32).
 *   - dtype: 0 = float32, 1 = float16, 2 = bfloat16.  D in {16,32,64,128,256}.
 *   - lens: int32 per batch entry (may be NULL = every sequence has length T);
 *     lens_stride in elements; values are clamped to [0, T].
 *   - Outputs are fully written, including the zeros at positions t >= lens[b];
 *     the caller need not clear them first.  Input positions t >= lens[b] are never
 *     read, so they may hold anything.
 *   - Return value: 0 on success, > 0 a hipError_t from the launch, < 0 one of SA_ERR_*.
 *   - Re-entrant.  The library's mutable state is the per-device, per-kernel attribute set-up
 *     (hipFuncSetAttribute on the first call of each kernel shape on each device, guarded by a
 *     mutex) and the variants pinned through sa_tune_override() (atomics; a measurement and test
 *     hook that no product caller needs).  Because of the former, the first call of each kernel
 *     shape on a device must be made outside a HIP graph capture.
 *   - The 16-bit dK/dV kernels at D >= 32 multiply K by -sm_scale*log2(e) and round the product to the
 *     element type before the score MFMA (what the reference does for prescale_qk=True,
 *     src/streaming_attention/kernel.py:1065-1066), whatever `prescale_qk` the caller of the Python
 *     operator passed: their probabilities differ from the forward's by about |score| * 2^-9 (bf16) /
 *     2^-12 (fp16) relative, inside the 16-bit accuracy bar.  Forward and dQ scale in float32.
 */
#ifndef STREAMING_ATTENTION_H
#define STREAMING_ATTENTION_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SA_DTYPE_F32 0
#define SA_DTYPE_F16 1
#define SA_DTYPE_BF16 2

#define SA_ERR_DTYPE (-1)
#define SA_ERR_HEAD_DIM (-2)
#define SA_ERR_ARG (-3)
#define SA_ERR_LAYOUT (-4)
#define SA_ERR_TOO_LARGE (-5)
#define SA_ERR_SCRATCH (-6)

/* Rows (B*H*T) that the static workspace of sa_backward_static holds: 8 MiB of float32 per GPU. */
#define SA_STATIC_MAX_ROWS (1 << 21)

/* Forward pass: O = softmax_window(sm_scale * Q K^T) V, LSE = log2 sum exp (scaled scores).
 * Replaces the launch of `_streaming_attn_fwd` inside `attention_forward_adapter`
 * (src/streaming_attention/kernel.py:1302-1333; kernel at :196-430).
 * `lse` may be NULL when the caller does not need it. */
int sa_forward(const void* q, const void* k, const void* v,
               const int32_t* lens, int64_t lens_stride,
               void* o, float* lse,
               const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
               int B, int H, int T, int D,
               int context_size, int back_contexts, float sm_scale,
               int dtype, void* stream);

/* delta[b,h,t] = sum_d O * dO in float32.
 * Replaces the launch of `_streaming_attn_bwd_precompute`
 * (src/streaming_attention/kernel.py:1380-1397; kernel at :433-514). */
int sa_bwd_delta(const void* o, const void* d_o, float* delta,
                 const int64_t* o_strides, const int64_t* do_strides,
                 int B, int H, int T, int D, int dtype, void* stream);

/* dQ.  Replaces the dQ workers of the fused launch `_streaming_attn_bwd`
 * (src/streaming_attention/kernel.py:1403-1440; workers at :638-773 and :940-1023). */
int sa_bwd_dq(const void* q, const void* k, const void* v,
              const int32_t* lens, int64_t lens_stride,
              const void* d_o, const float* lse, const float* delta,
              void* dq,
              const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
              const int64_t* do_strides,
              int B, int H, int T, int D,
              int context_size, int back_contexts, float sm_scale,
              int dtype, void* stream);

/* dK and dV.  Replaces the dK/dV workers of the same fused launch
 * (src/streaming_attention/kernel.py:1403-1440; workers at :776-937 and :1026-1129). */
int sa_bwd_dkdv(const void* q, const void* k, const void* v,
                const int32_t* lens, int64_t lens_stride,
                const void* d_o, const float* lse, const float* delta,
                void* dk, void* dv,
                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                const int64_t* do_strides,
                int B, int H, int T, int D,
                int context_size, int back_contexts, float sm_scale,
                int dtype, void* stream);

/* Whole backward on one stream; `delta` is a caller-provided [B,H,T] float32 workspace that holds
 * rowsum(O * dO) afterwards.  For float32 and for head dimensions 16 and 32 this is sa_bwd_delta +
 * sa_bwd_dkdv + sa_bwd_dq.  For float16 / bfloat16 at head dimensions 32, 64, 128 and 256 the dQ kernel
 * forms the row sums itself from the dO rows it holds anyway (it reads O once more and writes
 * `delta` for the dK/dV kernel, which runs after it), so the separate pass over O and dO -- the
 * reference's `_streaming_attn_bwd_precompute` launch, kernel.py:433-514 -- is not launched; the
 * sums are added in another order than sa_bwd_delta adds them, so the gradients agree with those
 * of the separate calls to rounding, not bit for bit.  Replaces the body of
 * `attention_backward_adapter` (src/streaming_attention/kernel.py:1363-1442). */
int sa_backward(const void* q, const void* k, const void* v,
                const int32_t* lens, int64_t lens_stride,
                const void* o, const void* d_o, const float* lse, float* delta,
                void* dq, void* dk, void* dv,
                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                const int64_t* o_strides, const int64_t* do_strides,
                int B, int H, int T, int D,
                int context_size, int back_contexts, float sm_scale,
                int dtype, void* stream);

/* sa_backward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same kernels, with the
 * [B,H,T] float32 row-sum workspace taken from a static device array inside the library instead
 * of a `delta` argument.  It has no counterpart in the reference.
 *   - B*H*T must not exceed SA_STATIC_MAX_ROWS (sa_query(10)); larger problems return
 *     SA_ERR_SCRATCH and launch nothing.
 *   - Calls nothing that allocates or frees.  The first call on a device looks the array's
 *     address up (hipGetSymbolAddress); make that call outside a graph capture.
 *   - Every call on one GPU uses that GPU's single array: calls that overlap on one GPU (two
 *     streams, two threads) race.  Calls on one stream are ordered and safe. */
int sa_backward_static(const void* q, const void* k, const void* v,
                       const int32_t* lens, int64_t lens_stride,
                       const void* o, const void* d_o, const float* lse,
                       void* dq, void* dk, void* dv,
                       const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                       const int64_t* o_strides, const int64_t* do_strides,
                       int B, int H, int T, int D,
                       int context_size, int back_contexts, float sm_scale,
                       int dtype, void* stream);

/* Static facts about the build, answerable without a GPU.  Replaces the reference's
 * launch-configuration tables (src/streaming_attention/kernel.py:17-85, 1143-1267) as the
 * place where tile shapes are looked up.
 *   what = 0: ABI version          1: waves per workgroup
 *          2: forward key tile (16-bit types)   3: forward key tile (fp32)
 *          4: dQ key tile          5: dK/dV query tile
 *          6: queries (or keys) owned by one workgroup
 *      (1-6 describe the kernels used for float32 and for D in {16, 32})
 *          7: 1 when the hand-scheduled (software-pipelined) kernels are part of this build, 0 when it was
 *             compiled with SA_NO_ASM_KERNELS and serves every call with the compiler-scheduled kernels
 *          8: waves per workgroup of the compiler-scheduled forward and dQ kernels used for the
 *             16-bit types at D in {64, 128, 256} (each wave owns 32 queries)
 *          9: number of context_size classes of the launch-configuration table (below)
 *         11: number of window classes of that table
 *         10: rows (B*H*T) the static workspace of sa_backward_static holds
 *   anything else: -1 */
int sa_query(int what);

/* The launch-configuration table for the 16-bit types at D in {64, 128}.  Replaces the reference's
 * per-head-dimension tile tables and autotune spaces (src/streaming_attention/kernel.py:17-85,
 * 1154-1193, 1212-1267): the reference searches block shapes at run time, this library ships the
 * outcome of an offline sweep on MI355X, indexed by head dimension, context_size class
 * (< 32, < 64, < 128, < 256, < 512, < 1024, >= 1024) and window class
 * (context_size * (back_contexts + 1) < 256, < 1024, < 4096, >= 4096).
 *   kernel = 0: forward   variant 0 = 4 waves (128 queries) per workgroup, 1 = software-pipelined kernel
 *                         (D = 128: 4 waves of 64 queries, one wave per SIMD)
 *   kernel = 1: dQ        variant 0 = 4 waves (128 queries), 1 = software-pipelined kernel (D = 128)
 *   kernel = 2: dK/dV     variant 0 = block-skipping kernel, 1 = software-pipelined kernel (D = 128),
 *                         2 = wave pairs (two waves per SIMD share 32 keys: one forms S and dV, the other dP and dK)
 * sa_launch_choice() returns the variant a call with these sizes runs (always variant 0 at D = 256, whose
 * kernels exist in one shape; -1 for a D outside {64, 128, 256},
 * a kernel id outside 0..2, context_size < 1 or back_contexts < 0).  Every variant computes the same
 * function. */
int sa_launch_choice(int D, int context_size, int back_contexts, int kernel);

/* Pins one variant of one kernel for all later calls of this process, or returns to the table with
 * variant = -1.  Meant for measurements (it is how the table was produced) and for tests that
 * exercise every variant; the counterpart of the reference's `autotune` switch
 * (src/streaming_attention/kernel.py:1154-1193).  A pinned software-pipelined variant applies to D = 128 only.
 * A measurement and test hook, not part of the operator.  The pinned variants are atomics, so a launch
 * on another thread sees either the old or the new variant, but which one is not ordered.  Returns 0 or
 * SA_ERR_ARG. */
int sa_tune_override(int kernel, int variant);

/* Human-readable text for a return code of the functions above (static storage). */
const char* sa_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif
