// extern "C" surface of libstreaming_attention.so: argument checks, parameter packing
// and dispatch on the element type.  See include/streaming_attention.h for the contract.
#include <mutex>
#include "../../include/streaming_attention.h"
#include "sa_launch.h"

using namespace sa;

// Workspace of sa_backward_static: the [B,H,T] float32 row sums that sa_backward takes from its
// caller.  One copy per GPU, held until the process ends.  In host code this name only stands
// for the symbol; the memory is reached through the address hipGetSymbolAddress returns.
static __device__ __align__(256) float sa_static_delta[SA_STATIC_MAX_ROWS];

namespace sa {
std::atomic<int> g_tune_override[3] = {{-1}, {-1}, {-1}};
}  // namespace sa

namespace {

constexpr float kLog2e = 1.4426950408889634f;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// strides are element counts; dim stride 1, the others whole 16-byte vectors.  The 16-bit kernels
// for D >= 32 address the rows of one (batch, head) slice with 32-bit byte offsets through a
// buffer descriptor; the others compute 64-bit addresses and have no such limit.  A zero stride along
// T (one row repeated) is refused: no caller needs it and no test covers it.
int check_layout(const void* p, const int64_t* s, int dtype, int T, int D) {
  if (!p || !s) return SA_ERR_ARG;
  const int64_t vec = dtype == SA_DTYPE_F32 ? 4 : 8;
  if (s[3] != 1) return SA_ERR_LAYOUT;
  if (!aligned16(p)) return SA_ERR_LAYOUT;
  for (int i = 0; i < 3; ++i)
    if (s[i] % vec != 0) return SA_ERR_LAYOUT;
  if (s[2] < 0 || (s[2] == 0 && T > 1)) return SA_ERR_LAYOUT;
  const bool offsets32 = dtype != SA_DTYPE_F32 && D >= 32;
  if (offsets32 && ((int64_t)T + 1024) * s[2] * 2 >= (int64_t(1) << 32)) return SA_ERR_TOO_LARGE;
  return SA_OK;
}

int check_common(int B, int H, int T, int D, int dtype) {
  if (dtype < 0 || dtype > 2) return SA_ERR_DTYPE;
  if (D != 16 && D != 32 && D != 64 && D != 128 && D != 256) return SA_ERR_HEAD_DIM;
  if (B < 0 || H < 0 || T < 0) return SA_ERR_ARG;
  return SA_OK;
}

// chunk ids only matter below T, so a larger context behaves like T; likewise R
void clamp_window(int T, int& C, int& R) {
  if (C > T) C = T;
  if (R > T) R = T;
}

template <typename F> int by_dtype(int dtype, F&& f) {
  switch (dtype) {
    case SA_DTYPE_F32: return f(float{});
    case SA_DTYPE_F16: return f(_Float16{});
    case SA_DTYPE_BF16: return f(__bf16{});
  }
  return SA_ERR_DTYPE;
}

}  // namespace

extern "C" {

int sa_forward(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
               void* o, float* lse, const int64_t* qs, const int64_t* ks, const int64_t* vs, int B, int H,
               int T, int D, int context_size, int back_contexts, float sm_scale, int dtype, void* stream) {
  if (int rc = check_common(B, H, T, D, dtype)) return rc;
  if (context_size < 1 || back_contexts < 0) return SA_ERR_ARG;
  if (B == 0 || H == 0 || T == 0) return SA_OK;
  if (int rc = check_layout(q, qs, dtype, T, D)) return rc;
  if (int rc = check_layout(k, ks, dtype, T, D)) return rc;
  if (int rc = check_layout(v, vs, dtype, T, D)) return rc;
  if (!o || !aligned16(o)) return o ? SA_ERR_LAYOUT : SA_ERR_ARG;
  FwdParams p{};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.lens = lens; p.lens_stride = lens_stride;
  p.q_sb = qs[0]; p.q_sh = qs[1]; p.q_st = qs[2];
  p.k_sb = ks[0]; p.k_sh = ks[1]; p.k_st = ks[2];
  p.v_sb = vs[0]; p.v_sh = vs[1]; p.v_st = vs[2];
  p.B = B; p.H = H; p.T = T; p.C = context_size; p.R = back_contexts;
  clamp_window(T, p.C, p.R);
  p.cdiv = chunk_div(p.C > 0 ? p.C : 1);
  p.scale_log2e = sm_scale * kLog2e;
  return by_dtype(dtype, [&](auto tag) {
    using E = decltype(tag);
    return D == 256 ? launch_fwd<E, 1>(p, D, (hipStream_t)stream) : launch_fwd<E, 0>(p, D, (hipStream_t)stream); });
}

int sa_bwd_delta(const void* o, const void* d_o, float* delta, const int64_t* os, const int64_t* gs, int B,
                 int H, int T, int D, int dtype, void* stream) {
  if (int rc = check_common(B, H, T, D, dtype)) return rc;
  if (B == 0 || H == 0 || T == 0) return SA_OK;
  if (int rc = check_layout(o, os, dtype, T, D)) return rc;
  if (int rc = check_layout(d_o, gs, dtype, T, D)) return rc;
  if (!delta) return SA_ERR_ARG;
  DeltaParams p{};
  p.o = o; p.d_o = d_o; p.delta = delta;
  p.o_sb = os[0]; p.o_sh = os[1]; p.o_st = os[2];
  p.do_sb = gs[0]; p.do_sh = gs[1]; p.do_st = gs[2];
  p.B = B; p.H = H; p.T = T;
  return by_dtype(dtype, [&](auto tag) {
    using E = decltype(tag);
    return D == 256 ? launch_delta<E, 1>(p, D, (hipStream_t)stream) : launch_delta<E, 0>(p, D, (hipStream_t)stream); });
}

static int fill_bwd(BwdParams& p, const void* q, const void* k, const void* v, const int32_t* lens,
                    int64_t lens_stride, const void* d_o, const float* lse, const float* delta,
                    const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* gs, int B, int H,
                    int T, int D, int context_size, int back_contexts, float sm_scale, int dtype) {
  if (int rc = check_common(B, H, T, D, dtype)) return rc;
  if (context_size < 1 || back_contexts < 0) return SA_ERR_ARG;
  if (B == 0 || H == 0 || T == 0) return SA_OK;
  if (int rc = check_layout(q, qs, dtype, T, D)) return rc;
  if (int rc = check_layout(k, ks, dtype, T, D)) return rc;
  if (int rc = check_layout(v, vs, dtype, T, D)) return rc;
  if (int rc = check_layout(d_o, gs, dtype, T, D)) return rc;
  if (!lse || !delta) return SA_ERR_ARG;
  p.q = q; p.k = k; p.v = v; p.d_o = d_o; p.lse = lse; p.delta = delta;
  p.lens = lens; p.lens_stride = lens_stride;
  p.q_sb = qs[0]; p.q_sh = qs[1]; p.q_st = qs[2];
  p.k_sb = ks[0]; p.k_sh = ks[1]; p.k_st = ks[2];
  p.v_sb = vs[0]; p.v_sh = vs[1]; p.v_st = vs[2];
  p.do_sb = gs[0]; p.do_sh = gs[1]; p.do_st = gs[2];
  p.B = B; p.H = H; p.T = T; p.C = context_size; p.R = back_contexts;
  clamp_window(T, p.C, p.R);
  p.cdiv = chunk_div(p.C > 0 ? p.C : 1);
  p.scale = sm_scale;
  p.scale_log2e = sm_scale * kLog2e;
  return SA_OK;
}

// dQ launch.  With o != null the kernel forms delta = rowsum(O * dO) itself and writes it to `delta` for
// the dK/dV launch that follows (the kernels that can: see delta_inside_dq()).
static int run_dq(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
                  const void* d_o, const float* lse, float* delta, void* dq, const int64_t* qs,
                  const int64_t* ks, const int64_t* vs, const int64_t* gs, int B, int H, int T, int D,
                  int context_size, int back_contexts, float sm_scale, int dtype, void* stream, const void* o,
                  const int64_t* os) {
  BwdParams p{};
  if (int rc = fill_bwd(p, q, k, v, lens, lens_stride, d_o, lse, delta, qs, ks, vs, gs, B, H, T, D,
                        context_size, back_contexts, sm_scale, dtype))
    return rc;
  if (B == 0 || H == 0 || T == 0) return SA_OK;
  if (!dq || !aligned16(dq)) return dq ? SA_ERR_LAYOUT : SA_ERR_ARG;
  p.dq = dq;
  if (o) {
    if (int rc = check_layout(o, os, dtype, T, D)) return rc;
    p.o = o; p.o_sb = os[0]; p.o_sh = os[1]; p.o_st = os[2];
    p.delta_out = delta;
  }
  return by_dtype(dtype, [&](auto tag) {
    using E = decltype(tag);
    return D == 256 ? launch_dq<E, 1>(p, D, (hipStream_t)stream) : launch_dq<E, 0>(p, D, (hipStream_t)stream); });
}

int sa_bwd_dq(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
              const void* d_o, const float* lse, const float* delta, void* dq, const int64_t* qs,
              const int64_t* ks, const int64_t* vs, const int64_t* gs, int B, int H, int T, int D,
              int context_size, int back_contexts, float sm_scale, int dtype, void* stream) {
  return run_dq(q, k, v, lens, lens_stride, d_o, lse, const_cast<float*>(delta), dq, qs, ks, vs, gs, B, H, T, D,
                context_size, back_contexts, sm_scale, dtype, stream, nullptr, nullptr);
}

int sa_bwd_dkdv(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
                const void* d_o, const float* lse, const float* delta, void* dk, void* dv,
                const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* gs, int B, int H,
                int T, int D, int context_size, int back_contexts, float sm_scale, int dtype, void* stream) {
  BwdParams p{};
  if (int rc = fill_bwd(p, q, k, v, lens, lens_stride, d_o, lse, delta, qs, ks, vs, gs, B, H, T, D,
                        context_size, back_contexts, sm_scale, dtype))
    return rc;
  if (B == 0 || H == 0 || T == 0) return SA_OK;
  if (!dk || !dv) return SA_ERR_ARG;
  if (!aligned16(dk) || !aligned16(dv)) return SA_ERR_LAYOUT;
  p.dk = dk; p.dv = dv;
  return by_dtype(dtype, [&](auto tag) {
    using E = decltype(tag);
    return D == 256 ? launch_dkdv<E, 1>(p, D, (hipStream_t)stream) : launch_dkdv<E, 0>(p, D, (hipStream_t)stream); });
}

// The dQ kernels for the 16-bit types at head dimensions 64, 128 and 256 hold each query's dO row and form
// delta = rowsum(O * dO) in their prologue; the separate pass over O and dO is then not launched.
static bool delta_inside_dq(int D, int dtype) { return dtype != SA_DTYPE_F32 && Cfg<__bf16>::fwd2(D); }

// The launches behind sa_backward and sa_backward_static: delta, dK/dV, dQ -- or dQ (forming delta), dK/dV.
static int backward_launches(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
                             const void* o, const void* d_o, const float* lse, float* delta, void* dq, void* dk,
                             void* dv, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                             const int64_t* gs, int B, int H, int T, int D, int context_size, int back_contexts,
                             float sm_scale, int dtype, void* stream) {
  if (int rc = check_common(B, H, T, D, dtype)) return rc;
  if (B > 0 && H > 0 && T > 0) {
    // every output is checked before the first launch: nothing is enqueued for a call that is going to fail
    if (!dq || !dk || !dv || !delta) return SA_ERR_ARG;
    if (!aligned16(dq) || !aligned16(dk) || !aligned16(dv)) return SA_ERR_LAYOUT;
    if (int rc = check_layout(o, os, dtype, T, D)) return rc;
    BwdParams probe{};
    if (int rc = fill_bwd(probe, q, k, v, lens, lens_stride, d_o, lse, delta, qs, ks, vs, gs, B, H, T, D,
                          context_size, back_contexts, sm_scale, dtype))
      return rc;
  }
  if (delta_inside_dq(D, dtype) && B > 0 && H > 0 && T > 0) {
    if (int rc = run_dq(q, k, v, lens, lens_stride, d_o, lse, delta, dq, qs, ks, vs, gs, B, H, T, D, context_size,
                        back_contexts, sm_scale, dtype, stream, o, os))
      return rc;
    return sa_bwd_dkdv(q, k, v, lens, lens_stride, d_o, lse, delta, dk, dv, qs, ks, vs, gs, B, H, T, D,
                       context_size, back_contexts, sm_scale, dtype, stream);
  }
  if (int rc = sa_bwd_delta(o, d_o, delta, os, gs, B, H, T, D, dtype, stream)) return rc;
  if (int rc = sa_bwd_dkdv(q, k, v, lens, lens_stride, d_o, lse, delta, dk, dv, qs, ks, vs, gs, B, H, T, D,
                           context_size, back_contexts, sm_scale, dtype, stream))
    return rc;
  return sa_bwd_dq(q, k, v, lens, lens_stride, d_o, lse, delta, dq, qs, ks, vs, gs, B, H, T, D, context_size,
                   back_contexts, sm_scale, dtype, stream);
}

int sa_backward(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
                const void* o, const void* d_o, const float* lse, float* delta, void* dq, void* dk, void* dv,
                const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os, const int64_t* gs,
                int B, int H, int T, int D, int context_size, int back_contexts, float sm_scale, int dtype,
                void* stream) {
  return backward_launches(q, k, v, lens, lens_stride, o, d_o, lse, delta, dq, dk, dv, qs, ks, vs, os, gs, B, H, T, D,
                           context_size, back_contexts, sm_scale, dtype, stream);
}

int sa_backward_static(const void* q, const void* k, const void* v, const int32_t* lens, int64_t lens_stride,
                       const void* o, const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                       const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
                       const int64_t* gs, int B, int H, int T, int D, int context_size, int back_contexts,
                       float sm_scale, int dtype, void* stream) {
  if (int rc = check_common(B, H, T, D, dtype)) return rc;
  if ((int64_t)B * H * T > (int64_t)SA_STATIC_MAX_ROWS) return SA_ERR_SCRATCH;
  // each device has its own copy of the array at its own address: look it up once per device
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static float* base[kMaxDevices] = {};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return SA_ERR_ARG;
  float* delta = nullptr;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!base[dev]) {
      void* ptr = nullptr;
      if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(sa_static_delta)); e != hipSuccess) return (int)e;
      base[dev] = static_cast<float*>(ptr);
    }
    delta = base[dev];
  }
  if (!delta) return SA_ERR_ARG;
  // every row the kernels read is written first, by the delta pass or by the dQ kernel: nothing to clear
  return backward_launches(q, k, v, lens, lens_stride, o, d_o, lse, delta, dq, dk, dv, qs, ks, vs, os, gs, B, H, T, D,
                           context_size, back_contexts, sm_scale, dtype, stream);
}

int sa_query(int what) {
  switch (what) {
    case 0: return 1;
    case 1: return Cfg<__bf16>::NW;
    case 2: return Cfg<__bf16>::FWD_TK;
    case 3: return Cfg<float>::FWD_TK;
    case 4: return Cfg<__bf16>::DQ_TK;
    case 5: return Cfg<__bf16>::DKDV_TQ;
    case 6: return Cfg<__bf16>::NW * 32;
    case 7: return kAsmKernels ? 1 : 0;
    case 8: return Cfg<__bf16>::NARROW_NW;
    case 9: return TUNE_CHUNK_CLASSES;
    case 10: return SA_STATIC_MAX_ROWS;
    case 11: return TUNE_WINDOW_CLASSES;
  }
  return -1;
}

int sa_launch_choice(int D, int context_size, int back_contexts, int kernel) {
  if ((D != 64 && D != 128 && D != 256) || context_size < 1 || back_contexts < 0 || kernel < 0 || kernel > 2) return -1;
  const LaunchChoice c = launch_choice(D, context_size, back_contexts);
  return kernel == 0 ? c.fwd : kernel == 1 ? c.dq : c.dkdv;
}

int sa_tune_override(int kernel, int variant) {
  if (kernel < 0 || kernel > 2) return SA_ERR_ARG;
  const int limit = kernel == 0 ? FWD_VARIANTS : kernel == 1 ? DQ_VARIANTS : DKDV_VARIANTS;
  if (variant < -1 || variant >= limit) return SA_ERR_ARG;
  g_tune_override[kernel].store(variant, std::memory_order_relaxed);
  return SA_OK;
}

const char* sa_error_string(int code) {
  switch (code) {
    case SA_OK: return "success";
    case SA_ERR_DTYPE: return "unsupported dtype id (0 = float32, 1 = float16, 2 = bfloat16)";
    case SA_ERR_HEAD_DIM: return "head dimension must be one of 16, 32, 64, 128, 256";
    case SA_ERR_ARG: return "invalid argument (null pointer, negative size, context_size < 1 or back_contexts < 0)";
    case SA_ERR_LAYOUT: return "unsupported layout (dim stride must be 1; pointers and strides 16-byte aligned)";
    case SA_ERR_TOO_LARGE: return "problem too large for one launch";
    case SA_ERR_SCRATCH: return "B*H*T exceeds the static workspace of sa_backward_static (see sa_query(10))";
  }
  return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
}

}  // extern "C"
