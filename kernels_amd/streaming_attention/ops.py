"""The operator boundary: ``alexdremov_streaming_attention::forward`` / ``::backward``.

Same dispatcher names, argument lists, fake implementations and autograd registration as
the reference (src/streaming_attention/kernel.py:1270-1530); the bodies enqueue the HIP
kernels of libstreaming_attention.so on the current stream instead of launching Triton
kernels.  ``autotune``, ``prescale_qk`` and ``precision`` are accepted for signature
compatibility and do not change the result: kernel variants are read from a table measured
on MI355X (head dimension, context_size class, window class), all accumulation is fp32, and
where the scale is applied is fixed per kernel: in float32 inside the exp2 argument in the forward
and dQ kernels (at least as accurate as either setting of ``prescale_qk``), folded into K and
rounded to the element type in the 16-bit dK/dV kernels at head dimensions 32 and up (what the
reference does under ``prescale_qk=True``, kernel.py:1065-1066).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib

_HEAD_DIMS = (16, 32, 64, 128, 256)
_VEC_BYTES = 16


_DTYPE_IDS = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}   # SA_DTYPE_* of the C ABI


def _dtype_id(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_IDS[dtype]
    except KeyError:
        raise AssertionError(f"unsupported dtype {dtype}: expected float32, float16 or bfloat16") from None


def _kernel_layout(t: torch.Tensor) -> torch.Tensor:
    """Return ``t`` itself when the kernels can read it in place (unit stride along the head
    dimension, every other stride and the base address a multiple of 16 bytes, a non-zero stride
    along T), otherwise a contiguous copy.  The 16-bit kernels for head dimensions 32 and up
    address the rows of one (batch, head) slice with 32-bit byte offsets (a contiguous tensor is
    within that range up to tens of millions of positions); the other kernels have no such limit."""
    es = t.element_size()
    offsets32 = es == 2 and t.shape[-1] >= 32
    if t.is_contiguous() and t.data_ptr() % _VEC_BYTES == 0 and t.shape[-1] * es % _VEC_BYTES == 0 \
            and (not offsets32 or (t.shape[-2] + 1024) * t.shape[-1] * es < 2**32):
        return t          # the common case, without looking at every stride
    vec = _VEC_BYTES // es
    ok = (
        t.stride(-1) == 1
        and all(s % vec == 0 for s in t.stride()[:-1])
        and (t.stride(-2) > 0 or t.shape[-2] <= 1)
        and t.data_ptr() % _VEC_BYTES == 0
        and (not offsets32 or (t.shape[-2] + 1024) * t.stride(-2) * es < 2**32)
    )
    return t if ok else t.contiguous()


def _lens_args(lens: Optional[torch.Tensor]):
    if lens is None:
        return None, 0
    return lens.data_ptr(), lens.stride(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream(device) -> int:
    """Handle of torch's current stream on ``device`` (what ``current_stream(device).cuda_stream``
    returns, without building the Stream object where this torch has the direct accessor)."""
    if _raw_stream is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """``torch.cuda.device(dev)`` that does nothing when ``dev`` is already current: entering the
    real context costs more than the launch of a small kernel."""

    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if device.index == _current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _validate_placement(q, k, v, lens, *others):
    """The kernels index k, v (and o, dO) with q's batch and head counts and dereference every
    pointer on q's device, so a tensor that lives elsewhere or has fewer batches / heads (an
    un-expanded grouped-query k or v) must be refused before any ``data_ptr()`` is taken."""
    assert q.ndim == 4 and k.ndim == 4 and v.ndim == 4
    assert k.shape[:2] == q.shape[:2] and v.shape[:2] == q.shape[:2], "k and v need q's batch and head sizes"
    assert k.device == q.device and v.device == q.device, "q, k and v must be on one device"
    assert lens is None or lens.device == q.device, "lens must be on the device of q"
    for t in others:
        assert t.shape == q.shape, "o and dO need q's shape"
        assert t.device == q.device, "o and dO must be on the device of q"


def _validate(q, k, v, lens, context_size, back_contexts, sm_scale, *others):
    # same conditions, same exception type as kernel.py:1288-1295
    shape, dev = q.shape, q.device
    plain = (len(shape) == 4 and k.shape == shape and v.shape == shape
             and k.device == dev and v.device == dev and (lens is None or lens.device == dev))
    for t in others:
        plain = plain and t.shape == shape and t.device == dev
    if not plain:   # name the condition that failed
        _validate_placement(q, k, v, lens, *others)
    batch, _, T, head_dim = shape
    assert back_contexts >= 0 and context_size >= 1
    assert head_dim in _HEAD_DIMS
    assert head_dim == k.shape[-1] and head_dim == v.shape[-1]
    assert T == k.shape[-2] and T == v.shape[-2]
    assert sm_scale is not None
    assert lens is None or (lens.dtype == torch.int32 and lens.ndim == 1 and batch == lens.shape[0])
    assert q.dtype == k.dtype == v.dtype


# The two ops are declared with the same schemas that the reference's ``torch.library.custom_op``
# decorators infer (kernel.py:1270-1284, 1360-1376) and carry the pt2-compliance tag that the
# decorator sets, but through ``torch.library.Library``: a call then goes from the dispatcher
# straight to the functions below, without the per-call Python wrappers of ``custom_op`` and of
# ``register_autograd``, which cost more host time per step than all four kernels of a small problem
# take on the GPU.
_LIBRARY = torch.library.Library("alexdremov_streaming_attention", "DEF")
_LIBRARY.define(
    "forward(Tensor q, Tensor k, Tensor v, Tensor? lens, SymInt context_size, SymInt back_contexts, "
    "float sm_scale, bool autotune, bool return_lse, bool prescale_qk, str precision) -> (Tensor, Tensor)",
    tags=(torch.Tag.pt2_compliant_tag,),
)
_LIBRARY.define(
    "backward(Tensor q, Tensor k, Tensor v, Tensor? lens, Tensor o, Tensor lse, Tensor do, "
    "SymInt context_size, SymInt back_contexts, float sm_scale, bool autotune, bool prescale_qk, "
    "str precision) -> (Tensor, Tensor, Tensor)",
    tags=(torch.Tag.pt2_compliant_tag,),
)


def attention_forward_adapter(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lens: Optional[torch.Tensor],
    context_size: int,
    back_contexts: int,
    sm_scale: float,
    autotune: bool,
    return_lse: bool,
    prescale_qk: bool,
    precision: str,
) -> tuple[torch.Tensor, torch.Tensor]:
    _validate(q, k, v, lens, context_size, back_contexts, sm_scale)
    B, H, T, D = q.shape
    lib = _lib.load()
    # the kernel writes every element (zeros at padded positions included)
    O = torch.empty_like(q, memory_format=torch.contiguous_format)
    LSE = torch.empty((B, H, T), dtype=torch.float32, device=q.device) if return_lse else None
    if q.numel() > 0:
        qk, kk, vk = _kernel_layout(q), _kernel_layout(k), _kernel_layout(v)
        lens_ptr, lens_stride = _lens_args(lens)
        with _on_device(q.device):
            rc = lib.sa_forward(
                qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), lens_ptr, lens_stride,
                O.data_ptr(), LSE.data_ptr() if LSE is not None else None,
                _lib.strides4(qk), _lib.strides4(kk), _lib.strides4(vk),
                B, H, T, D, min(int(context_size), 2**31 - 1), min(int(back_contexts), 2**31 - 1),
                float(sm_scale), _dtype_id(q.dtype), _stream(q.device),
            )
        _lib.check(rc, "sa_forward")
    if LSE is None:
        LSE = torch.empty(0)
    return O, LSE


_LIBRARY.impl("forward", attention_forward_adapter, "CUDA")


@torch.library.register_fake("alexdremov_streaming_attention::forward", lib=_LIBRARY)
def attention_forward_adapter_abstract(
    q, k, v, lens, context_size, back_contexts, sm_scale, autotune, return_lse, prescale_qk, precision
):
    return (
        torch.empty_like(q, memory_format=torch.contiguous_format),
        torch.empty(q.shape[:3], dtype=torch.float32, device=q.device) if return_lse else torch.empty(0),
    )


def attention_backward_adapter(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lens: Optional[torch.Tensor],
    o: torch.Tensor,
    lse: torch.Tensor,
    do: torch.Tensor,
    context_size: int,
    back_contexts: int,
    sm_scale: float,
    autotune: bool,
    prescale_qk: bool,
    precision: str,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _validate(q, k, v, lens, context_size, back_contexts, sm_scale, o, do)
    B, H, T, D = q.shape
    lib = _lib.load()
    DQ = torch.empty_like(q, memory_format=torch.contiguous_format)
    DK = torch.empty_like(k, memory_format=torch.contiguous_format)
    DV = torch.empty_like(v, memory_format=torch.contiguous_format)
    if q.numel() == 0:
        return DQ, DK, DV
    qk, kk, vk = _kernel_layout(q), _kernel_layout(k), _kernel_layout(v)
    # the upstream gradient may arrive in another dtype and with arbitrary strides
    # (tests/test_streaming_attention.py:224-248 hands an fp32 strided one to fp16 q/k/v)
    gk = _kernel_layout(do if do.dtype == q.dtype else do.to(q.dtype))
    ok = _kernel_layout(o if o.dtype == q.dtype else o.to(q.dtype))
    lens_ptr, lens_stride = _lens_args(lens)
    dt = _dtype_id(q.dtype)
    C = min(int(context_size), 2**31 - 1)
    R = min(int(back_contexts), 2**31 - 1)
    with _on_device(q.device):
        stream = _stream(q.device)
        if lse.numel() != B * H * T or lse.device != q.device:
            # forward was run with return_lse=False: rebuild the log-sum-exp
            lse = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
            scratch = torch.empty(q.shape, dtype=q.dtype, device=q.device)
            rc = lib.sa_forward(
                qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), lens_ptr, lens_stride,
                scratch.data_ptr(), lse.data_ptr(),
                _lib.strides4(qk), _lib.strides4(kk), _lib.strides4(vk),
                B, H, T, D, C, R, float(sm_scale), dt, stream,
            )
            _lib.check(rc, "sa_forward (log-sum-exp rebuild)")
        lse = lse.contiguous()
        if lse.dtype != torch.float32:
            lse = lse.float()
        delta = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
        rc = lib.sa_backward(
            qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), lens_ptr, lens_stride,
            ok.data_ptr(), gk.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            DQ.data_ptr(), DK.data_ptr(), DV.data_ptr(),
            _lib.strides4(qk), _lib.strides4(kk), _lib.strides4(vk), _lib.strides4(ok), _lib.strides4(gk),
            B, H, T, D, C, R, float(sm_scale), dt, stream,
        )
    _lib.check(rc, "sa_backward")
    return DQ, DK, DV


_LIBRARY.impl("backward", attention_backward_adapter, "CUDA")


@torch.library.register_fake("alexdremov_streaming_attention::backward", lib=_LIBRARY)
def attention_backward_adapter_abstract(
    q, k, v, lens, o, lse, do, context_size, back_contexts, sm_scale, autotune, prescale_qk, precision
):
    return (
        torch.empty_like(q, memory_format=torch.contiguous_format),
        torch.empty_like(k, memory_format=torch.contiguous_format),
        torch.empty_like(v, memory_format=torch.contiguous_format),
    )


class _StreamingAttention(torch.autograd.Function):
    """Autograd glue of the forward op (kernel.py:1467-1530): saves q, k, v, O, LSE and lens, hands
    dO to the backward op, lets no gradient flow through the log-sum-exp output (kernel.py:1498)."""

    @staticmethod
    def forward(ctx, q, k, v, lens, context_size, back_contexts, sm_scale, autotune, return_lse,
                prescale_qk, precision):
        with torch._C._AutoDispatchBelowAutograd():
            O, LSE = torch.ops.alexdremov_streaming_attention.forward(
                q, k, v, lens, context_size, back_contexts, sm_scale, autotune, return_lse, prescale_qk, precision)
        ctx.save_for_backward(q, k, v, O, LSE, lens)
        ctx.context_size = context_size
        ctx.back_contexts = back_contexts
        ctx.autotune = autotune
        ctx.sm_scale = sm_scale
        ctx.prescale_qk = prescale_qk
        ctx.precision = precision
        ctx.mark_non_differentiable(LSE)
        return O, LSE

    @staticmethod
    def backward(ctx, do, dlse):
        q, k, v, o, lse, lens = ctx.saved_tensors
        DQ, DK, DV = torch.ops.alexdremov_streaming_attention.backward(
            q, k, v, lens, o, lse, do, ctx.context_size, ctx.back_contexts, ctx.sm_scale,
            ctx.autotune, ctx.prescale_qk, ctx.precision)
        return DQ, DK, DV, None, None, None, None, None, None, None, None


_LIBRARY.impl("forward", _StreamingAttention.apply, "Autograd")


class _NoDoubleBackward(torch.autograd.Function):
    """Marks the outputs of the backward op as not differentiable a second time: the reference registers
    no autograd formula for ``::backward`` (kernel.py:1360-1442), so differentiating through it raises
    there; it raises here as well instead of silently returning detached gradients."""

    @staticmethod
    def forward(ctx, dq, dk, dv, *inputs):
        return dq.view_as(dq), dk.view_as(dk), dv.view_as(dv)

    @staticmethod
    def backward(ctx, *grads):
        raise RuntimeError(
            "alexdremov_streaming_attention::backward has no autograd formula: "
            "differentiating through the backward pass (double backward) is not supported")


def _backward_autograd(q, k, v, lens, o, lse, do, context_size, back_contexts, sm_scale, autotune,
                       prescale_qk, precision):
    with torch._C._AutoDispatchBelowAutograd():
        DQ, DK, DV = torch.ops.alexdremov_streaming_attention.backward(
            q, k, v, lens, o, lse, do, context_size, back_contexts, sm_scale, autotune, prescale_qk, precision)
    # under an ordinary .backward() gradient mode is off and nothing is recorded
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v, o, do)):
        return _NoDoubleBackward.apply(DQ, DK, DV, q, k, v, o, do)
    return DQ, DK, DV


_LIBRARY.impl("backward", _backward_autograd, "Autograd")
