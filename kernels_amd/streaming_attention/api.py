"""Public functions, signature-compatible with src/streaming_attention/kernel.py:1533-1652."""
from __future__ import annotations

import contextlib
import os
import threading

import torch
import torch.nn.functional as F

from . import ops  # noqa: F401  (registers the dispatcher ops)


def streaming_attention_reference(q, k, v, context_size, back_contexts, lens, scale=None):
    """Dense masked attention with the operator's semantics, in plain PyTorch.

    Same contract as the reference's function of this name (kernel.py:1533-1563): returns
    ``(output, valid_query_mask, fraction_of_allowed_pairs)``.  The mask lives on ``q``'s
    device, whichever that is.  Quadratic in T; meant for checking, not for use.
    """
    T = q.shape[-2]
    device = q.device
    chunk_id = torch.arange(T, device=device) // context_size
    gap = chunk_id.unsqueeze(1) - chunk_id.unsqueeze(0)
    attn_mask = (gap >= 0) & (gap <= back_contexts)
    if lens is not None:
        inside = torch.arange(T, device=device).unsqueeze(0) < lens.to(device).unsqueeze(-1)
        pair = inside.unsqueeze(-1) & inside.unsqueeze(-2)
        attn_mask = attn_mask.unsqueeze(0).unsqueeze(0) & pair.unsqueeze(1)
        res_mask = inside.unsqueeze(1).unsqueeze(-1)
    else:
        res_mask = torch.tensor([True], device=device)
    sparsity_fraction = attn_mask.sum().item() / attn_mask.numel()
    out = F.scaled_dot_product_attention(query=q, key=k, value=v, attn_mask=attn_mask, scale=scale)
    return out, res_mask, sparsity_fraction


def _forward_op(q, k, v, lens, context_size, back_contexts, sm_scale, autotune, return_lse,
                prescale_qk, precision):
    # the log-sum-exp is needed by the backward pass whenever a gradient is wanted
    requires_grad = any(i.requires_grad for i in (q, k, v))
    O, LSE = torch.ops.alexdremov_streaming_attention.forward(
        q, k, v, lens, context_size, back_contexts, sm_scale, autotune,
        return_lse or requires_grad, prescale_qk, precision,
    )
    if return_lse:
        return O, LSE
    return O


_compiled = None
_call_path = threading.local()


@contextlib.contextmanager
def compiled_wrapper(enabled: bool = True):
    """Route the calls of ``streaming_attention`` made inside the ``with`` block (on this thread) through the
    ``torch.compile(fullgraph=True, dynamic=True)`` wrapper that the reference puts around every call
    (kernel.py:1566-1596), or, with ``enabled=False``, straight to the op whatever the environment says.
    Results are identical either way; the wrapper costs guard checks per call."""
    previous = getattr(_call_path, "compiled", None)
    _call_path.compiled = bool(enabled)
    try:
        yield
    finally:
        _call_path.compiled = previous


def _use_compiled_wrapper() -> bool:
    """Which path a call takes: the ``compiled_wrapper`` context of this thread if one is active, else
    ``STREAMING_ATTENTION_COMPILED=1`` (wrapper) or ``STREAMING_ATTENTION_EAGER=0`` (wrapper; ``=1`` names the
    default), else the direct op call."""
    scoped = getattr(_call_path, "compiled", None)
    if scoped is not None:
        return scoped
    if os.environ.get("STREAMING_ATTENTION_COMPILED") == "1":
        return True
    return os.environ.get("STREAMING_ATTENTION_EAGER") == "0"


def _compiled_forward():
    """The reference wraps the op call in ``torch.compile(fullgraph=True, dynamic=True)``
    (kernel.py:1566).  The graph holds a single opaque op, so the ``aot_eager`` backend is
    used: Dynamo and AOTAutograd trace it, no code generator runs."""
    global _compiled
    if _compiled is None:
        _compiled = torch.compile(_forward_op, fullgraph=True, dynamic=True, backend="aot_eager")
    return _compiled


def streaming_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lens: torch.Tensor | None,
    context_size: int,
    back_contexts: int,
    sm_scale: float | None = None,
    autotune=False,
    return_lse=False,
    prescale_qk=False,
    precision="ieee",
):
    """Block-sparse self-attention with a chunked mask.

    Time is cut into chunks of ``context_size``; a query attends to every key of its own
    chunk and of the ``back_contexts`` chunks before it, limited to the first ``lens[b]``
    positions of sequence ``b``.  Work and memory grow linearly with the sequence length.

    Args:
        q, k, v: ``(batch, heads, time, head_dim)``, float32 / float16 / bfloat16
        lens: ``(batch,)`` int32 sequence lengths, or None
        context_size: chunk length
        back_contexts: number of earlier chunks a query can see
        sm_scale: softmax scale, ``head_dim ** -0.5`` by default
        return_lse: also return the base-2 log-sum-exp of the scaled scores, ``(batch, heads, time)``
        autotune, prescale_qk, precision: accepted for compatibility with the reference's
            signature (kernel.py:1599-1611); they do not change the result here.

    The op is called directly.  The reference routes every call through a
    ``torch.compile(fullgraph=True, dynamic=True)`` wrapper (kernel.py:1566-1596); that wrapper is
    kept and runs inside ``with compiled_wrapper():`` (per call site) or when
    ``STREAMING_ATTENTION_COMPILED=1`` is set (process-wide), but it is not the default: the
    graph it holds is this one opaque op, so it changes no result, and its guard checks and
    AOTAutograd wrappers cost about 0.1 ms of host time per forward+backward, as much as all four
    kernels of a small problem take on the GPU.
    """
    if sm_scale is None:
        sm_scale = q.size(-1) ** -0.5
    args = dict(
        q=q, k=k, v=v, lens=lens, context_size=context_size, back_contexts=back_contexts,
        sm_scale=sm_scale, autotune=autotune, return_lse=return_lse, prescale_qk=prescale_qk,
        precision=precision,
    )
    if torch.compiler.is_compiling() or not _use_compiled_wrapper():
        return _forward_op(**args)
    for t in (q, k, v):
        torch._dynamo.mark_static(t, 1)
        torch._dynamo.mark_static(t, 3)
    return _compiled_forward()(**args)
