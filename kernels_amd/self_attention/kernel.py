"""``alexdremov_flash_attention::forward`` and ``self_attention`` with the reference's names,
argument lists and conventions (src/self_attention/kernel.py:359-498).

One chunk that covers the whole sequence and no back-contexts turns the streaming mask into
``i < L_b and j < L_b``, which is exactly this operator's key-padding mask; outputs at
positions ``t >= lens[b]`` are zero, as the reference's ``zeros_like`` leaves them.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from streaming_attention import _lib
from streaming_attention.ops import _dtype_id, _kernel_layout, _lens_args, _on_device, _stream, _validate_placement

_HEAD_DIMS = (16, 32, 64, 128, 256)


@torch.library.custom_op("alexdremov_flash_attention::forward", mutates_args=(), device_types=("cuda",))
def attention_forward_adapter(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lens: Optional[torch.Tensor],
    sm_scale: float,
    autotune: bool,
    prescale: bool,
) -> torch.Tensor:
    _validate_placement(q, k, v, lens)
    batch, heads, T, head_dim = q.shape
    # same conditions as src/self_attention/kernel.py:372-379
    assert head_dim in _HEAD_DIMS
    assert head_dim == k.shape[-1] and head_dim == v.shape[-1]
    assert T == k.shape[-2] and T == v.shape[-2]
    assert sm_scale is not None
    assert lens is None or (lens.dtype == torch.int32 and batch == len(lens) and lens.ndim == 1)
    assert q.dtype == k.dtype == v.dtype

    lib = _lib.load()
    O = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if q.numel() == 0:
        return O
    qk, kk, vk = _kernel_layout(q), _kernel_layout(k), _kernel_layout(v)
    lens_ptr, lens_stride = _lens_args(lens)
    with _on_device(q.device):
        rc = lib.sa_forward(
            qk.data_ptr(), kk.data_ptr(), vk.data_ptr(), lens_ptr, lens_stride, O.data_ptr(), None,
            _lib.strides4(qk), _lib.strides4(kk), _lib.strides4(vk),
            batch, heads, T, head_dim, max(T, 1), 0, float(sm_scale), _dtype_id(q.dtype), _stream(q.device),
        )
    _lib.check(rc, "sa_forward (self attention)")
    return O


@torch.library.register_fake("alexdremov_flash_attention::forward")
def attention_forward_adapter_abstract(q, k, v, lens, sm_scale, autotune, prescale):
    return torch.empty_like(q, memory_format=torch.contiguous_format)


def _padding_masks(q, lens):
    T = q.shape[-2]
    if lens is None:
        return None, 1
    inside = (torch.arange(T, device=q.device).unsqueeze(0) < lens.unsqueeze(-1)).unsqueeze(-1)
    return (inside & inside.transpose(-1, -2)).unsqueeze(1), inside.unsqueeze(1)


def self_attention_reference(q, k, v, lens):
    """Masked SDPA with padded rows zeroed; returns ``(output, valid_query_mask)``."""
    attn_mask, res_mask = _padding_masks(q, lens)
    return F.scaled_dot_product_attention(query=q, key=k, value=v, attn_mask=attn_mask) * res_mask, res_mask


def self_attention_reference_naive(q, k, v, lens):
    """The same through an explicit softmax."""
    attn_mask, res_mask = _padding_masks(q, lens)
    scores = (q / (q.shape[-1] ** 0.5)) @ k.transpose(-1, -2)
    if attn_mask is not None:
        scores = torch.where(attn_mask, scores, -float("inf"))
    result = F.softmax(scores, dim=-1) @ v
    return (result if isinstance(res_mask, int) else torch.where(res_mask, result, 0)), res_mask


def self_attention(q, k, v, lens, sm_scale=None, autotune=True, prescale=False):
    """Dense attention over the first ``lens[b]`` positions of every sequence (all of them when
    ``lens`` is None).  ``autotune`` and ``prescale`` are accepted for signature compatibility."""
    if sm_scale is None:
        sm_scale = q.size(-1) ** -0.5
    return torch.ops.alexdremov_flash_attention.forward(q, k, v, lens, sm_scale, autotune, prescale)
