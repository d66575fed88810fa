"""Oracle for chunk-windowed ("streaming") attention, forward and backward.

TEST INFRASTRUCTURE ONLY -- the product path never imports this file.

Three independent formulations of the same operator, so that a mistake in one
(a dropped term, a wrong sign, a transposed operand) is caught by the others:

* ``dense_f64``       explicit float64 masked softmax (CPU tensors) and the closed-form
                      gradients (follows src/streaming_attention/kernel.py:1540-1551
                      for the mask, :239 for the ``lens`` clamp, :408 for the
                      base-2 log-sum-exp, :1017-1022 and :1119-1128 for dS/dQ/dK/dV).
* ``sdpa_reference``  what the reference's own oracle does: a dense boolean mask
                      handed to ``F.scaled_dot_product_attention``
                      (src/streaming_attention/kernel.py:1533-1563), with the device
                      taken from ``q`` instead of a hard-coded accelerator.
* ``windowed``        per query chunk, dense attention over the key slice
                      ``[max(0, c-R)*C, min((c+1)*C, L))`` only; linear memory in T, used
                      where a T x T mask cannot be materialised.

Pinned by tests/test_oracle.py against: a brute-force triple loop on tiny shapes,
``is_causal`` SDPA (C=1, R>=T), unmasked SDPA (C>=T), block-diagonal attention
(R=0), slice-and-pad equivalence for ``lens``, float64 ``gradcheck`` of the
autograd formulation, and the plain-C restatement in oracle/sa_oracle.c.
The value of LSE at padded rows (t >= lens[b]) is an implementation accident
of the reference (tile-size dependent, kernel.py:243-244 and :408) and is
"parity unpinned"; this oracle and the product both define it as 0.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

LOG2E = 1.4426950408889634


def clamp_lens(lens, B: int, T: int) -> np.ndarray:
    """L_b = min(lens[b], T), or T when lens is None (kernel.py:237-241)."""
    if lens is None:
        return np.full((B,), T, dtype=np.int64)
    arr = lens.detach().cpu().numpy() if isinstance(lens, torch.Tensor) else np.asarray(lens)
    return np.minimum(arr.astype(np.int64), T)


def allowed_mask(T: int, context_size: int, back_contexts: int, L: np.ndarray) -> np.ndarray:
    """Boolean [B, T, T]: allowed(b,i,j) = i<L_b and j<L_b and 0 <= i//C - j//C <= R.

    Follows kernel.py:1540-1551 (chunk-id difference window and-ed with the outer
    product of the key-padding mask with itself).
    """
    chunk = np.arange(T, dtype=np.int64) // int(context_size)
    diff = chunk[:, None] - chunk[None, :]
    window = (diff >= 0) & (diff <= int(back_contexts))
    valid = np.arange(T)[None, :] < np.asarray(L)[:, None]          # [B, T]
    return window[None] & valid[:, :, None] & valid[:, None, :]


def unmasked_pairs(T: int, context_size: int, back_contexts: int, L) -> int:
    """Number of allowed (query, key) pairs per head, summed over the batch.

    Closed form per chunk c: (rows of c below L) x (keys in [max(0,c-R)*C, min((c+1)*C, L))).
    """
    C, R = int(context_size), int(back_contexts)
    total = 0
    for Lb in np.asarray(L).tolist():
        Lb = int(min(Lb, T))
        c = 0
        while c * C < Lb:
            rows = min((c + 1) * C, Lb) - c * C
            keys = min((c + 1) * C, Lb) - max(0, c - R) * C
            total += rows * keys
            c += 1
    return total


def dense_f64(q, k, v, lens, context_size, back_contexts, sm_scale=None, d_out=None, round_dtype=None,
              prescaled_k=False):
    """Explicit float64 evaluation.  Returns dict with O, LSE (log2 units, 0 at padded
    rows) and, when ``d_out`` is given, dQ, dK, dV (all numpy float64).

    With ``round_dtype`` (torch.float16 / torch.bfloat16) the same formulas are evaluated the way
    a 16-bit kernel must evaluate them: the probabilities and dS are rounded to that type before
    the second matrix products (the reference does the same: kernel.py:370, 1020, 1121, 1127), the
    softmax denominator sums the rounded probabilities, and O is rounded before delta is formed.
    The difference between the two evaluations is the error that rounding alone causes.
    ``prescaled_k`` (with ``round_dtype``) also models the scores of the 16-bit dK/dV kernels for head
    dimensions 32 and up, which fold -scale*log2(e) into K and round the product to the element type
    before the score product (the reference's prescale_qk=True, kernel.py:1065-1066): dK and dV are then
    formed from probabilities exp2(q . round(k*scale*log2e) - lse), dQ from the unrounded scale."""
    qn, kn, vn = (t.detach().cpu().double() for t in (q, k, v))
    B, H, T, D = qn.shape
    s = float(D) ** -0.5 if sm_scale is None else float(sm_scale)
    L = clamp_lens(lens, B, T)
    # float64 torch tensors on the CPU: the same arithmetic as numpy, on all host threads
    mask = torch.from_numpy(allowed_mask(T, context_size, back_contexts, L))[:, None]   # [B,1,T,T]
    neg_inf = float("-inf")

    def rounded(x):
        return x if round_dtype is None else x.to(round_dtype).double()

    S = torch.matmul(qn, kn.transpose(-1, -2)) * s
    S = torch.where(mask, S, neg_inf)
    row_valid = mask.any(-1, keepdim=True)                            # [B,1,T,1]
    m = torch.where(row_valid, S.amax(-1, keepdim=True), 0.0)
    E = rounded(torch.where(mask, torch.exp(S - m), 0.0))
    l = E.sum(-1, keepdim=True)
    l_safe = torch.where(l == 0, 1.0, l)
    P = torch.where(row_valid, E / l_safe, 0.0)
    O = torch.matmul(P, vn)
    lse = torch.where(row_valid, (m + torch.log(l_safe)) * LOG2E, 0.0)[..., 0]
    lse = lse.broadcast_to((B, H, T)).contiguous()
    out = {"O": O.numpy(), "LSE": lse.numpy(), "P": P.numpy()}
    if d_out is not None:
        g = d_out.detach().cpu().double().broadcast_to(O.shape)
        if round_dtype is None:
            Pb, Ob = P, O
        else:
            # backward: P is rebuilt from the saved log-sum-exp and rounded for dV; O was stored rounded
            Pb = torch.where(mask, torch.exp(S - lse[..., None] / LOG2E), 0.0) * row_valid
            Ob = rounded(O)
        delta = (Ob * g).sum(-1, keepdim=True)
        dP = torch.matmul(g, vn.transpose(-1, -2))
        dS = Pb * (dP - delta)
        Pkv, dSkv = Pb, dS
        if round_dtype is not None and prescaled_k:
            S2 = torch.matmul(qn, rounded(kn * (s * LOG2E)).transpose(-1, -2))           # log2 units
            Pkv = torch.where(mask, torch.exp2(S2 - lse[..., None]), 0.0) * row_valid
            dSkv = Pkv * (dP - delta)
        Pkv, dS, dSkv = rounded(Pkv), rounded(dS), rounded(dSkv)
        out["dV"] = torch.matmul(Pkv.transpose(-1, -2), g).numpy()
        out["dQ"] = (s * torch.matmul(dS, kn)).numpy()
        out["dK"] = (s * torch.matmul(dSkv.transpose(-1, -2), qn)).numpy()
    return out


def sdpa_reference(q, k, v, context_size, back_contexts, lens, scale=None):
    """Mask + SDPA, the reference's own oracle (kernel.py:1533-1563); same return triple:
    (output, valid-query mask broadcastable to the output, fraction of allowed pairs)."""
    T = q.shape[-2]
    dev = q.device
    chunk = torch.arange(T, device=dev) // int(context_size)
    diff = chunk[:, None] - chunk[None, :]
    attn = (diff >= 0) & (diff < int(back_contexts) + 1)
    if lens is not None:
        valid = torch.arange(T, device=dev)[None, :] < lens.to(dev)[:, None]      # [B,T]
        attn = attn[None, None] & (valid[:, None, :, None] & valid[:, None, None, :])
        res_mask = valid[:, None, :, None]
    else:
        res_mask = torch.ones(1, dtype=torch.bool, device=dev)
    frac = attn.sum().item() / attn.numel()
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=attn, scale=scale)
    return out, res_mask, frac


def sdpa_fwd_bwd(q, k, v, lens, context_size, back_contexts, d_out, sm_scale=None):
    """Forward + backward the way the reference's test drives its oracle
    (tests/test_streaming_attention.py:152-161): inputs upcast to fp32, the upstream
    gradient multiplied by the valid-query mask before ``backward``."""
    qf, kf, vf = (t.detach().float().clone().requires_grad_() for t in (q, k, v))
    out, res_mask, _ = sdpa_reference(qf, kf, vf, context_size, back_contexts, lens, scale=sm_scale)
    g = d_out.detach().float() * res_mask.broadcast_to(out.shape)
    out.backward(g)
    o = out.detach() * res_mask.broadcast_to(out.shape)
    return o, qf.grad, kf.grad, vf.grad


def windowed(q, k, v, lens, context_size, back_contexts, d_out=None, sm_scale=None,
             dtype=torch.float32):
    """Chunk-by-chunk evaluation with memory linear in T (runs on q's device).

    For query chunk c the keys are the slice [max(0,c-R)*C, min((c+1)*C, L_b)); rows at or
    beyond L_b give zeros.  Gradients use the closed forms, accumulated per slice.
    Returns (O, LSE) or (O, LSE, dQ, dK, dV), all in ``dtype``.
    """
    B, H, T, D = q.shape
    C, R = int(context_size), int(back_contexts)
    s = float(D) ** -0.5 if sm_scale is None else float(sm_scale)
    L = clamp_lens(lens, B, T)
    qf, kf, vf = (t.detach().to(dtype) for t in (q, k, v))
    O = torch.zeros_like(qf)
    LSE = torch.zeros((B, H, T), dtype=dtype, device=q.device)
    want_grad = d_out is not None
    if want_grad:
        g = d_out.detach().to(dtype).broadcast_to(qf.shape)
        dQ, dK, dV = torch.zeros_like(qf), torch.zeros_like(kf), torch.zeros_like(vf)
    for b in range(B):
        Lb = int(L[b])
        c = 0
        while c * C < Lb:
            q0, q1 = c * C, min((c + 1) * C, Lb)
            k0, k1 = max(0, c - R) * C, q1
            qs, ks, vs = qf[b, :, q0:q1], kf[b, :, k0:k1], vf[b, :, k0:k1]
            S = torch.matmul(qs, ks.transpose(-1, -2)) * s
            lse_nat = torch.logsumexp(S, dim=-1, keepdim=True)
            P = torch.exp(S - lse_nat)
            o = torch.matmul(P, vs)
            O[b, :, q0:q1] = o
            LSE[b, :, q0:q1] = lse_nat[..., 0] * LOG2E
            if want_grad:
                gs = g[b, :, q0:q1]
                delta = (o * gs).sum(-1, keepdim=True)
                dP = torch.matmul(gs, vs.transpose(-1, -2))
                dS = P * (dP - delta)
                dV[b, :, k0:k1] += torch.matmul(P.transpose(-1, -2), gs)
                dQ[b, :, q0:q1] = s * torch.matmul(dS, ks)
                dK[b, :, k0:k1] += s * torch.matmul(dS.transpose(-1, -2), qs)
            c += 1
    if want_grad:
        return O, LSE, dQ, dK, dV
    return O, LSE


def brute_force(q, k, v, lens, context_size, back_contexts, sm_scale=None):
    """Triple Python loop in float64 for tiny shapes; forward only.  Deliberately written
    from the mask rule per element, sharing no code with the vectorised versions."""
    qn, kn, vn = (t.detach().cpu().double().numpy() for t in (q, k, v))
    B, H, T, D = qn.shape
    s = float(D) ** -0.5 if sm_scale is None else float(sm_scale)
    L = clamp_lens(lens, B, T)
    O = np.zeros_like(qn)
    lse = np.zeros((B, H, T))
    for b in range(B):
        for h in range(H):
            for i in range(min(int(L[b]), T)):
                js = [j for j in range(int(L[b]))
                      if 0 <= i // context_size - j // context_size <= back_contexts]
                sc = np.array([s * float(qn[b, h, i] @ kn[b, h, j]) for j in js])
                w = np.exp(sc - sc.max())
                O[b, h, i] = (w[:, None] * vn[b, h, js]).sum(0) / w.sum()
                lse[b, h, i] = (sc.max() + math.log(w.sum())) * LOG2E
    return O, lse
