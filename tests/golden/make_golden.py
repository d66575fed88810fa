"""Writes tests/golden/streaming_attention_small.npz.

Inputs come from a seeded CPU generator; expected outputs come from PyTorch's own
``scaled_dot_product_attention`` in float64 with the dense chunk-window mask (the library
routine the reference's oracle calls, src/streaming_attention/kernel.py:1558-1560) and from
autograd through it -- not from this repository's oracle or kernels, so the fixture pins both.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # name: (B, H, T, D, C, R, lens)
    "ragged": (2, 2, 48, 16, 8, 2, [48, 29]),
    "single_chunk_window": (1, 2, 40, 32, 10, 0, [37]),
    "causal_like": (1, 1, 24, 16, 1, 1000, None),
}


def main():
    out = {}
    for name, (B, H, T, D, C, R, lens) in CASES.items():
        g = torch.Generator().manual_seed(20)
        q, k, v, d_o = [torch.randn(B, H, T, D, generator=g, dtype=torch.float64) for _ in range(4)]
        q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
        chunk = torch.arange(T) // C
        diff = chunk[:, None] - chunk[None, :]
        mask = ((diff >= 0) & (diff <= R))[None, None].expand(B, 1, T, T).clone()
        valid = torch.ones(B, T, dtype=torch.bool)
        if lens is not None:
            valid = torch.arange(T)[None, :] < torch.tensor(lens)[:, None]
            mask &= valid[:, None, :, None] & valid[:, None, None, :]
        # rows with no allowed key would be NaN in SDPA: give them a dummy key and zero them after
        safe = mask | (~mask.any(-1, keepdim=True) & torch.eye(T, dtype=torch.bool)[None, None])
        o = F.scaled_dot_product_attention(q, k, v, attn_mask=safe) * valid[:, None, :, None]
        (o * d_o).sum().backward()
        out[f"{name}.shape"] = np.array([B, H, T, D, C, R], dtype=np.int64)
        out[f"{name}.lens"] = np.array(lens if lens is not None else [-1], dtype=np.int32)
        for key, t in (("q", q), ("k", k), ("v", v), ("d_o", d_o), ("o", o), ("dq", q.grad), ("dk", k.grad),
                       ("dv", v.grad)):
            out[f"{name}.{key}"] = t.detach().numpy()
    np.savez_compressed(os.path.join(HERE, "streaming_attention_small.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
