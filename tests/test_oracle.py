"""Pins the oracle (CPU only).  Each check is chosen so that a plausible mistake in the
oracle -- a wrong window bound, a dropped clamp, a transposed operand, a missing scale --
fails at least one of them: brute force per element, textbook special cases handled by a
library routine, invariants of softmax attention, autograd in float64, the independent C
restatement, and the committed golden vectors."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle, sa_oracle
from tests.helpers import make_inputs, tricky_lens

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "streaming_attention_small.npz")


def _f64(ts):
    return [t.double() for t in ts]


@pytest.mark.parametrize("C,R", [(1, 0), (3, 2), (8, 1), (5, 100), (100, 0)])
def test_mask_rule_brute_force(C, R):
    T = 23
    L = np.array([23, 7, 0, 30])
    m = sa_oracle.allowed_mask(T, C, R, np.minimum(L, T))
    for b, Lb in enumerate(np.minimum(L, T)):
        for i in range(T):
            for j in range(T):
                want = i < Lb and j < Lb and 0 <= i // C - j // C <= R
                assert m[b, i, j] == want, (b, i, j)
    assert sa_oracle.unmasked_pairs(T, C, R, L) == int(m.sum())


@pytest.mark.parametrize("C,R,lens", [(4, 1, None), (5, 2, [19, 8]), (1, 3, [1, 19]), (32, 0, [19, 20])])
def test_formulations_agree(C, R, lens):
    B, H, T, D = 2, 2, 19, 8
    q, k, v, d_o = _f64(make_inputs(B, H, T, D, seed=3))
    lt = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    dense = sa_oracle.dense_f64(q, k, v, lt, C, R, d_out=d_o)
    bo, bl = sa_oracle.brute_force(q, k, v, lt, C, R)
    np.testing.assert_allclose(dense["O"], bo, atol=1e-12)
    np.testing.assert_allclose(dense["LSE"], bl, atol=1e-12)
    cc = c_oracle.run(q.numpy(), k.numpy(), v.numpy(), None if lt is None else lt.numpy(), C, R, d_out=d_o.numpy())
    win = sa_oracle.windowed(q, k, v, lt, C, R, d_out=d_o, dtype=torch.float64)
    for name, w in zip(("O", "LSE", "dQ", "dK", "dV"), win):
        np.testing.assert_allclose(dense[name], cc[name], atol=1e-11, err_msg=f"C oracle {name}")
        np.testing.assert_allclose(dense[name], w.numpy(), atol=1e-11, err_msg=f"windowed {name}")
    so = sa_oracle.sdpa_fwd_bwd(q, k, v, lt, C, R, d_o)
    for name, w in zip(("O", "dQ", "dK", "dV"), so):
        np.testing.assert_allclose(dense[name], w.double().numpy(), atol=5e-6, err_msg=f"sdpa {name}")


def test_special_case_causal():
    # chunk 1 with unlimited history is token-causal attention
    B, H, T, D = 1, 2, 17, 8
    q, k, v, _ = _f64(make_inputs(B, H, T, D, seed=5))
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    got = sa_oracle.dense_f64(q, k, v, None, 1, T)["O"]
    np.testing.assert_allclose(got, want.numpy(), atol=1e-12)


def test_special_case_full_and_scale():
    # one chunk covering everything is plain bidirectional attention; explicit scale honoured
    B, H, T, D = 2, 1, 13, 8
    q, k, v, _ = _f64(make_inputs(B, H, T, D, seed=6))
    want = F.scaled_dot_product_attention(q, k, v, scale=0.37)
    got = sa_oracle.dense_f64(q, k, v, None, 1000, 0, sm_scale=0.37)["O"]
    np.testing.assert_allclose(got, want.numpy(), atol=1e-12)


def test_special_case_block_diagonal():
    # no history: every chunk is an independent dense attention
    B, H, T, D, C = 1, 2, 20, 8, 6
    q, k, v, _ = _f64(make_inputs(B, H, T, D, seed=7))
    got = sa_oracle.dense_f64(q, k, v, None, C, 0)["O"]
    for c0 in range(0, T, C):
        sl = slice(c0, min(c0 + C, T))
        want = F.scaled_dot_product_attention(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        np.testing.assert_allclose(got[:, :, sl], want.numpy(), atol=1e-12)


def test_lens_is_slice_and_pad():
    B, H, T, D, C, R = 3, 2, 21, 8, 4, 2
    q, k, v, d_o = _f64(make_inputs(B, H, T, D, seed=8))
    lens = torch.tensor([21, 9, 30], dtype=torch.int32)   # 30 > T must clamp
    full = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    for b, Lb in enumerate([21, 9, 21]):
        part = sa_oracle.dense_f64(q[b:b + 1, :, :Lb], k[b:b + 1, :, :Lb], v[b:b + 1, :, :Lb], None, C, R,
                                   d_out=d_o[b:b + 1, :, :Lb])
        for name in ("O", "dQ", "dK", "dV"):
            np.testing.assert_allclose(full[name][b, :, :Lb], part[name][0], atol=1e-12)
            assert not full[name][b, :, Lb:].any(), f"{name} must be zero at padded positions"
        assert not full["LSE"][b, :, Lb:].any()


def test_invariants():
    B, H, T, D, C, R = 2, 2, 18, 8, 5, 1
    q, k, v, d_o = _f64(make_inputs(B, H, T, D, seed=9))
    lens = torch.tensor([18, 11], dtype=torch.int32)
    r = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    P = r["P"]
    valid = (np.arange(T)[None, :] < lens.numpy()[:, None])[:, None, :]
    np.testing.assert_allclose(P.sum(-1)[np.broadcast_to(valid, P.shape[:3])], 1.0, atol=1e-12)
    # constant values give constant output on every valid row
    vc = torch.ones_like(v) * 2.5
    oc = sa_oracle.dense_f64(q, k, vc, lens, C, R)["O"]
    np.testing.assert_allclose(oc[np.broadcast_to(valid[..., None], oc.shape)], 2.5, atol=1e-12)
    # shifting all keys by a constant vector shifts every score of a row equally: O unchanged
    shift = torch.randn(1, 1, 1, D, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    o2 = sa_oracle.dense_f64(q, k, v, lens, C, R)["O"]
    # (q . (k + s)) = q.k + q.s, a per-row constant -> softmax invariant
    o3 = sa_oracle.dense_f64(q, k + shift, v, lens, C, R)["O"]
    np.testing.assert_allclose(o2, o3, atol=1e-10)
    # permuting the batch permutes the outputs
    perm = [1, 0]
    rp = sa_oracle.dense_f64(q[perm], k[perm], v[perm], lens[perm], C, R, d_out=d_o[perm])
    for name in ("O", "dQ", "dK", "dV", "LSE"):
        np.testing.assert_allclose(rp[name], r[name][perm], atol=1e-12)


def test_gradients_match_autograd_f64():
    # closed-form dQ/dK/dV against autograd through an explicit masked softmax
    B, H, T, D, C, R = 2, 2, 14, 4, 3, 2
    q, k, v, d_o = _f64(make_inputs(B, H, T, D, seed=10))
    lens = torch.tensor([14, 6], dtype=torch.int32)
    qa, ka, va = (t.clone().requires_grad_() for t in (q, k, v))
    mask = torch.from_numpy(sa_oracle.allowed_mask(T, C, R, sa_oracle.clamp_lens(lens, B, T)))[:, None]
    s = (qa @ ka.transpose(-1, -2)) * D ** -0.5
    p = torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1).nan_to_num(0.0)
    o = p @ va
    o.backward(d_o)
    r = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    np.testing.assert_allclose(r["O"], o.detach().numpy(), atol=1e-12)
    for name, t in (("dQ", qa), ("dK", ka), ("dV", va)):
        np.testing.assert_allclose(r[name], t.grad.numpy(), atol=1e-11, err_msg=name)


def test_gradcheck_small():
    # numerical differentiation of the windowed formulation's forward
    B, H, T, D, C, R = 1, 1, 6, 2, 2, 1

    def f(q, k, v):
        return sa_oracle.sdpa_reference(q, k, v, C, R, None)[0]

    g = torch.Generator().manual_seed(11)
    args = [torch.randn(B, H, T, D, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(3)]
    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-5)
    # and the closed forms agree with it
    d_o = torch.randn(B, H, T, D, generator=g, dtype=torch.float64)
    f(*args).backward(d_o)
    r = sa_oracle.dense_f64(*[a.detach() for a in args], None, C, R, d_out=d_o)
    for name, a in zip(("dQ", "dK", "dV"), args):
        np.testing.assert_allclose(r[name], a.grad.numpy(), atol=1e-10)


def test_lse_is_base2_logsumexp():
    B, H, T, D, C, R = 1, 1, 9, 4, 3, 1
    q, k, v, _ = _f64(make_inputs(B, H, T, D, seed=12))
    r = sa_oracle.dense_f64(q, k, v, None, C, R)
    s = (q @ k.transpose(-1, -2)) * D ** -0.5
    mask = torch.from_numpy(sa_oracle.allowed_mask(T, C, R, np.array([T])))[:, None]
    want = torch.logsumexp(s.masked_fill(~mask, float("-inf")), -1) / np.log(2.0)
    np.testing.assert_allclose(r["LSE"], want.numpy(), atol=1e-12)


def test_golden_vectors():
    data = np.load(GOLDEN, allow_pickle=False)
    names = sorted({k.split(".")[0] for k in data.files})
    assert names
    for name in names:
        B, H, T, D, C, R = data[f"{name}.shape"].tolist()
        lens = data[f"{name}.lens"]
        lt = None if lens[0] < 0 else torch.from_numpy(lens)
        q, k, v, d_o = (torch.from_numpy(data[f"{name}.{x}"]) for x in ("q", "k", "v", "d_o"))
        r = sa_oracle.dense_f64(q, k, v, lt, C, R, d_out=d_o)
        cc = c_oracle.run(q.numpy(), k.numpy(), v.numpy(), None if lt is None else lt.numpy(), C, R, d_out=d_o.numpy())
        for key, want in (("O", "o"), ("dQ", "dq"), ("dK", "dk"), ("dV", "dv")):
            np.testing.assert_allclose(r[key], data[f"{name}.{want}"], atol=1e-11, err_msg=f"{name} {key}")
            np.testing.assert_allclose(cc[key], data[f"{name}.{want}"], atol=1e-11, err_msg=f"{name} C {key}")


def test_tricky_lens_helper_is_seeded():
    a = tricky_lens(7, 100, 10, 5)
    b = tricky_lens(7, 100, 10, 5)
    assert torch.equal(a, b) and a.dtype == torch.int32
