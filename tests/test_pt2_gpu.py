"""pt2 surface of the operator on a real GPU: opcheck on both dispatcher ops
(tests/test_streaming_attention.py:224-268) and the bound on recompilations of the compiled
wrapper under changing batch and time sizes (tests/test_streaming_attention.py:271-310)."""
import os

import pytest
import torch

from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
@pytest.mark.parametrize("use_lens", [False, True])
def test_opcheck(dtype, use_lens):
    import streaming_attention  # noqa: F401

    dev = torch.device("cuda:0")
    B, H, T, D, C, R = 3, 2, 50, 64, 10, 2
    q, k, v, d_o = (t.to(dev) for t in make_inputs(B, H, T, D, seed=30, dtype=dtype))
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    lens = torch.tensor([50, 17, 51], dtype=torch.int32, device=dev) if use_lens else None
    fwd = torch.ops.alexdremov_streaming_attention.forward
    bwd = torch.ops.alexdremov_streaming_attention.backward
    atol = 1e-4 if dtype == torch.float32 else 1e-2
    torch.library.opcheck(
        fwd, args=(),
        kwargs=dict(q=q, k=k, v=v, lens=lens, context_size=C, back_contexts=R, sm_scale=D ** -0.5, autotune=False,
                    return_lse=False, prescale_qk=False, precision="ieee"),
        atol=atol, rtol=float("inf"),
    )
    o, lse = fwd(q.detach(), k.detach(), v.detach(), lens, C, R, D ** -0.5, False, True, False, "ieee")
    g = torch.zeros(B, H, T, 2 * D, dtype=torch.float32, device=dev)
    g[..., ::2] = d_o.float()
    torch.library.opcheck(
        bwd, args=(),
        kwargs=dict(q=q.detach(), k=k.detach(), v=v.detach(), lens=lens, o=o, lse=lse, do=g[..., ::2], context_size=C,
                    back_contexts=R, sm_scale=D ** -0.5, autotune=False, prescale_qk=False, precision="ieee"),
        test_utils=("test_schema", "test_faketensor"), atol=atol, rtol=float("inf"),
    )


@pytest.mark.parametrize("lens_mode", ["none", "random"])
def test_compiled_wrapper_does_not_recompile_per_shape(lens_mode, monkeypatch):
    monkeypatch.setenv("STREAMING_ATTENTION_COMPILED", "1")
    from streaming_attention import streaming_attention

    torch._dynamo.reset()
    torch._dynamo.utils.counters["stats"].clear()
    dev = torch.device("cuda:0")
    torch.empty(1, device=dev, requires_grad=True).backward()
    H, D = 4, 32
    g = torch.Generator().manual_seed(31)
    for B in range(1, 200, 48):
        for T in range(1, 400, 96):
            q, k, v = [torch.randn(B, H, T, D, generator=g).to(torch.float16).to(dev).requires_grad_() for _ in range(3)]
            lens = None
            if lens_mode == "random":
                lens = torch.randint(1, T + 1, (B,), generator=g, dtype=torch.int32).to(dev)
            out = streaming_attention(q, k, v, lens, context_size=16, back_contexts=2)
            out.backward(torch.randn_like(out))
            assert torch._dynamo.utils.counters["stats"]["unique_graphs"] <= 4
    torch.cuda.synchronize()


def test_inside_a_compiled_function(monkeypatch):
    monkeypatch.setenv("STREAMING_ATTENTION_COMPILED", "1")
    from oracle import sa_oracle
    from streaming_attention import streaming_attention
    from tests.helpers import assert_close

    torch._dynamo.reset()
    dev = torch.device("cuda:0")
    q, k, v, d_o = make_inputs(2, 2, 64, 64, seed=32)

    @torch.compile(fullgraph=True, backend="aot_eager")
    def f(q, k, v):
        return streaming_attention(q * 1.0, k, v, None, 16, 1) * 2.0

    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    out = f(qd, kd, vd)
    out.backward(d_o.to(dev))
    ref = sa_oracle.dense_f64(q, k, v, None, 16, 1, d_out=2.0 * d_o)
    assert_close("O", out, 2.0 * ref["O"], torch.float32)
    assert_close("dQ", qd.grad, ref["dQ"], torch.float32)
    assert_close("dV", vd.grad, ref["dV"], torch.float32)
