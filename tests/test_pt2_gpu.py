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
def test_compiled_wrapper_does_not_recompile_per_shape(lens_mode):
    """The reference's dynamic-shape sweep at its own size (tests/test_streaming_attention.py:271-310):
    32 x 32 (batch, time) sizes up to 993 x 993 through the compiled wrapper, at most 4 graphs."""
    from streaming_attention import compiled_wrapper, streaming_attention

    torch._dynamo.reset()
    torch._dynamo.utils.counters["stats"].clear()
    dev = torch.device("cuda:0")
    torch.empty(1, device=dev, requires_grad=True).backward()
    H, D = 4, 32
    g = torch.Generator(device=dev).manual_seed(31)
    with compiled_wrapper():
        for B in range(1, 1024, 32):
            for T in range(1, 1024, 32):
                q, k, v = [((torch.rand(B, H, T, D, generator=g, device=dev) - 0.5) * 0.02).to(torch.float16).requires_grad_()
                           for _ in range(3)]
                lens = None
                if lens_mode == "random":
                    lens = torch.randint(1, T + 1, (B,), generator=g, device=dev, dtype=torch.int32)
                out = streaming_attention(q, k, v, lens, context_size=16, back_contexts=2, autotune=False)
                out.backward(torch.randn(out.shape, generator=g, device=dev, dtype=out.dtype))
                assert torch._dynamo.utils.counters["stats"]["unique_graphs"] <= 4
    torch.cuda.synchronize()
    assert torch.isfinite(q.grad).all()


def test_call_path_selection(monkeypatch):
    """Direct op call by default; the compiled wrapper per call site, or process-wide through either
    environment variable; all paths give the same bits."""
    from streaming_attention import api, compiled_wrapper, streaming_attention

    for var in ("STREAMING_ATTENTION_COMPILED", "STREAMING_ATTENTION_EAGER"):
        monkeypatch.delenv(var, raising=False)
    assert not api._use_compiled_wrapper()
    with compiled_wrapper():
        assert api._use_compiled_wrapper()
        with compiled_wrapper(False):
            assert not api._use_compiled_wrapper()
        assert api._use_compiled_wrapper()
    assert not api._use_compiled_wrapper()
    monkeypatch.setenv("STREAMING_ATTENTION_EAGER", "1")
    assert not api._use_compiled_wrapper()
    monkeypatch.setenv("STREAMING_ATTENTION_EAGER", "0")
    assert api._use_compiled_wrapper()
    monkeypatch.delenv("STREAMING_ATTENTION_EAGER")
    monkeypatch.setenv("STREAMING_ATTENTION_COMPILED", "1")
    assert api._use_compiled_wrapper()
    with compiled_wrapper(False):
        assert not api._use_compiled_wrapper()
    monkeypatch.delenv("STREAMING_ATTENTION_COMPILED")
    dev = torch.device("cuda:0")
    q, k, v, _ = (t.to(dev) for t in make_inputs(2, 2, 70, 64, seed=33))
    direct = streaming_attention(q, k, v, None, 16, 1)
    with compiled_wrapper():
        wrapped = streaming_attention(q, k, v, None, 16, 1)
    assert torch.equal(direct, wrapped)


def test_double_backward_raises():
    """The reference registers no autograd formula for its backward op (kernel.py:1360-1442), so
    differentiating through the backward pass raises there; here too, instead of detaching silently."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    q, k, v, d_o = (t.to(dev).requires_grad_() for t in make_inputs(1, 2, 40, 64, seed=34))
    out = streaming_attention(q, k, v, None, 8, 1)
    (dq,) = torch.autograd.grad(out, q, d_o, create_graph=True)
    with pytest.raises(RuntimeError, match="double backward"):
        dq.sum().backward()
    # the ordinary backward is unaffected
    out = streaming_attention(q, k, v, None, 8, 1)
    out.backward(d_o.detach())
    assert torch.isfinite(q.grad).all()


def test_inside_a_compiled_function():
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
