"""Parity of the HIP path against the oracle, on a real MI355X.

Every call goes through the public API / dispatcher ops, which reach the kernels only
through the C ABI of libstreaming_attention.so.  Bars: fp32 <= 1e-4 abs; bf16/fp16 <= 2e-2 abs
+ 1e-2 rel, against the float64 (small shapes) or fp32 windowed (full-size shapes) oracle."""
import ctypes
import math
import os

import numpy as np
import pytest
import torch

from oracle import sa_oracle
from tests.helpers import (LSE_ATOL, TOL, assert_close, assert_close_lse, assert_close_rounding_aware, error_report,
                           make_inputs, tricky_lens)

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "streaming_attention_small.npz")


@pytest.fixture(scope="module", autouse=True)
def _library_loaded():
    from streaming_attention import _lib

    _lib.load()   # fail loudly here rather than silently somewhere else
    yield


def run_kernel(q, k, v, d_o, lens, C, R, **kw):
    """CPU tensors in, CPU tensors out; forward + backward on cuda:0."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    ld = lens.to(dev) if lens is not None else None
    out, lse = streaming_attention(qd, kd, vd, ld, C, R, return_lse=True, **kw)
    out.backward(d_o.to(dev))
    torch.cuda.synchronize()
    return out.detach().cpu(), lse.detach().cpu(), qd.grad.cpu(), kd.grad.cpu(), vd.grad.cpu()


def check_against_dense(q, k, v, d_o, lens, C, R, dtype, **kw):
    o, lse, dq, dk, dv = run_kernel(q, k, v, d_o, lens, C, R, **kw)
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=kw.get("sm_scale"), d_out=d_o)
    assert_close("O", o, ref["O"], dtype)
    assert_close("dQ", dq, ref["dQ"], dtype)
    assert_close("dK", dk, ref["dK"], dtype)
    assert_close("dV", dv, ref["dV"], dtype)
    assert_close_lse(lse, ref["LSE"], dtype)
    B, T = q.shape[0], q.shape[2]
    L = sa_oracle.clamp_lens(lens, B, T)
    for b in range(B):   # exact zeros at padded positions, as the reference's zeros_like gives
        for t in (o, dq, dk, dv):
            assert not t[b, :, int(L[b]):].any()
    return o, lse, dq, dk, dv


SHAPES = [(1, 1, 1), (40, 6, 10), (1, 6, 16), (40, 1, 16), (5, 3, 800)]
WINDOWS = [(1, 0), (1, 5), (10, 0), (10, 5), (10, 10000), (32, 5), (10000, 0), (10000, 10000)]


def strided_gradient_and_lens(d_o, lens):
    """The reference's "noncontiguous" inputs (tests/test_streaming_attention.py:98-150): the upstream
    gradient is float32 with every stride doubled (the last one included), lens has stride 2; q, k, v
    stay contiguous there (its slices are cloned)."""
    dev = torch.device("cuda:0")
    B, H, T, D = d_o.shape
    big = torch.zeros(2 * B, 2 * H, 2 * T, 2 * D, dtype=torch.float32, device=dev)
    big[1::2, 1::2, 1::2, 1::2] = d_o.to(dev).float()
    g = big[1::2, 1::2, 1::2, 1::2]
    assert g.stride(-1) == 2 and not g.is_contiguous()
    ld = None
    if lens is not None:
        lb = torch.zeros(2 * B, dtype=torch.int32, device=dev)
        lb[1::2] = lens.to(dev)
        ld = lb[1::2]
        assert ld.stride(0) == 2
    return g, ld


# (dtype, noncontiguous): the reference's grid has float32 and float16 on both settings of its
# "noncontiguous" axis and no bfloat16 at all; bfloat16 is added here on the contiguous setting
DTYPE_LAYOUTS = [(torch.float32, False), (torch.float32, True), (torch.float16, False), (torch.float16, True),
                 (torch.bfloat16, False)]


@pytest.mark.parametrize("dtype,noncontiguous", DTYPE_LAYOUTS, ids=lambda x: str(x))
@pytest.mark.parametrize("D", [16, 64])
@pytest.mark.parametrize("lens_mode", ["none", "tricky"])
@pytest.mark.parametrize("C,R", WINDOWS)
@pytest.mark.parametrize("B,H,T", SHAPES)
def test_reference_grid(B, H, T, D, C, R, noncontiguous, lens_mode, dtype):
    """The reference's own grid (tests/test_streaming_attention.py:11-31), reduced: batch 40 and 6
    heads at the short lengths, the long length at batch 5 (test_reference_grid_full_batch runs it at
    batch 40 with 6 heads), and its strided float32 upstream gradient and strided lens on every
    "noncontiguous" case (float32 and float16, as there)."""
    q, k, v, d_o = make_inputs(B, H, T, D, dtype=dtype)
    lens = tricky_lens(B, T, C, R) if lens_mode == "tricky" else None
    if not noncontiguous:
        check_against_dense(q, k, v, d_o, lens, C, R, dtype)
        return
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    g, ld = strided_gradient_and_lens(d_o, lens)
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    out = streaming_attention(qd, kd, vd, ld, C, R)
    out.backward(g)      # float32, strided; autograd casts it for the 16-bit types
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    for name, got in (("O", out), ("dQ", qd.grad), ("dK", kd.grad), ("dV", vd.grad)):
        assert_close(name, got, ref[name], dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
@pytest.mark.parametrize("D", [16, 64])
@pytest.mark.parametrize("lens_mode", ["none", "tricky"])
@pytest.mark.parametrize("C,R", [(1, 5), (10, 0), (10, 5), (32, 5), (10000, 10000)])
def test_reference_grid_full_batch(C, R, lens_mode, D, dtype):
    """The largest cell of the reference's grid at its real size (batch 40, 6 heads, T = 800,
    tests/test_streaming_attention.py:26-28), compared the way the reference's test compares: against
    dense-mask SDPA evaluated in float32 on the same GPU (tests/test_streaming_attention.py:152-222),
    which is the oracle's `sdpa_fwd_bwd` formulation."""
    from streaming_attention import streaming_attention

    B, H, T = 40, 6, 800
    dev = torch.device("cuda:0")
    q, k, v, d_o = (t.to(dev) for t in make_inputs(B, H, T, D, dtype=dtype))
    lens = tricky_lens(B, T, C, R).to(dev) if lens_mode == "tricky" else None
    qd, kd, vd = (t.clone().requires_grad_() for t in (q, k, v))
    out = streaming_attention(qd, kd, vd, lens, C, R)
    out.backward(d_o)
    want = sa_oracle.sdpa_fwd_bwd(q, k, v, lens, C, R, d_o)
    for name, got, ref in zip(("O", "dQ", "dK", "dV"), (out, qd.grad, kd.grad, vd.grad), want):
        got, ref = got.detach().float(), ref.float()
        atol, rtol = TOL[dtype]
        assert torch.isfinite(got).all(), name
        bad = (got - ref).abs() > atol + rtol * ref.abs()
        assert not bool(bad.any()), f"{name}: {int(bad.sum())} elements out of tolerance, max {(got - ref).abs().max().item():.3e}"


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("D", [16, 32, 64, 128, 256])
def test_all_head_dims(D, dtype):
    B, H, T, C, R = 2, 2, 200, 16, 2
    q, k, v, d_o = make_inputs(B, H, T, D, seed=21, dtype=dtype)
    lens = torch.tensor([T, 77], dtype=torch.int32)
    check_against_dense(q, k, v, d_o, lens, C, R, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("T,C,R", [(257, 64, 2), (513, 128, 1), (300, 256, 8), (1000, 96, 3), (640, 32, 20)])
def test_tile_edges_16bit(T, C, R, D, dtype):
    """Lengths and chunk sizes that straddle the kernels' 32/64/128/256-wide tiles."""
    B, H = 2, 2
    q, k, v, d_o = make_inputs(B, H, T, D, seed=22, dtype=dtype)
    lens = torch.tensor([T, max(1, T - 65)], dtype=torch.int32)
    check_against_dense(q, k, v, d_o, lens, C, R, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("C,R", [(16, 2), (20, 300), (48, 30), (100, 3), (200, 0), (200, 1), (300, 4), (600, 0), (1100, 1)])
def test_every_table_class_16bit(C, R, D, dtype):
    """One context_size per class of the launch-configuration table, windows in all four window
    classes (48 ... 6020 keys), run with the variants the table picks (head dimension 256 has one shape
    per kernel, in the short- and long-window forms)."""
    B, H, T = 2, 2, 1500
    q, k, v, d_o = make_inputs(B, H, T, D, seed=31, dtype=dtype)
    lens = torch.tensor([T, T - 333], dtype=torch.int32)
    check_against_dense(q, k, v, d_o, lens, C, R, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [64, 128])
def test_every_kernel_variant_16bit(D, dtype):
    """Each variant of the forward, dQ and dK/dV kernels pinned in turn (sa_tune_override), on chunk
    sizes below, at and above the workgroups' 128 / 256 rows; all must agree with the oracle."""
    from streaming_attention import _lib

    lib = _lib.load()
    B, H, T = 2, 2, 777
    q, k, v, d_o = make_inputs(B, H, T, D, seed=32, dtype=dtype)
    lens = torch.tensor([T, 500], dtype=torch.int32)
    # pipelined variants exist at head dimension 128 only: (forward, dQ, dK/dV) variant ids per kernel
    variants = ((0, 1) if D == 128 else (0,), (0, 1) if D == 128 else (0,), (0, 1, 2) if D == 128 else (0, 2))
    try:
        for kernel in range(3):
            for variant in variants[kernel]:
                assert lib.sa_tune_override(kernel, variant) == 0
                for C, R in ((24, 5), (128, 2), (256, 1), (320, 8)):
                    assert lib.sa_launch_choice(D, C, R, kernel) == variant
                    check_against_dense(q, k, v, d_o, lens, C, R, dtype)
            assert lib.sa_tune_override(kernel, -1) == 0
    finally:
        for kernel in range(3):
            lib.sa_tune_override(kernel, -1)


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.float16, 64), (torch.bfloat16, 128), (torch.float16, 32)],
                         ids=str)
def test_expanded_heads_and_repeated_rows(dtype, D):
    """k and v expanded over the head axis (stride 0, read in place: multi-query attention without a
    copy) and a v that repeats one row along T (stride 0 along T: the host makes a contiguous copy)."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    B, H, T, C, R = 2, 4, 200, 32, 2
    q, k1, v1, d_o = make_inputs(B, H, T, D, seed=33, dtype=dtype)
    k1, v1 = k1[:, :1], v1[:, :1]
    lens = torch.tensor([T, 77], dtype=torch.int32)
    for v_src in (v1, v1[:, :, :1].expand(B, 1, T, D)):
        qd = q.to(dev).requires_grad_()
        kd, vd = k1.to(dev).requires_grad_(), v_src.to(dev).requires_grad_()
        ke, ve = kd.expand(B, H, T, D), vd.expand(B, H, T, D)
        assert ke.stride(1) == 0
        o = streaming_attention(qd, ke, ve, lens.to(dev), C, R)
        o.backward(d_o.to(dev))
        ref = sa_oracle.dense_f64(q, k1.expand(B, H, T, D), v_src.expand(B, H, T, D), lens, C, R, d_out=d_o)
        assert_close("O", o.detach(), ref["O"], dtype)
        assert_close("dQ", qd.grad, ref["dQ"], dtype)
        # autograd sums the per-head gradients of the expanded tensors (in the element type, so the
        # bar widens with the number of heads summed)
        assert_close("dK", kd.grad.double().cpu() / H, ref["dK"].sum(1, keepdims=True) / H, dtype)
        assert_close("dV", vd.grad.double().cpu() / H, ref["dV"].sum(1, keepdims=True) / H, dtype)


def test_golden_vectors():
    data = np.load(GOLDEN, allow_pickle=False)
    for name in sorted({k.split(".")[0] for k in data.files}):
        B, H, T, D, C, R = data[f"{name}.shape"].tolist()
        lens = data[f"{name}.lens"]
        lt = None if lens[0] < 0 else torch.from_numpy(lens)
        q, k, v, d_o = (torch.from_numpy(data[f"{name}.{x}"]).float() for x in ("q", "k", "v", "d_o"))
        o, _, dq, dk, dv = run_kernel(q, k, v, d_o, lt, C, R)
        for key, got in (("o", o), ("dq", dq), ("dk", dk), ("dv", dv)):
            assert_close(f"{name}.{key}", got, data[f"{name}.{key}"], torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
def test_noncontiguous_inputs(dtype):
    """[B,T,H,D]-stored q/k/v (read in place), sliced views (copied by the host), a strided
    int32 lens and a strided fp32 upstream gradient."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    B, H, T, D, C, R = 3, 2, 70, 64, 16, 1
    q, k, v, d_o = make_inputs(B, H, T, D, seed=23, dtype=dtype)
    lens = torch.tensor([70, 33, 71], dtype=torch.int32)
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)

    def variants(t):
        bthd = t.to(dev).transpose(1, 2).contiguous().transpose(1, 2)
        big = torch.zeros(B, H, T, 2 * D, dtype=dtype, device=dev)
        big[..., 1::2] = t.to(dev)
        return bthd, big[..., 1::2]

    lens_big = torch.zeros(2 * B, dtype=torch.int32, device=dev)
    lens_big[::2] = lens.to(dev)
    for which in (0, 1):
        qd, kd, vd = (variants(t)[which].detach().requires_grad_() for t in (q, k, v))
        assert not qd.is_contiguous()
        out = streaming_attention(qd, kd, vd, lens_big[::2], C, R)
        g32 = torch.zeros(B, H, T, 2 * D, dtype=torch.float32, device=dev)
        g32[..., ::2] = d_o.to(dev).float()
        out.backward(g32[..., ::2].to(out.dtype) if which == 0 else variants(d_o)[1])
        assert out.is_contiguous()
        assert_close("O", out, ref["O"], dtype)
        assert_close("dQ", qd.grad, ref["dQ"], dtype)
        assert_close("dK", kd.grad, ref["dK"], dtype)
        assert_close("dV", vd.grad, ref["dV"], dtype)


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float32, 32), (torch.float16, 256)])
def test_packed_qkv_projection_is_read_in_place(dtype, D):
    """q, k, v as views of one [B, T, 3, H, D] projection output: no copies on the way in, and the
    gradient arrives in the packed tensor."""
    from streaming_attention import streaming_attention
    from streaming_attention.ops import _kernel_layout

    dev = torch.device("cuda:0")
    B, H, T, C, R = 2, 3, 200, 64, 1
    q, k, v, d_o = make_inputs(B, H, T, D, seed=29, dtype=dtype)
    lens = torch.tensor([200, 77], dtype=torch.int32)
    qkv = torch.stack([t.transpose(1, 2) for t in (q, k, v)], dim=2).to(dev).requires_grad_()   # [B,T,3,H,D]
    views = [qkv[:, :, i].transpose(1, 2) for i in range(3)]                                    # [B,H,T,D]
    assert all(_kernel_layout(x) is x and not x.is_contiguous() for x in views)
    out = streaming_attention(*views, lens.to(dev), C, R)
    out.backward(d_o.to(dev))
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    assert_close("O", out, ref["O"], dtype)
    for i, name in enumerate(("dQ", "dK", "dV")):
        assert_close(name, qkv.grad[:, :, i].transpose(1, 2), ref[name], dtype)


def test_backward_op_accepts_foreign_gradient_and_missing_lse():
    """The backward dispatcher op on its own: fp32 strided dO with fp16 q/k/v
    (tests/test_streaming_attention.py:224-248) and an empty lse (forward without return_lse)."""
    dev = torch.device("cuda:0")
    B, H, T, D, C, R = 2, 2, 90, 64, 10, 3
    dtype = torch.float16
    q, k, v, d_o = make_inputs(B, H, T, D, seed=24, dtype=dtype)
    lens = torch.tensor([90, 41], dtype=torch.int32)
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    fwd = torch.ops.alexdremov_streaming_attention.forward
    bwd = torch.ops.alexdremov_streaming_attention.backward
    o, lse = fwd(qd, kd, vd, lens.to(dev), C, R, D ** -0.5, False, False, False, "ieee")
    assert lse.numel() == 0 and lse.device.type == "cpu"
    g = torch.zeros(B, H, T, 2 * D, dtype=torch.float32, device=dev)
    g[..., ::2] = d_o.to(dev).float()
    dq, dk, dv = bwd(qd, kd, vd, lens.to(dev), o, lse, g[..., ::2], C, R, D ** -0.5, False, False, "ieee")
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    assert_close("dQ", dq, ref["dQ"], dtype)
    assert_close("dK", dk, ref["dK"], dtype)
    assert_close("dV", dv, ref["dV"], dtype)


@pytest.mark.parametrize("D,T,C,R", [(64, 200, 16, 2), (128, 700, 256, 8)])
def test_backward_op_reads_a_strided_forward_output(D, T, C, R):
    """The backward op with the forward output stored [B,T,H,D] (read in place through its strides): for
    16-bit inputs the dQ kernels form delta = rowsum(O * dO) from it themselves -- the narrow dQ kernel at
    D=64, the software-pipelined one at D=128 with a 2304-key window."""
    from streaming_attention import _lib
    from streaming_attention.ops import _kernel_layout

    dev = torch.device("cuda:0")
    B, H = 2, 2
    dtype = torch.bfloat16
    q, k, v, d_o = make_inputs(B, H, T, D, seed=33, dtype=dtype)
    lens = torch.tensor([T, T - 59], dtype=torch.int32)
    if D == 128:
        assert _lib.load().sa_launch_choice(D, C, R, 1) == 1   # the software-pipelined dQ kernel
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    fwd = torch.ops.alexdremov_streaming_attention.forward
    bwd = torch.ops.alexdremov_streaming_attention.backward
    o, lse = fwd(qd, kd, vd, lens.to(dev), C, R, D ** -0.5, False, True, False, "ieee")
    o_bthd = o.transpose(1, 2).contiguous().transpose(1, 2)
    assert not o_bthd.is_contiguous() and _kernel_layout(o_bthd) is o_bthd
    dq, dk, dv = bwd(qd, kd, vd, lens.to(dev), o_bthd, lse, d_o.to(dev), C, R, D ** -0.5, False, False, "ieee")
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, d_out=d_o)
    assert_close("dQ", dq, ref["dQ"], dtype)
    assert_close("dK", dk, ref["dK"], dtype)
    assert_close("dV", dv, ref["dV"], dtype)
    dq2, dk2, dv2 = bwd(qd, kd, vd, lens.to(dev), o, lse, d_o.to(dev), C, R, D ** -0.5, False, False, "ieee")
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)


def check_rounding_aware(q, k, v, d_o, lens, C, R, dtype, sm_scale=None, record=None):
    """16-bit results against the float64 oracle with the bar widened by what rounding P and dS to
    the input type costs in a float64 evaluation of the same formulas (no input is changed to fit)."""
    kw = {} if sm_scale is None else {"sm_scale": sm_scale}
    o, lse, dq, dk, dv = run_kernel(q, k, v, d_o, lens, C, R, **kw)
    exact = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=sm_scale, d_out=d_o)
    rounded = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=sm_scale, d_out=d_o, round_dtype=dtype,
                                  prescaled_k=q.shape[-1] >= 32)
    for name, got in (("O", o), ("dQ", dq), ("dK", dk), ("dV", dv)):
        assert_close_rounding_aware(name, got, exact[name], rounded[name], dtype)
        mx, rel, fro = error_report(got, exact[name])
        _, _, fro_r = error_report(rounded[name], exact[name])
        if record is not None:
            record.append(f"{name}: max abs {mx:.3e}, / max|ref| {rel:.3e}, Frobenius {fro:.3e} "
                          f"(rounded float64 evaluation: {fro_r:.3e})")
        # as a whole the result is as accurate as the type allows: a few unit roundoffs
        assert fro <= (2e-2 if dtype == torch.bfloat16 else 4e-3), f"{name}: relative Frobenius error {fro:.3e}"
    assert_close_lse(lse, exact["LSE"], dtype)
    B, T = q.shape[0], q.shape[2]
    L = sa_oracle.clamp_lens(lens, B, T)
    for b in range(B):
        for t in (o, dq, dk, dv):
            assert not t[b, :, int(L[b]):].any()


@pytest.mark.parametrize("scale", [0.37, -0.2, 0.0])
@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_softmax_scale(scale, dtype, capsys):
    """Explicit, negative and zero softmax scales, unchanged for every type.  With N(0,1) inputs a
    scale of 0.37 at D=64 gives scores of standard deviation 3 and gradients of magnitude ~5; what
    then exceeds the plain 16-bit bar is the rounding of P and dS before the second products, which
    the rounding-aware bar accounts for.  The errors are printed (pytest -s shows them)."""
    B, H, T, D, C, R = 2, 2, 100, 64, 32, 1
    q, k, v, d_o = make_inputs(B, H, T, D, seed=25, dtype=dtype)
    lens = torch.tensor([100, 64], dtype=torch.int32)
    if dtype == torch.float32:
        check_against_dense(q, k, v, d_o, lens, C, R, dtype, sm_scale=scale)
        return
    record = []
    check_rounding_aware(q, k, v, d_o, lens, C, R, dtype, sm_scale=scale, record=record)
    with capsys.disabled():
        print(f"\n[accuracy] {dtype} scale {scale}: " + "; ".join(record))


@pytest.mark.parametrize("dtype,D", [(torch.float32, 32), (torch.float16, 64), (torch.bfloat16, 128), (torch.bfloat16, 256)])
@pytest.mark.parametrize("T,C,R", [(150, 16, 2), (300, 64, 1), (520, 256, 0)])
def test_padding_is_never_read(T, C, R, dtype, D):
    """Positions t >= lens[b] of q, k, v and dO may hold anything (the reference masks its loads,
    kernel.py:246-274): NaN there must give bit-identical results to zeros there."""
    B, H = 3, 2
    q, k, v, d_o = make_inputs(B, H, T, D, seed=27, dtype=dtype)
    lens = torch.tensor([T - 1, max(T // 2 - 3, 1), 37], dtype=torch.int32)
    clean, dirty = [], []
    for t in (q, k, v, d_o):
        z, n = t.clone(), t.clone()
        for b in range(B):
            z[b, :, int(lens[b]):] = 0
            n[b, :, int(lens[b]):] = float("nan")
        clean.append(z)
        dirty.append(n)
    want = run_kernel(*clean, lens, C, R)
    got = run_kernel(*dirty, lens, C, R)
    for name, a, b in zip(("O", "LSE", "dQ", "dK", "dV"), got, want):
        assert torch.isfinite(a).all(), f"{name}: padding leaked into the result"
        assert torch.equal(a, b), f"{name}: result depends on the padded positions"


def _random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    D = int(rng.choice([16, 32, 64, 64, 128, 128, 256]))
    dtype = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    B, H = int(rng.integers(1, 5)), int(rng.integers(1, 4))
    T = int(rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 129, 255, 257, 300, 511, 640]))
    C = int(rng.choice([1, 2, 7, 16, 31, 32, 33, 64, 100, 128, 256, 10**6]))
    R = int(rng.choice([0, 0, 1, 2, 3, 8, 17, 10**6]))
    lens = None
    if rng.random() < 0.75:
        lens = torch.tensor(rng.integers(0, T + 3, B), dtype=torch.int32)
    scale = None if rng.random() < 0.5 else float(rng.choice([-1.0, 1.0]) * rng.uniform(0.02, 0.2))
    bthd = bool(rng.random() < 0.4)
    return B, H, T, D, C, R, lens, dtype, scale, bthd


@pytest.mark.parametrize("seed", range(64))
def test_random_problems(seed):
    """Seeded random draws over every axis at once: head dim, dtype, batch, heads, lengths around the
    tile sizes, chunk sizes that do and do not divide the tiles, unbounded windows, lens of 0 and
    beyond T, explicit and negative scales, [B,T,H,D]-stored inputs."""
    from streaming_attention import streaming_attention

    B, H, T, D, C, R, lens, dtype, scale, bthd = _random_case(seed)
    q, k, v, d_o = make_inputs(B, H, T, D, seed=500 + seed, dtype=dtype)
    dev = torch.device("cuda:0")

    def place(t):
        t = t.to(dev)
        return (t.transpose(1, 2).contiguous().transpose(1, 2) if bthd else t).requires_grad_()

    qd, kd, vd = place(q), place(k), place(v)
    kw = {} if scale is None else {"sm_scale": scale}
    out, lse = streaming_attention(qd, kd, vd, lens.to(dev) if lens is not None else None, C, R,
                                   return_lse=True, **kw)
    out.backward(d_o.to(dev))
    ref = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=scale, d_out=d_o)
    assert_close_lse(lse, ref["LSE"], dtype)
    results = (("O", out), ("dQ", qd.grad), ("dK", kd.grad), ("dV", vd.grad))
    if dtype == torch.float32 or scale is None:
        # the plain bar: 1e-4 for float32, 2e-2 + 1e-2 |ref| for the 16-bit types
        for name, got in results:
            assert_close(name, got, ref[name], dtype)
    else:
        # explicit scales up to 0.2 at head dimensions up to 256 give scores of standard deviation 3:
        # the bar allows for the rounding of P and dS, and of the pre-scaled K in the dK/dV kernels,
        # as a float64 evaluation with those roundings shows it (see check_rounding_aware)
        rnd = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=scale, d_out=d_o, round_dtype=dtype,
                                  prescaled_k=D >= 32)
        for name, got in results:
            assert_close_rounding_aware(name, got, ref[name], rnd[name], dtype)
    if dtype != torch.float32:
        for name, got in results:
            fro = error_report(got, ref[name])[2]
            assert fro <= (2e-2 if dtype == torch.bfloat16 else 4e-3), f"{name}: relative Frobenius error {fro:.3e}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("scale,q_gain", [(0.2, 1.0), (0.37, 1.0), (None, 6.0)])
def test_pinned_variants_large_scores(scale, q_gain, dtype, capsys):
    """Every forward, dQ and dK/dV variant at head dimension 128 pinned in turn on scores far from the
    default: explicit scales 0.2 and 0.37 (standard deviation 3.3 and 6 in base-2 units) and, with the
    default scale, queries multiplied by 6 (scores of standard deviation 8.7, maxima around 35-45 in
    base-2 units).  The dK/dV kernels rebuild their probabilities from K pre-multiplied by
    -scale*log2(e) and rounded to the element type, one more rounding than the forward pass makes;
    the bound is the plain bar plus what a float64 evaluation with exactly those roundings deviates
    from the exact one, head by head.  The margins are printed (pytest -s shows them)."""
    from streaming_attention import _lib

    lib = _lib.load()
    B, H, T, D, C, R = 2, 2, 600, 128, 128, 2
    q, k, v, d_o = make_inputs(B, H, T, D, seed=61, dtype=dtype)
    q = (q.float() * q_gain).to(dtype)
    lens = torch.tensor([T, 389], dtype=torch.int32)
    exact = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=scale, d_out=d_o)
    rounded = sa_oracle.dense_f64(q, k, v, lens, C, R, sm_scale=scale, d_out=d_o, round_dtype=dtype, prescaled_k=True)
    kw = {} if scale is None else {"sm_scale": scale}
    lines = []
    try:
        for kernel, name, variants in ((0, "fwd", (0, 1)), (1, "dq", (0, 1)), (2, "dkdv", (0, 1, 2))):
            for variant in variants:
                assert lib.sa_tune_override(kernel, variant) == 0
                assert lib.sa_launch_choice(D, C, R, kernel) == variant
                o, lse, dq, dk, dv = run_kernel(q, k, v, d_o, lens, C, R, **kw)
                assert_close_lse(lse, exact["LSE"], dtype)
                for tname, got in (("O", o), ("dQ", dq), ("dK", dk), ("dV", dv)):
                    assert_close_rounding_aware(tname, got, exact[tname], rounded[tname], dtype)
                    mx, _, fro = error_report(got, exact[tname])
                    ref_t = torch.from_numpy(exact[tname])
                    plain = (got.double() - ref_t).abs() - (TOL[dtype][0] + TOL[dtype][1] * ref_t.abs())
                    lines.append(f"{name}={variant} {tname}: max abs {mx:.2e}, Frobenius {fro:.2e}, over the plain bar by {max(plain.max().item(), 0.0):.2e}")
            assert lib.sa_tune_override(kernel, -1) == 0
    finally:
        for kernel in range(3):
            lib.sa_tune_override(kernel, -1)
    with capsys.disabled():
        print(f"\n[pinned variants] {dtype} scale {scale} q x {q_gain}: max |LSE| {np.abs(exact['LSE']).max():.1f}\n  " + "\n  ".join(lines))


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.bfloat16, 128), (torch.float16, 256)])
def test_results_are_deterministic(dtype, D):
    """No atomics and a fixed reduction order: two runs on the same inputs agree bit for bit."""
    q, k, v, d_o = make_inputs(2, 3, 333, D, seed=28, dtype=dtype)
    lens = torch.tensor([333, 170], dtype=torch.int32)
    first = run_kernel(q, k, v, d_o, lens, 48, 2)
    second = run_kernel(q, k, v, d_o, lens, 48, 2)
    for name, a, b in zip(("O", "LSE", "dQ", "dK", "dV"), first, second):
        assert torch.equal(a, b), name


def test_empty_inputs_and_zero_lengths():
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    for shape in ((0, 2, 8, 64), (2, 2, 0, 64)):
        q = torch.zeros(shape, device=dev, requires_grad=True)
        out = streaming_attention(q, q, q, None, 4, 1)
        assert out.shape == q.shape
    q, k, v, d_o = make_inputs(2, 2, 40, 64, seed=26)
    lens = torch.tensor([0, 40], dtype=torch.int32)
    o, lse, dq, dk, dv = check_against_dense(q, k, v, d_o, lens, 8, 1, torch.float32)
    assert not o[0].any() and not dq[0].any()


def test_c_abi_direct_calls():
    """ctypes straight into the shared library, no dispatcher in between."""
    from streaming_attention import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    B, H, T, D, C, R = 2, 3, 150, 128, 32, 2
    dtype = torch.bfloat16
    q, k, v, d_o = (t.to(dev) for t in make_inputs(B, H, T, D, seed=27, dtype=dtype))
    lens = torch.tensor([150, 99], dtype=torch.int32, device=dev)
    o = torch.empty_like(q)
    lse = torch.empty(B, H, T, dtype=torch.float32, device=dev)
    delta = torch.empty_like(lse)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    s4 = _lib.strides4
    st = torch.cuda.current_stream().cuda_stream
    sc = D ** -0.5
    assert lib.sa_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), lens.data_ptr(), 1, o.data_ptr(), lse.data_ptr(),
                          s4(q), s4(k), s4(v), B, H, T, D, C, R, sc, 2, st) == 0
    assert lib.sa_bwd_delta(o.data_ptr(), d_o.data_ptr(), delta.data_ptr(), s4(o), s4(d_o), B, H, T, D, 2, st) == 0
    assert lib.sa_bwd_dq(q.data_ptr(), k.data_ptr(), v.data_ptr(), lens.data_ptr(), 1, d_o.data_ptr(), lse.data_ptr(),
                         delta.data_ptr(), dq.data_ptr(), s4(q), s4(k), s4(v), s4(d_o), B, H, T, D, C, R, sc, 2, st) == 0
    assert lib.sa_bwd_dkdv(q.data_ptr(), k.data_ptr(), v.data_ptr(), lens.data_ptr(), 1, d_o.data_ptr(),
                           lse.data_ptr(), delta.data_ptr(), dk.data_ptr(), dv.data_ptr(), s4(q), s4(k), s4(v),
                           s4(d_o), B, H, T, D, C, R, sc, 2, st) == 0
    torch.cuda.synchronize()
    ref = sa_oracle.dense_f64(q.cpu(), k.cpu(), v.cpu(), lens.cpu(), C, R, d_out=d_o.cpu())
    for name, got in (("O", o), ("dQ", dq), ("dK", dk), ("dV", dv)):
        assert_close(name, got, ref[name], dtype)
    want_delta = (ref["O"] * d_o.double().cpu().numpy()).sum(-1)
    assert_close("delta", delta, want_delta, dtype)
    # sa_backward = the launches behind one entry point.  For 16-bit inputs at this head dimension the dQ
    # kernel forms delta itself (another summation order than the delta kernel's), so the results agree
    # with the separate launches to rounding, not bit for bit; the workspace holds the same row sums.
    dq2, dk2, dv2 = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    delta.fill_(float("nan"))
    assert lib.sa_backward(q.data_ptr(), k.data_ptr(), v.data_ptr(), lens.data_ptr(), 1, o.data_ptr(), d_o.data_ptr(),
                           lse.data_ptr(), delta.data_ptr(), dq2.data_ptr(), dk2.data_ptr(), dv2.data_ptr(),
                           s4(q), s4(k), s4(v), s4(o), s4(d_o), B, H, T, D, C, R, sc, 2, st) == 0
    torch.cuda.synchronize()
    for name, got in (("dQ", dq2), ("dK", dk2), ("dV", dv2)):
        assert_close(name, got, ref[name], dtype)
    for got, sep in ((dq2, dq), (dk2, dk), (dv2, dv)):
        assert (got.float() - sep.float()).abs().max().item() <= 2e-2
    assert_close("delta", delta, want_delta, dtype)
    # a layout the kernels cannot read in place is refused, not mis-read
    assert lib.sa_forward(q.data_ptr() + 2, k.data_ptr(), v.data_ptr(), None, 0, o.data_ptr(), None,
                          s4(q), s4(k), s4(v), B, H, T, D, C, R, sc, 2, st) == -4


# ---- the benchmark configurations at their real shapes --------------------------------

def _lens_for(mode, B, T, g):
    if mode == "full":
        return None
    if mode == "uniform_half_full":
        return torch.randint(T // 2, T + 1, (B,), generator=g, dtype=torch.int32)
    if mode == "uniform_256_512":
        return torch.randint(256, 513, (B,), generator=g, dtype=torch.int32)
    u = torch.rand(B, generator=g, dtype=torch.float64)
    return torch.exp(math.log(64.0) + u * (math.log(T) - math.log(64.0))).round().to(torch.int32)


CONFIGS = [
    ("cfg2_bf16_T4096_D64", 8, 16, 4096, 64, torch.bfloat16, 128, 4, "full", None),
    ("cfg3_headline_bf16_T16384_D128", 4, 16, 16384, 128, torch.bfloat16, 256, 8, "uniform_half_full", 1.0),
    ("cfg4_ragged_fp16_T2048_D128", 16, 8, 2048, 128, torch.float16, 64, 1, "loguniform", 1.0),
    ("cfg5_long_bf16_T65536_D128", 1, 32, 65536, 128, torch.bfloat16, 512, 16, "full", 1.0),
]


def test_baseline_config1_fp32():
    B, H, T, D, C, R = 2, 4, 512, 64, 64, 2
    g = torch.Generator().manual_seed(20)
    q, k, v, d_o = [torch.randn(B, H, T, D, generator=g) for _ in range(4)]
    lens = torch.randint(256, 513, (B,), generator=g, dtype=torch.int32)
    check_against_dense(q, k, v, d_o, lens, C, R, torch.float32)
    # and against the reference's own formulation (mask + SDPA, fp32)
    o, _, dq, dk, dv = run_kernel(q, k, v, d_o, lens, C, R)
    ro, rdq, rdk, rdv = sa_oracle.sdpa_fwd_bwd(q, k, v, lens, C, R, d_o)
    for name, a, b in (("O", o, ro), ("dQ", dq, rdq), ("dK", dk, rdk), ("dV", dv, rdv)):
        assert_close(name, a, b, torch.float32)


@pytest.mark.parametrize("name,B,H,T,D,dtype,C,R,lens_mode,qkv_scale", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_baseline_configs_full_size(name, B, H, T, D, dtype, C, R, lens_mode, qkv_scale):
    """Full-size shapes against the windowed fp32 oracle evaluated on the GPU with torch
    matmuls (a dense T x T mask does not fit), plus size-independent properties."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(20)
    lens = _lens_for(lens_mode, B, T, g)
    dg = torch.Generator(device=dev).manual_seed(20)
    sc = D ** -0.5 if qkv_scale is None else qkv_scale
    q, k, v = [(torch.randn(B, H, T, D, generator=dg, device=dev) * sc).to(dtype).requires_grad_() for _ in range(3)]
    d_o = torch.randn(B, H, T, D, generator=dg, device=dev).to(dtype)
    ld = lens.to(dev) if lens is not None else None
    out, lse = streaming_attention(q, k, v, ld, C, R, return_lse=True)
    out.backward(d_o)
    torch.cuda.synchronize()
    ro, rlse, rdq, rdk, rdv = sa_oracle.windowed(q, k, v, lens, C, R, d_out=d_o)
    for nm, a, b in (("O", out, ro), ("dQ", q.grad, rdq), ("dK", k.grad, rdk), ("dV", v.grad, rdv)):
        atol, rtol = TOL[dtype]
        err = (a.detach().float() - b).abs()
        bound = atol + rtol * b.abs()
        assert bool((err <= bound).all()), f"{name} {nm}: max err {err.max().item():.3e}"
        assert bool(torch.isfinite(a).all())
    # the float32 log-sum-exp output has its own absolute bar (the oracle here is float32 as well)
    lse_err = (lse - rlse).abs().max().item()
    assert lse_err <= LSE_ATOL[dtype] + 1e-4, f"{name} LSE: max err {lse_err:.3e}"
    assert bool(torch.isfinite(lse).all())
    L = sa_oracle.clamp_lens(lens, B, T)
    for b in range(B):
        for t in (out, q.grad, k.grad, v.grad):
            assert not bool(t[b, :, int(L[b]):].any()), "padded positions must be exactly zero"
    # determinism: the kernels use no atomics, a second run is bit-identical
    q2, k2, v2 = (t.detach().clone().requires_grad_() for t in (q, k, v))
    out2 = streaming_attention(q2, k2, v2, ld, C, R)
    out2.backward(d_o)
    assert torch.equal(out, out2) and torch.equal(q.grad, q2.grad) and torch.equal(k.grad, k2.grad)
    assert torch.equal(v.grad, v2.grad)
    # the backward pass is linear in dO: doubling dO (exact in binary floating point) doubles every
    # gradient bit for bit, and a zero dO gives exactly zero
    q5, k5, v5 = (t.detach().clone().requires_grad_() for t in (q, k, v))
    streaming_attention(q5, k5, v5, ld, C, R).backward(d_o * 2)
    for got, base in ((q5.grad, q.grad), (k5.grad, k.grad), (v5.grad, v.grad)):
        if dtype == torch.float16:   # fp16 intermediates reach the subnormal range, where rounding does not scale
            assert torch.allclose(got.float(), base.float() * 2, atol=2e-3, rtol=1e-2)
        else:
            assert torch.equal(got, base * 2)
    q6, k6, v6 = (t.detach().clone().requires_grad_() for t in (q, k, v))
    streaming_attention(q6, k6, v6, ld, C, R).backward(torch.zeros_like(d_o))
    assert not bool(q6.grad.any()) and not bool(k6.grad.any()) and not bool(v6.grad.any())
    if B > 1:
        # batch entries are independent: reversing the batch reverses the outputs bit for bit
        perm = torch.arange(B - 1, -1, -1, device=dev)
        q3, k3, v3 = (t.detach()[perm].clone().requires_grad_() for t in (q, k, v))
        out3 = streaming_attention(q3, k3, v3, ld[perm] if ld is not None else None, C, R)
        out3.backward(d_o[perm])
        assert torch.equal(out3, out[perm]) and torch.equal(q3.grad, q.grad[perm])
        assert torch.equal(k3.grad, k.grad[perm]) and torch.equal(v3.grad, v.grad[perm])
    if lens is not None:
        # a sequence of length L equals the same sequence cut to L positions
        b = int(np.argmin(L))
        Lb = int(L[b])
        q4, k4, v4 = (t.detach()[b:b + 1, :, :Lb].clone().requires_grad_() for t in (q, k, v))
        out4 = streaming_attention(q4, k4, v4, None, C, R)
        out4.backward(d_o[b:b + 1, :, :Lb])
        for a, bb in ((out4, out[b:b + 1, :, :Lb]), (q4.grad, q.grad[b:b + 1, :, :Lb]),
                      (k4.grad, k.grad[b:b + 1, :, :Lb]), (v4.grad, v.grad[b:b + 1, :, :Lb])):
            assert torch.allclose(a.float(), bb.float(), atol=1e-3, rtol=1e-3)
