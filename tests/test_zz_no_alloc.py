"""The allocation-free backward entry point (`sa_backward_static`) against `sa_backward`.

Same kernels, so the results must be identical bit for bit; the static entry point takes its
row-sum workspace from a device array inside the library.  Two calls in a row share that
array, the second on a smaller problem, and both must match.  Collected last on purpose: the
suite runs with `-x`."""
import pytest
import torch

from tests.helpers import assert_close, make_inputs

pytestmark = pytest.mark.gpu


def _run_both(lib, _lib, B, H, T, D, C, R, dtype, dt_id, seed, lens_list):
    dev = torch.device("cuda:0")
    q, k, v, d_o = (t.to(dev) for t in make_inputs(B, H, T, D, seed=seed, dtype=dtype))
    lens = torch.tensor(lens_list, dtype=torch.int32, device=dev) if lens_list is not None else None
    lp, ls = (lens.data_ptr(), 1) if lens is not None else (None, 0)
    o = torch.empty_like(q)
    lse = torch.empty(B, H, T, dtype=torch.float32, device=dev)
    s4 = _lib.strides4
    st = torch.cuda.current_stream().cuda_stream
    sc = D ** -0.5
    assert lib.sa_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, o.data_ptr(), lse.data_ptr(),
                          s4(q), s4(k), s4(v), B, H, T, D, C, R, sc, dt_id, st) == 0
    # reference results: the existing entry point with a caller-provided workspace
    delta = torch.empty_like(lse)
    want = [torch.empty_like(q) for _ in range(3)]
    assert lib.sa_backward(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, o.data_ptr(), d_o.data_ptr(),
                           lse.data_ptr(), delta.data_ptr(), *(t.data_ptr() for t in want),
                           s4(q), s4(k), s4(v), s4(o), s4(d_o), B, H, T, D, C, R, sc, dt_id, st) == 0
    # outputs pre-filled with garbage: the entry point must write every element itself
    got = [torch.full_like(q, float("nan")) for _ in range(3)]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    rc = lib.sa_backward_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), lp, ls, o.data_ptr(), d_o.data_ptr(),
                                lse.data_ptr(), *(t.data_ptr() for t in got),
                                s4(q), s4(k), s4(v), s4(o), s4(d_o), B, H, T, D, C, R, sc, dt_id, st)
    assert rc == 0, _lib.load().sa_error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    for name, g, w in zip(("dQ", "dK", "dV"), got, want):
        assert_close(name, g, w, dtype)
        assert torch.equal(g, w), f"{name}: same kernels, results must be identical"


def test_static_backward_matches_workspace_backward_twice():
    from streaming_attention import _lib

    lib = _lib.load()
    # first call: ragged bf16 problem; second call, right after, on a smaller fp32 one that
    # reuses (part of) the same static array
    _run_both(lib, _lib, 3, 4, 700, 128, 64, 2, torch.bfloat16, 2, 41, [700, 333, 512])
    _run_both(lib, _lib, 2, 2, 150, 64, 10, 3, torch.float32, 0, 42, [150, 77])
    _run_both(lib, _lib, 1, 2, 96, 64, 32, 1, torch.float16, 1, 43, None)
    # a window of 4608 keys at head dimension 128: the software-pipelined dQ and dK/dV kernels
    assert lib.sa_launch_choice(128, 512, 8, 1) == 1 and lib.sa_launch_choice(128, 512, 8, 2) == 1
    _run_both(lib, _lib, 1, 2, 5000, 128, 512, 8, torch.bfloat16, 2, 44, [4321])


def test_static_backward_rejects_oversize():
    from streaming_attention import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    x = torch.zeros(16, dtype=torch.bfloat16, device=dev)
    st4 = (_lib.ctypes.c_int64 * 4)(2**40, 2**30, 64, 1)
    p = x.data_ptr()
    limit = lib.sa_query(10)
    assert limit == 1 << 21
    # B*H*T one past the limit: refused before anything is launched or dereferenced
    rc = lib.sa_backward_static(p, p, p, None, 0, p, p, p, p, p, p, st4, st4, st4, st4, st4,
                                1, 1, limit + 1, 64, 4, 1, 0.125, 2, torch.cuda.current_stream().cuda_stream)
    assert rc == -6
    assert b"static workspace" in lib.sa_error_string(rc)
    torch.cuda.synchronize()
