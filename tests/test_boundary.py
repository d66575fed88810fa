"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, argument validation answers before any device work, the dispatcher ops carry
the reference's schemas, and the pieces of host logic behave."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "streaming_attention.h")


@pytest.fixture(scope="module")
def lib():
    from streaming_attention import _lib

    return _lib.load()


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sa_[a-z_]+)\s*\(", text)))


def test_header_symbols_exported(lib):
    names = _declared_symbols()
    assert names == ["sa_backward", "sa_backward_static", "sa_bwd_delta", "sa_bwd_dkdv", "sa_bwd_dq", "sa_error_string",
                     "sa_forward", "sa_launch_choice", "sa_query", "sa_tune_override"]
    for n in names:
        assert getattr(lib, n) is not None
    from streaming_attention import _lib

    assert sorted(_lib.SIGNATURES) == names


def test_query_and_error_strings(lib):
    assert lib.sa_query(0) >= 1
    assert lib.sa_query(1) in (4, 8)
    assert lib.sa_query(2) % 32 == 0 and lib.sa_query(3) % 32 == 0
    assert lib.sa_query(7) in (0, 1) and lib.sa_query(8) == 4 and lib.sa_query(9) == 7
    assert lib.sa_query(99) == -1
    assert b"success" in lib.sa_error_string(0)
    assert lib.sa_query(10) == 1 << 21
    assert lib.sa_query(11) == 4 and lib.sa_query(12) == -1
    # the launch-configuration table answers without a GPU and rejects what it does not cover
    for D in (64, 128):
        for C in (1, 31, 32, 100, 256, 5000):
            for R in (0, 3, 100, 2 ** 31 - 1):
                assert lib.sa_launch_choice(D, C, R, 0) in ((0, 1) if D == 128 else (0,))
                assert lib.sa_launch_choice(D, C, R, 1) in ((0, 1) if D == 128 else (0,))
                assert lib.sa_launch_choice(D, C, R, 2) in ((0, 1, 2) if D == 128 else (0, 2))
    assert [lib.sa_launch_choice(256, 256, 8, k) for k in range(3)] == [0, 0, 0]
    assert lib.sa_launch_choice(32, 64, 1, 0) == -1 and lib.sa_launch_choice(128, 0, 1, 0) == -1
    assert lib.sa_launch_choice(128, 64, 1, 3) == -1 and lib.sa_launch_choice(128, 64, -1, 0) == -1
    assert lib.sa_tune_override(0, 2) == -3 and lib.sa_tune_override(3, 0) == -3
    # a pinned software-pipelined variant applies at head dimension 128 only
    assert lib.sa_tune_override(0, 1) == 0 and lib.sa_launch_choice(64, 8, 0, 0) == 0
    assert lib.sa_launch_choice(128, 8, 0, 0) == lib.sa_query(7)
    assert lib.sa_tune_override(2, 1) == 0 and lib.sa_launch_choice(64, 512, 0, 2) == 0
    for k in range(3):
        assert lib.sa_tune_override(k, -1) == 0
    for code in (-1, -2, -3, -4, -5, -6):
        assert len(lib.sa_error_string(code)) > 10


def test_validation_codes_without_gpu(lib):
    """Bad arguments are rejected on the host, before any HIP call."""
    st = (ctypes.c_int64 * 4)(8 * 16 * 64, 16 * 64, 64, 1)
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf) & ~15
    common = dict(B=1, H=1, T=8, D=64, C=4, R=1, dtype=2)

    def fwd(**kw):
        a = dict(common, **kw)
        return lib.sa_forward(a.get("q", p), p, p, None, 0, a.get("o", p), None, a.get("qs", st), st, st,
                              a["B"], a["H"], a["T"], a["D"], a["C"], a["R"], 0.125, a["dtype"], None)

    assert fwd(dtype=7) == -1
    assert fwd(D=48) == -2
    assert fwd(C=0) == -3
    assert fwd(R=-1) == -3
    assert fwd(B=-1) == -3
    assert fwd(q=None) == -3
    assert fwd(q=p + 2) == -4                                     # misaligned base
    assert fwd(qs=(ctypes.c_int64 * 4)(8192, 1024, 64, 2)) == -4   # dim stride != 1
    assert fwd(qs=(ctypes.c_int64 * 4)(8192, 1024, 63, 1)) == -4   # row stride not a whole vector
    assert fwd(T=2**22, qs=(ctypes.c_int64 * 4)(2**33, 64, 2048, 1)) == -5   # row offsets beyond 32 bits
    assert fwd(qs=(ctypes.c_int64 * 4)(8192, 1024, 0, 1)) == -4    # one row repeated along T
    assert fwd(B=0) == 0 and fwd(T=0) == 0                         # empty problems are no-ops
    assert lib.sa_bwd_delta(p, p, None, st, st, 1, 1, 8, 64, 2, None) == -3
    # the static-workspace backward refuses what its array cannot hold, before any HIP call
    assert lib.sa_backward_static(p, p, p, None, 0, p, p, p, p, p, p, st, st, st, st, st,
                                  1, 33, 2**16, 64, 4, 1, 0.125, 2, None) == -6
    assert lib.sa_bwd_delta(p, p, p, st, st, 1, 1, 8, 17, 2, None) == -2


def test_missing_library_fails_loudly():
    code = ("import os, sys; os.environ['STREAMING_ATTENTION_LIB']='/nonexistent/lib.so';"
            f"sys.path.insert(0, {os.path.join(ROOT, 'kernels_amd')!r});"
            "from streaming_attention import _lib\n"
            "try:\n    _lib.load()\nexcept RuntimeError as e:\n    print('RAISED', e)\n")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert "RAISED" in out.stdout and "no fallback" in out.stdout.lower().replace("there is ", "")


def test_op_schemas_match_reference():
    import streaming_attention  # noqa: F401

    f = torch.ops.alexdremov_streaming_attention.forward.default._schema
    b = torch.ops.alexdremov_streaming_attention.backward.default._schema
    assert [a.name for a in f.arguments] == ["q", "k", "v", "lens", "context_size", "back_contexts", "sm_scale",
                                             "autotune", "return_lse", "prescale_qk", "precision"]
    assert [a.name for a in b.arguments] == ["q", "k", "v", "lens", "o", "lse", "do", "context_size",
                                             "back_contexts", "sm_scale", "autotune", "prescale_qk", "precision"]
    assert len(f.returns) == 2 and len(b.returns) == 3
    assert not any(a.alias_info for a in f.arguments + b.arguments)   # mutates nothing


def test_public_signature():
    import inspect

    from streaming_attention import streaming_attention, streaming_attention_reference

    params = list(inspect.signature(streaming_attention).parameters)
    assert params == ["q", "k", "v", "lens", "context_size", "back_contexts", "sm_scale", "autotune", "return_lse",
                      "prescale_qk", "precision"]
    assert list(inspect.signature(streaming_attention_reference).parameters) == [
        "q", "k", "v", "context_size", "back_contexts", "lens", "scale"]


def test_fake_impls_give_reference_metadata():
    from torch._subclasses.fake_tensor import FakeTensorMode

    import streaming_attention  # noqa: F401

    with FakeTensorMode():
        q = torch.empty(2, 3, 50, 64, dtype=torch.float16).transpose(1, 2).contiguous().transpose(1, 2)
        assert not q.is_contiguous()
        o, lse = torch.ops.alexdremov_streaming_attention.forward(q, q, q, None, 10, 2, 0.125, False, True, False, "ieee")
        assert o.shape == q.shape and o.is_contiguous() and o.dtype == q.dtype
        assert lse.shape == (2, 3, 50) and lse.dtype == torch.float32
        o2, lse2 = torch.ops.alexdremov_streaming_attention.forward(q, q, q, None, 10, 2, 0.125, False, False, False, "ieee")
        assert lse2.numel() == 0
        dq, dk, dv = torch.ops.alexdremov_streaming_attention.backward(q, q, q, None, o, lse, o.float(), 10, 2, 0.125,
                                                                      False, False, "ieee")
        assert all(t.shape == q.shape and t.is_contiguous() and t.dtype == q.dtype for t in (dq, dk, dv))


def test_validation_asserts_like_reference():
    from streaming_attention import ops

    q = torch.zeros(2, 2, 8, 64)
    lens = torch.tensor([8, 8], dtype=torch.int32)
    ops._validate(q, q, q, lens, 4, 1, 0.1)
    for bad in (dict(context_size=0), dict(back_contexts=-1), dict(sm_scale=None)):
        kw = dict(context_size=4, back_contexts=1, sm_scale=0.1)
        kw.update(bad)
        with pytest.raises(AssertionError):
            ops._validate(q, q, q, lens, **kw)
    with pytest.raises(AssertionError):
        ops._validate(torch.zeros(2, 2, 8, 48), q, q, lens, 4, 1, 0.1)          # head dim
    with pytest.raises(AssertionError):
        ops._validate(q, torch.zeros(2, 2, 9, 64), q, lens, 4, 1, 0.1)          # T mismatch
    with pytest.raises(AssertionError):
        ops._validate(q, q, q, lens.long(), 4, 1, 0.1)                          # lens dtype
    with pytest.raises(AssertionError):
        ops._validate(q, q, q, lens[:1], 4, 1, 0.1)                             # lens length


def test_placement_validation_launches_nothing():
    """A tensor on another device, or k / v with fewer batches or heads than q (an un-expanded
    grouped-query tensor), is refused with an AssertionError before any pointer is taken."""
    from streaming_attention import ops

    q = torch.zeros(2, 4, 8, 64)
    lens = torch.tensor([8, 8], dtype=torch.int32)
    meta = torch.zeros(2, 4, 8, 64, device="meta")
    with pytest.raises(AssertionError):
        ops._validate(q, meta, q, lens, 4, 1, 0.1)                              # k elsewhere
    with pytest.raises(AssertionError):
        ops._validate(q, q, meta, lens, 4, 1, 0.1)                              # v elsewhere
    with pytest.raises(AssertionError):
        ops._validate(q, q, q, lens.to("meta"), 4, 1, 0.1)                      # lens elsewhere
    with pytest.raises(AssertionError):
        ops._validate(q, torch.zeros(2, 1, 8, 64), q, lens, 4, 1, 0.1)          # k with one head
    with pytest.raises(AssertionError):
        ops._validate(q, q, torch.zeros(1, 4, 8, 64), lens, 4, 1, 0.1)          # v with one batch
    with pytest.raises(AssertionError):
        ops._validate(q, q, q, lens, 4, 1, 0.1, meta, q)                        # o elsewhere
    with pytest.raises(AssertionError):
        ops._validate(q, q, q, lens, 4, 1, 0.1, q, torch.zeros(2, 4, 9, 64))    # dO of another shape
    ops._validate(q, q, q, lens, 4, 1, 0.1, q, q)
    with pytest.raises(AssertionError):
        ops._validate_placement(q, q[:, :1], q, None)


def test_kernel_layout_rule():
    from streaming_attention.ops import _kernel_layout

    x = torch.zeros(2, 4, 16, 64, dtype=torch.float16)
    assert _kernel_layout(x) is x
    bthd = torch.zeros(2, 16, 4, 64, dtype=torch.float16).transpose(1, 2)       # [B,H,T,D] view of [B,T,H,D]
    assert _kernel_layout(bthd) is bthd
    sliced = torch.zeros(2, 4, 16, 128, dtype=torch.float16)[..., ::2]           # dim stride 2
    assert _kernel_layout(sliced).is_contiguous() and _kernel_layout(sliced) is not sliced
    odd = torch.zeros(2, 4, 16, 68, dtype=torch.float16)[..., 4:]                # base 8 bytes off, row 68
    assert _kernel_layout(odd).is_contiguous()


def test_bench_rejects_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                         text=True, timeout=300)
    assert out.returncode != 0 and "one GPU" in (out.stderr + out.stdout)


def test_flop_counter_matches_oracle():
    sys.path.insert(0, ROOT)
    import bench
    from oracle import sa_oracle

    for T, C, R, lens in ((512, 64, 2, [300, 512]), (100, 7, 3, [1, 99, 100]), (64, 1000, 0, [64])):
        assert bench.unmasked_pairs(T, C, R, lens) == sa_oracle.unmasked_pairs(T, C, R, lens)


def test_traffic_figures_match_profile_summaries():
    """`roofline.traffic` is quoted from profiles/hbm_traffic.json; every figure in it must be the
    'HBM bytes / launch' entry of the traffic table in the per-workload summary it is said to come from."""
    sys.path.insert(0, ROOT)
    import bench

    summaries = {
        "headline_bf16_T16384_D128": "streaming_attention_bf16_B4_H16_T16384_D128_C256_R8.md",
        "bf16_T4096_D64": "streaming_attention_bf16_B8_H16_T4096_D64_C128_R4.md",
        "ragged_fp16_T2048_D128": "streaming_attention_fp16_B16_H8_T2048_D128_C64_R1_ragged.md",
        "long_bf16_T65536_D128": "streaming_attention_bf16_B1_H32_T65536_D128_C512_R16.md",
    }
    quoted = bench.hbm_bytes_per_launch()
    assert set(quoted) == set(summaries)
    for workload, fname in summaries.items():
        text = open(os.path.join(ROOT, "profiles", fname)).read()
        section = text[text.index("## 2. HBM traffic"):text.index("## 3.")]
        header = next(ln for ln in section.splitlines() if ln.startswith("| kernel |"))
        col = [c.strip() for c in header.strip("|").split("|")].index("HBM bytes / launch")
        table = {}
        for ln in section.splitlines():
            cells = [c.strip() for c in ln.strip("|").split("|")]
            if ln.startswith("|") and len(cells) > col and cells[0] not in ("kernel", "---"):
                # fwd2 / fwd3 -> fwd, dq2 / dq3 -> dq, dkdv2 / dkdv3 / dkdv_split -> dkdv, delta
                table[re.sub(r"(_split|\d)+$", "", cells[0])] = float(cells[col])
        assert set(quoted[workload]) == set(table) == {"fwd", "dq", "dkdv", "delta"}, workload
        for kernel, value in quoted[workload].items():
            assert value == pytest.approx(table[kernel], rel=1e-9), (workload, kernel)
    assert set(quoted) <= set(bench.WORKLOADS)
