"""The hand-scheduled forward kernel on streams: launches that overlap on two streams, and launches replayed from a
captured graph with eager launches in between.  The library keeps no state between launches, so every result
must equal the first eager one bit for bit; the compiler-scheduled kernel is the tolerance check beside it."""
import pytest
import torch

pytestmark = pytest.mark.gpu

D = 128


def _problem(B, H, T, seed, dtype, lens_list):
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    q, k, v = ((torch.randn(B, H, T, D, generator=g, device=dev) * 0.5).to(dtype) for _ in range(3))
    lens = torch.tensor(lens_list, dtype=torch.int32, device=dev) if lens_list is not None else None
    return q, k, v, lens


def _forward(q, k, v, lens, C, R):
    from streaming_attention import streaming_attention

    return streaming_attention(q, k, v, lens, C, R, return_lse=True)


@pytest.fixture()
def pipelined_forward():
    from streaming_attention import _lib

    lib = _lib.load()
    if lib.sa_query(7) != 1:
        pytest.skip("library built without the hand-scheduled kernels")
    assert lib.sa_tune_override(0, 1) == 0
    yield lib
    lib.sa_tune_override(0, -1)


# the second problem: a number of (batch, head) pairs that is not a multiple of the 8 XCDs (the other branch of the
# block order), chunks smaller than a workgroup's 256 queries (waves of one workgroup walk different tile ranges)
@pytest.mark.parametrize("B,H,T,C,R,lens_list", [(5, 8, 4700, 256, 8, [4700, 0, 3111, 5000, 256]),
                                                 (3, 7, 6300, 96, 40, [6300, 6001, 17])], ids=["40 pairs", "21 pairs"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
def test_graph_replays_equal_eager_launches(pipelined_forward, dtype, B, H, T, C, R, lens_list):
    lib = pipelined_forward
    q, k, v, lens = _problem(B, H, T, 7, dtype, lens_list)
    # three launches in a row on one stream
    eager = [_forward(q, k, v, lens, C, R) for _ in range(3)]
    torch.cuda.synchronize()
    # captured, replayed twice with eager work in between
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _forward(q, k, v, lens, C, R)          # first call of the shape outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, lse_g = _forward(q, k, v, lens, C, R)
    for _ in range(2):
        o_g.fill_(float("nan"))
        graph.replay()
        between = _forward(q, k, v, lens, C, R)
        torch.cuda.synchronize()
        for o, lse in eager + [between]:
            assert torch.equal(o, o_g) and torch.equal(lse, lse_g)
    # and the compiler-scheduled kernel, to the 16-bit bar
    lib.sa_tune_override(0, 0)
    o_n, lse_n = _forward(q, k, v, lens, C, R)
    lib.sa_tune_override(0, 1)
    assert (o_n.float() - o_g.float()).abs().max().item() <= 2e-2
    assert (lse_n - lse_g).abs().max().item() <= 1e-4
    short = min(range(B), key=lambda b: lens_list[b])                  # the empty (or nearly empty) sequence
    n = min(lens_list[short], T)
    assert o_g[short, :, n:].abs().max().item() == 0.0 and lse_g[short, :, n:].abs().max().item() == 0.0


def test_forward_on_two_overlapping_streams(pipelined_forward):
    p1 = _problem(4, 8, 4608, 11, torch.bfloat16, [4608, 4000, 2222, 4608]) + (256, 8)
    p2 = _problem(2, 16, 5000, 12, torch.bfloat16, None) + (512, 4)
    want1, want2 = _forward(*p1), _forward(*p2)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got1, got2 = [], []
    for _ in range(8):          # nothing waits between the launches: the two streams overlap
        with torch.cuda.stream(s1):
            got1.append(_forward(*p1))
        with torch.cuda.stream(s2):
            got2.append(_forward(*p2))
    torch.cuda.synchronize()
    for o, lse in got1:
        assert torch.equal(o, want1[0]) and torch.equal(lse, want1[1])
    for o, lse in got2:
        assert torch.equal(o, want2[0]) and torch.equal(lse, want2[1])


@pytest.mark.parametrize("dtype,D_,C,R", [(torch.bfloat16, 128, 256, 8), (torch.float16, 128, 64, 1), (torch.bfloat16, 64, 128, 4),
                                         (torch.float32, 32, 16, 3)], ids=str)
def test_step_replayed_from_a_graph_equals_the_eager_step(dtype, D_, C, R):
    """Forward and backward through the public function, captured once and replayed three times with eager steps in
    between: every replay must reproduce the eager gradients bit for bit (a graph must hold nothing but the
    library's kernels and torch's own fill and copy kernels)."""
    from streaming_attention import streaming_attention

    dev = torch.device("cuda:0")
    B, H, T = 3, 4, 1500
    g = torch.Generator(device=dev).manual_seed(21)
    q, k, v, d_o = ((torch.randn(B, H, T, D_, generator=g, device=dev) * 0.5).to(dtype) for _ in range(4))
    lens = torch.tensor([1500, 700, 64], dtype=torch.int32, device=dev)
    for t in (q, k, v):
        t.requires_grad_()

    def step():
        q.grad = k.grad = v.grad = None
        out = streaming_attention(q, k, v, lens, C, R)
        out.backward(d_o)
        return out

    want_o = step().detach().clone()
    want = [t.grad.clone() for t in (q, k, v)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    q.grad = k.grad = v.grad = None
    with torch.cuda.graph(graph):
        out_g = streaming_attention(q, k, v, lens, C, R)
        out_g.backward(d_o)
    grads_g = [q.grad, k.grad, v.grad]          # static tensors of the graph
    for _ in range(3):
        for t in grads_g:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want_o)
        for got, w_ in zip(grads_g, want):
            assert torch.equal(got, w_)
        # eager work of the same kind between the replays, on fresh gradient tensors
        keep = [q.grad, k.grad, v.grad]
        step()
        q.grad, k.grad, v.grad = keep
        torch.cuda.synchronize()
