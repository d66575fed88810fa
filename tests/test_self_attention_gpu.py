"""The dense variable-length forward exposed under the reference's ``self_attention`` names
(tests/test_self_attention.py of the reference compares against masked SDPA with atol 1e-3)."""
import pytest
import torch

from oracle import sa_oracle
from tests.helpers import assert_close, make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [16, 128])
@pytest.mark.parametrize("B,H,T", [(1, 1, 1), (3, 2, 77), (2, 3, 700)])
@pytest.mark.parametrize("use_lens", [False, True])
def test_self_attention_forward(B, H, T, D, dtype, use_lens):
    from self_attention import self_attention, self_attention_reference

    dev = torch.device("cuda:0")
    q, k, v, _ = make_inputs(B, H, T, D, seed=40, dtype=dtype)
    lens = None
    if use_lens:
        g = torch.Generator().manual_seed(41)
        lens = torch.randint(1, T + 2, (B,), generator=g, dtype=torch.int32)
    out = self_attention(q.to(dev), k.to(dev), v.to(dev), lens.to(dev) if lens is not None else None)
    ref = sa_oracle.dense_f64(q, k, v, lens, max(T, 1), 0)
    assert_close("O", out, ref["O"], dtype)
    # and the package's own torch reference agrees with the oracle on the same inputs
    want, _ = self_attention_reference(q.float(), k.float(), v.float(), lens)
    assert_close("reference", want, ref["O"], torch.float32)


def test_self_attention_opcheck():
    import self_attention  # noqa: F401

    dev = torch.device("cuda:0")
    q, k, v, _ = (t.to(dev) for t in make_inputs(2, 2, 40, 64, seed=42, dtype=torch.float16))
    lens = torch.tensor([40, 13], dtype=torch.int32, device=dev)
    torch.library.opcheck(torch.ops.alexdremov_flash_attention.forward, (q, k, v, lens, 0.125, False, False),
                          test_utils=("test_schema", "test_faketensor"), atol=1e-2, rtol=float("inf"))
