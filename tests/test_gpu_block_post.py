"""The step after the layer (residual add / hyper-connection post mix): bit-exact against the oracle through the
C ABI, at decode and prefill sizes and for every supported number of residual streams."""
import numpy as np
import pytest
import torch

from tests.helpers import bf16_bits

pytestmark = pytest.mark.gpu


def _inputs(T, D, m, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((T, D), generator=g, device="cuda").to(torch.bfloat16)
    shape = (T, D) if m == 0 else (T, m, D)
    res = (torch.randn(shape, generator=g, device="cuda") * 3).to(torch.bfloat16)
    if m == 0:
        return x, res, None, None
    post = torch.sigmoid(torch.randn((T, m, 1), generator=g, device="cuda")) * 2.0       # deepseek_v4.zig:2310-2316
    comb = torch.softmax(torch.randn((T, m, m), generator=g, device="cuda"), dim=-1)
    return x, res, post, comb


@pytest.mark.parametrize("T,D,m", [(64, 4096, 4), (1, 64, 4), (2080, 4096, 4), (7, 1024, 1), (33, 512, 2),
                                   (5, 256, 8), (64, 4096, 0), (3, 8, 0), (8192, 4096, 0)])
def test_block_post_bit_exact(dmoe, orc, T, D, m):
    x, res, post, comb = _inputs(T, D, m, 100 + m)
    got = dmoe.block_post(x, res, post, comb)
    want = orc.block_post(bf16_bits(x), bf16_bits(res), None if post is None else post.cpu().numpy(),
                          None if comb is None else comb.cpu().numpy())
    np.testing.assert_array_equal(bf16_bits(got), want)


def test_block_post_empty_and_errors(dmoe):
    x = torch.zeros((0, 64), dtype=torch.bfloat16, device="cuda")
    assert dmoe.block_post(x, x.clone()).shape == (0, 64)
    x = torch.zeros((2, 12), dtype=torch.bfloat16, device="cuda")        # D not a multiple of 8
    with pytest.raises(dmoe.DmoeError):
        dmoe.block_post(x, x.clone())
    x = torch.zeros((2, 16), dtype=torch.bfloat16, device="cuda")
    res = torch.zeros((2, 9, 16), dtype=torch.bfloat16, device="cuda")   # more residual streams than supported
    with pytest.raises(dmoe.DmoeError):
        dmoe.block_post(x, res, torch.zeros((2, 9), device="cuda"), torch.zeros((2, 9, 9), device="cuda"))
