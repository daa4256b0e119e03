"""Block-fp8 W8A8 layers (the DeepSeek-V3-shaped configurations) on the GPU against the oracle:
routing bit-exact, activation quant bit-exact, layer output within the benchmark's tolerance."""
import numpy as np
import pytest
import torch

import oracle_lib as ol
from gpu_harness import assert_output_close, assert_routing_equal, both
from plow_amd import abi, layer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def check_layer(plan, dev, host):
    cfg = plan.cfg
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    assert np.array_equal(dev.np("xq"), host.np("xq"))
    assert np.array_equal(dev.np("xs").view(np.uint32), host.np("xs").view(np.uint32))
    # intermediate: dequantized fq * fs of live rows agrees to fp8 precision
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    fqd, fqh = dev.np("fq")[:rows][live], host.np("fq")[:rows][live]
    fsd, fsh = dev.np("fs")[:rows][live], host.np("fs")[:rows][live]
    same = (fqd == fqh).mean()
    print(f"[parity] fq bytes identical on {same * 100:.3f} % of live elements", flush=True)
    assert same > 0.98
    assert np.allclose(fsd, fsh, rtol=1e-4)
    pd, ph = dev.np("part"), host.np("part")
    assert np.all(np.isfinite(pd))
    err = np.abs(pd - ph).max() / np.abs(ph).max()
    print(f"[parity] part: max_abs/max|ref| = {err:.3e}", flush=True)
    assert err < 2e-2
    return assert_output_close(dev.np("out"), host.np("out"))


@pytest.mark.parametrize("T", [1, 7, 24, 100])
def test_small_dsv3_like_layer(moe, oracle, T):
    cfg = layer.MoeConfig("mini", H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True,
                          bias=True, n_group=4, topk_group=2, route_scale=2.5, enc="fp8blk",
                          arm="w8a8", n_shared=1, shared_mode="fold")
    check_layer(*both(moe, oracle, cfg, seed=T))


def test_rows_per_expert_beyond_one_tile(moe, oracle):
    """Few experts, many tokens: segments of 17..300 rows walk every row-tile arm of the kernel."""
    cfg = layer.MoeConfig("dense-ish", H=256, E=4, I=128, k=2, T=300, scoring="softmax",
                          norm_topk=True, enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold",
                          residual=True)
    check_layer(*both(moe, oracle, cfg, seed=3))


def test_dsv3_decode_b64_full_shape(moe, oracle):
    """The headline decode cell at its real shape (H 7168, 256 + 1 experts, I 2048, B = 64)."""
    cfg = layer.config("c2")
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    check_layer(plan, dev, host)
    cnt = host.np("meta")[cfg.E_all:2 * cfg.E_all]
    print(f"[c2] experts hit {int((cnt[:cfg.E] > 0).sum())} / {cfg.E}, max rows {int(cnt[:cfg.E].max())}", flush=True)
