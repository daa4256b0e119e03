"""The benchmark configurations at their real shapes: routing bit-exact, outputs within the
benchmark tolerance. Configurations too large for the oracle to replay whole (4096-token prefill)
are checked on routing for every token and on the layer output for a sample of tokens: a token's
output depends only on its own activation row and the weights, so the oracle replays the sampled
rows as a small batch over the same weights."""
import numpy as np
import pytest
import torch

import oracle_lib as ol
from gpu_harness import (assert_output_close, assert_routing_equal, both, run_device, run_oracle)
from plow_amd import abi, layer, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def test_c1_small_bf16_layer(moe, oracle):
    cfg = layer.config("c1")
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    assert_output_close(dev.np("out"), host.np("out"), "c1 out")


@pytest.mark.parametrize("B", [1, 16, 128])
def test_c4_kimi_k2_mxfp4_decode(moe, oracle, B):
    cfg = layer.config("c4", B)
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"), f"c4 B={B} out")


@pytest.mark.parametrize("arm", ["a16", "w8a8"])
@pytest.mark.parametrize("T", [1, 8, 64])
def test_c5_qwen3_per_channel_fp8(moe, oracle, T, arm):
    cfg = layer.config("c5", T)
    cfg.arm = arm
    plan, dev, host = both(moe, oracle, cfg, seed=0)
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"), f"c5 T={T} {arm} out")


def test_c3_dsv3_prefill_4k(moe, oracle):
    cfg = layer.config("c3")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, hot_expert=3.0)
    run_device(moe, plan, dev)
    check_prefill_sampled(oracle, cfg, plan, dev, want_skew=True)


@pytest.mark.parametrize("arm", ["w8a8", "a16"])
def test_c6_glm_tp8_slice_prefill_8k(moe, oracle, arm):
    """The shape of plow's own gfx950 prefill bench (288 experts, top-8, H 4096, I 256 per rank, 8192
    tokens), fp8 activations on the tiled kernels and bf16 activations on the four-row-group passes."""
    print(f"[case] c6 arm={arm}", flush=True)
    cfg = layer.config("c6")
    cfg.arm = arm
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=0, zipf=0.5)
    run_device(moe, plan, dev)
    check_prefill_sampled(oracle, cfg, plan, dev, want_skew=False)


def check_prefill_sampled(oracle, cfg, plan, dev, want_skew):
    w8a8 = cfg.arm == "w8a8"
    # routing and activation quant for all 4096 tokens, on the CPU
    host = synth.Bound(plan, "cpu")
    for name in ("logit", "table", "meta", "row_token", "row_partidx", "row_gate") + (("xq", "xs") if w8a8 else ()):
        host.alloc(name)
    for name in ("x", "Wr", "bias"):
        host.t[name] = dev.t[name].cpu()
    run_oracle(oracle, plan, host, labels=["score", "topk", "align"] + (["quant_x"] if w8a8 else []))
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    if w8a8:
        assert np.array_equal(dev.np("xq"), host.np("xq"))
        assert np.array_equal(dev.np("xs").view(np.uint32), host.np("xs").view(np.uint32))
    cnt = host.np("meta")[cfg.E_all:2 * cfg.E_all][:cfg.E]
    print(f"[{cfg.name}] rows/expert min {cnt.min()} median {np.median(cnt)} max {cnt.max()} "
          f"(x{cnt.max() / cnt.mean():.2f} mean), {int((cnt < 64).sum())} experts below 64 rows", flush=True)
    if want_skew:
        assert cnt.max() >= 2.0 * cnt.mean()        # the skew the configuration asks for
    # layer output of a sample of tokens against the oracle over the same weights
    pick = np.array([0, 1, 777, 2048, cfg.T - 1, 1234, 3001, 99])
    sub_cfg = layer.config(cfg.name, len(pick))
    sub_cfg.arm = cfg.arm
    sub = layer.plan_layer(sub_cfg)
    full_host = synth.to_host(dev)
    sh = synth.Bound(sub, "cpu")
    for name, sp in sub.specs.items():
        if sp.role in ("scratch", "out", "table"):
            sh.alloc(name)
    sh.t["x"] = full_host.t["x"][torch.from_numpy(pick)].contiguous()
    for name in ("Wr", "bias", "wtab", "stab"):
        sh.t[name] = full_host.t[name]
    sh.experts = full_host.experts
    run_oracle(oracle, sub, sh)
    assert np.array_equal(sh.np("table")["eid"].reshape(len(pick), -1),
                          host.np("table")["eid"].reshape(cfg.T, -1)[pick])
    assert_output_close(dev.np("out")[pick], sh.np("out"), f"{cfg.name} sampled out")
