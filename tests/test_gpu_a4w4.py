"""The fp4 x fp4 arm of ops 85 / 86 (mxfp4 weights, activations quantized to mxfp4 per 32 values) on the
GPU against the oracle: the quantized intermediate (codes and E8M0 bytes), the partials and the layer
output, on data where every sum is exact (any mistake in an operand layout, a scale byte or the
quantizer then shows as a different code) and on random data at many rows per expert."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as ol
from gpu_harness import assert_output_close, assert_routing_equal, both, run_device, run_oracle
from plow_amd import abi, layer, synth

pytestmark = pytest.mark.gpu

LADDER = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], np.float64)


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def dequant(codes, scales):
    """mxfp4 rows [R][n / 2] with E8M0 rows [R][n / 32] -> f64 [R][n]"""
    lo, hi = codes & 0xF, codes >> 4
    c = np.stack([lo, hi], axis=-1).reshape(codes.shape[0], -1)
    v = LADDER[c & 7] * np.where(c & 8, -1.0, 1.0)
    return v * np.repeat(np.exp2(scales.astype(np.float64) - 127.0), 32, axis=1)


def close(a, b, what, max_frac=2e-2, mean_rel=5e-3):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert np.all(np.isfinite(a)), what
    err = np.abs(a - b)
    mx = err.max() / max(np.abs(b).max(), 1e-30)
    mr = err.mean() / max(np.abs(b).mean(), 1e-30)
    print(f"[parity] {what}: max_abs/max|ref| = {mx:.3e}, mean rel = {mr:.3e}", flush=True)
    assert mx <= max_frac and mr <= mean_rel, (what, mx, mr)


def intermediate(plan, dev, host, rows):
    """live rows of the quantized intermediate, device and oracle"""
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    return (dev.np("fu4")[:rows][live], dev.np("fsc")[:rows][live],
            host.np("fu4")[:rows][live], host.np("fsc")[:rows][live])


def check_intermediate(plan, dev, host, rows, code_frac, scale_frac):
    """E8M0 bytes equal but for a few blocks whose amax sits on a power of two within an ulp; codes of
    the blocks with equal bytes equal but for a few values within an ulp of a rounding boundary, those
    one step apart; and the dequantized rows close."""
    dq, ds, hq, hs = intermediate(plan, dev, host, rows)
    sdiff = ds != hs
    print(f"[parity] fsc: {sdiff.mean():.3e} of the E8M0 bytes differ (<= {scale_frac})", flush=True)
    assert sdiff.mean() <= scale_frac
    assert np.all(np.abs(ds.astype(np.int32) - hs.astype(np.int32)) <= 1)
    same = np.repeat(~sdiff, 16, axis=1)
    dc = np.stack([dq & 0xF, dq >> 4], -1)[same]
    hc = np.stack([hq & 0xF, hq >> 4], -1)[same]
    cdiff = dc != hc
    print(f"[parity] fu4: {cdiff.mean():.3e} of the codes differ (<= {code_frac})", flush=True)
    assert cdiff.mean() <= code_frac
    # a differing pair is one ladder step apart (or +0 / -0.5-side neighbours across zero)
    signed = lambda c: np.where(c & 8, -1, 1) * (c & 7).astype(np.int32)
    assert np.all(np.abs(signed(dc[cdiff]) - signed(hc[cdiff])) <= 1)
    close(dequant(dq, ds), dequant(hq, hs), "fu (dequantized)")


def exact_data(dev, cfg, seed):
    """Rows and weights on which every fp4 x fp4 sum is exact in f32 in any order: x on the e2m1 ladder with
    a 6 in every 32-block (one scale for all blocks), weight E8M0 bytes within 2^3 of each other."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    lad = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    x = lad[torch.randint(0, 8, (cfg.T, cfg.H), generator=g)] * (torch.randint(0, 2, (cfg.T, cfg.H), generator=g) * 2 - 1)
    x[:, ::32] = 6.0
    dev.t["x"].copy_(x.to(torch.bfloat16).to(dev.device))
    for ws, ss in dev.experts:
        for w, s in zip(ws, ss):
            w.copy_(torch.randint(0, 256, tuple(w.shape), generator=g, dtype=torch.uint8).to(dev.device))
            s.copy_(torch.randint(113, 117, tuple(s.shape), generator=g, dtype=torch.uint8).to(dev.device))


@pytest.mark.parametrize("T,E,k", [(70, 4, 2), (333, 8, 2), (1030, 3, 1)])
def test_exact_sums_give_the_oracles_codes(moe, oracle, T, E, k):
    cfg = layer.MoeConfig("a4w4-exact", T=T, H=512, I=512, E=E, k=k, scoring="softmax", norm_topk=True,
                          enc="mxfp4", arm="a4w4")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=T)
    exact_data(dev, cfg, T)
    host = synth.to_host(dev)
    run_device(moe, plan, dev)
    run_oracle(oracle, plan, host)
    rows = assert_routing_equal(plan, dev, host)
    # gate and up are the same f32 on both sides; what may differ is the last bit of the activation
    check_intermediate(plan, dev, host, rows, code_frac=1e-3, scale_frac=1e-3)
    close(dev.np("part"), host.np("part"), "part")
    assert_output_close(dev.np("out"), host.np("out"))


@pytest.mark.parametrize("T,E,k,act", [(5, 8, 4, 1), (40, 8, 4, 1), (300, 8, 2, 4), (777, 8, 4, 2)])
def test_a4w4_layer(moe, oracle, T, E, k, act):
    cfg = layer.MoeConfig("a4w4-mini", T=T, H=768, I=512, E=E, k=k, scoring="sigmoid", norm_topk=True, bias=True,
                          route_scale=2.5, enc="mxfp4", arm="a4w4", act=act,
                          act_f=(0.0, 0.0) if act == 1 else (1.702, 1.5))
    plan, dev, host = both(moe, oracle, cfg, seed=T, x_std=1.0, w_std=0.05)
    rows = assert_routing_equal(plan, dev, host)
    check_intermediate(plan, dev, host, rows, code_frac=2e-3, scale_frac=2e-3)
    close(dev.np("part"), host.np("part"), "part")
    assert_output_close(dev.np("out"), host.np("out"))


def test_a4w4_bf16_partials_and_a_second_smaller_batch(moe, oracle):
    """arm 1 of op 86 (bf16 partials); then a smaller batch on the same context, whose staging block keeps
    the rows of the call before"""
    for T in (200, 9):
        cfg = layer.MoeConfig("a4w4-p16", T=T, H=512, I=768, E=4, k=2, scoring="softmax", norm_topk=False,
                              enc="mxfp4", arm="a4w4", part_bf16=True)
        plan, dev, host = both(moe, oracle, cfg, seed=T, w_std=0.05)
        rows = assert_routing_equal(plan, dev, host)
        check_intermediate(plan, dev, host, rows, code_frac=2e-3, scale_frac=2e-3)
        close(ol.bf2f(dev.np("part")), ol.bf2f(host.np("part")), "part (bf16)")
        assert_output_close(dev.np("out"), host.np("out"))


def clone(inst):
    c = abi.PlowDevInst()
    C.memmove(C.byref(c), C.byref(inst), C.sizeof(c))
    return c


def test_a4w4_refusals(moe):
    cfg = layer.MoeConfig("a4w4-refuse", T=4, H=512, I=512, E=4, k=2, scoring="softmax", enc="mxfp4", arm="a4w4")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=1)
    glu, down = plan.insts[plan.index("glu")], plan.insts[plan.index("down")]
    assert moe.check(glu, dev.table()) == 0 and moe.check(down, dev.table()) == 0
    for field, value in ((4, 0), (0, 384), (1, 640), (1, 256)):   # no T, I and H off the 256 grid, H too short
        bad = clone(glu)
        bad.i[field] = value
        assert moe.check(bad, dev.table()) == abi.E_INVAL, (field, value, moe.last_error())
    bad = clone(glu)
    bad.t[7] = abi.TENSOR_NONE
    assert moe.check(bad, dev.table()) == abi.E_INVAL
    bad = clone(down)
    bad.t[5] = abi.TENSOR_NONE
    assert moe.check(bad, dev.table()) == abi.E_INVAL
    bad = clone(down)
    bad.i[7] = 2   # the block-fp8 arm's number under the mxfp4 encoding
    assert moe.check(bad, dev.table()) == abi.E_UNSUPPORTED
    # the tiled kernel's directory counts row tiles in 16 bits: a stated row count that may exceed it is refused
    for op in (glu, down):
        bad = clone(op)
        bad.fj[2].u = 128 * 65535
        assert moe.check(bad, dev.table()) == abi.E_INVAL and "row tiles" in moe.last_error()
    # the staging of the quantized token rows belongs to the context and no op grows it: a batch beyond it is
    # refused before launch, and served once the caller has made room
    from plow_amd.lib import Moe
    own = Moe(0)
    big = clone(glu)
    big.i[1], big.i[4] = 7168, 20000                                # 76 MB of staging; a new context holds 32 MiB
    assert own.check(big, dev.table()) == abi.E_INVAL and "plow_moe_reserve_staging" in own.last_error()
    assert own.reserve_staging(20000, 7168) == 0
    assert own.check(big, dev.table()) == 0
    own.close()
    # the entry point that allocates nothing has no staging block
    err = C.create_string_buffer(256)
    rc = moe.lib.plow_moe_exec_noalloc(C.byref(glu), dev.table(), None, err, 256)
    assert rc == abi.E_UNSUPPORTED and b"context" in err.value, (rc, err.value)


def test_a4w4_skips_a_non_resident_expert_and_survives_a_token_past_the_batch(moe, oracle):
    """A null weight-table row (expert not resident on this rank): both ops leave its rows alone. A row whose
    token lies past the rows the op was told of (i4) is read from row 0 of the staged batch instead of from
    memory that was never staged: the layer's other rows are unaffected."""
    cfg = layer.MoeConfig("a4w4-null", H=512, E=4, I=512, k=2, T=150, scoring="softmax", norm_topk=True,
                          enc="mxfp4", arm="a4w4", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=11)
    dev.t["wtab"][1].zero_()                       # expert 1 is elsewhere
    dev.t["part"].fill_(0.25)                      # untouched rows must keep this
    dev.t["fu4"].fill_(0x77)
    host = synth.to_host(dev)
    host.t["wtab"][1].zero_()                      # (the host table holds host pointers of its own)
    run_device(moe, plan, dev)
    run_oracle(oracle, plan, host)
    rows = assert_routing_equal(plan, dev, host)
    pd, ph = dev.np("part"), host.np("part")
    untouched = (ph == 0.25).all(axis=1)
    assert untouched.any() and np.array_equal(pd[untouched], ph[untouched])
    assert_output_close(dev.np("out"), host.np("out"))
    # the GLU told of fewer rows than the row map names
    glu = clone(plan.insts[plan.index("glu")])
    glu.i[4] = 100
    want = dev.np("fu4").copy()
    moe.exec(glu, dev.table())
    torch.cuda.synchronize()
    tok = dev.np("row_token")[:rows]
    fine = (tok < 100) & (dev.np("row_partidx")[:rows] != abi.EXPERT_UNUSED)
    assert fine.any() and np.array_equal(dev.np("fu4")[:rows][fine], want[:rows][fine])
