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


# Share of the intermediate's e4m3 bytes that must equal the oracle's. A byte differs where the f32 sum of a
# 128-k block, added in the matrix instruction's order here and in index order there, lands on the other side
# of an e4m3 rounding boundary, or where the row's amax (and with it the scale) differs in its last bit. The
# floor is set a little under the smallest share measured over this file's cases (printed by every case).
FQ_SAME_FLOOR = 0.98


def check_layer(plan, dev, host):
    cfg = plan.cfg
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    if "xq" in dev.t:
        assert np.array_equal(dev.np("xq"), host.np("xq"))
        assert np.array_equal(dev.np("xs").view(np.uint32), host.np("xs").view(np.uint32))
    # intermediate: dequantized fq * fs of live rows agrees to fp8 precision
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    fqd, fqh = dev.np("fq")[:rows][live], host.np("fq")[:rows][live]
    fsd, fsh = dev.np("fs")[:rows][live], host.np("fs")[:rows][live]
    same = (fqd == fqh).mean()
    print(f"[parity] fq bytes identical on {same * 100:.3f} % of live elements", flush=True)
    assert same > FQ_SAME_FLOOR
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


@pytest.mark.parametrize("T,k,H,I,arm", [(1, 8, 512, 1024, "w8a8"), (2, 8, 512, 2048, "w8a8"), (4, 8, 512, 1408 + 128, "w8a8"),
                                         (3, 4, 512, 1024, "w8a8_p16"), (1, 8, 1024, 1024, "w8a8"), (4, 8, 2048 + 512, 1280, "w8a8"),
                                         (2, 6, 7168, 256, "w8a8")])
def test_few_tokens_as_matrix_vector_products(moe, oracle, T, k, H, I, arm):
    """With at most 36 routed rows and intermediate rows of a kilobyte or more the fp8 x fp8 DOWN runs as
    matrix-vector products (e4m3 rows widened to bf16 exactly, activation and weight block scales multiplied
    as in the streaming kernel): f32 and bf16 partials, rows of one and of several 1 KB pieces, experts with
    several rows, hidden sizes from 512 to 7168 (the GLU stays on its tile kernel at every one of them)."""
    print(f"[case] w8a8 gemv T={T} k={k} H={H} I={I} arm={arm}", flush=True)
    p16 = arm == "w8a8_p16"
    cfg = layer.MoeConfig("w8a8-gemv", H=H, E=16, I=I, k=k, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          route_scale=2.5, enc="fp8blk", arm="w8a8", part_bf16=p16, n_shared=1, shared_mode="fold")
    assert T * cfg.k_all <= 36
    plan, dev, host = both(moe, oracle, cfg, seed=11 * T + k)
    if p16:
        assert_routing_equal(plan, dev, host)
        assert_output_close(dev.np("part").reshape(-1), host.np("part").reshape(-1), "part (bf16)")
        assert_output_close(dev.np("out"), host.np("out"))
    else:
        check_layer(plan, dev, host)


@pytest.mark.parametrize("T", [1, 19, 100, 333, 700])
def test_glu_quantizes_bf16_rows_itself(moe, oracle, T):
    """Op 85 arm 6: bf16 rows in, quantized 1x128 where the kernel loads them, no quantizer op and no
    xq / xs tensors (plow runtime/amd/moe_pf_w8a8.h:118-121). The fq bytes and fs scales must also be the
    very ones the quantizer + arm 2 chain of the same library produces on the same inputs when that chain
    runs the same streaming kernel (few rows per expert)."""
    print(f"[case] w8a8 arm 6 T={T}", flush=True)
    kw = dict(H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True, n_group=4,
              topk_group=2, route_scale=2.5, enc="fp8blk", n_shared=1, shared_mode="fold")
    plan, dev, host = both(moe, oracle, layer.MoeConfig("mini-xq", arm="w8a8q", **kw), seed=T)
    assert "xq" not in dev.t and "quant_x" not in plan.names
    check_layer(plan, dev, host)
    # from 16 rows per expert on average the op runs as quantizer + tiled arm 2 over the context's staging (its i4
    # states the rows): the bytes must be those of the two-op chain, which runs the same two kernels
    if T * 5 >= 16 * 33:
        ref = both(moe, oracle, layer.MoeConfig("mini-x2", arm="w8a8", **kw), seed=T)[1]
        rows = int(dev.np("meta")[3 * plan.cfg.E_all]) * abi.MPF_BM
        live = dev.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
        assert np.array_equal(dev.np("fq")[:rows][live], ref.np("fq")[:rows][live])
        assert np.array_equal(dev.np("fs")[:rows][live].view(np.uint32), ref.np("fs")[:rows][live].view(np.uint32))
        assert np.array_equal(dev.np("out"), ref.np("out"))


@pytest.mark.parametrize("T,p16", [(1, False), (19, True), (100, False), (333, True), (700, False)])
def test_two_term_arms(moe, oracle, T, p16):
    """Ops 85 / 86 arms 4 / 5: the intermediate as two e4m3 terms per value, rows [hi I | lo I] with 1x128 scales
    (plow runtime/amd/moe_pf_w8a8.h:81-92, :115-117). The library multiplies the bf16 rows themselves where the
    reference multiplies their two terms (which stand for them to 2^-8), so the stored rows are compared as
    values, s * (hi + lo / 16), at the precision the two terms carry; few rows per expert (streaming kernels,
    matrix-vector form at one token) and many (tiled kernels)."""
    print(f"[case] w8a8 two-term T={T} p16={p16}", flush=True)
    cfg = layer.MoeConfig("mini-split", H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          n_group=4, topk_group=2, route_scale=2.5, enc="fp8blk", arm="w8a8split", part_bf16=p16,
                          n_shared=1, shared_mode="fold")
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    rows = assert_routing_equal(plan, dev, host)
    I = cfg.I
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    e4 = lambda b: torch.from_numpy(np.ascontiguousarray(b)).view(torch.float8_e4m3fn).float().numpy()
    def rows_of(t):
        fq, fs = t.np("fq")[:rows][live], t.np("fs")[:rows][live]
        return np.repeat(fs, 128, axis=1) * (e4(fq[:, :I]) + e4(fq[:, I:]) / 16.0), fs
    vd, fsd = rows_of(dev)
    vh, fsh = rows_of(host)
    assert np.allclose(fsd, fsh, rtol=1e-2)
    amax = np.repeat(np.abs(vh).reshape(vh.shape[0], -1, 128).max(2), 128, axis=1)
    err = (np.abs(vd - vh) / np.maximum(amax, 1e-20)).max()
    print(f"[parity] two-term rows: max |dev - ref| / group amax = {err:.3e}", flush=True)
    assert err < 2.0 ** -5
    relL2 = np.sqrt(((vd - vh) ** 2).sum() / (vh ** 2).sum())
    print(f"[parity] two-term rows: relL2 = {relL2:.3e}", flush=True)
    assert relL2 < 5e-3
    if p16:
        assert_output_close(dev.np("part").reshape(-1), host.np("part").reshape(-1), "part (bf16)")
    else:
        pd, ph = dev.np("part"), host.np("part")
        assert np.all(np.isfinite(pd))
        assert np.abs(pd - ph).max() / np.abs(ph).max() < 2e-2
    assert_output_close(dev.np("out"), host.np("out"))


def test_two_term_arm_refusals(moe):
    """The arms keep their aligned intermediate rows in the context's staging: a batch it does not hold, or a row
    count the op cannot know, is refused before anything is launched."""
    t = torch.zeros(64, device="cuda")
    from gpu_harness import dev_table
    tab = dev_table([t] * 8)
    big = abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, None, 7], i=[2048, 7168, 257, 1, 4096, 1, 0, abi.ARM_W8A8_SPLIT], slots=4096 * 9)
    assert moe.check(big, tab) == abi.E_INVAL and "staging" in moe.last_error()
    unknown = abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[512, 256, 33, 1, 0, 0, 0, abi.ARM_W8A8_SPLIT_P16])
    assert moe.check(unknown, tab) == abi.E_INVAL and "row count" in moe.last_error()
    ok = abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[512, 256, 33, 1, 0, 0, 0, abi.ARM_W8A8_SPLIT], slots=400)
    assert moe.check(ok, tab) == 0


@pytest.mark.parametrize("T,limit", [(1, 0.0), (19, 0.0), (100, 0.02), (333, 0.0), (700, 0.02)])  # from 16 rows per expert: tiled form
def test_atomic_chain_ops_188_189_190(moe, oracle, T, limit):
    """The block-fp8 chain with a bf16 intermediate (op 188), a slot-major quantized copy of it (op 189)
    and a bf16 atomic reduction straight into the layer output (op 190), no combine op
    (plow runtime/amd/op_moe_fp8_block128.h:7-88). The additions of op 190 come in no fixed order, each
    rounded to bf16: the output is held to a few bf16 roundings of the oracle's, everything before it to
    the usual bars."""
    print(f"[case] w8a8 atomic chain T={T} limit={limit}", flush=True)
    cfg = layer.MoeConfig("mini-atomic", H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          n_group=4, topk_group=2, route_scale=2.5, enc="fp8blk", arm="w8a8atomic", n_shared=1,
                          shared_mode="fold", act=4 if limit > 0 else 1, act_f=(0.0, limit))
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    assert "combine" not in plan.names
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("xq"), host.np("xq"))
    fd, fh = ol.bf2f(dev.np("fu")[:rows]), ol.bf2f(host.np("fu")[:rows])
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    assert not dev.np("fu")[:rows][~live].any()                  # pad rows of every tile are zeroed
    same = (dev.np("fu")[:rows] == host.np("fu")[:rows]).mean()
    print(f"[parity] fu bf16 identical on {same * 100:.3f} % of elements", flush=True)
    assert same > 0.98 and np.abs(fd - fh).max() <= 2.0 ** -7 * np.abs(fh).max()
    # the slot-major copy: dequantized values agree to fp8 precision
    deq = lambda h: (torch.from_numpy(h.np("hq")).view(torch.float8_e4m3fn).float().numpy() *
                     np.repeat(h.np("hs").T, 128, axis=1))
    hd, hh = deq(dev), deq(host)
    assert np.abs(hd - hh).max() <= 2.0 ** -3 * np.abs(hh).max()
    got, want = ol.bf2f(dev.np("out")), ol.bf2f(host.np("out"))
    assert np.all(np.isfinite(got))
    assert np.abs(got - want).max() <= 3e-2 * np.abs(want).max()
    assert np.abs(got - want).mean() <= 1e-2 * np.abs(want).mean()


@pytest.mark.parametrize("T,act,f", [(24, 2, (2.0, 1.5)), (24, 4, (0.0, 0.75)), (600, 2, (3.0, 0.0)), (600, 4, (0.0, 0.75))])
def test_pair_form_activations(moe, oracle, T, act, f):
    """Activations that transform the up branch too on op 85's block-fp8 W8A8 arm: 2 situ (beta, linear
    beta) and 4 clamped SwiGLU (limit in fj[1], small enough here to clamp), streaming and tiled forms."""
    print(f"[case] w8a8 act={act} f={f} T={T}", flush=True)
    cfg = layer.MoeConfig("mini-act", H=512, E=8, I=256, k=2, T=T, scoring="sigmoid", norm_topk=True,
                          bias=True, enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold", act=act, act_f=f)
    check_layer(*both(moe, oracle, cfg, seed=T + act))


def test_rows_longer_than_the_lds_scale_table(moe, oracle):
    """H = 16512 (129 blocks of 128 k): the direct-to-LDS GLU keeps a tile's weight block scales of all of K in
    an LDS table of 128 entries, so this shape must take the register form, which reads them as it goes (the
    tiled form does not serve it either); streaming row counts and tiled ones."""
    for T in (3, 80):
        print(f"[case] w8a8 long rows T={T}", flush=True)
        cfg = layer.MoeConfig("long-k", H=16512, E=4, I=256, k=2, T=T, scoring="sigmoid", norm_topk=True,
                              bias=True, enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold")
        check_layer(*both(moe, oracle, cfg, seed=T))


@pytest.mark.parametrize("enc,T,E,k", [("fp8blk", 600, 8, 2), ("fp8blk", 24, 8, 2), ("fp8pc", 640, 8, 4), ("fp8pc", 20, 8, 4)])
def test_ops_issued_alone_pick_their_form_on_the_device(moe, enc, T, E, k):
    """A caller that issues the ops one at a time and states no row count (plow's interpreter,
    runtime/amd/interp.hip:6556-6604): ops 86 / 81 / 82 know their rows only from meta, on the device. Both
    forms are launched behind a choice made there; the bytes must be those of the run that states the count
    (same form, same kernel), at tiled and at streaming row counts."""
    from plow_amd import synth
    print(f"[case] form on device enc={enc} T={T}", flush=True)
    shared = dict(n_shared=1, shared_mode="fold") if enc == "fp8blk" else {}
    cfg = layer.MoeConfig("alone", H=512, E=E, I=256, k=k, T=T, scoring="softmax", norm_topk=True, enc=enc, arm="w8a8", **shared)
    plan = layer.plan_layer(cfg)
    assert T * cfg.k_all > 36                                     # beyond the matrix-vector form, which only a stated count selects
    want = synth.bind(plan, "cuda", seed=T)
    moe.exec_many(plan.insts, want.table())
    torch.cuda.synchronize()
    got = synth.bind(plan, "cuda", seed=T)
    for d in plan.insts:
        d.fj[2].u = 0
        moe.exec(d, got.table())
    torch.cuda.synchronize()
    for name in ("meta", "part", "out") + (("fq", "fs") if enc == "fp8blk" else ("fu", "fu8")):
        rows = int(want.np("meta")[3 * cfg.E_all]) * abi.MPF_BM
        a, b = want.np(name), got.np(name)
        if name in ("fq", "fs", "fu", "fu8"):
            a, b = a[:rows], b[:rows]
        assert a.tobytes() == b.tobytes(), name
    assert np.isfinite(ol.bf2f(got.np("out"))).all()


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


@pytest.mark.parametrize("T,E,k", [(300, 4, 2), (700, 8, 4), (1030, 3, 1)])
def test_tiled_kernel_many_rows_per_expert(moe, oracle, T, E, k):
    """Row counts of 60..1030 per expert run the tiled (prefill) form: partial, full and multiple
    256-row tiles; routing bit-exact, output within tolerance."""
    cfg = layer.MoeConfig("tiled", H=384, E=E, I=256, k=k, T=T, scoring="softmax", norm_topk=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold", residual=True)
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    check_layer(plan, dev, host)


@pytest.mark.parametrize("T", [40, 700])
def test_bf16_partials(moe, oracle, T):
    """Arm 3: the down op writes bf16 partials and the combine reads them (streaming and tiled form)."""
    cfg = layer.MoeConfig("p16", H=384, E=8, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold", residual=True, part_bf16=True)
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("part").reshape(-1), host.np("part").reshape(-1), "part (bf16)")
    assert_output_close(dev.np("out"), host.np("out"))


def test_tiled_skips_non_resident_expert(moe, oracle):
    """A null weight-table row (expert not resident on this rank): the grouped ops leave its rows alone."""
    from gpu_harness import run_device, run_oracle
    from plow_amd import synth
    cfg = layer.MoeConfig("tiled-null", H=384, E=4, I=256, k=2, T=300, scoring="softmax", norm_topk=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=11)
    dev.t["wtab"][1].zero_()                       # expert 1 is elsewhere
    dev.t["part"].fill_(0.25)                      # untouched rows must keep this
    dev.t["fq"].fill_(7)
    host = synth.to_host(dev)
    host.t["wtab"][1].zero_()                      # (the host table holds host pointers of its own)
    run_device(moe, plan, dev)
    run_oracle(oracle, plan, host)
    assert_routing_equal(plan, dev, host)
    pd, ph = dev.np("part"), host.np("part")
    untouched = (ph == 0.25).all(axis=1)
    assert untouched.any() and np.array_equal(pd[untouched], ph[untouched])
    assert_output_close(dev.np("out"), host.np("out"))


def test_segment_entry_points(moe, oracle):
    """plow_moe_pf / plow_moe_dec: same results as op-by-op execution, the min-rows knob, and typed
    refusal of a mis-wired segment."""
    from gpu_harness import run_device, run_oracle
    from plow_amd import synth
    cfg = layer.MoeConfig("seg", H=256, E=8, I=128, k=2, T=40, scoring="sigmoid", norm_topk=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=5)
    host = synth.to_host(dev)
    run_oracle(oracle, plan, host)
    for entry in (moe.pf, moe.dec):
        for name in ("fq", "part", "out"):
            dev.t[name].zero_()
        assert entry(plan.insts, dev.table(), cfg.T) == 0
        torch.cuda.synchronize()
        assert_routing_equal(plan, dev, host)
        assert_output_close(dev.np("out"), host.np("out"))
    moe.set_min_rows(1, 64)                      # decode variant: segments below 64 rows roll back
    assert moe.dec(plan.insts, dev.table(), cfg.T) == abi.ROLLBACK
    assert moe.dec(plan.insts, dev.table(), 64) == 0
    moe.set_min_rows(0, 0)                       # prefill variant switched off
    assert moe.pf(plan.insts, dev.table(), cfg.T) == abi.ROLLBACK
    moe.set_min_rows(0, -1)
    moe.set_min_rows(1, -1)
    torch.cuda.synchronize()
    bad = [abi.PlowDevInst.from_buffer_copy(d) for d in plan.insts]
    bad[plan.index("down")].i[1] = cfg.I * 2     # DOWN's K no longer equals the GLU's N
    with pytest.raises(Exception) as ei:
        moe.pf(bad, dev.table(), cfg.T)
    assert "disagree" in str(ei.value)


@pytest.mark.parametrize("T", [24, 700])   # weight-streaming form, tiled form
def test_deterministic_fused_combine(moe, oracle, T):
    """Op 83 zeroes a [T][H] f64 accumulator, op 86 (i5) adds every live row's gate * acc into its token's
    row as an integer-valued double, op 87 (i4) reads it as one stream (plow runtime/amd/op_moe.h:2110-2165).
    The accumulator must equal, exactly, the integer sum of the quantized partials the plain chain of the
    same kernels writes (closed form over the device's own `part`), two runs must agree bit for bit
    (the additions commute), and the output must meet the layer tolerance against the oracle's."""
    import dataclasses
    from gpu_harness import run_device, run_oracle
    from plow_amd import synth
    from test_oracle_pins import det_closed_form
    print(f"[case] deterministic fused combine T={T}", flush=True)
    cfg = layer.MoeConfig("det", H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          n_group=4, topk_group=2, route_scale=2.5, enc="fp8blk", arm="w8a8", n_shared=1,
                          shared_mode="fold", residual=True)
    plain = layer.plan_layer(cfg)
    dp = synth.bind(plain, "cuda", seed=T)
    run_device(moe, plain, dp)
    want = det_closed_form(dp.t["part"].cpu().numpy(), cfg.T, cfg.k_all, cfg.H)
    det = layer.plan_layer(dataclasses.replace(cfg, det_combine=True))
    runs = []
    for rep in range(2):
        dd = synth.bind(det, "cuda", seed=T)
        dd.t["acc64"].fill_(float(rep + 1))          # op 83 must zero it
        run_device(moe, det, dd)
        runs.append((dd.t["acc64"].cpu().numpy(), dd.np("out")))
    assert np.array_equal(runs[0][0].view(np.uint64), runs[1][0].view(np.uint64))
    assert np.array_equal(runs[0][1], runs[1][1])
    assert np.array_equal(runs[0][0], want.astype(np.float64)), "accumulator differs from the integer sum of the partials"
    host = synth.to_host(dd)
    run_oracle(oracle, det, host)
    assert_output_close(runs[0][1], host.np("out"), f"det combine T={T} out")


def test_tiled_glu_silu_against_the_streaming_form(moe, oracle):
    """The tiled form's GLU epilogue takes SiLU from the hardware exp2 / reciprocal, the streaming form from
    expf and an IEEE division (plow's choice, runtime/amd/op_moe.h:209-215). Both forms accumulate the same
    matrix products in the same order, so running op 188 (bf16 intermediate) once per form over the same
    rows isolates that difference: how many bf16 values differ, and by how many steps. The form is picked
    through the routed-slot count in the descriptor (many slots: tiled; one slot: streaming, which is correct
    at every row count)."""
    T = 700
    print(f"[case] tiled vs streaming SiLU T={T}", flush=True)
    cfg = layer.MoeConfig("mini-atomic", H=512, E=32, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          n_group=4, topk_group=2, route_scale=2.5, enc="fp8blk", arm="w8a8atomic", n_shared=1,
                          shared_mode="fold", act=1)
    plan, dev, host = both(moe, oracle, cfg, seed=5)
    rows = assert_routing_equal(plan, dev, host)
    glu = plan.insts[plan.index("glu")]
    assert glu.fj[2].u >= 16 * (cfg.E + 1)                       # the run above took the tiled form
    tiled = dev.np("fu")[:rows].copy()
    dev.t["fu"].zero_()
    one = abi.PlowDevInst.from_buffer_copy(glu)
    one.fj[2].u = 1
    moe.exec(one, dev.table())
    torch.cuda.synchronize()
    stream = dev.np("fu")[:rows].copy()
    live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    a, b = tiled[live].astype(np.int32), stream[live].astype(np.int32)
    # bf16 bit patterns of one sign are ordered like the values: the difference of the patterns counts steps
    same_sign = (a >> 15) == (b >> 15)
    steps = np.where(same_sign, np.abs(a - b), (a & 0x7FFF) + (b & 0x7FFF))
    frac = float((steps != 0).mean())
    print(f"[parity] tiled vs streaming bf16 intermediate: {frac * 100:.4f} % of {steps.size} values differ, "
          f"max {int(steps.max())} step(s)", flush=True)
    assert frac <= 1e-3 and steps.max() <= 1
