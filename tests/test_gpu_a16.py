"""bf16-activation expert arms on the GPU against the oracle and the golden vectors of plow's CPU
kernels: bf16 weights (enc 0), block-fp8 W8A16 (enc 1 arm 0), mxfp4 W4A16 (enc 2 arm 8),
per-channel fp8 (ops 65 / 66 and the W8A8 pair 81 / 82), the slot-major decode ops 48 / 49 and the
dense shared expert (ops 20 / 8)."""
import os

import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from gpu_harness import (assert_output_close, assert_routing_equal, both, dev_table, from_dev, run_device, run_oracle,
                         to_dev)
from plow_amd import abi, layer, synth

pytestmark = pytest.mark.gpu

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "plow_cpu_golden.npz"))


@pytest.fixture(scope="module")
def moe():
    from plow_amd.lib import Moe
    m = Moe(0)
    yield m
    m.close()


def close(a, b, what, max_frac=2e-2, mean_rel=5e-3):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert np.all(np.isfinite(a)), what
    err = np.abs(a - b)
    mx = err.max() / max(np.abs(b).max(), 1e-30)
    mr = err.mean() / max(np.abs(b).mean(), 1e-30)
    print(f"[parity] {what}: max_abs/max|ref| = {mx:.3e}, mean rel = {mr:.3e}", flush=True)
    assert mx <= max_frac and mr <= mean_rel, (what, mx, mr)


def check_chain(plan, dev, host):
    rows = assert_routing_equal(plan, dev, host)
    assert np.array_equal(dev.np("logit").view(np.uint32), host.np("logit").view(np.uint32))
    if "fu" in dev.t:
        spec_rows = plan.specs["fu"].shape[0]
        if spec_rows == plan.cfg.R_max:   # gathered layout: compare live rows only
            live = host.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
            close(ol.bf2f(dev.np("fu")[:rows][live]), ol.bf2f(host.np("fu")[:rows][live]), "fu")
        else:
            close(ol.bf2f(dev.np("fu")), ol.bf2f(host.np("fu")), "fu")
    close(dev.np("part"), host.np("part"), "part")
    return assert_output_close(dev.np("out"), host.np("out"))


MINI = dict(H=512, E=16, I=256, k=4)


@pytest.mark.parametrize("T", [1, 5, 40])
def test_bf16_layer_with_dense_shared_experts(moe, oracle, T):
    cfg = layer.MoeConfig("bf16-mini", T=T, scoring="softmax", norm_topk=False, enc="bf16", arm="a16",
                          n_shared=2, shared_mode="dense", **MINI)
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    check_chain(plan, dev, host)
    close(ol.bf2f(dev.np("shared")), ol.bf2f(host.np("shared")), "shared")


@pytest.mark.parametrize("T", [3, 33])
def test_block_fp8_w8a16_layer(moe, oracle, T):
    cfg = layer.MoeConfig("w8a16-mini", T=T, scoring="sigmoid", norm_topk=True, bias=True, n_group=4,
                          topk_group=2, route_scale=2.5, enc="fp8blk", arm="a16", n_shared=1,
                          shared_mode="fold", residual=True, **MINI)
    check_chain(*both(moe, oracle, cfg, seed=T))


@pytest.mark.parametrize("T", [1, 16, 70])
def test_mxfp4_w4a16_layer(moe, oracle, T):
    cfg = layer.MoeConfig("mxfp4-mini", T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          route_scale=2.827, enc="mxfp4", arm="a16", n_shared=1, shared_mode="fold", **MINI)
    check_chain(*both(moe, oracle, cfg, seed=T))


@pytest.mark.parametrize("enc,act,f", [("mxfp4", 2, (2.0, 1.5)), ("fp8blk", 4, (0.0, 0.75)), ("bf16", 4, (0.0, 0.5))])
def test_pair_form_activations_bf16_arm(moe, oracle, enc, act, f):
    """Op 85 with bf16 activations under the activations that transform the up branch too (2 situ,
    4 clamped SwiGLU with a limit small enough to clamp)."""
    print(f"[case] a16 enc={enc} act={act} f={f}", flush=True)
    cfg = layer.MoeConfig("a16-act", T=20, scoring="sigmoid", norm_topk=True, bias=True, enc=enc, arm="a16",
                          n_shared=1, shared_mode="fold", act=act, act_f=f, **MINI)
    check_chain(*both(moe, oracle, cfg, seed=7 + act))


@pytest.mark.parametrize("arm", ["a16", "w8a8"])
@pytest.mark.parametrize("T", [2, 50])
def test_per_channel_fp8_layer(moe, oracle, T, arm):
    cfg = layer.MoeConfig("fp8pc-mini", T=T, scoring="softmax", norm_topk=True, enc="fp8pc", arm=arm, **MINI)
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    if arm == "w8a8":
        assert np.array_equal(dev.np("xq"), host.np("xq"))
        assert np.array_equal(dev.np("ascale").view(np.uint32), host.np("ascale").view(np.uint32))
    check_chain(plan, dev, host)


@pytest.mark.parametrize("enc,arm,T,E,k", [("bf16", "a16", 300, 4, 2), ("fp8blk", "a16", 1030, 3, 1), ("fp8blk", "a16", 333, 8, 4),
                                           ("fp8pc", "a16", 300, 4, 2), ("fp8pc", "a16", 1030, 3, 1), ("fp8pc", "a16", 777, 8, 4),
                                           ("mxfp4", "a16", 300, 4, 2)])
def test_bf16_activation_arms_many_rows(moe, oracle, enc, arm, T, E, k):
    """Experts with 40..1030 rows on the bf16-activation arms, all on the tiled kernels (from 16 rows per
    expert on average): fp8 weights (block and per-channel scales) and bf16 weights in 64-k blocks, mxfp4
    weights in 128-k blocks; partial, full and several 128-row tiles, pad rows, a folded shared expert of
    T rows."""
    print(f"[case] a16 many rows enc={enc} T={T} E={E} k={k}", flush=True)
    shared = dict(n_shared=1, shared_mode="fold") if enc != "fp8pc" else {}
    cfg = layer.MoeConfig("a16-rows", H=384, E=E, I=256, k=k, T=T, scoring="softmax", norm_topk=True, enc=enc, arm=arm, **shared)
    check_chain(*both(moe, oracle, cfg, seed=T))


@pytest.mark.parametrize("enc", ["bf16", "fp8blk", "mxfp4"])
@pytest.mark.parametrize("T", [1, 3, 12, 40])
def test_decode_expert_ops_48_49_in_a_layer(moe, oracle, enc, T):
    """The table-driven decode experts (ops 48 / 49, slot-major rows) as the layer's expert ops, every weight encoding:
    a handful of slots (the matrix-vector form lists its rows from the routing table itself, nothing is sorted),
    and more (the slots are sorted into the context's workspace first)."""
    print(f"[case] ops 48 / 49 layer enc={enc} T={T}", flush=True)
    cfg = layer.MoeConfig("a16-dec", H=512, E=16, I=256, k=4, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          enc=enc, arm="a16dec", n_shared=1, shared_mode="fold")
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    assert [i.op for i in plan.insts][3:5] == [abi.OP_MOE_GROUP_GLU_FP8_BLK, abi.OP_MOE_GROUP_DOWN_FP8_BLK]
    check_chain(plan, dev, host)


@pytest.mark.parametrize("enc,H,I,E,T", [("mxfp4", 2048, 512, 64, 64), ("mxfp4", 2048, 1536, 64, 64), ("mxfp4", 2048, 768, 64, 64),
                                         ("mxfp4", 4096, 512, 128, 96), ("fp8blk", 2048, 512, 64, 16), ("fp8pc", 2048, 512, 64, 16),
                                         ("bf16", 2048, 512, 64, 16)])
def test_streaming_form_wide_down_tiles_and_scale_chunks(moe, oracle, enc, H, I, E, T):
    """A few rows per expert on many experts: the weight-streaming form with the DOWN on tiles of 256 channels (two
    16-channel operands per wave), every encoding. mxfp4 brings its E8M0 bytes four 256-k steps at a time: rows of
    two steps (K = 512: every chunk is a tail), of six (one whole chunk and a tail), of three (K = 768, not whole
    16-byte pieces: the per-step loads), and two tiles per workgroup with the chunks running across the tile boundary
    (128 experts x 16 tiles)."""
    print(f"[case] a16 streaming wide enc={enc} H={H} I={I} E={E} T={T}", flush=True)
    shared = dict(n_shared=1, shared_mode="fold") if enc != "fp8pc" else {}
    cfg = layer.MoeConfig("a16-wide", H=H, E=E, I=I, k=4, T=T, scoring="softmax", norm_topk=True, enc=enc, arm="a16", **shared)
    check_chain(*both(moe, oracle, cfg, seed=H + I))


@pytest.mark.parametrize("T,E,k", [(300, 4, 2), (1030, 3, 1), (640, 8, 4)])
def test_per_channel_w8a8_tiled_many_rows(moe, oracle, T, E, k):
    """Ops 81 / 82 with 60..1030 rows per expert run the tiled (prefill) form: partial, full and
    multiple 128-row tiles, two and three 128-k blocks."""
    cfg = layer.MoeConfig("fp8pc-tiled", H=384, E=E, I=256, k=k, T=T, scoring="softmax", norm_topk=True,
                          enc="fp8pc", arm="w8a8")
    plan, dev, host = both(moe, oracle, cfg, seed=T)
    assert np.array_equal(dev.np("xq"), host.np("xq"))
    check_chain(plan, dev, host)


@pytest.mark.parametrize("enc,T,E,k", [("fp8blk", 333, 8, 4), ("fp8blk", 20, 8, 4), ("bf16", 300, 4, 2), ("bf16", 14, 4, 2)])
def test_bf16_activation_ops_issued_alone_pick_their_form_on_the_device(moe, enc, T, E, k):
    """Ops 85 / 86 on the bf16-activation arms issued one at a time with no row count stated: the tiled and the
    streaming form both go out behind a choice made on the device from meta; the bytes must be those of the run
    that states the count, at tiled and at streaming row counts."""
    print(f"[case] a16 form on device enc={enc} T={T}", flush=True)
    cfg = layer.MoeConfig("a16-alone", H=384, E=E, I=256, k=k, T=T, scoring="softmax", norm_topk=True, enc=enc, arm="a16",
                          n_shared=1, shared_mode="fold")
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
    rows = int(want.np("meta")[3 * cfg.E_all]) * abi.MPF_BM
    live = want.np("row_partidx")[:rows] != abi.EXPERT_UNUSED
    assert np.array_equal(want.np("fu")[:rows][live], got.np("fu")[:rows][live])
    for name in ("part", "out"):
        assert want.np(name).tobytes() == got.np(name).tobytes(), name


def test_mxfp4_decode_ops_match_plow_cpu_golden(moe):
    """Ops 48 / 49 at enc 2 against vectors written by plow's flat mxfp4 kernels (ops 150 / 151),
    including a sentinel slot (GLU writes nothing, DOWN writes zeros)."""
    Wgu, Sgu, Wd, Sd = (to_dev(G[f"mxdec/{n}"]) for n in ("Wgu", "Sgu", "Wd", "Sd"))
    x, tab = to_dev(G["mxdec/x"]), to_dev(G["mxdec/table"].view(np.int32))
    E, I2, K2 = G["mxdec/Wgu"].shape
    I, K, B, k = I2 // 2, K2 * 2, G["mxdec/x"].shape[0], 2
    es = Wgu.element_size()
    wtab = torch.tensor([[Wgu[e].data_ptr(), Wgu[e].data_ptr() + I * (K // 2), Wd[e].data_ptr()] for e in range(E)],
                        dtype=torch.int64).cuda()
    stab = torch.tensor([[Sgu[e].data_ptr(), Sgu[e].data_ptr() + I * (K // 32), Sd[e].data_ptr()] for e in range(E)],
                        dtype=torch.int64).cuda()
    # geometry of the fixture is below the kernels' 128-multiples: expect a typed refusal, not a launch
    fu = torch.full((B * k, I), 0x1234, dtype=torch.int16, device="cuda")
    inst = abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[0, 1, 2, 3, 4], i=[B * k, I, K, E, k, 1, 2])
    assert moe.check(inst, dev_table([fu, x, tab, wtab, stab])) == abi.E_INVAL


def run_decode_pair(moe, oracle, enc, seed, nslot_rows=(3, 2), pc=False):
    """Slot-major decode ops on random data incl. a sentinel slot and a non-resident expert."""
    r = cases.rng_of(seed)
    B, k = nslot_rows
    E, H, I = 6, 256, 128
    def weights(N, K):
        if enc == abi.ENC_BF16:
            return cases.randn_bf16(r, (N, K), 0.05), None
        if enc == abi.ENC_MXFP4:
            return (r.integers(0, 256, (N, K // 2), dtype=np.uint8), r.integers(120, 128, (N, K // 32), dtype=np.uint8))
        if pc:
            return cases.e4m3_bytes(r, (N, K)), (r.random(N) * 0.01 + 1e-3).astype(np.float32)
        return cases.e4m3_bytes(r, (N, K)), (r.random(((N + 127) // 128, K // 128)) * 0.02 + 1e-3).astype(np.float32)
    mats = []
    for _ in range(E):
        if pc:
            mats.append([weights(2 * I, H), weights(H, I)])
        else:
            mats.append([weights(I, H), weights(I, H), weights(H, I)])
    x = cases.randn_bf16(r, (B, H), 1.0)
    tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
    tab["eid"] = r.integers(0, E, B * k)
    tab["eid"][1] = abi.EXPERT_UNUSED
    tab["eid"][2] = 4                       # expert 4 is not resident
    tab["gate"] = (r.random(B * k) + 0.1).astype(np.float32)
    ncol = 2 if pc else 3
    def tables(get_ptr):
        wt = np.zeros((E, ncol), np.uint64)
        st = np.zeros((E, ncol), np.uint64)
        for e in range(E):
            for j in range(ncol):
                wt[e, j] = get_ptr(mats[e][j][0])
                st[e, j] = 0 if mats[e][j][1] is None else get_ptr(mats[e][j][1])
        wt[4] = 0
        return wt, st
    if pc:
        glu = abi.inst(abi.OP_MOE_EXPERT_GLU_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[k, I, H, E, 0, B, 1])
        down = abi.inst(abi.OP_MOE_EXPERT_DOWN_GEMMA_FP8, t=[0, 1, 2, 3, 4], i=[k, H, I, E, 0, B])
    else:
        st_h = 4 if enc != abi.ENC_BF16 else None
        glu = abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[0, 1, 2, 3, st_h], i=[B * k, I, H, E, k, 1, enc])
        down = abi.inst(abi.OP_MOE_GROUP_DOWN_FP8_BLK, t=[0, 1, 2, 3, st_h], i=[B * k, H, I, E, 0, 0, enc])
    # oracle
    wt, st = tables(lambda a: a.ctypes.data)
    fu_h = np.full((B * k, I), 0x1234, np.uint16)
    part_h = np.full((B * k, H), 9.0, np.float32)
    ol.run(oracle.plow_oracle_exec, glu, ol.table_of([fu_h, x, tab, wt, st]), 2)
    ol.run(oracle.plow_oracle_exec, down, ol.table_of([part_h, fu_h, tab, wt, st]), 2)
    # device
    keep = []
    def dptr(a):
        t = to_dev(a)
        keep.append(t)
        return t.data_ptr()
    wtd, std = tables(dptr)
    fu_d = torch.full((B * k, I), 0x1234, dtype=torch.int16, device="cuda")
    part_d = torch.full((B * k, H), 9.0, dtype=torch.float32, device="cuda")
    tbl = [None, to_dev(x), to_dev(tab), to_dev(wtd), to_dev(std)]
    print(f"[case] decode pair enc={enc} pc={pc}", flush=True)
    moe.exec(glu, dev_table([fu_d] + tbl[1:]))
    # DOWN reads the oracle's fu so that only the DOWN arithmetic is compared
    moe.exec(down, dev_table([part_d, to_dev(fu_h)] + tbl[2:]))
    torch.cuda.synchronize()
    fu_g = fu_d.cpu().numpy().view(np.uint16)
    served = np.array([e < E and e != 4 for e in tab["eid"]])
    assert np.all(fu_g[~served] == 0x1234)                   # skipped slots: GLU writes nothing
    close(ol.bf2f(fu_g[served]), ol.bf2f(fu_h[served]), "fu")
    part_g = part_d.cpu().numpy()
    assert np.all(part_g[~served] == 0.0)                    # skipped slots: DOWN writes zeros
    close(part_g, part_h, "part", mean_rel=1e-4, max_frac=1e-4)


@pytest.mark.parametrize("enc", [abi.ENC_BF16, abi.ENC_FP8BLK, abi.ENC_MXFP4])
def test_slot_major_decode_ops(moe, oracle, enc):
    run_decode_pair(moe, oracle, enc, seed=20 + enc)
    run_decode_pair(moe, oracle, enc, seed=30 + enc, nslot_rows=(1, 8))


def test_per_channel_decode_ops(moe, oracle):
    run_decode_pair(moe, oracle, abi.ENC_FP8BLK, seed=41, pc=True)


def test_dense_ops_match_plow_cpu_golden_shape_rules(moe):
    """The dense fixture (N 48) is below the kernels' 128-multiple rule: typed refusal."""
    x, wg = to_dev(G["dense/x"]), to_dev(G["dense/wg"])
    M, K = G["dense/x"].shape
    N = G["dense/wg"].shape[0]
    fu = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    inst = abi.inst(abi.OP_GEMM_GLU, t=[0, 1, 2, None, None, 5], i=[M, N, K, 0, 0, 1])
    assert moe.check(inst, dev_table([fu, x, wg, None, None, wg])) == abi.E_INVAL


def test_dense_ops_against_oracle(moe, oracle):
    r = cases.rng_of(50)
    M, N, K = 37, 256, 384
    x = cases.randn_bf16(r, (M + 2, K), 1.0)
    wg, wu, wd = cases.randn_bf16(r, (N, K), 0.05), cases.randn_bf16(r, (N, K), 0.05), cases.randn_bf16(r, (K, N), 0.05)
    glu = abi.inst(abi.OP_GEMM_GLU, t=[0, 1, 2, None, None, 5], i=[M + 2, N, K, 0, 0, 1])
    gemm = abi.inst(abi.OP_GEMM, t=[0, 1, 2], i=[M, K, N, 0, 2, 1])   # a_row0 = 2, c_row0 = 1
    fu_h, y_h = np.zeros((M + 2, N), np.uint16), np.zeros((M + 1, K), np.uint16)
    ol.run(oracle.plow_oracle_exec, glu, ol.table_of([fu_h, x, wg, None, None, wu]), 4)
    ol.run(oracle.plow_oracle_exec, gemm, ol.table_of([y_h, fu_h, wd]), 4)
    fu_d = torch.zeros((M + 2, N), dtype=torch.int16, device="cuda")
    y_d = torch.zeros((M + 1, K), dtype=torch.int16, device="cuda")
    moe.exec(glu, dev_table([fu_d, to_dev(x), to_dev(wg), None, None, to_dev(wu)]))
    moe.exec(gemm, dev_table([y_d, to_dev(fu_h), to_dev(wd)]))
    torch.cuda.synchronize()
    close(ol.bf2f(fu_d.cpu().numpy().view(np.uint16)), ol.bf2f(fu_h), "dense fu")
    yg = y_d.cpu().numpy().view(np.uint16)
    assert np.all(yg[0] == 0)
    close(ol.bf2f(yg[1:]), ol.bf2f(y_h[1:]), "dense y")


@pytest.mark.parametrize("M,N,K", [(16, 2816, 2048), (1, 1408, 2816), (64, 512, 5632), (7, 128, 1024), (100, 1408, 2048),
                                   (128, 512, 1024), (600, 1408, 2048), (1500, 256, 512)])
def test_dense_ops_split_k_or_run_tiled(moe, oracle, M, N, K):
    """Below 128 rows and with fewer channel tiles than CUs the dense ops run as K slices plus a second launch that
    adds the slices up (GLU: before the activation): shapes of the small bf16 layer's shared expert, a K whose step
    count has an odd factor, a single tile, two row passes. From 128 rows they run on the tiled kernel as a
    one-expert batch whose tables a set-up launch writes."""
    r = cases.rng_of(M + N + K)
    x = cases.randn_bf16(r, (M + 3, K), 1.0)
    wg, wu, wd = cases.randn_bf16(r, (N, K), 0.03), cases.randn_bf16(r, (N, K), 0.03), cases.randn_bf16(r, (K, N), 0.03)
    glu = abi.inst(abi.OP_GEMM_GLU, t=[0, 1, 2, None, None, 5], i=[M + 3, N, K, 0, 0, 1])
    gemm = abi.inst(abi.OP_GEMM, t=[0, 1, 2], i=[M, K, N, 0, 3, 1])   # a_row0 = 3, c_row0 = 1
    fu_h, y_h = np.zeros((M + 3, N), np.uint16), np.zeros((M + 1, K), np.uint16)
    ol.run(oracle.plow_oracle_exec, glu, ol.table_of([fu_h, x, wg, None, None, wu]), 4)
    ol.run(oracle.plow_oracle_exec, gemm, ol.table_of([y_h, fu_h, wd]), 4)
    fu_d = torch.zeros((M + 3, N), dtype=torch.int16, device="cuda")
    y_d = torch.zeros((M + 1, K), dtype=torch.int16, device="cuda")
    for _ in range(2):  # the scratch is reused: a second run over it gives the same rows
        moe.exec(glu, dev_table([fu_d, to_dev(x), to_dev(wg), None, None, to_dev(wu)]))
        moe.exec(gemm, dev_table([y_d, to_dev(fu_h), to_dev(wd)]))
    torch.cuda.synchronize()
    close(ol.bf2f(fu_d.cpu().numpy().view(np.uint16)), ol.bf2f(fu_h), "dense fu")
    yg = y_d.cpu().numpy().view(np.uint16)
    assert np.all(yg[0] == 0)
    close(ol.bf2f(yg[1:]), ol.bf2f(y_h[1:]), "dense y")


# the last three: activations that transform the up branch too (2 situ, 3 swiglu_oai), immediates in fj[0..1]
@pytest.mark.parametrize("layout,with_bias,act,fimm", [(1, False, 1, ()), (0, True, 0, ()), (0, False, 1, ()), (1, True, 1, ()),
                                                        (0, True, 3, (1.702, 7.0)), (1, True, 2, (2.0, 1.5)), (1, False, 2, (3.0, 0.0))])
def test_flat_mxfp4_ops(moe, oracle, layout, with_bias, act, fimm):
    """Reference ops 150 - 153 (flat [E][rows][K/2] tensors, blocked or interleaved gate / up rows, optional
    per-expert bias): slot-major decode incl. a sentinel slot, then the gathered-row twins after op 84."""
    print(f"[case] flat mxfp4 layout={layout} bias={with_bias} act={act}", flush=True)
    r = cases.rng_of(70 + 2 * layout + int(with_bias))
    E, I, K, k, B = 5, 128, 512, 2, 9
    Wgu = r.integers(0, 256, (E, 2 * I, K // 2), dtype=np.uint8)
    Sgu = r.integers(120, 128, (E, 2 * I, K // 32), dtype=np.uint8)
    Wd = r.integers(0, 256, (E, K, I // 2), dtype=np.uint8)
    Sd = r.integers(120, 128, (E, K, I // 32), dtype=np.uint8)
    bgu = cases.randn_bf16(r, (E, 2 * I), 2.0) if with_bias else None
    bd = cases.randn_bf16(r, (E, K), 2.0) if with_bias else None
    x = cases.randn_bf16(r, (B, K), 1.0)
    tab = np.zeros(B * k, dtype=ol.ROUTE_DT)
    tab["eid"] = r.integers(0, E, B * k)
    tab["eid"][3] = abi.EXPERT_UNUSED
    tab["gate"] = (r.random(B * k) + 0.1).astype(np.float32)
    tb = 5 if with_bias else None
    glu = abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4, tb], i=[k, I, K, E, layout, act, B], f=fimm)
    down = abi.inst(abi.OP_MOE_DOWN_MX, t=[0, 1, 2, 3, 4, tb], i=[k, K, I, E, 0, 0, B])
    fu_h = np.full((B * k, I), 0x1234, np.uint16)
    part_h = np.full((B * k, K), 9.0, np.float32)
    ol.run(oracle.plow_oracle_exec, glu, ol.table_of([fu_h, x, tab, Wgu, Sgu, bgu]), 4)
    ol.run(oracle.plow_oracle_exec, down, ol.table_of([part_h, fu_h, tab, Wd, Sd, bd]), 4)
    d = {n: to_dev(a) for n, a in dict(x=x, tab=tab, Wgu=Wgu, Sgu=Sgu, Wd=Wd, Sd=Sd, bgu=bgu, bd=bd, fu_h=fu_h).items()}
    fu_d = torch.full((B * k, I), 0x1234, dtype=torch.int16, device="cuda")
    part_d = torch.full((B * k, K), 9.0, dtype=torch.float32, device="cuda")
    moe.exec(glu, dev_table([fu_d, d["x"], d["tab"], d["Wgu"], d["Sgu"], d["bgu"]]))
    moe.exec(down, dev_table([part_d, d["fu_h"], d["tab"], d["Wd"], d["Sd"], d["bd"]]))
    torch.cuda.synchronize()
    fu_g = fu_d.cpu().numpy().view(np.uint16)
    served = tab["eid"] < E
    assert np.all(fu_g[~served] == 0x1234)
    close(ol.bf2f(fu_g[served]), ol.bf2f(fu_h[served]), "fu")
    part_g = part_d.cpu().numpy()
    assert np.all(part_g[~served] == 0.0)
    close(part_g, part_h, "part", mean_rel=1e-4, max_frac=1e-4)
    # gathered rows: 84, then 152 / 153 on the same table
    al = cases.align_arrays(tab, B, E, k)
    ol.run(oracle.plow_oracle_exec, cases.align_inst(B, E, k), ol.table_of(al), 1)
    rows = len(al[2])
    glu_pf = abi.inst(abi.OP_MOE_GLU_MX_PF, t=[0, 1, 2, 3, 4, 5, 6 if with_bias else None], i=[I, K, E, layout, 0, act], f=fimm)
    down_pf = abi.inst(abi.OP_MOE_DOWN_MX_PF, t=[0, 1, 2, 3, 4, 5 if with_bias else None, 6, 7], i=[K, I, E])
    fug_h = np.full((rows, I), 0x1234, np.uint16)
    partg_h = np.full((B * k, K), 9.0, np.float32)
    ol.run(oracle.plow_oracle_exec, glu_pf, ol.table_of([fug_h, x, Wgu, Sgu, al[0], al[2], bgu]), 4)
    ol.run(oracle.plow_oracle_exec, down_pf, ol.table_of([partg_h, fug_h, Wd, Sd, al[0], bd, al[3], al[4]]), 4)
    meta_d, rt_d, rp_d, rg_d, fug_hd = to_dev(al[0]), to_dev(al[2]), to_dev(al[3]), to_dev(al[4]), to_dev(fug_h)
    fug_d = torch.full((rows, I), 0x1234, dtype=torch.int16, device="cuda")
    partg_d = torch.full((B * k, K), 9.0, dtype=torch.float32, device="cuda")
    moe.exec(glu_pf, dev_table([fug_d, d["x"], d["Wgu"], d["Sgu"], meta_d, rt_d, d["bgu"]]))
    moe.exec(down_pf, dev_table([partg_d, fug_hd, d["Wd"], d["Sd"], meta_d, d["bd"], rp_d, rg_d]))
    torch.cuda.synchronize()
    live = al[2] != abi.EXPERT_UNUSED
    fug_g = fug_d.cpu().numpy().view(np.uint16)
    assert np.all(fug_g[~live] == 0x1234)                    # pad rows: nothing written
    close(ol.bf2f(fug_g[live]), ol.bf2f(fug_h[live]), "fu_g")
    partg_g = partg_d.cpu().numpy()
    assert np.all(partg_g[~served] == 9.0)                   # no row maps to a sentinel slot: untouched
    close(partg_g[served], partg_h[served], "part_g", mean_rel=1e-4, max_frac=1e-4)


def test_flat_mxfp4_refusals(moe):
    t = dev_table([torch.zeros(8, device="cuda")] * 8)
    ok = abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 128, 256, 4, 1, 1, 3])
    assert moe.check(ok, t) == 0
    assert moe.check(abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 128, 256, 4, 1, 3, 3], f=(1.702, 7.0)), t) == 0
    assert moe.check(abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 128, 256, 4, 1, 4, 3]), t) == abi.E_UNSUPPORTED
    assert moe.check(abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 128, 256, 4, 1, 5, 3]), t) == abi.E_UNSUPPORTED
    assert moe.check(abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 128, 256, 4, 2, 1, 3]), t) == abi.E_INVAL
    assert moe.check(abi.inst(abi.OP_MOE_GLU_MX, t=[0, 1, 2, 3, 4], i=[2, 64, 256, 4, 1, 1, 3]), t) == abi.E_INVAL
    assert moe.check(abi.inst(abi.OP_MOE_DOWN_MX_PF, t=[0, 1, 2, 3, 4], i=[256, 128, 4]), t) == abi.E_INVAL


@pytest.mark.parametrize("act,T,stated", [(0, 40, False), (1, 40, False), (1, 400, True), (0, 150, True)])
def test_bf16_grouped_fused_table_ops(moe, oracle, act, T, stated):
    """Reference ops 75 / 76 (bf16, fused table ewt[E][2]) on gathered rows with a non-resident expert and
    an expert of more than 16 rows; with the routed rows stated and 60 to 400 rows per expert they run the
    tiled kernel's bf16-weight form (partial, full and several 128-row tiles), which like the streaming form
    writes live rows only."""
    print(f"[case] ops 75/76 act={act} T={T} stated={stated}", flush=True)
    r = cases.rng_of(90 + act + T)
    E, I, H, k = 5, 256, 384, 2
    gu = [cases.randn_bf16(r, (2 * I, H), 0.05) for _ in range(E)]
    dn = [cases.randn_bf16(r, (H, I), 0.05) for _ in range(E)]
    x = cases.randn_bf16(r, (T, H), 1.0)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    tab["eid"] = np.where(r.random(T * k) < 0.5, 1, r.integers(0, E, T * k))     # expert 1 gets many rows
    tab["eid"][5] = abi.EXPERT_UNUSED
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    ol.run(oracle.plow_oracle_exec, cases.align_inst(T, E, k), ol.table_of(al), 1)
    rows = len(al[2])
    ewt_h = np.array([[g.ctypes.data, d.ctypes.data] for g, d in zip(gu, dn)], dtype=np.uint64)
    ewt_h[3] = 0
    glu = abi.inst(abi.OP_MOE_GROUP_GLU_GEMMA_PF, t=[0, 1, 2, 3, 4], i=[I, H, E, 0, 0, act], slots=T * k if stated else 0)
    down = abi.inst(abi.OP_MOE_GROUP_DOWN_GEMMA_PF, t=[0, 1, 2, 3, 4, 5], i=[H, I, E], slots=T * k if stated else 0)
    fu_h = np.full((rows, I), 0x1234, np.uint16)
    part_h = np.full((T * k, H), 9.0, np.float32)
    ol.run(oracle.plow_oracle_exec, glu, ol.table_of([fu_h, x, ewt_h, al[0], al[2]]), 4)
    ol.run(oracle.plow_oracle_exec, down, ol.table_of([part_h, fu_h, ewt_h, al[0], al[3], al[4]]), 4)
    gd, dd = [to_dev(a) for a in gu], [to_dev(a) for a in dn]
    ewt_d = np.array([[a.data_ptr(), b.data_ptr()] for a, b in zip(gd, dd)], dtype=np.uint64)
    ewt_d[3] = 0
    xd, ewtd, metad, rtd, rpd, rgd, fuhd = (to_dev(a) for a in (x, ewt_d, al[0], al[2], al[3], al[4], fu_h))
    fu_d = torch.full((rows, I), 0x1234, dtype=torch.int16, device="cuda")
    part_d = torch.full((T * k, H), 9.0, dtype=torch.float32, device="cuda")
    moe.exec(glu, dev_table([fu_d, xd, ewtd, metad, rtd]))
    moe.exec(down, dev_table([part_d, fuhd, ewtd, metad, rpd, rgd]))
    torch.cuda.synchronize()
    written = fu_h != 0x1234
    fu_g = fu_d.cpu().numpy().view(np.uint16)
    assert np.array_equal(fu_g != 0x1234, written)            # pad rows and expert 3: nothing written
    close(ol.bf2f(fu_g[written]), ol.bf2f(fu_h[written]), "fu")
    part_g = part_d.cpu().numpy()
    touched = part_h != 9.0
    assert np.array_equal(part_g != 9.0, touched)
    close(part_g[touched], part_h[touched], "part", mean_rel=1e-4, max_frac=1e-4)


@pytest.mark.parametrize("enc,H,I", [("bf16", 384, 256), ("bf16", 2048, 1408), ("fp8blk", 640, 384), ("fp8blk", 7168, 256),
                                     ("mxfp4", 768, 256), ("mxfp4", 3584, 512), ("fp8pc", 1536, 640)])
@pytest.mark.parametrize("T,k", [(1, 8), (2, 3), (1, 1)])
def test_matrix_vector_form_at_one_and_two_tokens(moe, oracle, enc, H, I, T, k):
    """Batches that route a handful of rows in all run the bf16-activation ops as matrix-vector products
    (every wave a share of one row's channels, weight rows of 16-byte pieces per lane): row lengths that
    are not whole kilobytes, rows of one to eight pieces, every encoding, gate folded into the DOWN."""
    print(f"[case] gemv enc={enc} H={H} I={I} T={T} k={k}", flush=True)
    cfg = layer.MoeConfig("gemv", T=T, H=H, E=16, I=I, k=k, scoring="sigmoid", norm_topk=True, bias=True,
                          route_scale=2.5, enc=enc, arm="a16", n_shared=1, shared_mode="fold")
    assert T * cfg.k_all <= 9
    check_chain(*both(moe, oracle, cfg, seed=H + T))


@pytest.mark.parametrize("enc,H,I,T,k", [("mxfp4", 768, 256, 14, 8), ("mxfp4", 3584, 512, 13, 8), ("fp8blk", 640, 384, 4, 8),
                                         ("fp8pc", 1536, 640, 2, 8)])
def test_matrix_vector_form_at_a_few_tokens(moe, oracle, enc, H, I, T, k):
    """The largest batches the matrix-vector form is chosen for, per encoding (mxfp4 up to 128 routed rows,
    block fp8 36, per-channel fp8 18): 16 experts, so every expert holds several rows and streams its weights
    once per row."""
    print(f"[case] gemv few tokens enc={enc} H={H} I={I} T={T} k={k}", flush=True)
    cfg = layer.MoeConfig("gemv-few", T=T, H=H, E=16, I=I, k=k, scoring="sigmoid", norm_topk=True, bias=True,
                          route_scale=2.5, enc=enc, arm="a16", n_shared=1, shared_mode="fold")
    check_chain(*both(moe, oracle, cfg, seed=H + T))


@pytest.mark.parametrize("enc,H,I,T", [("mxfp4", 512, 256, 40), ("mxfp4", 512, 256, 72), ("fp8pc", 256, 4096, 40)])
def test_matrix_vector_form_is_right_when_the_slot_count_is_understated(moe, oracle, enc, H, I, T):
    """The form is chosen from the routed-slot count the descriptor states. A count that is far too small
    still gives the layer's result: live rows are walked in windows of 256 (72 tokens route 360 rows: two
    windows), an expert's rows one after the other. With 200 rows in the window a wave's share of the
    per-channel case's 4096 GLU channels is more than the 64 whose sums (and channel scales) a wave holds
    at a time."""
    print(f"[case] gemv understated enc={enc} H={H} I={I} T={T}", flush=True)
    cfg = layer.MoeConfig("gemv-lie", T=T, H=H, E=8, I=I, k=4, scoring="softmax", norm_topk=True, enc=enc,
                          arm="a16", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    for name in ("glu", "down"):
        plan.insts[plan.index(name)].fj[2].u = 5          # 200 or 360 slots in truth
    dev = synth.bind(plan, "cuda", seed=3)
    host = synth.to_host(dev)
    run_device(moe, plan, dev)
    run_oracle(oracle, plan, host)
    check_chain(plan, dev, host)
