"""Expert pointer tables (plow_amd/tables.py): the three builders against the known answers of plow's own
unit tests (crates/plowrt/src/orch/moe.rs:127-250), the safetensors loader on a small block-fp8 layer
(CPU: table entries, expert-parallel ownership, refusals; GPU: a layer run over the loaded tables equals
the same layer over the tensors they were saved from, bit for bit)."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from plow_amd import tables


def test_routed_experts_resolve_in_gate_up_down_order():
    addrs = {"l1.shared.gate_up": 0x1000, "l1.shared.down": 0x2000, "l1.e0.gate": 0x3000, "l1.e0.up": 0x3100,
             "l1.e0.down": 0x3200, "l1.e1.gate": 0x4000, "l1.e1.up": 0x4100, "l1.e1.down": 0x4200}
    t = tables.build_expert_table([("l1.shared.gate_up", "l1.shared.down")],
                                  [[("l1.e0.gate", "l1.e0.up", "l1.e0.down"), ("l1.e1.gate", "l1.e1.up", "l1.e1.down")]],
                                  addrs.get)
    assert t == [0x1000, 0x2000, 0x3000, 0x3100, 0x3200, 0x4000, 0x4100, 0x4200]


def test_no_routed_names_is_shared_only_and_missing_names_are_skipped():
    t = tables.build_expert_table([("s.gu", "s.d")], [], {"s.gu": 7, "s.d": 8}.get)
    assert t == [7, 8]
    t = tables.build_expert_table([("s.gu", None)], [[("a", "b", "c")]], {"s.gu": 7, "a": 1, "c": 3}.get)
    assert t == [7, 1, 3]


def test_packed_table_dense_and_null_outside_the_local_block():
    assert tables.packed_expert_table(0x1000, 0x10, 3, range(0, 3)) == \
        [0x1000, 0x1010, 0x1020, 0x1030, 0x1040, 0x1050, 0x1060, 0x1070, 0x1080]
    t = tables.packed_expert_table(0x2000, 0x100, 4, range(2, 4))
    assert t[:6] == [0] * 6
    assert t[6:] == [0x2000, 0x2100, 0x2200, 0x2300, 0x2400, 0x2500]
    assert tables.packed_expert_table(0x2000, 0x100, 2, range(1, 5)) == [0, 0, 0, 0x2000, 0x2100, 0x2200]


def test_fused_table_is_base_plus_stride():
    assert tables.build_fused_expert_table(0x1000, 0x9000, 3, 0x100, 0x40) == \
        [0x1000, 0x9000, 0x1100, 0x9040, 0x1200, 0x9080]


def write_layer(path, prefix, E, I, H, shared, seed=0, drop=()):
    """A DeepSeek-V3 style block-fp8 layer in one safetensors file; returns {name: tensor}."""
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(seed)
    out = {}
    ids = [f"experts.{e}" for e in range(E)] + (["shared_experts"] if shared else [])
    for who in ids:
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            w = (torch.randn((n, k), generator=g) * 0.5).to(torch.float8_e4m3fn)
            s = torch.rand(((n + 127) // 128, (k + 127) // 128), generator=g) * 0.01 + 0.001
            out[f"{prefix}.{who}.{proj}.weight"] = w
            out[f"{prefix}.{who}.{proj}.weight_scale_inv"] = s.float()
    for name in drop:
        del out[name]
    out["model.norm.weight"] = torch.ones(H, dtype=torch.bfloat16)      # something the loader must ignore
    save_file(out, path)
    return out


def test_loader_fills_tables_over_what_it_loaded(tmp_path):
    prefix, E, I, H = "model.layers.3.mlp", 4, 256, 384
    path = str(tmp_path / "layer.safetensors")
    saved = write_layer(path, prefix, E, I, H, shared=True)
    L = tables.load_block_fp8_layer([path], prefix, E, "cpu", shared=True)
    assert (L.n_exp, L.n_all, L.inter, L.hidden) == (E, E + 1, I, H)
    assert tuple(L.wtab.shape) == (E + 1, 3) and L.wtab.dtype == torch.int64
    for e in range(E + 1):
        who = f"experts.{e}" if e < E else "shared_experts"
        for j, proj in enumerate(tables.PROJ):
            w, s = L.weights[(e, j)], L.scales[(e, j)]
            assert int(L.wtab[e, j]) == w.data_ptr() and int(L.stab[e, j]) == s.data_ptr()
            assert torch.equal(w, saved[f"{prefix}.{who}.{proj}.weight"].view(torch.uint8))
            assert torch.equal(s, saved[f"{prefix}.{who}.{proj}.weight_scale_inv"])
    # expert parallel: a rank that owns experts 2..3 leaves the others null, and holds nothing of them
    R = tables.load_block_fp8_layer([path], prefix, E, "cpu", owned=range(2, 4))
    assert not R.wtab[:2].any() and not R.stab[:2].any() and R.wtab[2:].all() and R.stab[2:].all()
    assert sorted({e for e, _ in R.weights}) == [2, 3]


def test_loader_refusals_and_partial_experts(tmp_path):
    prefix, E, I, H = "m", 2, 128, 256
    path = str(tmp_path / "a.safetensors")
    write_layer(path, prefix, E, I, H, shared=False, drop=(f"{prefix}.experts.1.down_proj.weight",
                                                           f"{prefix}.experts.1.down_proj.weight_scale_inv"))
    L = tables.load_block_fp8_layer([path], prefix, E, "cpu")
    assert L.wtab[0].all() and not L.wtab[1].any()          # an expert is resident as a whole or not at all
    path2 = str(tmp_path / "b.safetensors")
    write_layer(path2, prefix, E, I, H, shared=False, drop=(f"{prefix}.experts.0.up_proj.weight_scale_inv",))
    with pytest.raises(ValueError):
        tables.load_block_fp8_layer([path2], prefix, E, "cpu")
    from safetensors.torch import save_file
    path3 = str(tmp_path / "c.safetensors")
    save_file({f"{prefix}.experts.0.gate_proj.weight": torch.zeros((I, H), dtype=torch.bfloat16)}, path3)
    with pytest.raises(ValueError):
        tables.load_block_fp8_layer([path3], prefix, 1, "cpu")


@pytest.mark.gpu
def test_layer_over_loaded_tables_equals_direct_binding(tmp_path):
    from safetensors.torch import save_file
    from gpu_harness import run_device
    from plow_amd import layer, synth
    from plow_amd.lib import Moe
    print("[case] checkpoint round trip through safetensors", flush=True)
    cfg = layer.MoeConfig("ckpt", H=512, E=8, I=256, k=2, T=40, scoring="sigmoid", norm_topk=True, bias=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=5)
    moe = Moe(0)
    run_device(moe, plan, dev)
    want = dev.t["out"].clone()
    prefix, out = "model.layers.7.mlp", {}
    for e, (ws, ss) in enumerate(dev.experts):
        who = f"experts.{e}" if e < cfg.E else "shared_experts"
        for j, proj in enumerate(tables.PROJ):
            out[f"{prefix}.{who}.{proj}.weight"] = ws[j].cpu().view(torch.float8_e4m3fn)
            out[f"{prefix}.{who}.{proj}.weight_scale_inv"] = ss[j].cpu()
    path = str(tmp_path / "layer.safetensors")
    save_file(out, path)
    L = tables.load_block_fp8_layer([path], prefix, cfg.E, "cuda", shared=True)
    assert (L.n_all, L.inter, L.hidden) == (cfg.E_all, cfg.I, cfg.H)
    assert not torch.equal(L.wtab, dev.t["wtab"])            # other allocations, same bytes
    dev.t["wtab"], dev.t["stab"] = L.wtab, L.stab
    dev._table = None
    dev.t["out"].zero_()
    run_device(moe, plan, dev)
    assert torch.equal(dev.t["out"].view(torch.int16), want.view(torch.int16))
    # the expert-parallel half: experts 0..3 only; the others contribute deterministic zeros
    Lh = tables.load_block_fp8_layer([path], prefix, cfg.E, "cuda", owned=range(0, 4), shared=True)
    dev.t["wtab"], dev.t["stab"] = Lh.wtab, Lh.stab
    dev._table = None
    run_device(moe, plan, dev)
    assert torch.isfinite(dev.t["out"].float()).all()
    moe.close()


# ---- mxfp4 checkpoint layouts -----------------------------------------------------------------------

def mxfp4_layer_tensors(E, I, H, seed=0):
    """Per expert (gate, up, down) quantized with plow's mxfp4 rule: packed rows + E8M0 bytes."""
    from plow_amd import synth
    out = []
    for e in range(E):
        ws = [synth.randn_bf16(shape, 0.02, torch.device("cpu"), seed * 100 + 3 * e + j)
              for j, shape in enumerate(((I, H), (I, H), (H, I)))]
        out.append([synth.quant_mxfp4(w) for w in ws])
    return out


def write_gptoss_layer(path, prefix, experts, with_bias, seed=0):
    """The GPT-OSS layout (plow runtime/common/dev_isa.h:1285-1303): one tensor per projection over all
    experts, gate / up rows interleaved, blocks as [E][rows][K/32][16]."""
    from safetensors.torch import save_file
    E = len(experts)
    (gq, gs), (uq, us), (dq, ds) = experts[0]
    I, H = gq.shape[0], dq.shape[0]
    gu_b = torch.zeros((E, 2 * I, H // 2), dtype=torch.uint8)
    gu_s = torch.zeros((E, 2 * I, H // 32), dtype=torch.uint8)
    d_b = torch.zeros((E, H, I // 2), dtype=torch.uint8)
    d_s = torch.zeros((E, H, I // 32), dtype=torch.uint8)
    for e, ((gq, gs), (uq, us), (dq, ds)) in enumerate(experts):
        gu_b[e, 0::2], gu_b[e, 1::2] = gq, uq
        gu_s[e, 0::2], gu_s[e, 1::2] = gs, us
        d_b[e], d_s[e] = dq, ds
    out = {f"{prefix}.experts.gate_up_proj_blocks": gu_b.view(E, 2 * I, H // 32, 16).contiguous(),
           f"{prefix}.experts.gate_up_proj_scales": gu_s, f"{prefix}.experts.down_proj_blocks": d_b.view(E, H, I // 32, 16).contiguous(),
           f"{prefix}.experts.down_proj_scales": d_s}
    if with_bias:
        g = torch.Generator().manual_seed(seed)
        out[f"{prefix}.experts.gate_up_proj_bias"] = (torch.randn((E, 2 * I), generator=g) * 0.1).bfloat16()
        out[f"{prefix}.experts.down_proj_bias"] = (torch.randn((E, H), generator=g) * 0.1).bfloat16()
    out["model.norm.weight"] = torch.ones(H, dtype=torch.bfloat16)
    save_file(out, path)
    return out


def test_gptoss_flat_loader_binds_the_checkpoint_tensors_verbatim(tmp_path):
    prefix, E, I, H = "model.layers.2.mlp", 3, 128, 256
    experts = mxfp4_layer_tensors(E, I, H)
    path = str(tmp_path / "oss.safetensors")
    saved = write_gptoss_layer(path, prefix, experts, with_bias=True)
    L = tables.load_mxfp4_flat_layer([path], prefix, "cpu")
    assert (L.n_exp, L.inter, L.hidden, L.layout) == (E, I, H, 0)
    assert L.gate_up_blocks.shape == (E, 2 * I, H // 2) and L.down_scales.shape == (E, H, I // 32)
    assert torch.equal(L.gate_up_blocks.reshape(-1), saved[f"{prefix}.experts.gate_up_proj_blocks"].reshape(-1))
    assert torch.equal(L.gate_up_blocks[1, 0::2], experts[1][0][0]) and torch.equal(L.gate_up_blocks[1, 1::2], experts[1][1][0])
    assert torch.equal(L.gate_up_bias, saved[f"{prefix}.experts.gate_up_proj_bias"])
    # refusals: a projection without its scales; scales of the wrong shape
    from safetensors.torch import save_file
    bad = {k: v for k, v in saved.items() if not k.endswith("down_proj_scales")}
    p2 = str(tmp_path / "bad.safetensors")
    save_file(bad, p2)
    with pytest.raises(ValueError):
        tables.load_mxfp4_flat_layer([p2], prefix, "cpu")
    bad = dict(saved)
    bad[f"{prefix}.experts.down_proj_scales"] = saved[f"{prefix}.experts.down_proj_scales"][:, :, :-1].contiguous()
    save_file(bad, p2)
    with pytest.raises(ValueError):
        tables.load_mxfp4_flat_layer([p2], prefix, "cpu")


def write_mxfp4_twin_layer(path, prefix, experts, shared_last):
    from safetensors.torch import save_file
    out = {}
    n = len(experts) - (1 if shared_last else 0)
    for e, triple in enumerate(experts):
        who = f"experts.{e}" if e < n else "shared_experts"
        for (q, s), proj in zip(triple, tables.PROJ):
            out[f"mxfp4/{prefix}.{who}.{proj}.weight"] = q
            out[f"mxfp4/{prefix}.{who}.{proj}.weight_scale"] = s
    save_file(out, path)
    return out


def test_mxfp4_twin_loader_fills_tables(tmp_path):
    prefix, E, I, H = "model.layers.5.mlp", 4, 128, 256
    experts = mxfp4_layer_tensors(E + 1, I, H)
    path = str(tmp_path / "mx.safetensors")
    saved = write_mxfp4_twin_layer(path, prefix, experts, shared_last=True)
    L = tables.load_mxfp4_layer([path], prefix, E, "cpu", shared=True)
    assert (L.n_exp, L.n_all, L.inter, L.hidden) == (E, E + 1, I, H)
    for e in range(E + 1):
        for j in range(3):
            assert int(L.wtab[e, j]) == L.weights[(e, j)].data_ptr() and int(L.stab[e, j]) == L.scales[(e, j)].data_ptr()
            assert torch.equal(L.weights[(e, j)], experts[e][j][0]) and torch.equal(L.scales[(e, j)], experts[e][j][1])
    R = tables.load_mxfp4_layer([path], prefix, E, "cpu", owned=range(1, 3))
    assert not R.wtab[0].any() and not R.wtab[3:].any() and R.wtab[1:3].all()
    from safetensors.torch import save_file
    bad = {k: v for k, v in saved.items() if k != f"mxfp4/{prefix}.experts.2.up_proj.weight_scale"}
    p2 = str(tmp_path / "bad.safetensors")
    save_file(bad, p2)
    with pytest.raises(ValueError):
        tables.load_mxfp4_layer([p2], prefix, E, "cpu")


@pytest.mark.gpu
def test_mxfp4_layers_over_loaded_checkpoints_equal_the_direct_binding(tmp_path):
    """One mxfp4 layer three ways, bit for bit: the synthetic binding (ops 85 / 86 over wtab / stab), the
    same experts saved as plow's per-expert twins and loaded back into tables, and the same experts saved
    in the GPT-OSS flat layout (interleaved gate / up rows) and run through ops 152 / 153 on the tensors
    the flat loader bound."""
    from gpu_harness import run_device
    from plow_amd import abi, layer, synth
    from plow_amd.lib import Moe
    print("[case] mxfp4 checkpoint round trips", flush=True)
    cfg = layer.MoeConfig("ckpt-mx", H=512, E=6, I=256, k=2, T=40, scoring="sigmoid", norm_topk=True, bias=True,
                          enc="mxfp4", arm="a16")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=9)
    moe = Moe(0)
    run_device(moe, plan, dev)
    want_fu, want = dev.t["fu"].clone(), dev.t["out"].clone()
    experts = [[(ws[j].cpu(), ss[j].cpu()) for j in range(3)] for ws, ss in dev.experts]
    prefix = "model.layers.1.mlp"
    p1 = str(tmp_path / "twin.safetensors")
    write_mxfp4_twin_layer(p1, prefix, experts, shared_last=False)
    L = tables.load_mxfp4_layer([p1], prefix, cfg.E, "cuda")
    assert (L.inter, L.hidden) == (cfg.I, cfg.H)
    dev.t["wtab"], dev.t["stab"] = L.wtab, L.stab
    dev._table = None
    dev.t["out"].zero_()
    run_device(moe, plan, dev)
    assert torch.equal(dev.t["out"].view(torch.int16), want.view(torch.int16))
    # GPT-OSS flat layout through the gathered-row flat ops
    p2 = str(tmp_path / "oss.safetensors")
    write_gptoss_layer(p2, prefix, experts, with_bias=False)
    F = tables.load_mxfp4_flat_layer([p2], prefix, "cuda")
    R = dev.t["fu"].shape[0]
    fu = torch.zeros((R, cfg.I), dtype=torch.bfloat16, device="cuda")
    part = torch.zeros_like(dev.t["part"])
    t = [fu, dev.t["x"], F.gate_up_blocks, F.gate_up_scales, dev.t["meta"], dev.t["row_token"], part,
         F.down_blocks, F.down_scales, dev.t["row_partidx"], dev.t["row_gate"]]
    table = (C.c_void_p * len(t))(*[a.data_ptr() for a in t])
    glu = abi.inst(abi.OP_MOE_GLU_MX_PF, t=[0, 1, 2, 3, 4, 5], i=[cfg.I, cfg.H, cfg.E, F.layout, 0, cfg.act], slots=cfg.T * cfg.k)
    down = abi.inst(abi.OP_MOE_DOWN_MX_PF, t=[6, 0, 7, 8, 4, None, 9, 10], i=[cfg.H, cfg.I, cfg.E], slots=cfg.T * cfg.k)
    moe.exec_many([glu, down], table)
    torch.cuda.synchronize()
    rows = int(dev.np("meta")[3 * cfg.E]) * 64
    live = torch.from_numpy(dev.np("row_partidx")[:rows] != abi.EXPERT_UNUSED).cuda()
    assert torch.equal(fu[:rows][live].view(torch.int16), want_fu[:rows][live].view(torch.int16))
    assert torch.equal(part.view(torch.int32), dev.t["part"].view(torch.int32))
    moe.close()
