"""The device code objects for an unmodified plowrt (plow_amd/moe_fp8_pf_gfx950.elf, the expert GEMMs;
plow_amd/moe_w8a8_dec_gfx950.elf, the decode pair; plow_amd/moe_combine_gfx950.elf, the combine;
plow_amd/router_decode_gfx950.elf, the decode router): each ELF carries the kernel symbols, the ABI markers and a
launch shape plowrt can use (CPU tests); launched the way plowrt launches them (1-D grid, 512 / 256
threads, no dynamic LDS, one by-value argument block) they match the oracle (GPU tests)."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ELF = os.path.join(ROOT, "plow_amd", "moe_fp8_pf_gfx950.elf")
ELF_COMBINE = os.path.join(ROOT, "plow_amd", "moe_combine_gfx950.elf")
COMBINE_KERNEL = "plow_moe_combine_fixed_order_gfx950"                           # amd.rs:11668
COMBINE_MARKERS = ["plow_moe_combine_fixed_order_abi_1", "plow_moe_combine_fixed_order_slots16_1",
                   "plow_moe_combine_materialized_f32_1", "plow_moe_combine_wave64_1",
                   "plow_moe_combine_no_spill_1"]                                  # amd.rs:11669-11675
ELF_DEC = os.path.join(ROOT, "plow_amd", "moe_w8a8_dec_gfx950.elf")
DEC_MARKER = "plow_moe_w8a8_dec_abi_1"                                            # amd.rs:10810
DEC_KERNELS = {"plow_moe_w8a8_dec_glu": 96, "plow_moe_w8a8_dec_down": 80, "plow_moe_w8a8_dec_pair": 192}  # amd.rs:10827-10840
ELF_ROUTER = os.path.join(ROOT, "plow_amd", "router_decode_gfx950.elf")
ROUTER_MARKER, ROUTER_KERNEL = "plow_router_decode_abi_3", "plow_router_decode"  # amd.rs:10765-10767
KERNELS = ["plow_moe_fp8_glu_pf_gfx950", "plow_moe_fp8_down_pf_gfx950", "plow_moe_w8a8_glu_pf_gfx950",
           "plow_moe_w8a8_down_pf_gfx950", "plow_moe_w8a8_down_acc_pf_gfx950"]   # amd.rs:11720-11740


def elf_symbols(path):
    """Names in .symtab / .dynsym of a 64-bit little-endian ELF."""
    b = open(path, "rb").read()
    assert b[:4] == b"\x7fELF" and b[4] == 2 and b[5] == 1, "not a raw 64-bit ELF (plowrt loads unbundled objects)"
    shoff, = struct.unpack_from("<Q", b, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", b, 0x3A)
    secs = [struct.unpack_from("<IIQQQQIIQQ", b, shoff + i * shentsize) for i in range(shnum)]
    names = set()
    for (_, typ, _, _, off, size, link, _, _, entsize) in secs:
        if typ not in (2, 11):          # SHT_SYMTAB, SHT_DYNSYM
            continue
        stroff = secs[link][4]
        for k in range(size // entsize):
            st_name, = struct.unpack_from("<I", b, off + k * entsize)
            end = b.index(b"\0", stroff + st_name)
            names.add(b[stroff + st_name:end].decode())
    return names, b


def test_code_object_symbols_and_launch_shape():
    if not os.path.exists(ELF):
        pytest.fail(f"{ELF} is not built; run `python -m plow_amd.build`")
    names, blob = elf_symbols(ELF)
    assert "plow_moe_fp8_pf_abi_2" in names          # the marker plowrt insists on (amd.rs:11750-11753)
    for k in KERNELS:
        assert k in names and k + ".kd" in names, k  # entry point and kernel descriptor
    # every kernel declares 512 threads and static LDS within the CU's 160 KB (metadata note, msgpack text keys)
    assert blob.count(b".max_flat_workgroup_size") >= len(KERNELS)
    import re
    import subprocess
    readelf = "/opt/rocm/llvm/bin/llvm-readelf"
    if os.path.exists(readelf):
        notes = subprocess.run([readelf, "--notes", ELF], capture_output=True, text=True).stdout
        for k in KERNELS:
            m = re.search(r"\.group_segment_fixed_size: (\d+)\n(?:.*\n)*?\s*\.max_flat_workgroup_size: (\d+)\n\s*\.name:\s+" + k + r"\n", notes)
            assert m, k
            assert int(m.group(1)) <= 160 * 1024 and int(m.group(2)) == 512, (k, m.groups())


def test_combine_object_symbols_and_launch_shape():
    """plowrt takes the combine object only with its kernel, five markers, a 48-byte argument block (or
    48 + 256 bytes of hidden arguments), no LDS, no private memory and room for 256 threads
    (plow crates/plowrt/src/exec/amd.rs:11666-11716)."""
    if not os.path.exists(ELF_COMBINE):
        pytest.fail(f"{ELF_COMBINE} is not built; run `python -m plow_amd.build`")
    names, _ = elf_symbols(ELF_COMBINE)
    assert COMBINE_KERNEL in names and COMBINE_KERNEL + ".kd" in names
    for mk in COMBINE_MARKERS:
        assert mk in names, mk
    import re
    import subprocess
    readelf = "/opt/rocm/llvm/bin/llvm-readelf"
    if os.path.exists(readelf):
        notes = subprocess.run([readelf, "--notes", ELF_COMBINE], capture_output=True, text=True).stdout
        kernels = re.findall(r"\.name:\s+(\S+)\n", notes)
        assert [k for k in kernels if k.startswith("plow_") or k.startswith("_Z")] == [COMBINE_KERNEL]
        field = lambda f: int(re.search(r"\." + f + r":\s+(\d+)", notes).group(1))
        assert field("group_segment_fixed_size") == 0
        assert field("private_segment_fixed_size") == 0
        assert field("kernarg_segment_size") in (48, 48 + 256)
        assert field("max_flat_workgroup_size") >= 256
        assert field("wavefront_size") == 64
        assert field("sgpr_spill_count") == 0 and field("vgpr_spill_count") == 0


def test_decode_object_symbols_and_launch_shape():
    """plowrt takes the decode object only with its marker, three kernels whose argument segments are 96,
    80 and 192 bytes (or those + 256 bytes of hidden arguments) and no private memory; it launches 256
    threads with no dynamic LDS (plow crates/plowrt/src/exec/amd.rs:10799-10852, :17748-17790)."""
    if not os.path.exists(ELF_DEC):
        pytest.fail(f"{ELF_DEC} is not built; run `python -m plow_amd.build`")
    names, _ = elf_symbols(ELF_DEC)
    assert DEC_MARKER in names
    for k in DEC_KERNELS:
        assert k in names and k + ".kd" in names, k
    import re
    import subprocess
    readelf = "/opt/rocm/llvm/bin/llvm-readelf"
    if os.path.exists(readelf):
        notes = subprocess.run([readelf, "--notes", ELF_DEC], capture_output=True, text=True).stdout
        blocks = re.split(r"\n\s+- \.agpr_count:", notes)
        seen = 0
        for blk in blocks:
            m = re.search(r"\.name:\s+(plow_moe_w8a8_dec_\w+)\n", blk)
            if not m:
                continue
            seen += 1
            field = lambda f: int(re.search(r"\." + f + r":\s+(\d+)", blk).group(1))
            want = DEC_KERNELS[m.group(1)]
            assert field("kernarg_segment_size") in (want, want + 256), (m.group(1), field("kernarg_segment_size"))
            assert field("private_segment_fixed_size") == 0
            assert field("sgpr_spill_count") == 0 and field("vgpr_spill_count") == 0
            assert field("max_flat_workgroup_size") >= 256
            assert field("group_segment_fixed_size") <= 64 * 1024
        assert seen == 3


def test_router_object_symbols_and_launch_shape():
    """plowrt takes the router object only with its marker, its kernel, a 104-byte argument segment (or 104 +
    256 bytes of hidden arguments) and no private memory; it launches 512 threads with no dynamic LDS
    (plow crates/plowrt/src/exec/amd.rs:10755-10800, :17811-17832)."""
    if not os.path.exists(ELF_ROUTER):
        pytest.fail(f"{ELF_ROUTER} is not built; run `python -m plow_amd.build`")
    names, _ = elf_symbols(ELF_ROUTER)
    assert ROUTER_MARKER in names and ROUTER_KERNEL in names and ROUTER_KERNEL + ".kd" in names
    import re
    import subprocess
    readelf = "/opt/rocm/llvm/bin/llvm-readelf"
    if os.path.exists(readelf):
        notes = subprocess.run([readelf, "--notes", ELF_ROUTER], capture_output=True, text=True).stdout
        assert re.findall(r"\.name:\s+(plow_\S+)\n", notes) == [ROUTER_KERNEL]
        field = lambda f: int(re.search(r"\." + f + r":\s+(\d+)", notes).group(1))
        assert field("kernarg_segment_size") in (104, 104 + 256)
        assert field("private_segment_fixed_size") == 0
        assert field("sgpr_spill_count") == 0 and field("vgpr_spill_count") == 0
        assert field("max_flat_workgroup_size") >= 512
        assert field("group_segment_fixed_size") <= 160 * 1024
        assert field("wavefront_size") == 64


# ---- GPU: launch it the way plowrt does --------------------------------------------------------------

class GluArgs(C.Structure):       # plow crates/plowrt/src/exec/amd.rs:1784-1807, 96 bytes
    _fields_ = [(n, C.c_uint64) for n in ("out", "x", "weight_table", "scale_table", "meta", "row_token", "x_scale", "out_scale")] + \
               [("inter", C.c_uint32), ("hidden", C.c_uint32), ("experts", C.c_uint32), ("act", C.c_uint32),
                ("beta", C.c_float), ("linear_beta", C.c_float), ("x_pitch", C.c_uint32), ("reserved", C.c_uint32)]


class DownArgs(C.Structure):      # amd.rs:1809-1828, 80 bytes
    _fields_ = [(n, C.c_uint64) for n in ("part", "fu", "weight_table", "scale_table", "meta", "row_partidx", "row_gate", "fu_scale")] + \
               [("hidden", C.c_uint32), ("inter", C.c_uint32), ("experts", C.c_uint32), ("reserved", C.c_uint32)]


class CombineArgs(C.Structure):   # amd.rs:1768-1782, 48 bytes
    _fields_ = [(n, C.c_uint64) for n in ("out", "residual", "shared", "part")] + \
               [(n, C.c_uint32) for n in ("hidden", "topk", "tokens", "reserved")]


class DecPairArgs(C.Structure):   # amd.rs:3420-3430, 192 bytes
    _fields_ = [("glu", GluArgs), ("down", DownArgs), ("ctr", C.c_uint64), ("grid_glu", C.c_uint32), ("reserved", C.c_uint32)]


class RouterDecodeArgs(C.Structure):   # amd.rs:955-982, 104 bytes
    _fields_ = [(n, C.c_uint64) for n in ("logit", "x", "w", "table", "bias", "ctr", "signal")] + \
               [(n, C.c_uint32) for n in ("rows", "n_exp", "k_dim", "topk", "flags", "shared_tail", "n_group", "topk_group")] + \
               [("route_scale", C.c_float), ("per_row", C.c_uint32), ("signal_add", C.c_uint32), ("pad", C.c_uint32)]


assert C.sizeof(RouterDecodeArgs) == 104
assert C.sizeof(GluArgs) == 96 and C.sizeof(DownArgs) == 80 and C.sizeof(CombineArgs) == 48
assert C.sizeof(DecPairArgs) == 192


class Module:
    def __init__(self, elf=ELF, markers=("plow_moe_fp8_pf_abi_2",)):
        self.hip = C.CDLL("libamdhip64.so")
        self.mod = C.c_void_p()
        assert self.hip.hipModuleLoad(C.byref(self.mod), elf.encode()) == 0
        for mk in markers:
            dptr, size = C.c_void_p(), C.c_size_t()
            assert self.hip.hipModuleGetGlobal(C.byref(dptr), C.byref(size), self.mod, mk.encode()) == 0, mk
            assert size.value == 4
            self.marker = dptr.value

    def launch(self, name, args, grid, threads=512):
        f = C.c_void_p()
        assert self.hip.hipModuleGetFunction(C.byref(f), self.mod, name.encode()) == 0, name
        size = C.c_size_t(C.sizeof(args))
        extra = (C.c_void_p * 5)(1, C.cast(C.byref(args), C.c_void_p), 2, C.cast(C.byref(size), C.c_void_p), 3)
        rc = self.hip.hipModuleLaunchKernel(f, grid, 1, 1, threads, 1, 1, 0, None, None, extra)
        assert rc == 0, (name, rc)


@pytest.mark.gpu
@pytest.mark.parametrize("arm,T,grid", [("w8a8", 300, 37), ("w8a8", 24, 256), ("a16", 300, 37), ("a16", 24, 5)])
def test_code_object_launched_like_plowrt(oracle, arm, T, grid):
    import torch
    from gpu_harness import assert_output_close, assert_routing_equal, run_oracle
    from plow_amd import abi, layer, synth
    from plow_amd.lib import Moe
    print(f"[case] plowrt object arm={arm} T={T} grid={grid}", flush=True)
    cfg = layer.MoeConfig("obj", H=512, E=8, I=256, k=2, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          enc="fp8blk", arm=arm, n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    dev = synth.bind(plan, "cuda", seed=T)
    host = synth.to_host(dev)
    run_oracle(oracle, plan, host)
    moe, m = Moe(0), Module()
    marker = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert m.hip.hipMemcpy(C.c_void_p(marker.data_ptr()), C.c_void_p(m.marker), 4, 3) == 0   # device to device
    assert int(marker.item()) == 1
    table = dev.table()
    glu, down = plan.insts[plan.index("glu")], plan.insts[plan.index("down")]
    # everything before the GLU through the library, the two expert ops through the object, combine through the library
    pre = [d for n, d in zip(plan.names, plan.insts) if n not in ("glu", "down", "combine")]
    moe.exec_many(pre, table)
    torch.cuda.synchronize()
    p = lambda name: dev.t[name].data_ptr() if name in dev.t else 0
    Ea = cfg.E_all
    if arm == "w8a8":
        ga = GluArgs(p("fq"), p("xq"), p("wtab"), p("stab"), p("meta"), p("row_token"), p("xs"), p("fs"),
                     cfg.I, cfg.H, Ea, cfg.act, 0.0, 0.0, glu.i[4], 0)
        da = DownArgs(p("part"), p("fq"), p("wtab"), p("stab"), p("meta"), p("row_partidx"), p("row_gate"), p("fs"),
                      cfg.H, cfg.I, Ea, 0)
        m.launch("plow_moe_w8a8_glu_pf_gfx950", ga, grid)
        m.launch("plow_moe_w8a8_down_pf_gfx950", da, grid)
    else:
        ga = GluArgs(p("fu"), p("x"), p("wtab"), p("stab"), p("meta"), p("row_token"), 0, 0,
                     cfg.I, cfg.H, Ea, cfg.act, 0.0, 0.0, 0, 0)
        da = DownArgs(p("part"), p("fu"), p("wtab"), p("stab"), p("meta"), p("row_partidx"), p("row_gate"), 0,
                      cfg.H, cfg.I, Ea, 0)
        m.launch("plow_moe_fp8_glu_pf_gfx950", ga, grid)
        m.launch("plow_moe_fp8_down_pf_gfx950", da, grid)
    torch.cuda.synchronize()
    moe.exec_many([plan.insts[plan.index("combine")]], table)
    torch.cuda.synchronize()
    assert_routing_equal(plan, dev, host)
    pd, ph = dev.np("part"), host.np("part")
    assert np.all(np.isfinite(pd))
    assert np.abs(pd - ph).max() / np.abs(ph).max() < 2e-2
    assert_output_close(dev.np("out"), host.np("out"))
    if arm == "w8a8":
        # the fused-combine DOWN adds gate * acc into a bf16 [T][H] output seeded with zeros: the same
        # sums as combine, rounded to bf16 after every addition in an order that depends on timing
        acc = torch.zeros((cfg.T, cfg.H), dtype=torch.bfloat16, device="cuda")
        da.part, da.reserved = acc.data_ptr(), cfg.k_all
        m.launch("plow_moe_w8a8_down_acc_pf_gfx950", da, grid)
        torch.cuda.synchronize()
        got, want = acc.float().cpu().numpy(), host.np("out").astype(np.uint32)
        want = (want << 16).view(np.float32)
        assert np.abs(got - want).max() <= 3e-2 * np.abs(want).max()
        assert np.abs(got - want).mean() <= 1e-2 * np.abs(want).mean()
    moe.close()


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,k,res,shr", [(1, 512, 16, True, True), (37, 1024, 8, True, False), (700, 512, 9, False, True),
                                           (1500, 2048, 16, True, True), (64, 520, 3, False, False)])
def test_combine_object_launched_like_plowrt(T, H, k, res, shr):
    """min(tokens, 512) workgroups of 256 threads (amd.rs:4018-4036): bit-exact with the library's op 87 and
    with the f32 sum in slot order on top of residual + shared, rounded to bf16 once
    (plow runtime/cpu/dev/golden/moe_route.c:130-147)."""
    import torch
    print(f"[case] plowrt combine object T={T} H={H} k={k} residual={res} shared={shr}", flush=True)
    g = torch.Generator(device="cpu").manual_seed(T * 131 + k)
    part = torch.randn((T * k, H), generator=g, dtype=torch.float32)
    residual = torch.randn((T, H), generator=g, dtype=torch.float32).bfloat16()
    shared = torch.randn((T, H), generator=g, dtype=torch.float32).bfloat16()
    want = torch.zeros((T, H), dtype=torch.float32)
    if res:
        want = want + residual.float()
    if shr:
        want = want + shared.float()
    p3 = part.view(T, k, H)
    for j in range(k):
        want = want + p3[:, j, :]
    want = want.bfloat16()
    d_part, d_res, d_shr = part.cuda(), residual.cuda(), shared.cuda()
    out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
    m = Module(ELF_COMBINE, COMBINE_MARKERS)
    a = CombineArgs(out.data_ptr(), d_res.data_ptr() if res else 0, d_shr.data_ptr() if shr else 0,
                    d_part.data_ptr(), H, k, T, 0)
    m.launch(COMBINE_KERNEL, a, min(T, 512), threads=256)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
    # and the library's own op 87 on the same buffers
    from plow_amd import abi
    from plow_amd.lib import Moe
    moe = Moe(0)
    out2 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
    d = abi.inst(87, t=[0, 1 if res else None, 2 if shr else None, 3], i=[H, k, T])
    table = (C.c_void_p * 4)(out2.data_ptr(), d_res.data_ptr(), d_shr.data_ptr(), d_part.data_ptr())
    moe.exec_many([d], table)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    moe.close()


@pytest.mark.gpu
@pytest.mark.parametrize("T,shrink", [(24, 1), (5, 1), (70, 3)])
def test_decode_object_launched_like_plowrt(oracle, T, shrink):
    """The decode pair (op 85 arm 6 + op 86 arm 2) through `moe_w8a8_dec_gfx950.elf`: GLU and DOWN back to
    back on plowrt's grids (2 * tiles * I / 128 and 2 * tiles * H / 256 workgroups of 256 threads,
    amd.rs:3519-3520; `shrink` divides them, any grid must serve), then both in one launch of the pair
    kernel with its counter scratch. Same arithmetic as the library's streaming kernel: bit-identical to
    the library's own ops on the same inputs, and within tolerance of the oracle."""
    import torch
    from gpu_harness import assert_output_close, assert_routing_equal, run_oracle
    from plow_amd import abi, layer, synth
    from plow_amd.lib import Moe
    print(f"[case] plowrt decode object T={T} shrink={shrink}", flush=True)
    cfg = layer.MoeConfig("dec-obj", H=1024, E=8, I=256, k=2, T=T, scoring="sigmoid", norm_topk=True, bias=True,
                          enc="fp8blk", arm="w8a8q", n_shared=1, shared_mode="fold")
    plan = layer.plan_layer(cfg)
    plan.insts[plan.index("glu")].i[4] = 0          # no row count of x stated: the op keeps its streaming form at every size
    dev = synth.bind(plan, "cuda", seed=T)
    host = synth.to_host(dev)
    run_oracle(oracle, plan, host)
    moe = Moe(0)
    table = dev.table()
    moe.exec_many(plan.insts, table)               # the library's own run: the bits to reproduce
    torch.cuda.synchronize()
    assert_routing_equal(plan, dev, host)
    assert_output_close(dev.np("out"), host.np("out"))
    want = {n: dev.t[n].clone() for n in ("fq", "fs", "part")}
    Ea = cfg.E_all
    tiles = int(dev.np("meta")[3 * Ea])             # 64-row tiles of this batch (plowrt passes a bound on it)
    grid_glu = max(1, 2 * tiles * (cfg.I // 128) // shrink)
    grid_down = max(1, 2 * tiles * ((cfg.H + 255) // 256) // shrink)
    p = lambda name: dev.t[name].data_ptr()
    ga = GluArgs(p("fq"), p("x"), p("wtab"), p("stab"), p("meta"), p("row_token"), 0, p("fs"),
                 cfg.I, cfg.H, Ea, cfg.act, 0.0, 0.0, 0, 0)
    da = DownArgs(p("part"), p("fq"), p("wtab"), p("stab"), p("meta"), p("row_partidx"), p("row_gate"), p("fs"),
                  cfg.H, cfg.I, Ea, 0)
    m = Module(ELF_DEC, (DEC_MARKER,))

    def wipe():
        dev.t["fq"].fill_(0x55)
        dev.t["fs"].fill_(7.0)
        dev.t["part"].fill_(float("nan"))
        torch.cuda.synchronize()

    def check(what):
        live = dev.np("row_partidx")[:tiles * 64] != abi.EXPERT_UNUSED
        for n in ("fq", "fs"):
            got, ref = dev.t[n][:tiles * 64].cpu().numpy()[live], want[n][:tiles * 64].cpu().numpy()[live]
            assert np.array_equal(got.view(np.uint8), ref.view(np.uint8)), (what, n)
        assert torch.equal(dev.t["part"].view(torch.int32), want["part"].view(torch.int32)), (what, "part")

    wipe()
    print(f"[launch] dec_glu grid={grid_glu}, dec_down grid={grid_down}", flush=True)
    m.launch("plow_moe_w8a8_dec_glu", ga, grid_glu, threads=256)
    m.launch("plow_moe_w8a8_dec_down", da, grid_down, threads=256)
    torch.cuda.synchronize()
    check("back to back")

    wipe()
    ctr = torch.zeros(4 * max(tiles, 1), dtype=torch.int32, device="cuda")
    pa = DecPairArgs(ga, da, ctr.data_ptr(), grid_glu, 0)
    for rep in range(2):                            # the second launch finds the scratch the first left
        print(f"[launch] dec_pair grid={grid_glu}+{grid_down} rep={rep}", flush=True)
        m.launch("plow_moe_w8a8_dec_pair", pa, grid_glu + grid_down, threads=256)
        torch.cuda.synchronize()
        check(f"pair rep {rep}")
        assert int(ctr.abs().sum().item()) == 0
        wipe()

    # A DOWN item whose bounded wait gives up: forced from the host with a poll limit of 1 (the pair block's
    # `reserved` word) and a GLU share of one workgroup, so most DOWN items poll before their expert's GLU
    # items are done. Every kernel still runs to its end. Each 256-channel block of each live slot row must
    # then hold either the right values or NaN (the item said it could not compute), never what was there
    # before; the scratch must come back zeroed; and a normal launch on that scratch must be exact again.
    dev.t["fq"].fill_(0x55)
    dev.t["fs"].fill_(7.0)
    dev.t["part"].fill_(123.0)
    torch.cuda.synchronize()
    pa1 = DecPairArgs(ga, da, ctr.data_ptr(), 1, 1)
    print(f"[launch] dec_pair grid=1+{grid_down} poll limit 1", flush=True)
    m.launch("plow_moe_w8a8_dec_pair", pa1, 1 + grid_down, threads=256)
    torch.cuda.synchronize()
    assert int(ctr.abs().sum().item()) == 0
    got = dev.t["part"].cpu().numpy().reshape(-1, cfg.H // 256, 256)
    ref = want["part"].cpu().numpy().reshape(-1, cfg.H // 256, 256)
    live_slots = host.np("table")["eid"] < Ea
    blk_nan = np.isnan(got).all(axis=2)
    blk_ok = (got.view(np.uint32) == ref.view(np.uint32)).all(axis=2)
    assert (blk_nan | blk_ok)[live_slots].all(), "a block holds neither the result nor the poison"
    print(f"[pair] {int(blk_nan[live_slots].sum())} of {int(live_slots.sum()) * (cfg.H // 256)} blocks poisoned, the rest exact", flush=True)
    wipe()
    m.launch("plow_moe_w8a8_dec_pair", pa, grid_glu + grid_down, threads=256)
    torch.cuda.synchronize()
    check("pair after a launch whose waits gave up")
    assert int(ctr.abs().sum().item()) == 0
    moe.close()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,E,H,k,tail,groups", [(1, 256, 1024, 8, 1, (8, 4)), (3, 384, 768, 8, 1, (1, 1)), (7, 128, 512, 6, 0, (1, 1)),
                                                    (1, 72, 520, 4, 0, (1, 1)), (20, 512, 256, 8, 1, (4, 2))])
def test_router_object_launched_like_plowrt(rows, E, H, k, tail, groups):
    """rows * ceil(n_exp / 8) workgroups of 512 threads, no dynamic LDS (amd.rs:1009, :17811-17832): logits and
    table are the bytes of the library's op 180 followed by op 83, the arrival counters are back at zero, a
    second launch gives the same, and a launch that signals adds its increment to the counter it names.
    H = 520 is a row length the few-token score kernel does not serve (the object's plain loop runs)."""
    import torch
    from plow_amd import abi
    from plow_amd.lib import Moe
    print(f"[case] plowrt router object rows={rows} E={E} H={H} k={k} tail={tail} groups={groups}", flush=True)
    g = torch.Generator(device="cpu").manual_seed(rows * 1000 + E)
    x = torch.randn((rows, H), generator=g).bfloat16().cuda()
    w = (torch.randn((E, H), generator=g) * 0.05).bfloat16().cuda()
    bias = (torch.randn(E, generator=g) * 0.01).float().cuda()
    flags = abi.ROUTE_SIGMOID | abi.ROUTE_NORM_TOPK | abi.ROUTE_BIAS | abi.ROUTE_F32_LOGIT
    ng, tg = groups
    # the library's two ops
    moe = Moe(0)
    logit_ref = torch.zeros((rows, E), dtype=torch.float32, device="cuda")
    table_ref = torch.zeros((rows * (k + tail), 2), dtype=torch.int32, device="cuda")
    tab = (C.c_void_p * 5)(logit_ref.data_ptr(), x.data_ptr(), w.data_ptr(), table_ref.data_ptr(), bias.data_ptr())
    moe.exec_many([abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[rows, E, H]),
                   abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[3, 0, None, 4], i=[0, E, k, flags, rows, tail, ng, tg], f=[2.5, 0.0])], tab)
    torch.cuda.synchronize()
    moe.close()
    m = Module(ELF_ROUTER, (ROUTER_MARKER,))
    per_row = (E + 7) // 8
    ctr = torch.zeros(rows * 32, dtype=torch.int32, device="cuda")
    signal = torch.zeros(64, dtype=torch.int32, device="cuda")
    for rep, add in enumerate((0, 0, 5)):
        if add and rows != 1:
            break                                   # plowrt signals from one-row routers only
        logit = torch.full((rows, E), float("nan"), dtype=torch.float32, device="cuda")
        table = torch.full((rows * (k + tail), 2), -1, dtype=torch.int32, device="cuda")
        a = RouterDecodeArgs(logit.data_ptr(), x.data_ptr(), w.data_ptr(), table.data_ptr(), bias.data_ptr(), ctr.data_ptr(),
                             signal.data_ptr() + 16 * 4, rows, E, H, k, flags, tail, ng, tg, 2.5, per_row, add, 0)
        m.launch(ROUTER_KERNEL, a, rows * per_row, threads=512)
        torch.cuda.synchronize()
        assert torch.equal(logit.view(torch.int32), logit_ref.view(torch.int32)), rep
        assert torch.equal(table, table_ref), rep
        assert not ctr.any()
        assert int(signal[16]) == add and int(signal.sum()) == add
