"""Expert pointer tables and a checkpoint loader for them: the host-side step before the operator.

The expert ops never see an expert's tensors by name, only two tables of device addresses,
``wtab[E][3]`` / ``stab[E][3]`` = {gate, up, down} (plow runtime/amd/op_moe.h:18-21, :1242-1249), or
``ewt[E][2]`` = {gate_up fused, down} for fused tensors. A zero entry is not an omission but the
interface: the ops skip such an expert (GLU writes nothing, DOWN zeroes or skips its rows), which is how
an expert-parallel rank leaves out the experts it does not hold. The three builders mirror plow's
(crates/plowrt/src/orch/moe.rs:21-55, :84-97, :110-124) and keep their argument meaning; the loader
reads one layer of a block-fp8 checkpoint in the DeepSeek-V3 safetensors layout (e4m3 ``weight`` [N][K]
with f32 ``weight_scale_inv`` [ceil(N/128)][ceil(K/128)], multiplied on dequantization: the layout the
ops read, runtime/common/dev_isa.h:442-445) and fills both tables over the tensors it loaded."""
from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch

PROJ = ("gate_proj", "up_proj", "down_proj")


def build_expert_table(shared: Iterable[Tuple[Optional[str], Optional[str]]],
                       layers: Iterable[Iterable[Tuple[str, str, str]]],
                       resolve: Callable[[str], Optional[int]]) -> List[int]:
    """Flat base table: the shared experts' (gate_up, down) first, then per routed layer each expert's
    (gate, up, down) in id order. A name that does not resolve is skipped
    (crates/plowrt/src/orch/moe.rs:29-55)."""
    bases: List[int] = []
    for pair in shared:
        for name in pair:
            if name is not None:
                addr = resolve(name)
                if addr is not None:
                    bases.append(addr)
    for layer in layers:
        for triple in layer:
            for name in triple:
                addr = resolve(name)
                if addr is not None:
                    bases.append(addr)
    return bases


def packed_expert_table(base: int, stride: int, n_exp: int, owned: range) -> List[int]:
    """The [E][3] table of one layer whose owned experts are packed into one buffer, slot k at
    base + k * stride in (expert, projection) order; an expert outside `owned` keeps zeros
    (crates/plowrt/src/orch/moe.rs:84-97)."""
    table = [0] * (n_exp * 3)
    for slot, e in enumerate(e for e in owned if e < n_exp):
        for j in range(3):
            table[e * 3 + j] = base + (slot * 3 + j) * stride
    return table


def build_fused_expert_table(gate_up_base: int, down_base: int, num_experts: int, gate_up_stride: int,
                             down_stride: int) -> List[int]:
    """The [E][2] table over fused 3-D tensors gate_up [E][2I][H] and down [E][H][I]: per-expert byte
    offsets into the two tensors (crates/plowrt/src/orch/moe.rs:110-124)."""
    bases: List[int] = []
    for e in range(num_experts):
        bases.append(gate_up_base + e * gate_up_stride)
        bases.append(down_base + e * down_stride)
    return bases


class BlockFp8Layer:
    """One layer's experts on a device: the tensors (kept alive here) and the two tables."""

    def __init__(self):
        self.weights: Dict[Tuple[int, int], torch.Tensor] = {}
        self.scales: Dict[Tuple[int, int], torch.Tensor] = {}
        self.wtab: Optional[torch.Tensor] = None   # int64 [E_all][3] on the device
        self.stab: Optional[torch.Tensor] = None
        self.n_exp = 0        # routed experts
        self.n_all = 0        # + the folded shared expert, if any
        self.inter = 0
        self.hidden = 0


def load_block_fp8_layer(files: Sequence[str], prefix: str, n_exp: int, device,
                         owned: Optional[range] = None, shared: bool = False) -> BlockFp8Layer:
    """Read `{prefix}.experts.{e}.{gate,up,down}_proj.weight` (+ `.weight_scale_inv`) for the experts in
    `owned` (default: all) from safetensors files and build wtab / stab. With `shared`, the layer's
    `{prefix}.shared_experts.*` becomes expert id n_exp (the folded form, routed to by every token).
    Experts outside `owned`, and tensors missing from the files, leave zero entries. Nothing but
    safetensors' own reader touches the files."""
    from safetensors import safe_open
    want: Dict[str, Tuple[int, int, bool]] = {}
    owned = range(n_exp) if owned is None else owned
    for e in owned:
        if e >= n_exp:
            continue
        for j, proj in enumerate(PROJ):
            want[f"{prefix}.experts.{e}.{proj}.weight"] = (e, j, False)
            want[f"{prefix}.experts.{e}.{proj}.weight_scale_inv"] = (e, j, True)
    if shared:
        for j, proj in enumerate(PROJ):
            want[f"{prefix}.shared_experts.{proj}.weight"] = (n_exp, j, False)
            want[f"{prefix}.shared_experts.{proj}.weight_scale_inv"] = (n_exp, j, True)
    L = BlockFp8Layer()
    L.n_exp, L.n_all = n_exp, n_exp + (1 if shared else 0)
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                hit = want.get(name)
                if hit is None:
                    continue
                e, j, is_scale = hit
                t = f.get_tensor(name)
                if is_scale:
                    if t.dtype != torch.float32:
                        raise ValueError(f"{name}: scales must be f32, found {t.dtype}")
                    L.scales[(e, j)] = t.contiguous().to(device)
                else:
                    if t.dtype != torch.float8_e4m3fn:
                        raise ValueError(f"{name}: weights must be float8_e4m3fn, found {t.dtype}")
                    L.weights[(e, j)] = t.contiguous().view(torch.uint8).to(device)
    for (e, j), wt in L.weights.items():
        sc = L.scales.get((e, j))
        n, k = wt.shape
        if sc is None or tuple(sc.shape) != ((n + 127) // 128, (k + 127) // 128):
            raise ValueError(f"expert {e} projection {PROJ[j]}: scale grid missing or not [ceil(N/128)][ceil(K/128)]")
        if j == 0:
            L.inter, L.hidden = n, k
    wtab = torch.zeros((L.n_all, 3), dtype=torch.int64)
    stab = torch.zeros((L.n_all, 3), dtype=torch.int64)
    for e in range(L.n_all):
        if all((e, j) in L.weights for j in range(3)):        # an expert is resident as a whole or not at all
            for j in range(3):
                wtab[e, j] = L.weights[(e, j)].data_ptr()
                stab[e, j] = L.scales[(e, j)].data_ptr()
    L.wtab, L.stab = wtab.to(device), stab.to(device)
    return L


class Mxfp4FlatLayer:
    """One layer's experts in the GPT-OSS checkpoint layout, bound verbatim: flat fused-expert tensors
    that ops 150 - 153 index by expert themselves (plow runtime/common/dev_isa.h:1285-1303)."""

    def __init__(self):
        self.gate_up_blocks: Optional[torch.Tensor] = None   # u8 [E][2I][K/2]   (checkpoint [E][2I][K/32][16])
        self.gate_up_scales: Optional[torch.Tensor] = None   # u8 [E][2I][K/32]  E8M0
        self.gate_up_bias: Optional[torch.Tensor] = None     # bf16 [E][2I] or None
        self.down_blocks: Optional[torch.Tensor] = None      # u8 [E][H][I/2]
        self.down_scales: Optional[torch.Tensor] = None      # u8 [E][H][I/32]
        self.down_bias: Optional[torch.Tensor] = None        # bf16 [E][H] or None
        self.n_exp = self.inter = self.hidden = 0
        self.layout = 0      # gate / up rows interleaved (row 2n = gate_n, 2n + 1 = up_n): op 150 / 152's i4 / i3 = 0


def load_mxfp4_flat_layer(files: Sequence[str], prefix: str, device) -> Mxfp4FlatLayer:
    """Read `{prefix}.experts.{gate_up,down}_proj_{blocks,scales,bias}` (GPT-OSS: prefix
    `model.layers.N.mlp`; plow binds them under these checkpoint names, crates/devgen/src/gptoss.rs:382-398).
    The tensors go to the device as they are: [E][rows][K/32][16] blocks are already the fp4 rows
    [E][rows][K/2] the ops read (low nibble = even k), scales are E8M0 bytes, rows of gate_up interleaved."""
    from safetensors import safe_open
    names = {f"{prefix}.experts.{p}_proj_{part}": (p, part) for p in ("gate_up", "down") for part in ("blocks", "scales", "bias")}
    got: Dict[Tuple[str, str], torch.Tensor] = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                if name in names:
                    got[names[name]] = f.get_tensor(name)
    L = Mxfp4FlatLayer()
    for p in ("gate_up", "down"):
        blk, sc = got.get((p, "blocks")), got.get((p, "scales"))
        if blk is None or sc is None:
            raise ValueError(f"{prefix}.experts.{p}_proj: blocks or scales missing")
        if blk.dtype != torch.uint8 or sc.dtype != torch.uint8:
            raise ValueError(f"{prefix}.experts.{p}_proj: blocks and scales must be uint8")
        if blk.dim() == 4:                                  # [E][rows][K/32][16] -> [E][rows][K/2]
            if blk.shape[3] != 16:
                raise ValueError(f"{prefix}.experts.{p}_proj_blocks: last dimension {blk.shape[3]} is not 16")
            blk = blk.reshape(blk.shape[0], blk.shape[1], blk.shape[2] * 16)
        if blk.dim() != 3 or sc.dim() != 3 or tuple(sc.shape) != (blk.shape[0], blk.shape[1], blk.shape[2] // 16):
            raise ValueError(f"{prefix}.experts.{p}_proj: scales {tuple(sc.shape)} do not match blocks {tuple(blk.shape)}")
        bias = got.get((p, "bias"))
        if bias is not None and (bias.dtype != torch.bfloat16 or tuple(bias.shape) != tuple(blk.shape[:2])):
            raise ValueError(f"{prefix}.experts.{p}_proj_bias: must be bf16 [E][rows]")
        setattr(L, f"{p}_blocks", blk.contiguous().to(device))
        setattr(L, f"{p}_scales", sc.contiguous().to(device))
        setattr(L, f"{p}_bias", None if bias is None else bias.contiguous().to(device))
    E, rows_gu, kh = L.gate_up_blocks.shape
    Ed, H, ih = L.down_blocks.shape
    if Ed != E or rows_gu % 2 or rows_gu // 2 != ih * 2 or kh * 2 != H:
        raise ValueError(f"{prefix}: gate_up {tuple(L.gate_up_blocks.shape)} and down {tuple(L.down_blocks.shape)} do not describe one layer")
    L.n_exp, L.inter, L.hidden = E, rows_gu // 2, H
    return L


class Mxfp4Layer(BlockFp8Layer):
    """Per-expert mxfp4 tensors behind wtab / stab (e2m1 rows [N][K/2] + E8M0 bytes [N][K/32])."""


def load_mxfp4_layer(files: Sequence[str], prefix: str, n_exp: int, device, owned: Optional[range] = None,
                     shared: bool = False) -> Mxfp4Layer:
    """Read plow's mxfp4 weight twins `mxfp4/{prefix}.experts.{e}.{gate,up,down}_proj.weight` (u8 [N][K/2],
    low nibble = even k) and `..._scale` (u8 [N][K/32], E8M0) — the format of plow's quantizer
    (perf-data/tools/quantize_mxfp4.py:4-9) — for the experts in `owned`, and build wtab / stab [E][3] for
    ops 85 / 86 (enc 2, bf16 activations) and 48 / 49. With `shared`, `{prefix}.shared_experts.*` becomes
    expert id n_exp. Experts outside `owned` and experts with a tensor missing keep zero entries."""
    from safetensors import safe_open
    want: Dict[str, Tuple[int, int, bool]] = {}
    owned = range(n_exp) if owned is None else owned
    who = [(e, f"experts.{e}") for e in owned if e < n_exp] + ([(n_exp, "shared_experts")] if shared else [])
    for e, w in who:
        for j, proj in enumerate(PROJ):
            want[f"mxfp4/{prefix}.{w}.{proj}.weight"] = (e, j, False)
            want[f"mxfp4/{prefix}.{w}.{proj}.weight_scale"] = (e, j, True)
    L = Mxfp4Layer()
    L.n_exp, L.n_all = n_exp, n_exp + (1 if shared else 0)
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                hit = want.get(name)
                if hit is None:
                    continue
                e, j, is_scale = hit
                t = f.get_tensor(name)
                if t.dtype != torch.uint8 or t.dim() != 2:
                    raise ValueError(f"{name}: must be a 2-D uint8 tensor, found {t.dtype} {tuple(t.shape)}")
                (L.scales if is_scale else L.weights)[(e, j)] = t.contiguous().to(device)
    for (e, j), wt in L.weights.items():
        sc = L.scales.get((e, j))
        n, kh = wt.shape
        if sc is None or tuple(sc.shape) != (n, kh // 16) or kh % 16:
            raise ValueError(f"expert {e} projection {PROJ[j]}: E8M0 scales missing or not [N][K/32]")
        if j == 0:
            L.inter, L.hidden = n, kh * 2
    wtab = torch.zeros((L.n_all, 3), dtype=torch.int64)
    stab = torch.zeros((L.n_all, 3), dtype=torch.int64)
    for e in range(L.n_all):
        if all((e, j) in L.weights for j in range(3)):
            for j in range(3):
                wtab[e, j] = L.weights[(e, j)].data_ptr()
                stab[e, j] = L.scales[(e, j)].data_ptr()
    L.wtab, L.stab = wtab.to(device), stab.to(device)
    return L
