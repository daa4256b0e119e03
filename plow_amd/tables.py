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
