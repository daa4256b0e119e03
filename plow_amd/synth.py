"""Synthetic, seeded inputs for a MoE layer plan and the tensor table that binds them.

One PRNG: ``torch.Generator`` (Philox on a GPU, MT19937 on the CPU) seeded per tensor from the
layer seed, so every tensor is reproducible on its own. Distributions follow the benchmark
definition: activations ~N(0,1), expert / shared / router weights ~N(0,0.02), router bias
~N(0,0.01), all rounded to bf16 first and then quantized with the reference's quantizer rules:

  block-fp8   e4m3 with one f32 scale per 128x128 block, scale = amax_block / 448
              (DeepSeek ``weight_scale_inv`` convention; layout runtime/common/dev_isa.h:442-445)
  per-channel e4m3 with one f32 scale per output row, scale = amax_row / 448
              (perf-data/tools/quantize_fp8.py:204-207)
  mxfp4       e2m1 + E8M0 per 32: scale 2^e with amax / 2^e in (3, 6], round to nearest with ties
              toward zero, all-zero block -> 2^-3 (perf-data/tools/quantize_mxfp4.py:38-55)

torch is used here for storage and random numbers only; none of it is on the operator's path.
"""
import ctypes as C
from typing import Dict, Optional

import numpy as np
import torch

from . import abi
from .layer import LayerPlan, MoeConfig

_TORCH_DT = {"bf16": torch.bfloat16, "f32": torch.float32, "f64": torch.float64, "u8": torch.uint8,
             "i32": torch.int32, "u32": torch.int32, "u64": torch.int64}

E4M3_MAX = 448.0


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def randn_bf16(shape, std, device, seed):
    return (torch.randn(shape, generator=_gen(device, seed), device=device, dtype=torch.float32) * std
            ).to(torch.bfloat16)


def quant_fp8_block128(w: torch.Tensor):
    """w [N, K] (any float dtype) -> (e4m3 bytes u8 [N, K], f32 scales [ceil(N/128), ceil(K/128)])."""
    N, K = w.shape
    nb, kb = (N + 127) // 128, (K + 127) // 128
    wp = torch.zeros((nb * 128, kb * 128), dtype=torch.float32, device=w.device)
    wp[:N, :K] = w.float()
    blk = wp.view(nb, 128, kb, 128)
    amax = blk.abs().amax(dim=(1, 3))
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    q = (blk / scale[:, None, :, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    q = q.view(nb * 128, kb * 128)[:N, :K].contiguous().view(torch.uint8)
    return q, scale.contiguous()


def quant_fp8_channel(w: torch.Tensor):
    """w [N, K] -> (e4m3 bytes u8 [N, K], f32 scales [N])."""
    amax = w.float().abs().amax(dim=1)
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    q = (w.float() / scale[:, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).contiguous(), scale.contiguous()


def quant_mxfp4(w: torch.Tensor):
    """w [N, K] -> (packed e2m1 u8 [N, K/2] low nibble = even k, E8M0 u8 [N, K/32])."""
    N, K = w.shape
    assert K % 32 == 0
    blk = w.float().view(N, K // 32, 32)
    amax = blk.abs().amax(dim=2)
    mant, ex = torch.frexp(amax)                       # amax = mant * 2^ex, mant in [0.5, 1)
    e = ex - 2 - (mant <= 0.75).to(ex.dtype)           # amax / 2^e in (3, 6]
    e = torch.where(amax > 0, e, torch.full_like(e, -3)).clamp(-127, 127)
    v = (blk / torch.exp2(e.float()).unsqueeze(2)).clamp(-6.0, 6.0)
    mid = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], device=w.device)
    code = torch.bucketize(v.abs(), mid) | ((v < 0).to(torch.int64) << 3)   # ties -> lower code
    code = code.view(N, K)
    packed = (code[:, 0::2] | (code[:, 1::2] << 4)).to(torch.uint8)
    return packed.contiguous(), (e + 127).to(torch.uint8).contiguous()


class Bound:
    """Tensors of one plan on one device plus the handle table pointing at them."""

    def __init__(self, plan: LayerPlan, device):
        self.plan, self.device = plan, torch.device(device)
        self.t: Dict[str, torch.Tensor] = {}
        self.experts = []          # keeps the per-expert weight tensors alive
        self._table = None

    def alloc(self, name: str, fill: Optional[float] = None) -> torch.Tensor:
        sp = self.plan.specs[name]
        if sp.dtype == "route":
            t = torch.zeros((sp.shape[0], 2), dtype=torch.int32, device=self.device)
        else:
            t = torch.zeros(sp.shape, dtype=_TORCH_DT[sp.dtype], device=self.device)
        if fill is not None:
            t.fill_(fill)
        self.t[name] = t
        self._table = None
        return t

    def table(self):
        """ctypes ``void*[]`` handle table (device or host pointers, by where the tensors live)."""
        if self._table is None:
            n = len(self.plan.slots)
            arr = (C.c_void_p * n)()
            for name, h in self.plan.slots.items():
                arr[h] = self.t[name].data_ptr() if name in self.t else None
            self._table = arr
        return self._table

    def np(self, name: str) -> np.ndarray:
        """Host copy of a tensor as a numpy array (bf16 as its uint16 bits; routes as (eid, gate))."""
        t = self.t[name].detach().cpu().contiguous()
        sp = self.plan.specs[name]
        if sp.dtype == "bf16":
            return t.view(torch.int16).numpy().view(np.uint16)
        if sp.dtype == "u32":
            return t.numpy().view(np.uint32)
        if sp.dtype == "u64":
            return t.numpy().view(np.uint64)
        if sp.dtype == "route":
            a = t.numpy()
            out = np.zeros(a.shape[0], dtype=[("eid", np.uint32), ("gate", np.float32)])
            out["eid"] = a[:, 0].view(np.uint32)
            out["gate"] = a[:, 1].view(np.float32)
            return out
        return t.numpy()


def skewed_bias(E: int, hot: float, device, seed: int) -> torch.Tensor:
    """Router bias ~N(0, 0.01) with expert 0 raised so that it draws about ``hot`` x the mean load."""
    b = torch.randn(E, generator=_gen(device, seed), device=device) * 0.01
    if hot > 1.0:
        b[0] += 0.0175 * hot
    return b


def zipf_bias(E: int, s: float, device, seed: int, alpha: float = 0.01) -> torch.Tensor:
    """Selection bias alpha * ln(rank ** -s) over a seeded permutation of the experts: expert
    popularity falls off Zipf-like with exponent ``s`` while gates stay the unbiased scores."""
    perm = torch.randperm(E, generator=_gen("cpu", seed)).to(device)
    rank = torch.empty(E, device=device)
    rank[perm] = torch.arange(1, E + 1, device=device, dtype=torch.float32)
    return (-s * alpha) * torch.log(rank)


def bind(plan: LayerPlan, device, seed: int = 0, x_std: float = 1.0, w_std: float = 0.02,
         hot_expert: float = 0.0, experts_alias: int = 0, zipf: float = 0.0,
         share: Optional[Bound] = None) -> Bound:
    """Allocate and fill every tensor of ``plan`` on ``device``.

    ``experts_alias`` > 0 generates only that many distinct expert weight sets and lets the pointer
    tables cycle through them (for memory-limited CPU tests; 0 = every expert distinct).
    ``share``: a binding of the same layer (same seed, same expert geometry, any batch size) on the same
    device whose router and expert weights and pointer tables are reused instead of generated again.
    """
    cfg: MoeConfig = plan.cfg
    b = Bound(plan, device)
    dev = b.device
    for name, sp in plan.specs.items():
        if sp.role in ("scratch", "out", "table"):
            b.alloc(name)
    b.t["x"] = randn_bf16((cfg.T, cfg.H), x_std, dev, seed * 1000 + 1)
    if share is not None:
        sc = share.plan.cfg
        assert (sc.H, sc.E, sc.I, sc.enc, sc.E_all) == (cfg.H, cfg.E, cfg.I, cfg.enc, cfg.E_all) and share.device == dev
    b.t["Wr"] = share.t["Wr"] if share is not None else randn_bf16((cfg.E, cfg.H), w_std, dev, seed * 1000 + 2)
    if cfg.bias:
        b.t["bias"] = (zipf_bias(cfg.E, zipf, dev, seed * 1000 + 3) if zipf
                       else skewed_bias(cfg.E, hot_expert, dev, seed * 1000 + 3) if hot_expert
                       else torch.randn(cfg.E, generator=_gen(dev, seed * 1000 + 3), device=dev) * 0.01)
    if cfg.residual:
        b.t["residual"] = randn_bf16((cfg.T, cfg.H), x_std, dev, seed * 1000 + 4)
    if cfg.shared_mode == "dense":
        Is = cfg.I_shared
        b.t["Ws_gate"] = randn_bf16((Is, cfg.H), w_std, dev, seed * 1000 + 5)
        b.t["Ws_up"] = randn_bf16((Is, cfg.H), w_std, dev, seed * 1000 + 6)
        b.t["Ws_down"] = randn_bf16((cfg.H, Is), w_std, dev, seed * 1000 + 7)

    Ea = cfg.E_all
    wname, sname = ("ewt", "est") if cfg.enc == "fp8pc" else ("wtab", "stab")
    if share is not None:
        b.experts = share.experts
        b.t[wname] = share.t[wname]
        if sname in plan.slots:
            b.t[sname] = share.t[sname]
        b._table = None
        return b
    n_distinct = min(Ea, experts_alias) if experts_alias else Ea
    sets = []
    for e in range(n_distinct):
        base = seed * 1000 + 100 + 3 * e
        g = randn_bf16((cfg.I, cfg.H), w_std, dev, base)
        u = randn_bf16((cfg.I, cfg.H), w_std, dev, base + 1)
        d = randn_bf16((cfg.H, cfg.I), w_std, dev, base + 2)
        if cfg.enc == "bf16":
            sets.append(((g, u, d), (None, None, None)))
        elif cfg.enc == "fp8blk":
            q = [quant_fp8_block128(w) for w in (g, u, d)]
            sets.append((tuple(a for a, _ in q), tuple(s for _, s in q)))
        elif cfg.enc == "mxfp4":
            q = [quant_mxfp4(w) for w in (g, u, d)]
            sets.append((tuple(a for a, _ in q), tuple(s for _, s in q)))
        elif cfg.enc == "fp8pc":
            gu = torch.cat([g, u], dim=0)
            (qgu, sgu), (qd, sd) = quant_fp8_channel(gu), quant_fp8_channel(d)
            sets.append(((qgu, qd), (sgu, sd)))
        else:
            raise ValueError(cfg.enc)
        del g, u, d
    b.experts = sets
    width = 2 if cfg.enc == "fp8pc" else 3
    wt = torch.zeros((Ea, width), dtype=torch.int64)
    st = torch.zeros((Ea, width), dtype=torch.int64)
    for e in range(Ea):
        ws, ss = sets[e % n_distinct]
        for j in range(width):
            wt[e, j] = ws[j].data_ptr()
            st[e, j] = ss[j].data_ptr() if ss[j] is not None else 0
    b.t[wname] = wt.to(dev)
    if sname in plan.slots:
        b.t[sname] = st.to(dev)
    b._table = None
    return b


def to_host(b: Bound) -> Bound:
    """A host twin of a device binding: same bytes, pointer tables rebuilt over the host copies."""
    plan = b.plan
    h = Bound(plan, "cpu")
    for name, t in b.t.items():
        if name not in ("wtab", "stab", "ewt", "est"):
            h.t[name] = t.detach().cpu().clone()
    h.experts = [(tuple(w.cpu() for w in ws), tuple(None if s is None else s.cpu() for s in ss))
                 for ws, ss in b.experts]
    cfg = plan.cfg
    wname, sname = ("ewt", "est") if cfg.enc == "fp8pc" else ("wtab", "stab")
    width = 2 if cfg.enc == "fp8pc" else 3
    wt = torch.zeros((cfg.E_all, width), dtype=torch.int64)
    st = torch.zeros((cfg.E_all, width), dtype=torch.int64)
    nd = len(h.experts)
    for e in range(cfg.E_all):
        ws, ss = h.experts[e % nd]
        for j in range(width):
            wt[e, j] = ws[j].data_ptr()
            st[e, j] = ss[j].data_ptr() if ss[j] is not None else 0
    h.t[wname] = wt
    if sname in plan.slots:
        h.t[sname] = st
    return h
