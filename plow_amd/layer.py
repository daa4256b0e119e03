"""Host-side emitter of one MoE FFN layer as a run of op descriptors.

This mirrors what plow's device-blob emitter produces for a MoE layer (operand wiring of the router
tail + align in crates/devgen/src/mla.rs:11227-11291 and of the GLU / DOWN / combine ops in
crates/devgen/src/k3.rs:1405-1461): a fixed chain

    router score (180) -> router top-k (83) -> align (84) -> [activation quant (184 / 32)]
      -> grouped gate|up + GLU (85 / 81) -> [intermediate quant (32)] -> grouped down (86 / 82)
      -> [dense shared expert (20, 8)] -> combine (87)

over a table of tensor handles. The same descriptors run on the HIP operator (device pointers in the
table) and on the CPU oracle (host pointers), which is how the parity tests compare them.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from . import abi


@dataclass
class MoeConfig:
    name: str
    H: int
    E: int
    I: int
    k: int
    T: int
    scoring: str = "sigmoid"        # or "softmax", "sqrtsoftplus"
    norm_topk: bool = True
    bias: bool = False
    n_group: int = 1
    topk_group: int = 1
    route_scale: float = 1.0
    enc: str = "fp8blk"             # "bf16" | "fp8blk" | "mxfp4" | "fp8pc" (per-channel)
    arm: str = "w8a8"               # "a16" (bf16 activations) | "w8a8" | "w8a8q" (block-fp8 only: the GLU
                                    # quantizes the bf16 rows itself, plow's arm 6; no quantizer op) |
                                    # "w8a8atomic" (block-fp8 only: ops 184, 188, 189, 190 - bf16
                                    # intermediate, slot-major quantized copy, bf16 atomic reduction into
                                    # the output; no combine op, no residual / dense shared expert)
    n_shared: int = 0
    shared_mode: Optional[str] = None  # "fold" (slot {E, 1.0}) | "dense" (ops 20 + 8) | None
    act: int = abi.ACT_SILU
    act_f: Tuple[float, float] = (0.0, 0.0)  # the activation's immediates (fj[0], fj[1]) for the pair forms 2 / 3 / 4
    residual: bool = False
    part_bf16: bool = False         # block-fp8 W8A8 only: bf16 partials (arm 3) instead of f32
    router_raw: bool = False        # the score op carries its top-k (op 180 with the router mark): one launch at decode
    emit_align: bool = True         # False: no op 84 in a chain whose expert ops are table driven (ops 65 / 66 sort the slots
                                    # themselves; plow's decode chain for them is 56 -> 65 -> 66 -> 43)
    det_combine: bool = False       # block-fp8 W8A8 only: the deterministic fused down -> combine (op 83 zeroes a
                                    # [T][H] f64 fixed-point accumulator, op 86 adds into it, op 87 reads it as
                                    # one stream; plow runtime/amd/op_moe.h:2110-2165); no part tensor

    @property
    def tail(self) -> int:
        return 1 if self.shared_mode == "fold" else 0

    @property
    def E_all(self) -> int:      # experts the align / grouped ops see
        return self.E + self.tail

    @property
    def k_all(self) -> int:
        return self.k + self.tail

    @property
    def I_shared(self) -> int:
        return self.I * self.n_shared

    @property
    def R_max(self) -> int:
        return abi.max_rows(self.T, self.k_all, self.E_all)

    @property
    def flags(self) -> int:
        f = abi.ROUTE_F32_LOGIT
        if self.scoring == "sigmoid":
            f |= abi.ROUTE_SIGMOID
        if self.scoring == "sqrtsoftplus":
            f |= abi.ROUTE_SQRT_SOFTPLUS
        if self.norm_topk:
            f |= abi.ROUTE_NORM_TOPK
        if self.bias:
            f |= abi.ROUTE_BIAS
        return f


# The five benchmark configurations (shapes of the reference's headline cells).
def config(name: str, T: Optional[int] = None) -> MoeConfig:
    if name == "c1":   # small bf16 layer runnable on plow's CPU path
        return MoeConfig("c1", H=2048, E=64, I=1408, k=6, T=T or 16, scoring="softmax",
                         norm_topk=False, enc="bf16", arm="a16", n_shared=2, shared_mode="dense")
    if name in ("c2", "c3"):  # DeepSeek-V3-shaped block-fp8
        return MoeConfig(name, H=7168, E=256, I=2048, k=8, T=T or (64 if name == "c2" else 4096),
                         scoring="sigmoid", norm_topk=True, bias=True, n_group=8, topk_group=4,
                         route_scale=2.5, enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold")
    if name == "c4":   # Kimi-K2-shaped mxfp4, bf16 activations
        return MoeConfig("c4", H=7168, E=384, I=2048, k=8, T=T or 16, scoring="sigmoid",
                         norm_topk=True, bias=True, route_scale=2.827, enc="mxfp4", arm="a16",
                         n_shared=1, shared_mode="fold")
    if name == "c5":   # Qwen3-MoE-shaped per-channel fp8, no shared expert
        return MoeConfig("c5", H=4096, E=128, I=1536, k=8, T=T or 64, scoring="softmax",
                         norm_topk=True, enc="fp8pc", arm="a16")
    if name == "c6":   # GLM-5.3-Flash-shaped block-fp8, one rank's slice of TP8 (the shape of plow's
        # own gfx950 prefill bench, runtime/bench/amd/moe_fp8_pf_bench.hip:1-7)
        return MoeConfig("c6", H=4096, E=288, I=256, k=8, T=T or 8192, scoring="sigmoid",
                         norm_topk=True, bias=True, enc="fp8blk", arm="w8a8")
    raise KeyError(name)


@dataclass
class TensorSpec:
    dtype: str                 # "bf16" "f32" "u8" "i32" "u32" "u64" "route"
    shape: Tuple[int, ...]
    role: str                  # "in" | "weight" | "scratch" | "out" | "table"


@dataclass
class LayerPlan:
    cfg: MoeConfig
    slots: Dict[str, int] = field(default_factory=dict)
    specs: Dict[str, TensorSpec] = field(default_factory=dict)
    insts: List[abi.PlowDevInst] = field(default_factory=list)
    names: List[str] = field(default_factory=list)   # one label per instruction

    def _t(self, name: str, dtype: str, shape, role: str) -> int:
        if name not in self.slots:
            self.slots[name] = len(self.slots)
            self.specs[name] = TensorSpec(dtype, tuple(int(s) for s in shape), role)
        return self.slots[name]

    def _emit(self, label: str, d: abi.PlowDevInst):
        self.insts.append(d)
        self.names.append(label)

    def index(self, label: str) -> int:
        return self.names.index(label)


def plan_layer(cfg: MoeConfig, with_router_score: bool = True) -> LayerPlan:
    """Emit the op chain of one layer. Returns the plan: descriptors + the tensor slots to bind."""
    p = LayerPlan(cfg)
    T, H, E, I, k = cfg.T, cfg.H, cfg.E, cfg.I, cfg.k
    Ea, ka, R = cfg.E_all, cfg.k_all, cfg.R_max
    x = p._t("x", "bf16", (T, H), "in")
    wr = p._t("Wr", "bf16", (E, H), "weight")
    logit = p._t("logit", "f32", (T, E), "scratch")
    bias = p._t("bias", "f32", (E,), "weight") if cfg.bias else None
    table = p._t("table", "route", (T * ka,), "scratch")
    meta = p._t("meta", "i32", (3 * Ea + 1,), "scratch")
    row_token = p._t("row_token", "u32", (R,), "scratch")
    row_partidx = p._t("row_partidx", "u32", (R,), "scratch")
    row_gate = p._t("row_gate", "f32", (R,), "scratch")
    p16 = cfg.part_bf16 and ((cfg.enc == "fp8blk" and cfg.arm in ("w8a8", "w8a8q", "w8a8split")) or
                             (cfg.enc == "mxfp4" and cfg.arm == "a4w4"))
    det = cfg.det_combine and cfg.enc == "fp8blk" and cfg.arm in ("w8a8", "w8a8q")
    assert not (det and p16)
    part = (p._t("acc64", "f64", (T, H), "scratch") if det
            else p._t("part", "bf16" if p16 else "f32", (T * ka, H), "scratch"))
    out = p._t("out", "bf16", (T, H), "out")
    residual = p._t("residual", "bf16", (T, H), "in") if cfg.residual else None

    if cfg.router_raw:
        # plow's raw router segment (crates/devgen/src/mla.rs:3294-3312): per-row arrival counters, 128 bytes apart
        assert with_router_score and not det
        ctr = p._t("router_ctr", "u32", (T * 32,), "scratch")
        p._emit("score", abi.inst(abi.OP_GEMM_F32, t=[logit, x, wr, table, bias, ctr],
                                  i=[T, E, H, k, cfg.flags, cfg.tail, cfg.n_group | (cfg.topk_group << 16),
                                     abi.ROUTER_RAW_MARK], f=[cfg.route_scale, 0.0]))
    elif with_router_score:
        p._emit("score", abi.inst(abi.OP_GEMM_F32, t=[logit, x, wr], i=[T, E, H]))
    if not cfg.router_raw:
        p._emit("topk", abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[table, logit, part if det else None, bias],
                                 i=[H if det else 0, E, k, cfg.flags, T, cfg.tail, cfg.n_group, cfg.topk_group],
                                 f=[cfg.route_scale, 0.0]))
    slot_major = (cfg.enc == "fp8pc" and cfg.arm != "w8a8") or cfg.arm == "a16dec"
    if cfg.emit_align or not slot_major:
        p._emit("align", abi.inst(abi.OP_MOE_ALIGN_PF, t=[meta, table, row_token, row_partidx, row_gate],
                                  i=[T, Ea, ka]))

    if cfg.enc == "fp8pc":
        ewt = p._t("ewt", "u64", (Ea, 2), "table")
        est = p._t("est", "u64", (Ea, 2), "table")
        if cfg.arm == "w8a8":
            xq = p._t("xq", "u8", (T, H), "scratch")
            ascale = p._t("ascale", "f32", (T,), "scratch")
            fu = p._t("fu", "bf16", (R, I), "scratch")
            fu8 = p._t("fu8", "u8", (R, I), "scratch")
            fscale = p._t("fscale", "f32", (R,), "scratch")
            p._emit("quant_x", abi.inst(abi.OP_QUANT_FP8, t=[xq, x, ascale], i=[T, H]))
            p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_GEMMA_PF_W8A8,
                                    t=[fu, xq, ewt, meta, row_token, ascale, est],
                                    i=[I, H, Ea, 0, 0, cfg.act], slots=T * ka))
            p._emit("quant_fu", abi.inst(abi.OP_QUANT_FP8, t=[fu8, fu, fscale], i=[R, I]))
            p._emit("down", abi.inst(abi.OP_MOE_GROUP_DOWN_GEMMA_PF_W8A8,
                                     t=[part, fu8, ewt, meta, row_partidx, row_gate, est, fscale],
                                     i=[H, I, Ea], slots=T * ka))
        else:
            # per-channel fp8 weights with bf16 activations: the decode ops 65/66, table driven.
            fu = p._t("fu", "bf16", (T * ka, I), "scratch")
            p._emit("glu", abi.inst(abi.OP_MOE_EXPERT_GLU_GEMMA_FP8, t=[fu, x, table, ewt, est],
                                    i=[ka, I, H, Ea, 0, T, cfg.act]))
            p._emit("down", abi.inst(abi.OP_MOE_EXPERT_DOWN_GEMMA_FP8, t=[part, fu, table, ewt, est],
                                     i=[ka, H, I, Ea, 0, T]))
    else:
        enc = {"bf16": abi.ENC_BF16, "fp8blk": abi.ENC_FP8BLK, "mxfp4": abi.ENC_MXFP4}[cfg.enc]
        wtab = p._t("wtab", "u64", (Ea, 3), "table")
        stab = p._t("stab", "u64", (Ea, 3), "table") if enc != abi.ENC_BF16 else None
        if cfg.arm == "a16dec":
            # plow's decode experts (ops 48 / 49): bf16 activations, table driven, slot-major rows, no op 84
            fu = p._t("fu", "bf16", (T * ka, I), "scratch")
            p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[fu, x, table, wtab, stab],
                                    i=[T * ka, I, H, Ea, ka, cfg.act, enc]))
            p._emit("down", abi.inst(abi.OP_MOE_GROUP_DOWN_FP8_BLK, t=[part, fu, table, wtab, stab],
                                     i=[T * ka, H, I, Ea, 0, 0, enc]))
        elif enc == abi.ENC_FP8BLK and cfg.arm == "w8a8atomic":
            assert cfg.shared_mode != "dense" and not cfg.residual, "the atomic chain has no combine op"
            xq = p._t("xq", "u8", (T, H), "scratch")
            xs = p._t("xs", "f32", (H // 128, T), "scratch")
            fu = p._t("fu", "bf16", (R, I), "scratch")
            hq = p._t("hq", "u8", (T * ka, I), "scratch")
            hs = p._t("hs", "f32", (I // 128, T * ka), "scratch")
            p._emit("quant_x", abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[xq, x, xs], i=[T, H]))
            p._emit("glu", abi.inst(abi.OP_MOE_GLU_FP8_BLOCK128, t=[fu, xq, xs, wtab, stab, meta, row_token],
                                    i=[I, H, Ea, T], f=[0.0, cfg.act_f[1] if cfg.act == 4 else 0.0], slots=T * ka))
            p._emit("quant_fu", abi.inst(abi.OP_MOE_QUANT_FP8_BLOCK128, t=[hq, fu, hs, meta, row_partidx, out],
                                         i=[I, Ea, ka, T, H]))
            p._emit("down", abi.inst(abi.OP_MOE_DOWN_FP8_BLOCK128,
                                     t=[out, hq, hs, wtab, stab, meta, row_partidx, row_gate],
                                     i=[I, H, Ea, ka, T], slots=T * ka))
            return p
        if cfg.arm == "a16dec":
            pass
        elif enc == abi.ENC_FP8BLK and cfg.arm in ("w8a8", "w8a8q", "w8a8split"):
            two = cfg.arm == "w8a8split"   # two e4m3 terms per value: rows [hi I | lo I]
            fq = p._t("fq", "u8", (R, 2 * I if two else I), "scratch")
            fs = p._t("fs", "f32", (R, I // 128), "scratch")
            if two:
                assert not det, "the deterministic combine is the plain arm's"
                p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_PF,
                                        t=[fq, x, wtab, stab, meta, row_token, None, fs],
                                        i=[I, H, Ea, enc, T, cfg.act, 0, abi.ARM_W8A8_SPLIT], f=cfg.act_f, slots=T * ka))
            elif cfg.arm == "w8a8q":
                p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_PF,
                                        t=[fq, x, wtab, stab, meta, row_token, None, fs],
                                        i=[I, H, Ea, enc, T, cfg.act, 0, abi.ARM_W8A8_XQ], f=cfg.act_f, slots=T * ka))
            else:
                xq = p._t("xq", "u8", (T, H), "scratch")
                xs = p._t("xs", "f32", (H // 128, T), "scratch")
                p._emit("quant_x", abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[xq, x, xs], i=[T, H, T]))
                p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_PF,
                                        t=[fq, xq, wtab, stab, meta, row_token, xs, fs],
                                        i=[I, H, Ea, enc, T, cfg.act, 0, abi.ARM_W8A8], f=cfg.act_f, slots=T * ka))
            p._emit("down", abi.inst(abi.OP_MOE_GROUP_DOWN_PF,
                                     t=[part, fq, wtab, stab, meta, fs, row_partidx, row_gate],
                                     i=[H, I, Ea, enc, 0, (256 + ka) if det else 0, 0,
                                        (abi.ARM_W8A8_SPLIT_P16 if p16 else abi.ARM_W8A8_SPLIT) if two
                                        else (abi.ARM_W8A8_P16 if p16 else abi.ARM_W8A8)], slots=T * ka))
        elif enc == abi.ENC_MXFP4 and cfg.arm == "a4w4":
            # fp4 on both operands: the GLU quantizes its bf16 rows per 32 and writes the intermediate as
            # mxfp4 with E8M0 rows; i4 = T (the rows of x) is what this library's quantizer pass needs
            fu4 = p._t("fu4", "u8", (R, I // 2), "scratch")
            fsc = p._t("fsc", "u8", (R, I // 32), "scratch")
            p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_PF,
                                    t=[fu4, x, wtab, stab, meta, row_token, row_partidx, fsc],
                                    i=[I, H, Ea, enc, T, cfg.act, 0, abi.ARM_A4W4], f=cfg.act_f, slots=T * ka))
            p._emit("down", abi.inst(abi.OP_MOE_GROUP_DOWN_PF,
                                     t=[part, fu4, wtab, stab, meta, fsc, row_partidx, row_gate],
                                     i=[H, I, Ea, enc, 0, 0, 0, abi.ARM_A4W4_P16 if p16 else abi.ARM_A4W4],
                                     slots=T * ka))
        else:
            arm = abi.ARM_W4A16 if enc == abi.ENC_MXFP4 else abi.ARM_A16
            fu = p._t("fu", "bf16", (R, I), "scratch")
            p._emit("glu", abi.inst(abi.OP_MOE_GROUP_GLU_PF,
                                    t=[fu, x, wtab, stab, meta, row_token],
                                    i=[I, H, Ea, enc, 0, cfg.act, 0, arm], f=cfg.act_f, slots=T * ka))
            p._emit("down", abi.inst(abi.OP_MOE_GROUP_DOWN_PF,
                                     t=[part, fu, wtab, stab, meta, None, row_partidx, row_gate],
                                     i=[H, I, Ea, enc, 0, 0, 0, arm], slots=T * ka))

    shared = None
    if cfg.shared_mode == "dense":
        Is = cfg.I_shared
        wsg = p._t("Ws_gate", "bf16", (Is, H), "weight")
        wsu = p._t("Ws_up", "bf16", (Is, H), "weight")
        wsd = p._t("Ws_down", "bf16", (H, Is), "weight")
        sfu = p._t("shared_fu", "bf16", (T, Is), "scratch")
        shared = p._t("shared", "bf16", (T, H), "scratch")
        p._emit("shared_glu", abi.inst(abi.OP_GEMM_GLU, t=[sfu, x, wsg, None, None, wsu],
                                       i=[T, Is, H, 0, 0, cfg.act]))
        p._emit("shared_down", abi.inst(abi.OP_GEMM, t=[shared, sfu, wsd], i=[T, H, Is]))
    p._emit("combine", abi.inst(abi.OP_MOE_COMBINE_PF, t=[out, residual, shared, part],
                                i=[H, 1 if det else ka, T, 0, 1 if det else 0, 0, 0, 1 if p16 else 0]))
    return p
