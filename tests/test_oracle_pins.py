"""Pins for the parts of the oracle that plow's CPU kernels cannot replay (tests/test_golden.py
covers the rest): number formats, group-limited routing, the 1x128 activation quant and the
block-fp8 arms. Each check is independent of the oracle's own formula: a closed form, a library
routine (torch float8 / bfloat16 casts, integer matmul), brute force, or an invariant."""
import numpy as np
import pytest
import torch

import cases
import oracle_lib as ol
from plow_amd import abi


def run(oracle, inst, arrays, nthreads=1):
    ol.run(oracle.plow_oracle_exec, inst, ol.table_of(arrays), nthreads)


# ---- number formats ------------------------------------------------------------------------------

def test_bf16_round_matches_torch(oracle):
    r = cases.rng_of(1)
    v = np.concatenate([r.standard_normal(20000).astype(np.float32) * 10.0 ** r.integers(-20, 20, 20000),
                        # exact ties and their neighbours around every rounding boundary
                        (np.arange(0x3F800000, 0x3F800000 + 0x40000, 0x4000, dtype=np.uint32) + 0x8000).view(np.float32),
                        (np.arange(0x3F800000, 0x3F800000 + 0x40000, 0x4000, dtype=np.uint32) + 0x7FFF).view(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38, 1e-40], np.float32)]).astype(np.float32)
    got = np.zeros(v.size, np.uint16)
    oracle.plow_oracle_f2bf_n(got.ctypes.data, np.ascontiguousarray(v).ctypes.data, v.size)
    want = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(ol.f2bf(v), want)
    nan = oracle.plow_oracle_f2bf(float("nan"))
    assert (nan & 0x7F80) == 0x7F80 and (nan & 0x7F) != 0


def test_e4m3_decode_table_matches_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = np.array([oracle.plow_oracle_e4m3_to_f32(int(c)) for c in codes], np.float32)
    fin = np.isfinite(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    assert np.isnan(got[0x7F]) and np.isnan(got[0xFF]) and fin.sum() == 254
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def test_e4m3_encode_is_nearest_even_by_brute_force(oracle):
    codes = np.array([c for c in range(128) if c != 0x7F], np.uint8)
    grid = np.array([oracle.plow_oracle_e4m3_to_f32(int(c)) for c in codes], np.float64)
    r = cases.rng_of(2)
    mids = (grid[:-1] + grid[1:]) / 2
    v = np.concatenate([r.standard_normal(4000) * 10.0 ** r.integers(-4, 3, 4000), mids,
                        np.nextafter(mids.astype(np.float32), np.float32(0)),
                        np.nextafter(mids.astype(np.float32), np.float32(1e9)), grid,
                        [447.9, 448.0, 463.9, 464.0, 1e9, 1e-12, 0.0]]).astype(np.float32)
    v = np.concatenate([v, -v])
    got = np.zeros(v.size, np.uint8)
    oracle.plow_oracle_e4m3_encode_n(got.ctypes.data, np.ascontiguousarray(v).ctypes.data, v.size)
    for x, c in zip(v, got):
        a = abs(float(x))
        if a >= 448.0:
            want = 0x7E
        else:
            d = np.abs(grid - a)
            best = np.flatnonzero(d == d.min())
            want = int(codes[best[0]]) if len(best) == 1 else int(codes[[b for b in best if codes[b] % 2 == 0][0]])
        assert (c & 0x7F) == want, (x, hex(c), hex(want))
        assert (c >> 7) == (1 if np.signbit(x) else 0)
    # the same answers from torch's cast wherever it is defined without saturation
    inr = np.abs(v) < 448.0
    tq = torch.from_numpy(v[inr]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(tq, got[inr])
    assert oracle.plow_oracle_f32_to_e4m3(float("nan")) & 0x7F == 0x7F
    assert oracle.plow_oracle_f32_to_e4m3(float("inf")) == 0x7E


def test_e2m1_and_e8m0_closed_forms(oracle):
    mags = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for n in range(16):
        v = oracle.plow_oracle_e2m1(n)
        assert abs(v) == mags[n & 7] and (np.signbit(v) == bool(n & 8))
    assert oracle.plow_oracle_e8m0(0) == 0.0 and np.isinf(oracle.plow_oracle_e8m0(255))
    for s in range(1, 255):
        assert oracle.plow_oracle_e8m0(s) == 2.0 ** (s - 127)


# ---- routing: closed forms and invariants --------------------------------------------------------

def route(oracle, logit, bias, E, k, flags, **kw):
    T = logit.shape[0]
    tail = kw.get("tail", 0)
    table = np.zeros(T * (k + tail), dtype=ol.ROUTE_DT)
    run(oracle, cases.route_inst(E, k, T, flags, bias is not None, **kw), [table, logit, None, bias])
    return table.reshape(T, k + tail)


def test_all_equal_logits_pick_lowest_ids(oracle):
    lg = np.full((3, 40), 0.25, np.float32)
    for flags in (8, 8 | 1, 8 | 2):
        tab = route(oracle, lg, None, 40, 6, flags, route_scale=1.0)
        assert np.array_equal(tab["eid"], np.tile(np.arange(6, dtype=np.uint32), (3, 1)))


def test_softmax_norm_gates_sum_to_scale(oracle):
    lg = (cases.rng_of(3).standard_normal((50, 128)) * 3).astype(np.float32)
    tab = route(oracle, lg, None, 128, 8, 8 | 2, route_scale=1.0)
    assert np.allclose(tab["gate"].sum(1), 1.0, atol=1e-6)
    tab = route(oracle, lg, None, 128, 8, 8 | 2, route_scale=2.5)
    assert np.allclose(tab["gate"].sum(1), 2.5, atol=1e-5)


def test_flat_selection_is_descending_argsort(oracle):
    r = cases.rng_of(4)
    for E, k in ((7, 3), (16, 16), (130, 8)):
        lg = r.standard_normal((20, E)).astype(np.float32)
        bias = (r.standard_normal(E) * 0.3).astype(np.float32)
        tab = route(oracle, lg, bias, E, k, 8 | 1 | 4, route_scale=1.0)
        score = (1.0 / (1.0 + np.exp(-lg.astype(np.float64)))).astype(np.float32)
        sel = score + bias
        for t in range(20):
            order = sorted(range(E), key=lambda e: (-sel[t, e], e))[:k]
            assert list(tab["eid"][t]) == order
            # gates are the UNBIASED scores (to libm rounding), not the selection values
            assert np.allclose(tab["gate"][t], score[t, order], rtol=1e-6)


def test_sqrt_softplus_scores_and_selection(oracle):
    """Flag bit 5: score = sqrt(softplus(logit)), checked against float64 (the gate of an un-normalized, unscaled
    table is the score itself), selection = descending argsort of score + bias, bit 0 ignored beside it, and the
    closed-form ends: softplus(l) -> l for large l, -> exp(l) for very negative l, softplus(0) = ln 2."""
    r = cases.rng_of(41)
    E, k, T = 96, 8, 30
    lg = (r.standard_normal((T, E)) * 4).astype(np.float32)
    bias = (r.standard_normal(E) * 0.2).astype(np.float32)
    ref = np.sqrt(np.logaddexp(0.0, lg.astype(np.float64)))
    tab = route(oracle, lg, bias, E, k, 8 | 4 | 32, route_scale=1.0)
    sel = ref.astype(np.float32) + bias
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-sel[t, e], e))[:k]
        assert list(tab["eid"][t]) == order
        assert np.allclose(tab["gate"][t], ref[t, order], rtol=3e-7, atol=0)
    both = route(oracle, lg, bias, E, k, 8 | 4 | 32 | 1, route_scale=1.0)
    assert np.array_equal(both.view(np.uint8), tab.view(np.uint8))
    sig = route(oracle, lg, bias, E, k, 8 | 4 | 1, route_scale=1.0)
    assert not np.array_equal(sig["gate"], tab["gate"])
    ends = np.array([[0.0, 30.0, 100.0, -30.0, -100.0, 3e38, -3e38, np.inf, -np.inf, 1.0]], np.float32)
    e = route(oracle, ends, None, 10, 10, 8 | 32, route_scale=1.0)
    got = dict(zip(e["eid"][0].tolist(), e["gate"][0].tolist()))
    assert got[0] == np.float32(np.sqrt(np.log(2.0)))
    assert got[1] == np.float32(np.sqrt(30.0)) and got[2] == np.float32(10.0)
    assert np.isclose(got[3], np.exp(-15.0), rtol=1e-6) and got[4] == 0.0   # exp(-100) is below the f32 range
    assert got[5] == np.float32(np.sqrt(np.float64(np.float32(3e38)))) and got[6] == 0.0
    assert got[7] == np.inf and got[8] == 0.0
    norm = route(oracle, lg, bias, E, k, 8 | 4 | 32 | 2, route_scale=2.0)
    assert np.allclose(norm["gate"].sum(1), 2.0, rtol=1e-5)


def test_logit_scale_and_shared_tail(oracle):
    lg = (cases.rng_of(5).standard_normal((6, 32))).astype(np.float32)
    a = route(oracle, lg * np.float32(0.5), None, 32, 4, 8 | 1)
    b = route(oracle, lg, None, 32, 4, 8 | 1, logit_scale=0.5)
    assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    c = route(oracle, lg * np.float32(0.5), None, 32, 4, 8 | 1, tail=1)
    assert np.array_equal(c[:, :4].copy().view(np.uint8), a.view(np.uint8))
    assert np.all(c["eid"][:, 4] == 32) and np.all(c["gate"][:, 4] == 1.0)


def noaux_tc(score, bias, k, n_group, topk_group):
    """Independent restatement of group-limited selection in the DeepSeek-V3 modelling code's terms:
    mask whole groups, then a plain top-k over what is left."""
    sel = score + bias
    E = sel.shape[0]
    gs = np.sort(sel.reshape(n_group, -1), axis=1)[:, -2:]
    gscore = (gs[:, 1] + gs[:, 0]).astype(np.float32)      # m1 + m2 in f32
    keep = sorted(range(n_group), key=lambda g: (-gscore[g], g))[:topk_group]
    masked = np.full(E, -np.inf)
    for g in keep:
        lo = g * (E // n_group)
        masked[lo:lo + E // n_group] = sel[lo:lo + E // n_group]
    return sorted(range(E), key=lambda e: (-masked[e], e))[:k], set(keep)


@pytest.mark.parametrize("E,k,ng,tg", [(256, 8, 8, 4), (64, 6, 4, 2), (128, 8, 8, 1), (288, 8, 18, 2)])
def test_group_limited_selection(oracle, E, k, ng, tg):
    r = cases.rng_of(6)
    T = 40
    lg = (r.standard_normal((T, E)) * 1.5).astype(np.float32)
    bias = (r.standard_normal(E) * 0.1).astype(np.float32)
    tab = route(oracle, lg, bias, E, k, 8 | 1 | 2 | 4, n_group=ng, topk_group=tg)
    flat = route(oracle, lg, bias, E, k, 8 | 1 | 2 | 4)
    # the scores the oracle used are those of the flat arm, which plow's CPU kernel pins bit for bit
    score = np.zeros((T, E), np.float32)
    full = route(oracle, lg, None, E, 16, 8 | 1, route_scale=1.0)  # probe: unbiased scores of top 16
    differs = 0
    for t in range(T):
        sc = (1.0 / (1.0 + np.exp(-lg[t].astype(np.float64)))).astype(np.float32)
        sc[full["eid"][t]] = full["gate"][t]            # exact libm bits where we have them
        score[t] = sc
        want, keep = noaux_tc(sc, bias, k, ng, tg)
        got = list(tab["eid"][t])
        assert {e // (E // ng) for e in got} <= keep    # every winner lies in a kept group
        assert got == want
        differs += got != list(flat["eid"][t])
    assert differs > 0                                   # the mask really changes the selection
    for off in ((1, 0), (0, 0), (ng, tg and ng)):        # inactive shapes are the flat arm exactly
        same = route(oracle, lg, bias, E, k, 8 | 1 | 2 | 4, n_group=off[0], topk_group=off[1])
        assert np.array_equal(same.view(np.uint8), flat.view(np.uint8))


def test_align_structure(oracle):
    r = cases.rng_of(7)
    T, E, k = 200, 24, 4
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["eid"][r.choice(T * k, 30, replace=False)] = abi.EXPERT_UNUSED
    tab["gate"] = r.random(T * k).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    meta, rt, rp, rg = al[0], al[2], al[3], al[4]
    rowoff, cnt, tilep = meta[:E], meta[E:2 * E], meta[2 * E:]
    live = tab["eid"] < E
    assert cnt.sum() == live.sum()
    assert np.array_equal(cnt, np.bincount(tab["eid"][live], minlength=E))
    assert np.array_equal(rowoff, 64 * tilep[:E]) and tilep[E] == ((cnt + 63) // 64).sum()
    for e in range(E):
        seg = rp[rowoff[e]:rowoff[e] + cnt[e]]
        assert np.array_equal(seg, np.flatnonzero(tab["eid"] == e))      # ascending slot order
        assert np.array_equal(rt[rowoff[e]:rowoff[e] + cnt[e]], seg // k)
        assert np.array_equal(rg[rowoff[e]:rowoff[e] + cnt[e]], tab["gate"][seg])
        pad = slice(rowoff[e] + cnt[e], rowoff[e] + 64 * ((cnt[e] + 63) // 64))
        assert np.all(rt[pad] == abi.EXPERT_UNUSED) and np.all(rp[pad] == abi.EXPERT_UNUSED)
        assert np.all(rg[pad] == 0.0)


# ---- 1x128 activation quant ----------------------------------------------------------------------

def test_quant_block128_closed_form(oracle):
    r = cases.rng_of(8)
    M, K, pitch = 5, 384, 9
    x = cases.randn_bf16(r, (M, K), 2.0)
    x[2, 128:256] = 0                                   # all-zero group: amax floor 1e-10
    xq, xs = np.zeros((M, K), np.uint8), np.full((K // 128, pitch), -1.0, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[M, K, pitch]), [xq, x, xs], 2)
    xf = ol.bf2f(x).reshape(M, K // 128, 128)
    amax = np.maximum(np.abs(xf).max(2), np.float32(1e-10))
    s = (amax * np.float32(1.0 / 448.0)).astype(np.float32)
    assert np.array_equal(xs[:, :M].T.view(np.uint32), s.view(np.uint32)) and np.all(xs[:, M:] == -1.0)
    inv = (np.float32(1.0) / s).astype(np.float32)
    want = torch.from_numpy((xf * inv[:, :, None]).astype(np.float32).clip(-448, 448)).to(
        torch.float8_e4m3fn).view(torch.uint8).numpy().reshape(M, K)
    assert np.array_equal(xq, want)
    # decode(q) * s reproduces x to within half an e4m3 step of the group's amax
    deq = torch.from_numpy(xq).view(torch.float8_e4m3fn).float().numpy().reshape(M, K // 128, 128) * s[:, :, None]
    assert np.all(np.abs(deq - xf) <= amax[:, :, None] * (0.0625 / 1.75 + 1e-6))


# ---- block-fp8 experts ----------------------------------------------------------------------------

def identity_align(T, E_of_row, E):
    """Row maps for hand-made segments: token t is routed (k = 1) to expert E_of_row[t]."""
    tab = np.zeros(T, dtype=ol.ROUTE_DT)
    tab["eid"], tab["gate"] = E_of_row, 1.0
    return tab


def build_fp8(oracle, r, E, T, H, I, small_int, scales_one):
    """Tiny block-fp8 layer, k = 1. small_int: payloads are the integers -3..3 (exact in e4m3)."""
    def payload(shape):
        if small_int:
            v = r.integers(-3, 4, size=shape).astype(np.float32)
            b = np.zeros(v.size, np.uint8)
            oracle.plow_oracle_e4m3_encode_n(b.ctypes.data, np.ascontiguousarray(v).ctypes.data, v.size)
            return b.reshape(shape), v
        b = cases.e4m3_bytes(r, shape)
        v = torch.from_numpy(b).view(torch.float8_e4m3fn).float().numpy()
        return b, v
    W = {n: [payload(s) for _ in range(E)] for n, s in (("g", (I, H)), ("u", (I, H)), ("d", (H, I)))}
    def grid(N, K):
        g = np.ones((N // 128, K // 128), np.float32)
        return g if scales_one else (r.random(g.shape) * 0.02 + 0.001).astype(np.float32)
    S = {n: [grid(*s) for _ in range(E)] for n, s in (("g", (I, H)), ("u", (I, H)), ("d", (H, I)))}
    wtab = np.array([[W[n][e][0].ctypes.data for n in "gud"] for e in range(E)], dtype=np.uint64)
    stab = np.array([[S[n][e].ctypes.data for n in "gud"] for e in range(E)], dtype=np.uint64)
    return W, S, wtab, stab


def dequant(Wv, S):
    return Wv.astype(np.float64) * np.kron(S.astype(np.float64), np.ones((128, 128)))


@pytest.mark.parametrize("arm", [abi.ARM_A16, abi.ARM_W8A8])
def test_fp8blk_unit_scales_small_integers_is_exact_integer_gemm(oracle, arm):
    """All scales 1 and integer payloads: every partial sum is an integer below 2^24, so the DOWN
    arm must equal an integer matmul exactly, whatever the summation order."""
    r = cases.rng_of(9)
    E, T, H, I = 3, 7, 256, 128
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, True, True)
    eids = r.integers(0, E, T).astype(np.uint32)
    tab = identity_align(T, eids, E)
    tab["gate"] = r.integers(1, 4, T).astype(np.float32)
    al = cases.align_arrays(tab, T, E, 1)
    run(oracle, cases.align_inst(T, E, 1), al)
    R = al[2].shape[0]
    fi = r.integers(-3, 4, size=(R, I)).astype(np.float32)
    part = np.zeros((T, H), np.float32)
    if arm == abi.ARM_A16:
        fu = ol.f2bf(fi)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[H, I, E, 1, 0, 0, 0, 0]),
            [part, fu, wtab, stab, al[0], None, al[3], al[4]], 2)
    else:
        fq = np.zeros(fi.size, np.uint8)
        oracle.plow_oracle_e4m3_encode_n(fq.ctypes.data, np.ascontiguousarray(fi).ctypes.data, fi.size)
        fs = np.ones((R, I // 128), np.float32)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E, 1, 0, 0, 0, 2]),
            [part, fq.reshape(R, I), wtab, stab, al[0], fs, al[3], al[4]], 2)
    for row in range(int(al[0][-1]) * 64):
        t = al[3][row]
        if t == abi.EXPERT_UNUSED:
            continue
        e = eids[t]
        want = tab["gate"][t] * (W["d"][e][1].astype(np.int64) @ fi[row].astype(np.int64))
        assert np.array_equal(part[t], want.astype(np.float32))


def test_fp8blk_one_hot_activation_reads_back_a_dequantized_column(oracle):
    r = cases.rng_of(10)
    E, H, I = 2, 256, 128
    W, S, wtab, stab = build_fp8(oracle, r, E, 4, H, I, False, False)
    T = 4
    hot = [3, 130, 200, 255]
    x = np.zeros((T, H), np.float32)
    x[np.arange(T), hot] = 1.0
    eids = np.array([0, 1, 1, 0], np.uint32)
    tab = identity_align(T, eids, E)
    al = cases.align_arrays(tab, T, E, 1)
    run(oracle, cases.align_inst(T, E, 1), al)
    R = al[2].shape[0]
    part = np.zeros((T, I), np.float32)
    # use the GATE matrix as a "down" matrix of shape [I][H] so that the output is its column
    wt2 = wtab.copy(); st2 = stab.copy()
    wt2[:, 2], st2[:, 2] = wtab[:, 0], stab[:, 0]
    xr = np.zeros((R, H), np.uint16)
    for row in range(int(al[0][-1]) * 64):
        if al[3][row] != abi.EXPERT_UNUSED:
            xr[row] = ol.f2bf(x[al[3][row]])
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[I, H, E, 1, 0, 0, 0, 0]),
        [part, xr, wt2, st2, al[0], None, al[3], al[4]])
    for t in range(T):
        col = dequant(W["g"][eids[t]][1], S["g"][eids[t]])[:, hot[t]]
        assert np.array_equal(part[t], col.astype(np.float32))


@pytest.mark.parametrize("arm", [abi.ARM_A16, abi.ARM_W8A8])
def test_fp8blk_layer_against_f64_over_the_same_bytes(oracle, arm):
    """GLU -> DOWN at a small shape vs an f64 evaluation of the same quantized operands. The W8A8 arm
    re-derives its own intermediate quantization from the oracle's fq / fs (so that only the GEMM
    arithmetic is under test here; the quant rule is pinned above)."""
    r = cases.rng_of(11)
    E, T, H, I, k = 4, 9, 256, 256, 2
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, False, False)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    R = al[2].shape[0]
    x = cases.randn_bf16(r, (T, H), 1.0)
    part = np.zeros((T * k, H), np.float32)
    silu = lambda g: g / (1.0 + np.exp(-g))
    if arm == abi.ARM_A16:
        fu = np.zeros((R, I), np.uint16)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5], i=[I, H, E, 1, 0, 1, 0, 0]),
            [fu, x, wtab, stab, al[0], al[2]], 2)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[H, I, E, 1, 0, 0, 0, 0]),
            [part, fu, wtab, stab, al[0], None, al[3], al[4]], 2)
        xa = ol.bf2f(x).astype(np.float64)
        fa = ol.bf2f(fu).astype(np.float64)
    else:
        xq, xs = np.zeros((T, H), np.uint8), np.zeros((H // 128, T), np.float32)
        run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[T, H, T]), [xq, x, xs])
        fq, fs = np.zeros((R, I), np.uint8), np.zeros((R, I // 128), np.float32)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[I, H, E, 1, T, 1, 0, 2]),
            [fq, xq, wtab, stab, al[0], al[2], xs, fs], 2)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E, 1, 0, 0, 0, 2]),
            [part, fq, wtab, stab, al[0], fs, al[3], al[4]], 2)
        xa = torch.from_numpy(xq).view(torch.float8_e4m3fn).double().numpy() * np.repeat(xs.T.astype(np.float64), 128, axis=1)
        fa = torch.from_numpy(fq).view(torch.float8_e4m3fn).double().numpy() * np.repeat(fs.astype(np.float64), 128, axis=1)
    for row in range(int(al[0][-1]) * 64):
        s = al[3][row]
        if s == abi.EXPERT_UNUSED:
            continue
        e, t = tab["eid"][s], s // k
        g = dequant(W["g"][e][1], S["g"][e]) @ xa[t]
        u = dequant(W["u"][e][1], S["u"][e]) @ xa[t]
        v = silu(g) * u
        # the stored intermediate (bf16, or e4m3 x scale) is the f64 value to format precision
        tol = 2.0 ** -8 if arm == abi.ARM_A16 else 2.0 ** -4
        assert np.all(np.abs(fa[row] - v) <= tol * np.abs(v).max() + 1e-6)
        y = tab["gate"][s] * (dequant(W["d"][e][1], S["d"][e]) @ fa[row])
        assert np.allclose(part[s], y, rtol=2e-5, atol=2e-5 * np.abs(y).max())


def test_fp8blk_two_term_arms_against_f64_over_bf16_activations(oracle):
    """Arms 4 (GLU) and 4 / 5 (DOWN): two e4m3 terms per value, s * (hi + lo / 16). Pinned by what the two terms are
    for: (1) the stored rows [hi | lo] decode to the f64 GLU of the bf16 inputs to about bf16 precision (2^-7 of the
    group's amax; a dropped lo term or a wrong 1/16 leaves the single term's 2^-4), (2) over a sweep of the whole
    e4m3 range hi is the nearest e4m3 value and hi + lo / 16 lies within 2^-8 of the value (2^-14 absolute at the
    bottom), (3) the DOWN equals an f64 product over the decoded rows, and lands several times closer to the all-f64
    layer than the single-term arm 2 does, (4) arm 5 is arm 4 rounded to bf16."""
    r = cases.rng_of(31)
    E, T, H, I, k = 4, 9, 256, 256, 2
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, False, False)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    R = al[2].shape[0]
    x = cases.randn_bf16(r, (T, H), 1.0)
    e4 = lambda b: torch.from_numpy(np.ascontiguousarray(b)).view(torch.float8_e4m3fn).double().numpy()
    fq, fs = np.zeros((R, 2 * I), np.uint8), np.zeros((R, I // 128), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, None, 7], i=[I, H, E, 1, T, 1, 0, 4]),
        [fq, x, wtab, stab, al[0], al[2], None, fs], 2)
    part = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E, 1, 0, 0, 0, 4]),
        [part, fq, wtab, stab, al[0], fs, al[3], al[4]], 2)
    p16 = np.zeros((T * k, H), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E, 1, 0, 0, 0, 5]),
        [p16, fq, wtab, stab, al[0], fs, al[3], al[4]], 2)
    # the single-term chain on the same inputs
    xq, xs = np.zeros((T, H), np.uint8), np.zeros((H // 128, T), np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[T, H, T]), [xq, x, xs])
    fq1, fs1 = np.zeros((R, I), np.uint8), np.zeros((R, I // 128), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[I, H, E, 1, T, 1, 0, 2]),
        [fq1, xq, wtab, stab, al[0], al[2], xs, fs1], 2)
    part1 = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E, 1, 0, 0, 0, 2]),
        [part1, fq1, wtab, stab, al[0], fs1, al[3], al[4]], 2)
    # (2)
    sweep = np.concatenate([np.linspace(-448, 448, 200001), np.geomspace(2.0 ** -12, 448, 50000), [0.0, 448.0, -448.0]]).astype(np.float32)
    bh, bl = np.zeros(sweep.size, np.uint8), np.zeros(sweep.size, np.uint8)
    oracle.plow_oracle_split_e4m3_n(bh.ctypes.data, bl.ctypes.data, sweep.ctypes.data, sweep.size)
    assert np.array_equal(bh, torch.from_numpy(sweep).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    two = e4(bh) + e4(bl) / 16.0
    assert np.all(np.abs(two - sweep) <= np.maximum(np.abs(sweep.astype(np.float64)) * 2.0 ** -8, 2.0 ** -14))
    assert np.mean(np.abs(e4(bh) - sweep) > np.abs(sweep) * 2.0 ** -6) > 0.3   # which one term alone does not reach
    silu = lambda g: g / (1.0 + np.exp(-g))
    xa = ol.bf2f(x).astype(np.float64)
    sc = np.repeat(fs.astype(np.float64), 128, axis=1)
    hi, lo = e4(fq[:, :I]), e4(fq[:, I:])
    fa = sc * (hi + lo / 16.0)
    err2 = err1 = ref2 = 0.0
    for row in range(int(al[0][-1]) * 64):
        s = al[3][row]
        if s == abi.EXPERT_UNUSED:
            continue
        e, t = tab["eid"][s], s // k
        v = silu(dequant(W["g"][e][1], S["g"][e]) @ xa[t]) * (dequant(W["u"][e][1], S["u"][e]) @ xa[t])
        amax = np.abs(v).reshape(-1, 128).max(1).repeat(128)
        assert np.all(np.abs(fa[row] - v) <= amax * 2.0 ** -7 + 1e-9)                   # (1)
        assert np.abs(sc[row] * hi[row] - v).max() > np.abs(fa[row] - v).max() * 4      # lo carries real bits
        y = tab["gate"][s] * (dequant(W["d"][e][1], S["d"][e]) @ fa[row])
        assert np.all(np.abs(part[s] - y) <= 1e-5 * np.abs(y).max() + 1e-6)             # (3)
        yref = tab["gate"][s] * (dequant(W["d"][e][1], S["d"][e]) @ v)
        err2 += ((part[s] - yref) ** 2).sum(); err1 += ((part1[s] - yref) ** 2).sum(); ref2 += (yref ** 2).sum()
        assert np.array_equal(p16[s], ol.f2bf(part[s]))                                 # (4)
    rel2, rel1 = np.sqrt(err2 / ref2), np.sqrt(err1 / ref2)
    print(f"two-term relL2 {rel2:.2e}, single-term {rel1:.2e}")
    assert rel2 < 4e-3 and rel2 * 8 < rel1


def test_fp8blk_inline_quant_arm_equals_quantizer_plus_plain_arm(oracle):
    """Op 85 arm 6 takes the bf16 rows and quantizes each 1x128 group itself: by definition the quantizer
    op followed by arm 2, bit for bit (plow runtime/amd/moe_pf_w8a8.h:118-121)."""
    r = cases.rng_of(23)
    E, T, H, I, k = 5, 21, 384, 256, 2
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, False, False)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    R = al[2].shape[0]
    x = cases.randn_bf16(r, (T, H), 1.0)
    x[3, 128:256] = 0                     # an all-zero group: the floored amax
    xq, xs = np.zeros((T, H), np.uint8), np.zeros((H // 128, T), np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[T, H, T]), [xq, x, xs])
    fq2, fs2 = np.full((R, I), 0x55, np.uint8), np.full((R, I // 128), 7.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[I, H, E, 1, T, 1, 0, abi.ARM_W8A8]),
        [fq2, xq, wtab, stab, al[0], al[2], xs, fs2], 2)
    fq6, fs6 = np.full((R, I), 0x55, np.uint8), np.full((R, I // 128), 7.0, np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, None, 7], i=[I, H, E, 1, 0, 1, 0, abi.ARM_W8A8_XQ]),
        [fq6, x, wtab, stab, al[0], al[2], None, fs6], 3)
    assert np.array_equal(fq6, fq2)
    assert np.array_equal(fs6.view(np.uint32), fs2.view(np.uint32))
    assert (fq6 != 0x55).any()


def test_fp8blk_atomic_chain_against_f64_and_the_plain_quantizer(oracle):
    """Ops 188 / 189 / 190 (bf16 intermediate, slot-major quantized copy, bf16 reduction into the output;
    plow runtime/amd/op_moe_fp8_block128.h:7-88): the GLU against an f64 evaluation of the same quantized
    operands with the pad rows of every tile zeroed, the scatter quantizer bit for bit against the plain
    1x128 quantizer applied to the rows put in slot order by hand, the reduction against f64 within the
    rounding of k bf16 additions; the clamp limit of fj[1] acts on gate (above) and up (both sides)."""
    r = cases.rng_of(31)
    E, T, H, I, k = 4, 11, 256, 256, 2
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, False, False)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    meta, row_token, row_partidx, row_gate = al[0], al[2], al[3], al[4]
    R = row_token.shape[0]
    ntile = int(meta[3 * E])
    x = cases.randn_bf16(r, (T, H), 1.0)
    xq, xs = np.zeros((T, H), np.uint8), np.zeros((H // 128, T), np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[T, H]), [xq, x, xs])
    xa = torch.from_numpy(xq).view(torch.float8_e4m3fn).double().numpy() * np.repeat(xs.T.astype(np.float64), 128, axis=1)
    silu = lambda g: g / (1.0 + np.exp(-g))
    for limit in (0.0, 0.05):
        fu = np.full((R, I), 0x7FC0, np.uint16)
        run(oracle, abi.inst(abi.OP_MOE_GLU_FP8_BLOCK128, t=[0, 1, 2, 3, 4, 5, 6], i=[I, H, E, T], f=[0.0, limit]),
            [fu, xq, xs, wtab, stab, meta, row_token], 3)
        fa = ol.bf2f(fu).astype(np.float64)
        clamped = 0
        for row in range(ntile * 64):
            s_ = row_partidx[row]
            if s_ == abi.EXPERT_UNUSED:
                assert not fu[row].any()                        # pad rows of a tile are zeroed
                continue
            e, t = tab["eid"][s_], s_ // k
            g = dequant(W["g"][e][1], S["g"][e]) @ xa[t]
            u = dequant(W["u"][e][1], S["u"][e]) @ xa[t]
            if limit > 0:
                clamped += int((g > limit).sum() + (np.abs(u) > limit).sum())
                g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
            v = silu(g) * u
            assert np.all(np.abs(fa[row] - v) <= 2.0 ** -8 * np.abs(v).max() + 1e-6)
        assert (fu[ntile * 64:] == 0x7FC0).all()                # nothing beyond the last tile is touched
        assert limit == 0.0 or clamped > 0
    # (fu now holds the clamped run) scatter quantizer == plain quantizer over the rows in slot order
    slots = T * k
    hq, hs = np.full((slots, I), 0x55, np.uint8), np.full((I // 128, slots), 7.0, np.float32)
    out = np.full((T, H), 0x7FC0, np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_QUANT_FP8_BLOCK128, t=[0, 1, 2, 3, 4, 5], i=[I, E, k, T, H]),
        [hq, fu, hs, meta, row_partidx, out], 3)
    assert not out.any()
    by_slot = np.zeros((slots, I), np.uint16)
    for row in range(ntile * 64):
        if row_partidx[row] != abi.EXPERT_UNUSED:
            by_slot[row_partidx[row]] = fu[row]
    hq2, hs2 = np.zeros((slots, I), np.uint8), np.zeros((I // 128, slots), np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8_BLOCK128, t=[0, 1, 2], i=[slots, I]), [hq2, by_slot, hs2])
    assert np.array_equal(hq, hq2) and np.array_equal(hs.view(np.uint32), hs2.view(np.uint32))
    # the reduction
    run(oracle, abi.inst(abi.OP_MOE_DOWN_FP8_BLOCK128, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[I, H, E, k, T]),
        [out, hq, hs, wtab, stab, meta, row_partidx, row_gate], 2)
    ha = torch.from_numpy(hq).view(torch.float8_e4m3fn).double().numpy() * np.repeat(hs.T.astype(np.float64), 128, axis=1)
    want = np.zeros((T, H))
    for s_ in range(slots):
        want[s_ // k] += float(tab["gate"][s_]) * (dequant(W["d"][tab["eid"][s_]][1], S["d"][tab["eid"][s_]]) @ ha[s_])
    got = ol.bf2f(out).astype(np.float64)
    assert np.abs(got - want).max() <= k * 2.0 ** -8 * np.abs(want).max()


def test_fp8blk_constant_block_scale_factors_out(oracle):
    """A constant scale grid c equals c times the unit-scale result (c a power of two: exactly)."""
    r = cases.rng_of(12)
    E, T, H, I = 2, 5, 256, 128
    W, S, wtab, stab = build_fp8(oracle, r, E, T, H, I, False, True)
    tab = identity_align(T, r.integers(0, E, T).astype(np.uint32), E)
    al = cases.align_arrays(tab, T, E, 1)
    run(oracle, cases.align_inst(T, E, 1), al)
    R = al[2].shape[0]
    fu = cases.randn_bf16(r, (R, I), 1.0)
    outs = []
    for c in (1.0, 0.25):
        for e in range(E):
            S["d"][e][:] = c
        part = np.zeros((T, H), np.float32)
        run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[H, I, E, 1, 0, 0, 0, 0]),
            [part, fu, wtab, stab, al[0], None, al[3], al[4]])
        outs.append(part)
    assert np.array_equal(outs[1], outs[0] * np.float32(0.25))


def test_mxfp4_grouped_arm_equals_decode_arm(oracle):
    """Ops 85/86 at enc 2 / arm 8 are the arithmetic of the decode ops 48/49 (pinned by plow's flat
    mxfp4 kernels in tests/test_golden.py) applied to gathered rows: same bits, row for row."""
    r = cases.rng_of(13)
    E, T, H, I, k = 5, 6, 128, 64, 2
    Wg, Wu = [r.integers(0, 256, (I, H // 2), dtype=np.uint8) for _ in range(E)], [r.integers(0, 256, (I, H // 2), dtype=np.uint8) for _ in range(E)]
    Wd = [r.integers(0, 256, (H, I // 2), dtype=np.uint8) for _ in range(E)]
    Sg, Su = [r.integers(120, 128, (I, H // 32), dtype=np.uint8) for _ in range(E)], [r.integers(120, 128, (I, H // 32), dtype=np.uint8) for _ in range(E)]
    Sd = [r.integers(120, 128, (H, I // 32), dtype=np.uint8) for _ in range(E)]
    wtab = np.array([[Wg[e].ctypes.data, Wu[e].ctypes.data, Wd[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    stab = np.array([[Sg[e].ctypes.data, Su[e].ctypes.data, Sd[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = r.random(T * k).astype(np.float32)
    x = cases.randn_bf16(r, (T, H), 1.0)
    fu_d = np.zeros((T * k, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_FP8_BLK, t=[0, 1, 2, 3, 4], i=[T * k, I, H, E, k, 1, 2]), [fu_d, x, tab, wtab, stab])
    part_d = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_FP8_BLK, t=[0, 1, 2, 3, 4], i=[T * k, H, I, E, 0, 0, 2]), [part_d, fu_d, tab, wtab, stab])
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    R = al[2].shape[0]
    fu_g = np.zeros((R, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5], i=[I, H, E, 2, 0, 1, 0, 8]), [fu_g, x, wtab, stab, al[0], al[2]], 2)
    part_g = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, None, 6, 7], i=[H, I, E, 2, 0, 0, 0, 8]),
        [part_g, fu_g, wtab, stab, al[0], None, al[3], al[4]], 2)
    for row in range(int(al[0][-1]) * 64):
        if al[3][row] != abi.EXPERT_UNUSED:
            assert np.array_equal(fu_g[row], fu_d[al[3][row]])
    assert np.array_equal(part_g.view(np.uint32), part_d.view(np.uint32))


def test_per_channel_w8a8_against_f64(oracle):
    """Ops 32 -> 81 -> 32 -> 82 vs f64 over the same quantized bytes (sequential-sum f32 arithmetic,
    as the reference's own GPU test checks them: runtime/tests/moe_gemma_gfx950_test.c:1140-1200)."""
    r = cases.rng_of(14)
    E, T, H, I, k = 3, 8, 128, 64, 2
    gu8 = [cases.e4m3_bytes(r, (2 * I, H)) for _ in range(E)]
    d8 = [cases.e4m3_bytes(r, (H, I)) for _ in range(E)]
    sgu = [(r.random(2 * I) * 0.01 + 1e-3).astype(np.float32) for _ in range(E)]
    sd = [(r.random(H) * 0.01 + 1e-3).astype(np.float32) for _ in range(E)]
    ewt = np.array([[a.ctypes.data, b.ctypes.data] for a, b in zip(gu8, d8)], dtype=np.uint64)
    est = np.array([[a.ctypes.data, b.ctypes.data] for a, b in zip(sgu, sd)], dtype=np.uint64)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = (r.random(T * k) + 0.1).astype(np.float32)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    R = al[2].shape[0]
    x = cases.randn_bf16(r, (T, H), 1.0)
    xq, asc = np.zeros((T, H), np.uint8), np.zeros(T, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[T, H]), [xq, x, asc])
    fu = np.zeros((R, I), np.uint16)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_GEMMA_PF_W8A8, t=[0, 1, 2, 3, 4, 5, 6], i=[I, H, E, 0, 0, 1]),
        [fu, xq, ewt, al[0], al[2], asc, est], 2)
    fu8, fsc = np.zeros((R, I), np.uint8), np.zeros(R, np.float32)
    run(oracle, abi.inst(abi.OP_QUANT_FP8, t=[0, 1, 2], i=[R, I]), [fu8, fu, fsc])
    part = np.zeros((T * k, H), np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_GEMMA_PF_W8A8, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[H, I, E]),
        [part, fu8, ewt, al[0], al[3], al[4], est, fsc], 2)
    dec = lambda b: torch.from_numpy(np.ascontiguousarray(b)).view(torch.float8_e4m3fn).double().numpy()
    for row in range(int(al[0][-1]) * 64):
        s = al[3][row]
        if s == abi.EXPERT_UNUSED:
            continue
        e, t = tab["eid"][s], s // k
        gu = (dec(gu8[e]) @ dec(xq[t])) * asc[t] * sgu[e]
        v = gu[:I] / (1 + np.exp(-gu[:I])) * gu[I:]
        assert np.all(np.abs(ol.bf2f(fu[row]) - v) <= 2.0 ** -8 * np.abs(v) + 1e-7)
        y = tab["gate"][s] * ((dec(d8[e]) @ dec(fu8[row])) * fsc[row] * sd[e])
        assert np.allclose(part[s], y, rtol=1e-5, atol=1e-6)


def det_closed_form(part, T, k, H):
    """The deterministic fused combine's accumulator from the f32 partials of the plain chain, in exact
    integer arithmetic: acc[t][h] = sum_j rint(clamp(part[t*k+j][h], +-2^17) * 2^32) (Python integers)."""
    p = np.clip(part.astype(np.float64).reshape(T, k, H), -131072.0, 131072.0) * 4294967296.0
    q = np.rint(p)                                  # |q| <= 2^49: exact in f64 and in int64
    return q.astype(np.int64).sum(axis=1)


def test_deterministic_fused_combine_closed_form_and_thread_independence(oracle):
    """Op 86 with i5 (plow runtime/amd/op_moe.h:2110-2165): the [T][H] f64 accumulator must hold, exactly,
    the integer sum of the quantized contributions the plain arm writes to `part` (closed form in integer
    arithmetic), whatever the number of workers (the additions commute); op 83 zeroes it; op 87 with i4
    reads it as one stream: out = bf16(residual + (float)(acc * 2^-32)). The clamp at +-2^17 is reached
    with a huge gate."""
    import dataclasses
    from gpu_harness import run_oracle
    from plow_amd import layer, synth
    cfg = layer.MoeConfig("det", H=256, E=6, I=128, k=3, T=21, scoring="sigmoid", norm_topk=True, bias=True,
                          enc="fp8blk", arm="w8a8", n_shared=1, shared_mode="fold", residual=True)
    plain = layer.plan_layer(cfg)
    hp = synth.bind(plain, "cpu", seed=5)
    run_oracle(oracle, plain, hp)
    det = layer.plan_layer(dataclasses.replace(cfg, det_combine=True))
    assert "part" not in det.slots and det.insts[det.index("down")].i[5] == 256 + cfg.k_all
    outs = []
    for nthreads in (1, 7, 16):
        hd = synth.bind(det, "cpu", seed=5)
        hd.t["acc64"].fill_(123.0)                  # op 83 must zero it
        run_oracle(oracle, det, hd, nthreads=nthreads)
        outs.append((hd.t["acc64"].numpy().copy(), hd.np("out").copy()))
    want = det_closed_form(hp.t["part"].numpy(), cfg.T, cfg.k_all, cfg.H)
    for acc, out in outs:
        assert np.array_equal(acc, want.astype(np.float64)) and np.all(acc == np.rint(acc))
        assert np.array_equal(out, outs[0][1])
    res = ol.bf2f(hp.np("residual")).astype(np.float32)
    expect = ol.f2bf(res + (want.astype(np.float64) * 2.0 ** -32).astype(np.float32))
    assert np.array_equal(outs[0][1], expect)
    # against the plain chain's output: same values up to the order of the f32 additions and 2^-32 steps
    a, b = ol.bf2f(outs[0][1]).astype(np.float64), ol.bf2f(hp.np("out")).astype(np.float64)
    assert np.abs(a - b).max() <= 2.0 ** -7 * np.abs(b).max()
    # the clamp: a gate of 1e9 drives every contribution to +-2^17 * 2^32 = +-2^49
    big = synth.bind(det, "cpu", seed=5)
    run_oracle(oracle, det, big, labels=["score", "topk", "align", "quant_x", "glu"])
    big.t["row_gate"].fill_(1e9)
    run_oracle(oracle, det, big, labels=["down"])
    acc = big.t["acc64"].numpy()
    assert np.abs(acc).max() <= cfg.k_all * 2.0 ** 49 and (np.abs(acc) >= 2.0 ** 49).any()


def test_deterministic_fused_combine_reference_shift_encoding(oracle):
    """i5 = log2(k) + 1 (the reference's encoding, power-of-two k) selects the same rows as 256 + k."""
    import dataclasses
    from gpu_harness import run_oracle
    from plow_amd import layer, synth
    cfg = layer.MoeConfig("det4", H=128, E=5, I=128, k=4, T=9, scoring="softmax", norm_topk=True,
                          enc="fp8blk", arm="w8a8", det_combine=True)
    plan = layer.plan_layer(cfg)
    a = synth.bind(plan, "cpu", seed=2)
    run_oracle(oracle, plan, a)
    plan.insts[plan.index("down")].i[5] = 3         # log2(4) + 1
    b = synth.bind(plan, "cpu", seed=2)
    run_oracle(oracle, plan, b)
    assert np.array_equal(a.t["acc64"].numpy(), b.t["acc64"].numpy()) and np.abs(a.t["acc64"].numpy()).max() > 0


# ---- the fp4 x fp4 arm of ops 85 / 86: its activation quantizer and its GEMMs ---------------------

E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def test_mx_act_e8m0_is_the_smallest_power_of_two_that_brings_the_amax_below_six(oracle):
    """Exact rational arithmetic instead of the float's bit fields: 2^(b - 127) is the smallest power of two
    s with amax / s < 6 (so the block's largest value lands on e2m1's 3, 4 or just under 6), clamped to the
    bytes 1..254; zero, negative, infinite and NaN amax give 127."""
    from fractions import Fraction
    r = cases.rng_of(21)
    vals = [np.float32(v) for v in r.integers(4, 0x7F800000, 4000, dtype=np.uint32).view(np.float32)]
    for n in range(-140, 128):
        for m in (1.0, 1.25, 1.5, 1.75):
            v = np.float32(m * 2.0 ** n)
            if v > 0 and np.isfinite(v):
                vals += [v, np.nextafter(v, np.float32(0)), np.nextafter(v, np.float32(np.inf))]
    for a in vals:
        if not np.isfinite(a) or a.view(np.uint32) < 4:
            continue
        F = Fraction(float(a))
        e = int(np.frexp(float(a))[1])
        while F >= 6 * Fraction(2) ** e:
            e += 1
        while F < 6 * Fraction(2) ** (e - 1):
            e -= 1
        want = min(max(e + 127, 1), 254)
        assert oracle.plow_oracle_mx_act_e8m0(float(a)) == want, (a, want)
    for a in (0.0, -1.0, float("inf"), float("nan"), float(np.uint32(3).view(np.float32))):
        assert oracle.plow_oracle_mx_act_e8m0(a) == 127


def test_mx_act_fp4_is_the_nearest_e2m1_value_with_midpoints_away_from_zero(oracle):
    from fractions import Fraction
    r = cases.rng_of(22)
    vals = list(r.uniform(-8, 8, 3000).astype(np.float32)) + list(r.standard_normal(500).astype(np.float32) * 1e-3)
    for a, b in zip(E2M1[:-1], E2M1[1:]):
        mid = np.float32((a + b) / 2)
        for v in (mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(9)), np.float32(a), np.float32(b)):
            vals += [v, -v]
    vals += [np.float32(v) for v in (6.0, 6.5, 100.0, 3e38, float("inf"), -float("inf"), 1e-40, -1e-40)]
    for v in vals:
        F = Fraction(float(abs(v))) if np.isfinite(v) else Fraction(10)
        best = min(range(8), key=lambda n: (abs(F - Fraction(float(E2M1[n]))), -n))   # ties: the larger magnitude
        want = (8 if v < 0 else 0) | best
        assert oracle.plow_oracle_mx_act_fp4(float(v)) == want, (v, want)
    assert oracle.plow_oracle_mx_act_fp4(-0.0) == 0
    assert oracle.plow_oracle_mx_act_fp4(float("nan")) == 7


def mx_dequant(codes, scales):
    c = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(codes.shape[0], -1)
    v = E2M1[c & 7] * np.where(c & 8, -1.0, 1.0)
    return v * np.repeat(np.exp2(scales.astype(np.float64) - 127.0), 32, axis=1)


def mx_act_quant(oracle, v):
    v = np.ascontiguousarray(v, np.float32)
    out, sc = np.zeros((v.shape[0], v.shape[1] // 2), np.uint8), np.zeros((v.shape[0], v.shape[1] // 32), np.uint8)
    oracle.plow_oracle_mx_act_quant(out.ctypes.data, sc.ctypes.data, v.ctypes.data, v.size // 32)
    return out, sc


def test_mx_act_quant_returns_representable_blocks_unchanged(oracle):
    """A block of e2m1 values up to 4, times 2^s, with a 4 in it: the byte is s + 127 and the block survives
    exactly. With a 6 as its amax the byte is one more (6 / 2^s is not below 6) and the block comes back as
    its halves, rounded away from zero onto the ladder."""
    r = cases.rng_of(23)
    n = 64
    s = r.integers(-20, 20, (n, 1))
    v = E2M1[r.integers(0, 7, (n, 32))] * r.choice([-1.0, 1.0], (n, 32))
    v[:, 5] = 4.0
    x = (v * np.exp2(s)).astype(np.float32)
    q, sc = mx_act_quant(oracle, x)
    assert np.array_equal(sc[:, 0], (s[:, 0] + 127).astype(np.uint8))
    assert np.array_equal(mx_dequant(q, sc), x.astype(np.float64))
    v[:, 5] = -6.0
    x = (v * np.exp2(s)).astype(np.float32)
    q, sc = mx_act_quant(oracle, x)
    assert np.array_equal(sc[:, 0], (s[:, 0] + 128).astype(np.uint8))
    half = np.abs(v) / 2                                    # 0 .25 .5 .75 1 1.5 2 3: .25 -> .5 and .75 -> 1
    want = np.where(half == 0.25, 0.5, np.where(half == 0.75, 1.0, half)) * np.sign(v) * 2 * np.exp2(s)
    assert np.array_equal(mx_dequant(q, sc), want)


@pytest.mark.parametrize("p16", [False, True])
def test_a4w4_arm_against_f64_over_the_same_bytes(oracle, p16):
    """Op 85 at enc 2 / arm 0 quantizes each gathered row per 32 values, multiplies in fp4 x fp4, applies the
    GLU in f32 and leaves mxfp4 rows with E8M0 rows; op 86 reads them back. Against numpy f64 over the
    dequantized bytes, with the pad rows left untouched."""
    r = cases.rng_of(31)
    E, T, H, I, k = 4, 9, 128, 64, 2
    Wg = [r.integers(0, 256, (I, H // 2), dtype=np.uint8) for _ in range(E)]
    Wu = [r.integers(0, 256, (I, H // 2), dtype=np.uint8) for _ in range(E)]
    Wd = [r.integers(0, 256, (H, I // 2), dtype=np.uint8) for _ in range(E)]
    Sg = [r.integers(118, 124, (I, H // 32), dtype=np.uint8) for _ in range(E)]
    Su = [r.integers(118, 124, (I, H // 32), dtype=np.uint8) for _ in range(E)]
    Sd = [r.integers(118, 124, (H, I // 32), dtype=np.uint8) for _ in range(E)]
    wtab = np.array([[Wg[e].ctypes.data, Wu[e].ctypes.data, Wd[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    stab = np.array([[Sg[e].ctypes.data, Su[e].ctypes.data, Sd[e].ctypes.data] for e in range(E)], dtype=np.uint64)
    tab = np.zeros(T * k, dtype=ol.ROUTE_DT)
    for t in range(T):
        tab["eid"][t * k:(t + 1) * k] = r.choice(E, k, replace=False)
    tab["gate"] = r.random(T * k).astype(np.float32)
    x = cases.randn_bf16(r, (T, H), 1.0)
    al = cases.align_arrays(tab, T, E, k)
    run(oracle, cases.align_inst(T, E, k), al)
    meta, _, row_token, row_partidx, row_gate = al
    R = row_token.shape[0]
    fu4, fsc = np.full((R, I // 2), 0xAA, np.uint8), np.full((R, I // 32), 0x55, np.uint8)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_GLU_PF, t=[0, 1, 2, 3, 4, 5, 6, 7], i=[I, H, E, 2, T, 1, 0, abi.ARM_A4W4]),
        [fu4, x, wtab, stab, meta, row_token, row_partidx, fsc], 2)
    part = np.zeros((T * k, H), np.uint16 if p16 else np.float32)
    run(oracle, abi.inst(abi.OP_MOE_GROUP_DOWN_PF, t=[0, 1, 2, 3, 4, 5, 6, 7],
                         i=[H, I, E, 2, 0, 0, 0, abi.ARM_A4W4_P16 if p16 else abi.ARM_A4W4]),
        [part, fu4, wtab, stab, meta, fsc, row_partidx, row_gate], 2)

    xq = mx_dequant(*mx_act_quant(oracle, ol.bf2f(x)))      # the quantizer is pinned by the three tests above
    seen = 0
    for e in range(E):
        r0, cnt = int(meta[e]), int(meta[E + e])
        g64, u64, d64 = mx_dequant(Wg[e], Sg[e]), mx_dequant(Wu[e], Su[e]), mx_dequant(Wd[e], Sd[e])
        for row in range(r0, r0 + cnt):
            a = xq[row_token[row]]
            gt, up = (g64 @ a).astype(np.float32).astype(np.float64), (u64 @ a).astype(np.float32).astype(np.float64)
            v = (gt / (1.0 + np.exp(-gt)) * up).astype(np.float32)
            wq, ws = mx_act_quant(oracle, v[None, :])
            # the oracle's f32 SiLU and this f64 one may differ in the last bit: a value on a rounding boundary
            # may take the neighbouring code
            got, want = mx_dequant(fu4[row:row + 1], fsc[row:row + 1])[0], mx_dequant(wq, ws)[0]
            assert np.array_equal(fsc[row], ws[0]) and np.mean(got != want) <= 1 / 32, row
            np.testing.assert_allclose(got, want, rtol=0, atol=0.5 * np.abs(want).max())
            p = (d64 @ got) * float(row_gate[row])
            have = ol.bf2f(part[row_partidx[row]]) if p16 else part[row_partidx[row]]
            np.testing.assert_allclose(have, p, rtol=2 ** -8 if p16 else 1e-6, atol=1e-30)
            seen += 1
    assert seen == T * k
    pad = row_partidx == abi.EXPERT_UNUSED
    assert pad.any() and np.all(fu4[pad] == 0xAA) and np.all(fsc[pad] == 0x55)


def test_router_score_that_carries_its_topk_is_the_op_pair(oracle):
    """Op 180 with the router mark writes the logits of op 180 and the table of op 83 over them (the pair is
    pinned above and by plow's golden vectors); the counters stay as they were."""
    r = cases.rng_of(41)
    T, E, H, k = 5, 64, 256, 4
    x, w = cases.randn_bf16(r, (T, H), 1.0), cases.randn_bf16(r, (E, H), 0.05)
    bias = (r.standard_normal(E) * 0.01).astype(np.float32)
    flags = abi.ROUTE_SIGMOID | abi.ROUTE_NORM_TOPK | abi.ROUTE_BIAS | abi.ROUTE_F32_LOGIT
    logit = np.zeros((T, E), np.float32)
    table = np.zeros(T * (k + 1), dtype=ol.ROUTE_DT)
    run(oracle, abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2], i=[T, E, H]), [logit, x, w], 3)
    run(oracle, abi.inst(abi.OP_MOE_ROUTER_TOPK_PF, t=[0, 1, None, 3], i=[0, E, k, flags, T, 1, 8, 4], f=[2.5, 0.0]),
        [table, logit, None, bias], 3)
    logit2, table2 = np.zeros_like(logit), np.zeros_like(table)
    ctr = np.full(T * 32, 7, np.uint32)
    run(oracle, abi.inst(abi.OP_GEMM_F32, t=[0, 1, 2, 3, 4, 5], i=[T, E, H, k, flags, 1, 8 | (4 << 16), abi.ROUTER_RAW_MARK],
                         f=[2.5, 0.0]), [logit2, x, w, table2, bias, ctr], 3)
    assert np.array_equal(logit.view(np.uint32), logit2.view(np.uint32))
    assert np.array_equal(table, table2) and table["eid"].max() == E and np.all(ctr == 7)
