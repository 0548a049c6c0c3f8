"""Pins oracle.fused_moe (restatement of ck_tile host/reference/reference_fused_moe.hpp:42-204):
ck_tile's own function (bit-exact in strict order), the committed golden outputs, an independent
dense float64 formulation that never touches the sorted arrays, and a triple loop on tiny shapes."""
import hashlib
import os

import numpy as np
import pytest

import oracle
from therock_amd import inputs as mi

DT = {"bf16": oracle.DT_BF16, "fp8": oracle.DT_E4M3, "int8": oracle.DT_I8}


def sha(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def rel_l2(x, ref):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    return np.linalg.norm(x - ref) / max(np.linalg.norm(ref), 1e-30)


def dense_moe_f64(cfg, inp, mask=None):
    """O[t] = sum_k w[t,k] * FFN_{e(t,k)}(x_t) in float64, without any sorting."""
    dt = DT[cfg.dtype]
    a = oracle.to_f32(inp["a"], dt).astype(np.float64)
    g = oracle.to_f32(inp["g"], dt).astype(np.float64)
    d = oracle.to_f32(inp["d"], dt).astype(np.float64)
    if inp["a_scale"] is not None:
        a *= inp["a_scale"][:, None]
        g *= inp["g_scale"][:, :, None]
        d *= inp["d_scale"][:, :, None]
    out = np.zeros((cfg.tokens, cfg.hidden))
    remap = np.arange(cfg.experts) if mask is None else np.cumsum(mask) - 1
    for e in range(cfg.experts):
        if mask is not None and mask[e] == 0:
            continue
        t, k = np.nonzero(inp["topk_ids"] == e)
        if len(t) == 0:
            continue
        le = remap[e]  # weights are indexed by the local expert id the sort emits
        acc = a[t] @ g[le].T
        gate, up = acc[:, :cfg.inter], acc[:, cfg.inter:]
        y = gate / (1.0 + np.exp(-gate)) * up
        out[t] += (y @ d[le].T) * inp["topk_weight"][t, k][:, None]
    return out


def run_oracle(cfg, inp, **kw):
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit,
                           local_expert_mask=kw.pop("mask", None))
    dt = DT[cfg.dtype]
    return oracle.fused_moe(inp["a"], dt, inp["g"], dt, inp["d"], dt, *s, cfg.unit, cfg.tokens, cfg.experts,
                            cfg.hidden, cfg.inter, cfg.topk, a_scale=inp["a_scale"], g_scale=inp["g_scale"],
                            d_scale=inp["d_scale"], **kw)


def test_cfg1_matches_golden_ck_output(golden_dir):
    g = np.load(os.path.join(golden_dir, "cfg1_ck_reference.npz"))
    cfg = mi.CONFIGS["cfg1_cpu_ref_bf16"]
    inp = mi.make_inputs_np(cfg, 0)
    assert str(g["input_sha"]) == sha(inp["a"], inp["g"], inp["d"]), "input generator changed: regenerate tests/golden"
    assert np.array_equal(inp["topk_ids"], g["topk_ids"]) and np.array_equal(inp["topk_weight"], g["topk_weight"])
    s_ids, s_w, s_eid, pp = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit)
    assert pp == int(g["post_pad"]) and np.array_equal(s_ids[:pp], g["sorted_ids"])
    assert np.array_equal(s_w[:pp], g["sorted_w"]) and np.array_equal(s_eid[:pp // cfg.unit], g["sorted_eid"])
    strict = run_oracle(cfg, inp, strict=True)
    assert np.array_equal(strict, g["out_bf16"])  # same summation order => same bits
    fast = run_oracle(cfg, inp)
    assert rel_l2(oracle.bf16_to_f32(fast), oracle.bf16_to_f32(g["out_bf16"])) < 2e-4
    assert (fast != g["out_bf16"]).mean() < 5e-3


@pytest.mark.parametrize("key", ["fp8", "int8"])
def test_small_quantised_matches_golden_ck_output(key, golden_dir):
    from tests.golden.make_golden import SMALL_QUANT
    g = np.load(os.path.join(golden_dir, "small_quant_ck_reference.npz"))
    cfg = SMALL_QUANT[key]
    inp = mi.make_inputs_np(cfg, 0)
    assert str(g[f"{key}_input_sha"]) == sha(inp["a"], inp["g"], inp["d"], inp["a_scale"], inp["g_scale"], inp["d_scale"])
    assert np.array_equal(run_oracle(cfg, inp, strict=True), g[f"{key}_out_bf16"])


@pytest.mark.parametrize("name", ["gelu", "silu_gate_only", "gelu_gate_only"])
def test_activation_variants_match_golden_ck_output(name, golden_dir):
    from tests.golden.make_golden import ACT_VARIANT_CFG as cfg, ACT_VARIANTS
    g = np.load(os.path.join(golden_dir, "act_variants_ck_reference.npz"))
    inp = mi.make_inputs_np(cfg, 11)
    assert str(g["input_sha"]) == sha(inp["a"], inp["g"], inp["d"]), "input generator changed: regenerate tests/golden"
    act, gate_only = ACT_VARIANTS[name]
    if gate_only:
        inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
    assert np.array_equal(run_oracle(cfg, inp, strict=True, activation=act, gate_only=gate_only), g[name])


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_matches_dense_float64_formulation(dtype):
    cfg = mi.MoeConfig("t", 37, 256, 192, 12, 3, dtype, "softmax_renorm", unit=16)
    inp = mi.make_inputs_np(cfg, 4)
    ref = dense_moe_f64(cfg, inp)
    got = run_oracle(cfg, inp, out_dt=oracle.DT_F32)
    assert rel_l2(got, ref) < 5e-6
    got_bf16 = oracle.bf16_to_f32(run_oracle(cfg, inp))
    assert rel_l2(got_bf16, ref) < 3e-3  # one bf16 rounding: 2^-9 relative at most
    # local expert mask: masked experts contribute nothing, weights are indexed by local id
    mask = (np.arange(cfg.experts) % 3 != 1).astype(np.int32)
    nloc = int(mask.sum())
    inp_l = dict(inp, g=inp["g"][:nloc], d=inp["d"][:nloc],
                 g_scale=None if inp["g_scale"] is None else inp["g_scale"][:nloc],
                 d_scale=None if inp["d_scale"] is None else inp["d_scale"][:nloc])
    cfg_l = cfg.scaled(experts=cfg.experts)
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit, local_expert_mask=mask)
    dt = DT[dtype]
    got = oracle.fused_moe(inp_l["a"], dt, inp_l["g"], dt, inp_l["d"], dt, *s, cfg.unit, cfg.tokens, nloc,
                           cfg.hidden, cfg.inter, cfg.topk, a_scale=inp["a_scale"], g_scale=inp_l["g_scale"],
                           d_scale=inp_l["d_scale"], out_dt=oracle.DT_F32)
    assert rel_l2(got, dense_moe_f64(cfg_l, inp_l, mask)) < 5e-6


def test_tiny_triple_loop_and_partials():
    cfg = mi.MoeConfig("tiny", 5, 8, 6, 3, 2, "bf16", "softmax_renorm", unit=4)
    inp = mi.make_inputs_np(cfg, 9)
    a, g, d = (oracle.bf16_to_f32(inp[k]).astype(np.float64) for k in ("a", "g", "d"))
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit)
    o, part = oracle.fused_moe(inp["a"], 1, inp["g"], 1, inp["d"], 1, *s, cfg.unit, cfg.tokens, cfg.experts,
                               cfg.hidden, cfg.inter, cfg.topk, out_dt=oracle.DT_F32, want_partials=True)
    for t in range(cfg.tokens):
        for k in range(cfg.topk):
            e = inp["topk_ids"][t, k]
            y = np.zeros(cfg.inter)
            for n in range(cfg.inter):
                gate = sum(a[t, h] * g[e, n, h] for h in range(cfg.hidden))
                up = sum(a[t, h] * g[e, n + cfg.inter, h] for h in range(cfg.hidden))  # up rows follow gate rows
                y[n] = gate / (1 + np.exp(-gate)) * up
            for h in range(cfg.hidden):
                want = sum(y[n] * d[e, h, n] for n in range(cfg.inter)) * inp["topk_weight"][t, k]
                assert part[t, k, h] == pytest.approx(want, rel=1e-5, abs=1e-9)
    assert np.allclose(o, part.sum(axis=1), rtol=1e-6)
    # gate-only variant: y = silu(gate), G has `inter` rows
    og = oracle.fused_moe(inp["a"], 1, inp["g"][:, :cfg.inter], 1, inp["d"], 1, *s, cfg.unit, cfg.tokens, cfg.experts,
                          cfg.hidden, cfg.inter, cfg.topk, out_dt=oracle.DT_F32, gate_only=True)
    t, e = 0, inp["topk_ids"][0]
    want = np.zeros(cfg.hidden)
    for k in range(cfg.topk):
        gate = a[t] @ g[e[k], :cfg.inter].T
        want += ((gate / (1 + np.exp(-gate))) @ d[e[k]].T) * inp["topk_weight"][t, k]
    assert np.allclose(og[0], want, rtol=1e-5, atol=1e-8)


@pytest.mark.skipif(oracle.ck_ref() is None, reason="oracle/_ref not built")
@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
@pytest.mark.parametrize("activation,gate_only", [(1, False), (0, False), (1, True), (0, True)])
def test_bit_exact_with_ck_tile_reference(dtype, activation, gate_only):
    cfg = mi.MoeConfig("t", 19, 128, 96, 6, 2, dtype, "softmax_renorm", unit=8)
    inp = mi.make_inputs_np(cfg, 11)
    if gate_only:  # G holds the gate rows only
        inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
        if inp["g_scale"] is not None:
            inp["g_scale"] = np.ascontiguousarray(inp["g_scale"][:, :cfg.inter])
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit)
    mine = run_oracle(cfg, inp, strict=True, activation=activation, gate_only=gate_only)
    kw = dict(activation=activation, gate_only=gate_only)
    if dtype == "bf16":
        ck = oracle.ck_fused_moe(inp["a"], inp["g"], inp["d"], *s, cfg.unit, cfg.tokens, cfg.experts, cfg.hidden,
                                 cfg.inter, cfg.topk, **kw)
    else:
        dt = DT[dtype]
        ck = oracle.ck_fused_moe(oracle.to_f32(inp["a"], dt) * inp["a_scale"][:, None],
                                 oracle.to_f32(inp["g"], dt) * inp["g_scale"][:, :, None],
                                 oracle.to_f32(inp["d"], dt) * inp["d_scale"][:, :, None],
                                 *s, cfg.unit, cfg.tokens, cfg.experts, cfg.hidden, cfg.inter, cfg.topk, f32_inputs=True,
                                 **kw)
    assert np.array_equal(mine, ck)


@pytest.mark.skipif(oracle.ck_ref() is None, reason="oracle/_ref not built")
@pytest.mark.parametrize("activation,gate_only", [(1, False), (0, False), (1, True)])
def test_fp16_bit_exact_with_ck_tile_reference(activation, gate_only):
    """ck_tile's other instance: fp16 operands and output.  The oracle takes the fp16 values as float32 and rounds its
    fp32 result to fp16 once; reference_fused_moe instantiated with half_t must give the same bits."""
    cfg = mi.MoeConfig("t", 19, 128, 96, 6, 2, "fp16", "softmax_renorm", unit=8)
    inp = mi.make_inputs_np(cfg, 13)
    if gate_only:
        inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit)
    kw = dict(activation=activation, gate_only=gate_only)
    mine = oracle.fused_moe_f16(inp["a"].view(np.float16), inp["g"].view(np.float16), inp["d"].view(np.float16), *s,
                                cfg.unit, cfg.tokens, cfg.experts, cfg.hidden, cfg.inter, cfg.topk, strict=True, **kw)
    ck = oracle.ck_fused_moe(inp["a"], inp["g"], inp["d"], *s, cfg.unit, cfg.tokens, cfg.experts, cfg.hidden, cfg.inter,
                             cfg.topk, f16=True, **kw)
    assert np.array_equal(mine.view(np.uint16), ck)
    # and it is not the bf16 result in disguise: fp16 keeps three more bits
    assert mine.dtype == np.float16 and np.isfinite(mine.astype(np.float32)).all()
