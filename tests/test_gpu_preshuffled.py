"""Weights in ck_tile's pre-shuffled layout (FusedMoeGemmWeightPermuteEnum::b_nr_kr_kw_nw_kv, what its device
kernel takes and its example produces before the call): the GEMM kernels read them in place.  The layout is pinned
on ck_tile::reference_permute in the CPU tests of the permutation tool; here the tool's output goes in with
weight_permute = 1 and the result has to be the row-major run's, bit for bit - every kernel family fetches the
same bytes into the same LDS positions either way - and stay within tolerance of the oracle."""
import numpy as np
import pytest
import torch

import oracle
import therock_amd as ta
from therock_amd import inputs as mi

pytestmark = pytest.mark.gpu

# decode tiles, 64-row decode tiles, 128-row small tiles, 320-row tiles; ragged K depths where the layout allows them
# (rows of whole 64-byte blocks: hidden and inter multiples of 32 for 16-bit types, of 64 for 8-bit types)
SHAPES = [
    ("decode", 24, 1088, 320, 16, 4, 32),
    ("decode_two_blocks", 160, 512, 256, 8, 2, 32),
    ("small_tiles", 384, 576, 384, 8, 2, 32),
    ("large_tiles", 2048, 512, 256, 8, 2, 32),
    ("large_tiles_unit64", 640, 256, 1536, 4, 4, 64),
    ("small_tiles_unit8", 700, 256, 384, 3, 2, 8),
]


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp8", "int8"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: s[0])
def test_preshuffled_weights_give_the_same_bits(shape, dtype):
    from tests.gpu_util import rel_l2, run_fused_moe
    name, T, H, I, E, K, unit = shape
    if dtype in ("fp8", "int8"):
        H, I = (H + 63) // 64 * 64, (I + 63) // 64 * 64
    if dtype == "fp8":
        I = (I + 127) // 128 * 128
    cfg = mi.MoeConfig(name, T, H, I, E, K, dtype, "softmax_renorm", unit)
    print(f"pre-shuffled {cfg}", flush=True)
    inp = mi.make_inputs_np(cfg, 3)
    plain, buf = run_fused_moe(cfg, inp)
    rows = buf and ta.fused_moe_tile_rows(ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, prec_o="fp16" if dtype == "fp16" else "bf16",
                                                               block_m=unit), T, E, K, H, I)
    shuffled, _ = run_fused_moe(cfg, inp, weight_permute=1)
    assert np.array_equal(plain, shuffled), f"{name} {dtype}: tile rows {rows}"
    unfused, _ = run_fused_moe(cfg, inp, weight_permute=1, unfused=True)
    assert np.array_equal(plain, unfused)
    if dtype != "fp16":  # against the oracle as well (the row-major run has its own tests; this guards the comparison itself)
        s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], E, unit)
        dt = {"bf16": oracle.DT_BF16, "fp8": oracle.DT_E4M3, "int8": oracle.DT_I8}[dtype]
        ref = oracle.bf16_to_f32(oracle.fused_moe(inp["a"], dt, inp["g"], dt, inp["d"], dt, *s, unit, T, E, H, I, K,
                                                  a_scale=inp["a_scale"], g_scale=inp["g_scale"], d_scale=inp["d_scale"]))
        assert rel_l2(oracle.bf16_to_f32(shuffled), ref) <= (1e-2 if dtype == "bf16" else 3e-2)


def test_preshuffled_variants():
    """Gate-only weights, GELU, the expert mask, the int8 path with re-quantised intermediate activations, and the fp8
    path whose tile height the sort chooses on the device."""
    from tests.gpu_util import run_fused_moe
    for cfg, kw in ((mi.MoeConfig("v", 300, 512, 384, 8, 2, "bf16", "softmax_renorm"), dict(gate_only=1)),
                    (mi.MoeConfig("v", 48, 512, 256, 16, 4, "int8", "sigmoid_renorm"), dict(activation=0)),
                    (mi.MoeConfig("v", 2048, 512, 256, 8, 2, "int8", "softmax_renorm"), dict(fused_quant=2)),
                    (mi.MoeConfig("v", 64, 256, 256, 8, 2, "int8", "softmax_renorm"), dict(fused_quant=2)),
                    (mi.MoeConfig("v", 256, 512, 2048, 64, 4, "fp8", "zipf"), {}),
                    (mi.MoeConfig("v", 144, 512, 256, 8, 2, "bf16", "softmax_renorm"),
                     dict(mask=np.array([1, 0, 1, 1, 0, 1, 0, 1], dtype=np.int32)))):
        print(f"pre-shuffled {cfg} {kw}", flush=True)
        inp = mi.make_inputs_np(cfg, 4)
        if kw.get("mask") is not None:
            nloc = int(kw["mask"].sum())
            for k in ("g", "d", "g_scale", "d_scale"):
                if inp[k] is not None:
                    inp[k] = inp[k][:nloc]
        if kw.get("gate_only"):
            inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
        plain, _ = run_fused_moe(cfg, inp, **kw)
        shuffled, _ = run_fused_moe(cfg, inp, weight_permute=1, **kw)
        assert np.array_equal(plain, shuffled), (cfg, kw)


def test_preshuffled_argument_checks():
    """Rows that are not whole 64-byte blocks have no pre-shuffled form; an unknown layout code has no kernel."""
    t = ta.fused_moe_traits(prec_i="int8", prec_w="int8", block_m=32, weight_permute=1)
    assert ta.fused_moe_get_workspace_size(t, 64, 8, 2, 256, 256) > 0
    t2 = ta.fused_moe_traits(prec_i="int8", prec_w="int8", block_m=32, weight_permute=2)
    assert ta.fused_moe_get_workspace_size(t2, 64, 8, 2, 256, 256) == 0
    cfg = mi.MoeConfig("bad", 64, 96, 160, 8, 2, "int8", "softmax_renorm")  # 96-byte and 160-byte rows
    inp = mi.make_inputs_np(cfg, 0)
    from tests.gpu_util import dev
    buf = ta.MoeBuffers(t, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, "cuda")
    args = ta.make_args(t, buf, dev(inp["a"]).view(torch.int8), dev(inp["g"]).view(torch.int8), dev(inp["d"]).view(torch.int8),
                        dev(inp["topk_ids"]), dev(inp["topk_weight"]), a_scale=dev(inp["a_scale"]),
                        g_scale=dev(inp["g_scale"]), d_scale=dev(inp["d_scale"]))
    assert ta.fused_moe(t, args) == -1.0
