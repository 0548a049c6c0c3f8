"""Seeded random problem shapes through mi355_fused_moe against the oracle: every dtype, sort units from 8 to
128 rows, row counts per expert from a fraction of a row to several hundred (all three GEMM kernel families
and the boundaries between them), local-expert masks, padded token rows, the unfused entry points.  The
shapes are drawn so that the CPU oracle needs at most about a second per case."""
import numpy as np
import pytest

from therock_amd import inputs as mi
from tests.test_gpu_fused_moe import check

pytestmark = pytest.mark.gpu

ROUTERS = ("softmax_renorm", "softmax", "sigmoid_renorm", "zipf")


def draw(rng, dtype):
    experts = int(rng.choice([1, 2, 3, 5, 8, 16, 33, 64]))
    topk = int(rng.integers(1, min(experts, 8) + 1))
    hidden = 32 * int(rng.integers(1, 33))                       # 32 .. 1024
    inter = (128 if dtype == "fp8" else 32) * int(rng.integers(1, 9 if dtype == "fp8" else 25))
    budget = 1.2e9 / (6.0 * topk * hidden * inter)                # oracle flops
    tokens = int(min(max(1, rng.integers(1, 1200)), max(1, budget)))
    unit = int(rng.choice([8, 16, 32, 48, 64, 128]))
    return mi.MoeConfig("rnd", tokens, hidden, inter, experts, topk, dtype, str(rng.choice(ROUTERS)), unit=unit)


def draw_many_rows(rng, dtype):
    """Few experts, hundreds of rows each, K depths the 320-row kernel takes (multiples of 128 bytes)."""
    experts = int(rng.integers(1, 5))
    topk = int(rng.integers(1, experts + 1))
    hidden = 128 * int(rng.integers(1, 5))
    inter = 128 * int(rng.integers(1, 5))
    rows = int(rng.integers(170, 900))                            # per expert, on average
    tokens = max(1, rows * experts // topk)
    unit = int(rng.choice([16, 32, 48, 64, 128]))
    return mi.MoeConfig("rnd", tokens, hidden, inter, experts, topk, dtype, str(rng.choice(ROUTERS)), unit=unit)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_random_shapes_many_rows_per_expert(dtype):
    import therock_amd as ta
    rng = np.random.default_rng({"bf16": 11, "fp8": 22, "int8": 33}[dtype])
    for case in range(10):
        cfg = draw_many_rows(rng, dtype)
        traits = ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, block_m=cfg.unit)
        assert ta.fused_moe_tile_rows(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter) == 320
        kw = {0: {}, 1: {"unfused": True}, 2: {"stride_pad": 64}, 3: {"gate_only": 1}}[int(rng.integers(0, 4))]
        check(cfg, seed=2000 + case, **kw)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_random_shapes(dtype):
    rng = np.random.default_rng({"bf16": 101, "fp8": 202, "int8": 303}[dtype])
    for case in range(24):
        cfg = draw(rng, dtype)
        kw = {}
        mask = None
        mode = int(rng.integers(0, 6))
        if mode == 1 and cfg.experts > 1:
            mask = (rng.random(cfg.experts) < 0.7).astype(np.int32)
            mask[int(rng.integers(0, cfg.experts))] = 1
        elif mode == 2:
            kw["unfused"] = True
        elif mode == 3:
            kw["stride_pad"] = 32 * int(rng.integers(1, 4))
        elif mode == 4:
            kw["activation"] = 0
        elif mode == 5:
            kw["gate_only"] = 1
        # a handful of rows in fp8 is too small a sample for the rel-L2 of Y's e4m3 rounding to be stable
        if dtype == "fp8" and cfg.tokens * cfg.topk < 16:
            cfg = cfg.scaled(tokens=max(cfg.tokens, 16 // cfg.topk + 1))
        check(cfg, seed=1000 + case, mask=mask, **kw)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_random_shapes_preshuffled_weights(dtype):
    """The same draw with g and d in ck_tile's pre-shuffled layout (rows of whole 64-byte blocks), against the oracle."""
    rng = np.random.default_rng({"bf16": 111, "fp8": 222, "int8": 333}[dtype])
    for case in range(16):
        cfg = (draw_many_rows if case % 4 == 3 else draw)(rng, dtype)
        if dtype != "bf16":
            cfg = cfg.scaled(hidden=(cfg.hidden + 63) // 64 * 64, inter=(cfg.inter + (127 if dtype == "fp8" else 63)) // (128 if dtype == "fp8" else 64) * (128 if dtype == "fp8" else 64))
        if dtype == "fp8" and cfg.tokens * cfg.topk < 16:
            cfg = cfg.scaled(tokens=max(cfg.tokens, 16 // cfg.topk + 1))
        kw = {0: {}, 1: {"unfused": True}, 2: {"activation": 0}, 3: {"gate_only": 1}, 4: {"stride_pad": 64}}[int(rng.integers(0, 5))]
        check(cfg, seed=5000 + case, weight_permute=1, **kw)


def test_random_shapes_fp16():
    from tests.test_gpu_fused_moe import check_fp16
    rng = np.random.default_rng(404)
    for case in range(12):
        cfg = (draw_many_rows if case % 4 == 3 else draw)(rng, "fp16")
        kw = {0: {}, 1: {"unfused": True}, 2: {"activation": 0}, 3: {"gate_only": 1}}[int(rng.integers(0, 4))]
        check_fp16(cfg, seed=3000 + case, **kw)


@pytest.mark.parametrize("fq", [1, 2])
def test_random_shapes_int8_fused_quant(fq):
    """Re-quantised intermediate activations over random shapes and sort units (all three down-GEMM kernels)."""
    from tests.test_gpu_fused_quant import run
    rng = np.random.default_rng(500 + fq)
    for case in range(12):
        cfg = (draw_many_rows if case % 3 == 2 else draw)(rng, "int8")
        # the row-wise int8 rounding of Y needs a few hundred values per row and a few rows for a stable rel-L2
        cfg = cfg.scaled(inter=max(cfg.inter, 128), tokens=max(cfg.tokens, 16 // cfg.topk + 1))
        run(cfg, fq, seed=4000 + case)
