"""GPU parity of mi355_fused_moe / mi355_fused_moegemm against the oracle.

Tolerances are the ones the build targets: rel-L2 <= 1e-2 for bf16, <= 3e-2 for fp8 and int8
(fp32 accumulation in both GEMMs; the intermediate activations are stored in bf16, or block-scaled
e4m3 on the fp8 path, which the oracle keeps in fp32)."""
import os

import numpy as np
import pytest

import oracle
from therock_amd import inputs as mi

pytestmark = pytest.mark.gpu

DT = {"bf16": oracle.DT_BF16, "fp8": oracle.DT_E4M3, "int8": oracle.DT_I8}
TOL = {"bf16": 1e-2, "fp8": 3e-2, "int8": 3e-2}


def oracle_out(cfg, inp, mask=None, activation=1, gate_only=0):
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit, local_expert_mask=mask)
    dt = DT[cfg.dtype]
    o = oracle.fused_moe(inp["a"], dt, inp["g"], dt, inp["d"], dt, *s, cfg.unit, cfg.tokens, inp["g"].shape[0],
                         cfg.hidden, cfg.inter, cfg.topk, a_scale=inp["a_scale"], g_scale=inp["g_scale"],
                         d_scale=inp["d_scale"], activation=activation, gate_only=bool(gate_only))
    return oracle.bf16_to_f32(o), s


def check(cfg, seed=0, mask=None, **kw):
    from tests.gpu_util import rel_l2, run_fused_moe
    inp = mi.make_inputs_np(cfg, seed)
    if mask is not None:  # weights of the local experts only, indexed by local id
        nloc = int(mask.sum())
        for k in ("g", "d", "g_scale", "d_scale"):
            if inp[k] is not None:
                inp[k] = inp[k][:nloc]
    if kw.get("gate_only"):  # G holds the gate rows only
        inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
        if inp["g_scale"] is not None:
            inp["g_scale"] = np.ascontiguousarray(inp["g_scale"][:, :cfg.inter])
    print(f"fused_moe {cfg} seed={seed} mask={mask is not None} {kw}", flush=True)
    got, buf = run_fused_moe(cfg, inp, mask=mask, **kw)
    ref, s = oracle_out(cfg, inp, mask, kw.get("activation", 1), kw.get("gate_only", 0))
    pp = s[3]
    assert int(buf.total[0]) == pp
    assert np.array_equal(buf.sorted_ids[:pp].cpu().numpy(), s[0][:pp])
    assert np.array_equal(buf.sorted_eid[:pp // cfg.unit].cpu().numpy(), s[2][:pp // cfg.unit])
    err = rel_l2(oracle.bf16_to_f32(got), ref)
    print(f"  rel-L2 = {err:.3e} (tolerance {TOL[cfg.dtype]:.0e})", flush=True)
    assert np.all(np.isfinite(oracle.bf16_to_f32(got)))
    assert err <= TOL[cfg.dtype]
    return err


@pytest.mark.parametrize("dtype", ["bf16", "int8", "fp8"])
def test_small_single_tile(dtype):
    # one expert tile, one K tile pair: the smallest problem that touches every code path
    check(mi.MoeConfig("s", 8, 128, 128, 4, 2, dtype, "softmax_renorm"))


@pytest.mark.parametrize("dtype", ["bf16", "int8", "fp8"])
def test_medium_multi_tile(dtype):
    check(mi.MoeConfig("m", 300, 512, 384, 8, 2, dtype, "softmax_renorm"))
    check(mi.MoeConfig("m", 48, 512, 256, 16, 4, dtype, "sigmoid_renorm"))


def test_cfg1_against_oracle_and_ck_golden(golden_dir):
    from tests.gpu_util import rel_l2, run_fused_moe
    cfg = mi.CONFIGS["cfg1_cpu_ref_bf16"]
    check(cfg)
    g = np.load(os.path.join(golden_dir, "cfg1_ck_reference.npz"))
    got, buf = run_fused_moe(cfg, mi.make_inputs_np(cfg, 0))
    pp = int(g["post_pad"])
    assert np.array_equal(buf.sorted_ids[:pp].cpu().numpy(), g["sorted_ids"])
    assert np.array_equal(buf.sorted_w[:pp].cpu().numpy(), g["sorted_w"])
    assert rel_l2(oracle.bf16_to_f32(got), oracle.bf16_to_f32(g["out_bf16"])) <= 1e-2


@pytest.mark.parametrize("key", ["fp8", "int8"])
def test_small_quantised_against_ck_golden(key, golden_dir):
    from tests.golden.make_golden import SMALL_QUANT
    from tests.gpu_util import rel_l2, run_fused_moe
    g = np.load(os.path.join(golden_dir, "small_quant_ck_reference.npz"))
    cfg = SMALL_QUANT[key]
    got, _ = run_fused_moe(cfg, mi.make_inputs_np(cfg, 0))
    assert rel_l2(oracle.bf16_to_f32(got), oracle.bf16_to_f32(g[f"{key}_out_bf16"])) <= 3e-2


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_ragged_shapes_and_units(dtype):
    # intermediate not a multiple of the 128-column tile, hidden not a multiple of 256, odd counts
    inter = 384 if dtype == "fp8" else 416
    check(mi.MoeConfig("r", 77, 320, inter, 12, 3, dtype, "softmax_renorm", unit=32), seed=3)
    check(mi.MoeConfig("r", 130, 1152, 256, 6, 2, dtype, "softmax_renorm", unit=64), seed=4)
    check(mi.MoeConfig("r", 200, 256, 128, 3, 1, dtype, "softmax_renorm", unit=128), seed=5)
    check(mi.MoeConfig("r", 50, 256, 128, 16, 4, dtype, "softmax", unit=16), seed=6)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_local_expert_mask_and_unfused_entry(dtype):
    cfg = mi.MoeConfig("e", 96, 256, 256, 10, 3, dtype, "softmax_renorm")
    mask = (np.arange(cfg.experts) % 3 != 1).astype(np.int32)
    check(cfg, seed=7, mask=mask)
    check(cfg, seed=7, unfused=True)
    check(cfg, seed=8, stride_pad=64)


def test_skewed_routing_with_empty_experts():
    check(mi.MoeConfig("z", 3000, 256, 128, 64, 6, "bf16", "zipf"), seed=2)


def test_decode_shapes_int8():
    for T in (16, 64):
        check(mi.CONFIGS["cfg4_decode_int8_t64"].scaled(tokens=T, hidden=1024, inter=512))


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_decode_kernel_ragged(dtype):
    # <= 32 rows per expert selects the decode kernel (64 weight rows, 512-byte K runs split over the four
    # waves): K depths that are not a multiple of 512 bytes, column tails, a single token, empty experts
    inter = 384 if dtype == "fp8" else 288
    check(mi.MoeConfig("d", 24, 1056, inter, 16, 4, dtype, "softmax_renorm"), seed=1)
    # (a single fp8 token is too small a sample for a stable rel-L2 of the e4m3 rounding of Y: four there)
    check(mi.MoeConfig("d", 4 if dtype == "fp8" else 1, 480, 128, 8, 2, dtype, "softmax"), seed=2)
    check(mi.MoeConfig("d", 40, 2080, 640, 64, 8, dtype, "sigmoid_renorm", unit=16), seed=3)


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "int8"])
def test_two_block_decode_tiles(dtype):
    """28 .. 56 rows per expert with 16-bit or int8 operands: the decode kernel with two 32-row token blocks per
    tile (64-row tiles).  Ragged K depths and column tails, experts with more than 64 rows (two tiles) and with
    none, a sort unit that is not a multiple of 32, the expert mask, GELU and gate-only."""
    import therock_amd as ta
    chk = check_fp16 if dtype == "fp16" else check
    for i, (T, H, I, E, K, router, unit) in enumerate(((160, 512, 256, 8, 2, "softmax_renorm", 32),
                                                      (330, 1056, 288, 16, 2, "sigmoid_renorm", 16),
                                                      (100, 480, 128, 6, 2, "softmax", 8),
                                                      (640, 512, 256, 128, 8, "sigmoid_renorm", 32))):
        cfg = mi.MoeConfig("d2", T, H, I, E, K, dtype, router, unit)
        traits = ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, prec_o="fp16" if dtype == "fp16" else "bf16", block_m=unit)
        assert ta.fused_moe_tile_rows(traits, T, E, K, H, I) == 64, cfg
        chk(cfg, seed=i)
    cfg = mi.MoeConfig("d2", 160, 512, 256, 8, 2, dtype, "softmax_renorm")
    chk(cfg, seed=5, activation=0)
    chk(cfg, seed=6, gate_only=1)
    if dtype != "fp16":
        # 240 tokens over the five local experts of eight: about 36 rows each after the foreign slots drop out
        check(mi.MoeConfig("d2", 144, 512, 256, 8, 2, dtype, "softmax_renorm"), seed=7, mask=np.array([1, 0, 1, 1, 0, 1, 0, 1], dtype=np.int32))
    # a skewed routing: a few experts with several 64-row tiles, the tail with a handful of rows or none
    chk(mi.MoeConfig("d2_zipf", 320, 512, 256, 16, 2, dtype, "zipf"), seed=8)


def test_skewed_fp8_batch_takes_the_large_tiles_on_the_device():
    """fp8, 16 rows per expert on average: the host picks decode tiles.  With Zipf routing the experts that have
    tokens hold 48 padded rows or more each, and the sort, which has the counts, builds the work list for the 320-row
    tiles instead; both kernel families are launched and one of them finds nothing to do.  Same shapes with uniform
    routing, and with too few active experts to fill the chip, stay on the decode tiles.  Parity either way, also
    through the expert mask, gate-only weights and on a second call with another routing on the same workspace."""
    import torch
    import therock_amd as ta
    from tests.gpu_util import rel_l2, run_fused_moe

    def run(cfg, seed, want_rows, **kw):
        inp = mi.make_inputs_np(cfg, seed)
        mask = kw.get("mask")
        if mask is not None:
            nloc = int(mask.sum())
            for k in ("g", "d", "g_scale", "d_scale"):
                inp[k] = inp[k][:nloc]
        if kw.get("gate_only"):
            inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
            inp["g_scale"] = np.ascontiguousarray(inp["g_scale"][:, :cfg.inter])
        print(f"fused_moe {cfg} seed={seed} {kw}", flush=True)
        got, buf = run_fused_moe(cfg, inp, **kw)  # (unfused: mi355_moe_sorting + mi355_fused_moegemm, whose tile-list pass chooses)
        traits = ta.fused_moe_traits(prec_i="fp8", prec_w="fp8", block_m=cfg.unit, local_expert_masking=mask is not None,
                                     gate_only=kw.get("gate_only", 0))
        shape = (cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter)
        assert ta.fused_moe_tile_rows(traits, *shape) == 32
        rows = ta.fused_moe_chosen_tile_rows(traits, buf, *shape)
        ref, s = oracle_out(cfg, inp, mask, 1, kw.get("gate_only", 0))
        active = len(set(s[2][:s[3] // cfg.unit].tolist()))
        print(f"  tile rows chosen on the device: {rows}; {active} active experts, {s[3]} padded rows", flush=True)
        assert rows == want_rows
        assert np.array_equal(buf.sorted_ids[:s[3]].cpu().numpy(), s[0][:s[3]])
        err = rel_l2(oracle.bf16_to_f32(got), ref)
        print(f"  rel-L2 = {err:.3e} (tolerance {TOL['fp8']:.0e})", flush=True)
        assert np.all(np.isfinite(oracle.bf16_to_f32(got))) and err <= TOL["fp8"]

    zipf = mi.MoeConfig("skew", 256, 512, 2048, 64, 4, "fp8", "zipf")
    run(zipf, 1, 320)
    run(mi.MoeConfig("skew", 256, 512, 2048, 64, 4, "fp8", "softmax_renorm"), 2, 32)   # uniform: 16 rows per expert
    run(mi.MoeConfig("skew", 256, 512, 256, 64, 4, "fp8", "zipf"), 3, 32)              # two column tiles per expert: too few
    run(mi.MoeConfig("skew", 192, 512, 2048, 64, 4, "fp8", "zipf", unit=16), 4, 320)   # 16-row sort units, ragged tiles
    run(mi.MoeConfig("skew", 256, 512, 4096, 64, 4, "fp8", "zipf"), 5, 320, gate_only=1)  # (half the column tiles per expert)
    run(zipf, 6, 320, mask=np.array(([1, 1, 1, 1, 1, 1, 1, 0] * 8), dtype=np.int32))
    # 512 experts: the multi-phase sort (count / scan / scatter kernels) makes the same choice
    run(mi.MoeConfig("skew", 1024, 256, 2048, 512, 4, "fp8", "zipf"), 7, 320)
    run(mi.MoeConfig("skew", 1024, 256, 2048, 512, 4, "fp8", "softmax_renorm"), 8, 32)
    # the sort and the grouped GEMMs as two calls: the GEMM entry point's own tile-list pass makes the same choice
    run(zipf, 9, 320, unfused=True)
    run(mi.MoeConfig("skew", 256, 512, 2048, 64, 4, "fp8", "softmax_renorm"), 10, 32, unfused=True)
    run(zipf, 11, 320, unfused=True, mask=np.array(([1, 1, 1, 1, 1, 1, 1, 0] * 8), dtype=np.int32))


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_many_rows_per_expert_with_small_sort_units(dtype):
    # hundreds of rows per expert, but expert boundaries on multiples of 8 or 24 rows only: the 320-row kernel
    # (whose tiles start on whole 16-row slabs of the intermediate buffer) must not be chosen for unit 8 or 24
    import therock_amd as ta
    for unit, rows in ((8, 128), (24, 128), (16, 320), (48, 320)):
        cfg = mi.MoeConfig("u", 700, 256, 384, 3, 2, dtype, "softmax_renorm", unit=unit)
        traits = ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, block_m=unit)
        assert ta.fused_moe_tile_rows(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter) == rows
        check(cfg, seed=unit)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_large_tile_kernel_partial_tiles(dtype):
    # from about 28 (fp8) or 57 (other types) rows per expert on, and with enough tiles to fill the chip, the 320-row
    # kernel runs with mostly empty tiles: it then fetches only the 64-row slab groups a tile has (1 to 5 per step)
    import therock_amd as ta
    for cfg, seed in ((mi.MoeConfig("p", 640 if dtype == "fp8" else 960, 256, 512, 64, 4, dtype, "softmax_renorm"), 1),
                      (mi.MoeConfig("p", 1500, 256, 512, 64, 4, dtype, "zipf"), 2),
                      (mi.MoeConfig("p", 4000, 384, 512, 64, 6, dtype, "zipf", unit=64), 3)):
        traits = ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, block_m=cfg.unit)
        assert ta.fused_moe_tile_rows(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter) == 320
        check(cfg, seed=seed)


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
@pytest.mark.parametrize("activation,gate_only", [(0, 0), (1, 1), (0, 1)])
def test_gelu_and_gate_only(dtype, activation, gate_only):
    # the other activation of fused_moe_traits (gelu, erf form) and gate-only weights ([e, inter, hidden],
    # y = act(gate)), through each of the three GEMM kernels: small tiles, decode tiles, 320-row tiles
    kw = dict(activation=activation, gate_only=gate_only)
    inter = 384 if dtype == "fp8" else 416  # not a multiple of the 256 columns a gate-only tile covers
    check(mi.MoeConfig("a", 77, 320, inter, 12, 3, dtype, "softmax_renorm"), seed=3, **kw)
    check(mi.MoeConfig("a", 24, 1056, 384 if dtype == "fp8" else 288, 16, 4, dtype, "softmax_renorm"), seed=1, **kw)
    check(mi.MoeConfig("a", 700, 256, 384, 3, 2, dtype, "softmax_renorm"), seed=2, **kw)
    check(mi.MoeConfig("a", 96, 256, 256, 10, 3, dtype, "softmax_renorm"), seed=4, unfused=True, **kw)


def _check_routing(cfg, ids, w, seed=0):
    """check() with a hand-made routing instead of the generator's."""
    from tests.gpu_util import rel_l2, run_fused_moe
    inp = mi.make_inputs_np(cfg, seed)
    inp["topk_ids"], inp["topk_weight"] = ids.astype(np.int32), w.astype(np.float32)
    print(f"fused_moe {cfg} hand-made routing", flush=True)
    got, buf = run_fused_moe(cfg, inp)
    ref, s = oracle_out(cfg, inp)
    assert int(buf.total[0]) == s[3]
    assert np.array_equal(buf.sorted_ids[:s[3]].cpu().numpy(), s[0][:s[3]])
    err = rel_l2(oracle.bf16_to_f32(got), ref)
    print(f"  rel-L2 = {err:.3e}", flush=True)
    assert err <= TOL[cfg.dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp8", "int8"])
def test_extreme_routings(dtype):
    rng = np.random.default_rng(5)
    # every token picks the same experts: one bucket per slot holds all tokens, every other expert is empty
    cfg = mi.MoeConfig("x", 700, 256, 256, 16, 3, dtype, "softmax")
    _check_routing(cfg, np.tile(np.array([11, 2, 7]), (cfg.tokens, 1)), rng.random((cfg.tokens, 3)))
    # top-k = experts: every token visits every expert, in a different order per token
    cfg = mi.MoeConfig("x", 40, 128, 128, 8, 8, dtype, "softmax")
    _check_routing(cfg, np.stack([rng.permutation(8) for _ in range(cfg.tokens)]), rng.random((cfg.tokens, 8)))
    # a single expert, a single slot; zero and negative top-k weights
    cfg = mi.MoeConfig("x", 33, 128, 128, 1, 1, dtype, "softmax")
    _check_routing(cfg, np.zeros((cfg.tokens, 1)), rng.standard_normal((cfg.tokens, 1)) * (rng.random((cfg.tokens, 1)) < 0.7))
    # the most experts the path takes, a wide top-k, a handful of tokens
    cfg = mi.MoeConfig("x", 5, 128, 128, 1024, 48, dtype, "softmax")
    _check_routing(cfg, np.stack([rng.permutation(1024)[:48] for _ in range(cfg.tokens)]), rng.random((cfg.tokens, 48)))


@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
def test_no_local_expert(dtype):
    # a rank that owns none of the experts: nothing is sorted, no tile exists, the output is all zeros
    from tests.gpu_util import run_fused_moe
    cfg = mi.MoeConfig("m", 50, 128, 128, 6, 2, dtype, "softmax")
    inp = mi.make_inputs_np(cfg, 1)
    mask = np.zeros(cfg.experts, dtype=np.int32)
    for k in ("g", "d", "g_scale", "d_scale"):  # one expert's worth of storage, never read
        if inp[k] is not None:
            inp[k] = inp[k][:1]
    got, buf = run_fused_moe(cfg, inp, mask=mask)
    assert int(buf.total[0]) == 0
    assert np.all(oracle.bf16_to_f32(got) == 0.0)


def test_invalid_sizes_are_rejected():
    import torch
    import therock_amd as ta
    t = ta.fused_moe_traits()
    z = lambda *sh, dt=torch.bfloat16: torch.zeros(sh, dtype=dt, device="cuda")

    def call(T, E, K, H, I, traits=t):
        buf = ta.MoeBuffers(ta.fused_moe_traits(), T, E, K, 128, 128, "cuda")
        buf.out = z(T, H)
        args = ta.make_args(traits, buf, z(T, H), z(E, 2 * I, H), z(E, H, I), z(T, K, dt=torch.int32), z(T, K, dt=torch.float32))
        return ta.fused_moegemm(traits, args)

    assert call(4, 4, 2, 100, 128) == -1.0      # hidden not a multiple of 32
    assert call(4, 4, 2, 128, 96 + 16) == -1.0  # intermediate not a multiple of 32
    with pytest.raises(RuntimeError, match="bad sizes"):
        call(4, 2000, 2, 128, 128)               # more experts than the path takes
    t8 = ta.fused_moe_traits(prec_i="fp8", prec_w="fp8")
    buf = ta.MoeBuffers(t8, 4, 4, 2, 128, 96, "cuda")
    u8 = lambda *sh: torch.zeros(sh, dtype=torch.uint8, device="cuda")
    f32 = lambda *sh: torch.ones(sh, dtype=torch.float32, device="cuda")
    args = ta.make_args(t8, buf, u8(4, 128), u8(4, 192, 128), u8(4, 128, 96), z(4, 2, dt=torch.int32), f32(4, 2),
                        a_scale=f32(4), g_scale=f32(4, 192), d_scale=f32(4, 128))
    assert ta.fused_moegemm(t8, args) == -1.0    # fp8 keeps one scale per 32 Y columns in groups of four: inter % 128


def test_no_tokens():
    import torch
    import therock_amd as ta
    t = ta.fused_moe_traits()
    buf = ta.MoeBuffers(t, 0, 4, 2, 128, 128, "cuda")
    z = lambda *sh, dt=torch.bfloat16: torch.zeros(sh, dtype=dt, device="cuda")
    args = ta.make_args(t, buf, z(0, 128), z(4, 256, 128), z(4, 128, 128), z(0, 2, dt=torch.int32), z(0, 2, dt=torch.float32))
    args.stride_token = 128
    assert ta.fused_moe(t, args) == 0.0
    torch.cuda.synchronize()


def test_traits_without_kernel_return_minus_one():
    import torch
    import therock_amd as ta
    for kw in (dict(prec_i="fp16", prec_w="fp16"), dict(activation=2), dict(gate_only=2), dict(prec_o="fp32")):
        assert ta.fused_moe(ta.fused_moe_traits(**kw), ta.fused_moe_args()) == -1.0
    t = ta.fused_moe_traits()
    buf = ta.MoeBuffers(t, 4, 4, 2, 128, 128, "cuda")
    a = torch.zeros((4, 128), dtype=torch.bfloat16, device="cuda")
    g = torch.zeros((4, 256, 128), dtype=torch.bfloat16, device="cuda")
    d = torch.zeros((4, 128, 128), dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros((4, 2), dtype=torch.int32, device="cuda")
    w = torch.zeros((4, 2), dtype=torch.float32, device="cuda")
    args = ta.make_args(t, buf, a, g, d, ids, w)
    args.workspace = None
    with pytest.raises(RuntimeError, match="workspace"):
        ta.fused_moe(t, args)


@pytest.mark.parametrize("dtype", ["bf16", "fp8"])
def test_large_tile_kernel(dtype):
    # >= 160 rows per expert selects the 256-row tile kernel (global->LDS DMA ring): full tiles,
    # ragged tiles, padding ids, column tails and a K depth that is not a multiple of the ring
    check(mi.MoeConfig("b", 1024, 512, 384, 8, 2, dtype, "softmax_renorm"), seed=1)
    check(mi.MoeConfig("b", 700, 320, 128, 4, 1, dtype, "softmax_renorm", unit=64), seed=2)
    check(mi.MoeConfig("b", 2000, 192, 256, 6, 3, dtype, "zipf"), seed=3)
    check(mi.MoeConfig("b", 600, 64, 128, 2, 1, dtype, "softmax_renorm"), seed=4)


# ---- fp16 operands and output: ck_tile's other instance (fused_moegemm_pipeline_flatmm_policy.hpp:790-807)
def check_fp16(cfg, seed=0, **kw):
    from tests.gpu_util import rel_l2, run_fused_moe
    inp = mi.make_inputs_np(cfg, seed)
    if kw.get("gate_only"):
        inp["g"] = np.ascontiguousarray(inp["g"][:, :cfg.inter])
    print(f"fused_moe {cfg} seed={seed} {kw}", flush=True)
    got, buf = run_fused_moe(cfg, inp, **kw)
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], cfg.experts, cfg.unit)
    ref = oracle.fused_moe_f16(inp["a"].view(np.float16), inp["g"].view(np.float16), inp["d"].view(np.float16), *s, cfg.unit,
                               cfg.tokens, cfg.experts, cfg.hidden, cfg.inter, cfg.topk, activation=kw.get("activation", 1),
                               gate_only=bool(kw.get("gate_only", 0))).astype(np.float32)
    got = got.view(np.float16).astype(np.float32)
    assert np.all(np.isfinite(got))
    err = rel_l2(got, ref)
    print(f"  rel-L2 = {err:.3e} (tolerance 1e-02)", flush=True)
    assert err <= 1e-2
    return err


@pytest.mark.parametrize("cfg", [
    mi.MoeConfig("f16_decode", 8, 128, 128, 4, 2, "fp16"),
    mi.MoeConfig("f16_mid", 300, 512, 384, 8, 2, "fp16"),
    mi.MoeConfig("f16_mid_sigmoid", 48, 512, 256, 16, 4, "fp16", "sigmoid_renorm"),
    mi.MoeConfig("f16_big", 2048, 512, 256, 8, 2, "fp16"),
], ids=lambda c: c.name)
def test_fp16(cfg):
    err = check_fp16(cfg)
    assert err <= 2e-3  # fp16 Y and partial rows: three more bits than the bf16 path's 3.3e-3


def test_fp16_variants():
    check_fp16(mi.MoeConfig("f16_gelu", 128, 256, 256, 8, 2, "fp16"), activation=0)
    check_fp16(mi.MoeConfig("f16_gate_only", 128, 256, 256, 8, 2, "fp16"), gate_only=1)
    check_fp16(mi.MoeConfig("f16_unfused", 128, 256, 256, 8, 2, "fp16"), unfused=True)
