"""GPU parity of the int8 and fp8 paths with fused_quant 1 (smooth-dynamic-quant) and 2 (dynamic-quant) of ck_tile's
fused_moe_traits: the intermediate activations are re-quantised to int8 (e4m3) per row between the two GEMMs, with the
per-expert smooth scale of FusedMoeGemmHostArgs::y_smooth_scale_ptr (fused_moegemm_kernel.hpp:103) for variant 1,
whose activations arrive as one quantised row per (slot, token) ([topk, tokens, hidden] with scales
[topk, tokens], moe_sorting_kernel.hpp:82-83).

ck_tile 1.2.0 ships no instance of these variants and its host reference ignores every scale tensor, so the
reference is the de-quantised one used for all quantised paths: the oracle fed float operands.  The smooth
scale enters it folded into the de-quantised down weights ((y * s) . d = y . (s * d)); the per-(slot, token)
activations enter it as tokens * topk pseudo tokens with one slot each, whose fp32 partial rows are then summed
in slot order and rounded once, like reference_fused_moe.hpp:186-197 does.  Tolerance: rel-L2 <= 3e-2 (int8, fp8)."""
import numpy as np
import pytest
import torch

import oracle
import therock_amd as ta
from therock_amd import inputs as mi

pytestmark = pytest.mark.gpu

TOL = 3e-2
QDT = {"int8": oracle.DT_I8, "fp8": oracle.DT_E4M3}
VIEW = {"int8": torch.int8, "fp8": torch.float8_e4m3fn}


def reference(cfg, inp, fq, sm_y, a_q, a_scale, mask=None):
    T, K, H, I, E = cfg.tokens, cfg.topk, cfg.hidden, cfg.inter, cfg.experts
    assert mask is None or fq == 2
    qdt = QDT[cfg.dtype]
    d = oracle.to_f32(inp["d"], qdt) * inp["d_scale"][:, :, None]
    if fq == 1:
        d = d * sm_y[:, None, :]
        # pseudo token slot * T + token, one slot each
        s_ids, s_w, s_eid, pp = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], E, cfg.unit)
        slot = (s_ids.astype(np.uint32) >> 24).astype(np.int64)
        tok = (s_ids & 0xffffff).astype(np.int64)
        real = tok < T
        pid = np.where(real, slot * T + tok, T * K).astype(np.int32)
        o, part = oracle.fused_moe(a_q.reshape(K * T, H), qdt, inp["g"], qdt, d, oracle.DT_F32, pid, s_w,
                                   s_eid, pp, cfg.unit, K * T, E, H, I, 1, a_scale=a_scale.reshape(K * T),
                                   g_scale=inp["g_scale"], want_partials=True)
        acc = np.zeros((T, H), dtype=np.float32)
        for k in range(K):  # slot order
            acc += part[k * T:(k + 1) * T, 0]
        return oracle.bf16_to_f32(oracle.f32_to_bf16(acc))
    s = oracle.moe_sorting(inp["topk_ids"], inp["topk_weight"], E, cfg.unit, local_expert_mask=mask)
    o = oracle.fused_moe(a_q, qdt, inp["g"], qdt, d, oracle.DT_F32, *s, cfg.unit, T, inp["g"].shape[0], H, I,
                         K, a_scale=a_scale, g_scale=inp["g_scale"])
    return oracle.bf16_to_f32(o)


def run(cfg, fq, seed=0, mask=None):
    from tests.gpu_util import dev, rel_l2
    print(f"fused_quant={fq} {cfg} seed={seed} mask={mask is not None}", flush=True)
    inp = mi.make_inputs_np(cfg, seed)
    if mask is not None:  # weights of the local experts only, indexed by local id
        nloc = int(mask.sum())
        for k in ("g", "d", "g_scale", "d_scale"):
            inp[k] = inp[k][:nloc]
    rng = np.random.Generator(np.random.Philox(seed + 77))
    T, K, H, I, E = cfg.tokens, cfg.topk, cfg.hidden, cfg.inter, cfg.experts
    sm_y = None
    if fq == 1:
        sm_x = rng.uniform(0.5, 2.0, size=(E, H)).astype(np.float32)
        sm_y = rng.uniform(0.25, 4.0, size=(E, I)).astype(np.float32)
        x = mi.bf16_bits_to_f32(inp["a_bf16"])
        a_q, a_scale = oracle.smoothquant(x, sm_x, inp["topk_ids"], QDT[cfg.dtype])  # [K, T, H], [K, T]
    else:
        a_q, a_scale = inp["a"], inp["a_scale"]
    ref = reference(cfg, inp, fq, sm_y, a_q, a_scale, mask)

    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit, fused_quant=fq,
                                 local_expert_masking=mask is not None)
    buf = ta.MoeBuffers(traits, T, E, K, H, I, "cuda")
    buf.ws.fill_(0x5A)  # a dirty workspace
    view = VIEW[cfg.dtype]
    a_dev = dev(a_q).view(view)
    args = ta.make_args(traits, buf, a_dev.reshape(-1, H)[:T], dev(inp["g"]).view(view), dev(inp["d"]).view(view),
                        dev(inp["topk_ids"]), dev(inp["topk_weight"]), a_scale=dev(a_scale), g_scale=dev(inp["g_scale"]),
                        d_scale=dev(inp["d_scale"]), local_expert_mask=None if mask is None else dev(mask.astype(np.int32)),
                        num_experts=E)
    args.a_ptr = a_dev.data_ptr()
    keep = None
    if fq == 1:
        keep = dev(sm_y)
        args.y_smooth_scale_ptr = keep
    assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    got = oracle.bf16_to_f32(buf.out.view(torch.uint16).cpu().numpy())
    assert np.all(np.isfinite(got))
    err = rel_l2(got, ref)
    print(f"  rel-L2 = {err:.3e} (tolerance {TOL:.0e})", flush=True)
    assert err <= TOL
    return got


# 16 rows per expert: decode kernel; 40: decode kernel with two token blocks per tile; 128: 128-row tiles;
# 512 / 640: large-tile kernel (I % 128 == 0)
SHAPES = [
    mi.MoeConfig("fq_decode", 64, 256, 256, 8, 2, "int8", "softmax_renorm"),
    mi.MoeConfig("fq_decode_two_blocks", 160, 512, 256, 8, 2, "int8", "softmax_renorm"),
    mi.MoeConfig("fq_mid", 384, 512, 384, 8, 2, "int8", "softmax_renorm"),
    mi.MoeConfig("fq_big", 2048, 512, 256, 8, 2, "int8", "softmax_renorm"),
    mi.MoeConfig("fq_big_unit64", 640, 256, 1536, 4, 4, "int8", "sigmoid_renorm", 64),
]


@pytest.mark.parametrize("fq", [1, 2])
@pytest.mark.parametrize("dtype", ["int8", "fp8"])
@pytest.mark.parametrize("cfg", SHAPES, ids=lambda c: c.name)
def test_fused_quant_matches_dequantised_reference(cfg, fq, dtype):
    run(cfg.scaled(dtype=dtype), fq)


def test_fused_quant_with_local_expert_mask():
    """A rank that owns some of the experts: the sort renumbers them, the re-quantisation pass and the down GEMM see
    local ids, slots of foreign experts drop out."""
    mask = np.array([1, 0, 1, 1, 0, 1, 0, 1], dtype=np.int32)
    run(SHAPES[2], 2, mask=mask)
    run(SHAPES[3], 2, mask=mask)
    run(SHAPES[3].scaled(dtype="fp8"), 2, mask=mask)


def test_fused_quant_is_deterministic():
    cfg = SHAPES[3]
    a = run(cfg, 2)
    b = run(cfg, 2)
    assert np.array_equal(a, b)


def test_fused_quant_argument_checks():
    """y_smooth_scale goes with fused_quant 1 and only with it; fused_quant needs int8 or fp8 operands."""
    from tests.gpu_util import dev
    cfg = SHAPES[0]
    inp = mi.make_inputs_np(cfg, 0)
    T, K, H, I, E = cfg.tokens, cfg.topk, cfg.hidden, cfg.inter, cfg.experts
    for fq, with_scale in ((1, False), (2, True), (0, True)):
        traits = ta.fused_moe_traits(prec_i="int8", prec_w="int8", block_m=cfg.unit, fused_quant=fq)
        buf = ta.MoeBuffers(traits, T, E, K, H, I, "cuda")
        a_rows = K * T if fq == 1 else T
        a = torch.zeros((a_rows, H), dtype=torch.int8, device="cuda")
        args = ta.make_args(traits, buf, a[:T], dev(inp["g"]).view(torch.int8), dev(inp["d"]).view(torch.int8),
                            dev(inp["topk_ids"]), dev(inp["topk_weight"]),
                            a_scale=torch.ones((a_rows,), dtype=torch.float32, device="cuda"),
                            g_scale=dev(inp["g_scale"]), d_scale=dev(inp["d_scale"]))
        sm = torch.ones((E, I), dtype=torch.float32, device="cuda")
        args.y_smooth_scale_ptr = sm if with_scale else None
        with pytest.raises(RuntimeError):
            ta.fused_moe(traits, args)
    traits = ta.fused_moe_traits(prec_i="bf16", prec_w="bf16", block_m=32, fused_quant=2)
    assert ta.fused_moe_get_workspace_size(traits, T, E, K, H, I) == 0
