"""Parity at the full benchmark sizes, where the oracle cannot run the whole problem.

* moe_sorting: bit-exact against the oracle on the full routing (the oracle's sort is fast).
* fused MoE: a token's output depends only on that token, its experts and their weights, so a
  handful of sampled tokens are re-run through the oracle as a compact sub-problem (their experts
  renumbered 0..E'-1, weights copied to the host) and compared within the stated tolerance.
* size-independent properties: two runs give identical bits (no atomics anywhere in the path), and
  doubling every top-k weight doubles every output exactly (power-of-two scaling commutes with all
  roundings on the path)."""
import numpy as np
import pytest
import torch

import oracle
import therock_amd as ta
from therock_amd import inputs as mi

pytestmark = pytest.mark.gpu

DT = {"bf16": oracle.DT_BF16, "fp8": oracle.DT_E4M3, "int8": oracle.DT_I8}
NPV = {"bf16": torch.uint16, "fp8": torch.uint8, "int8": torch.int8}
TOL = {"bf16": 1e-2, "fp8": 3e-2, "int8": 3e-2}


def host(t, cfg):
    return t.contiguous().view(NPV[cfg.dtype]).cpu().numpy()


def sampled_oracle(cfg, inp, tokens):
    """Oracle output [len(tokens), H] (float32 of the bf16 result) for the sampled tokens."""
    ids = inp["topk_ids"][tokens].cpu().numpy()
    w = inp["topk_weight"][tokens].cpu().numpy()
    experts = np.unique(ids)
    remap = {int(e): i for i, e in enumerate(experts)}
    ids_c = np.vectorize(remap.get)(ids).astype(np.int32)
    et = torch.from_numpy(experts).to(inp["g"].device).long()
    byte_view = lambda x: x.view(torch.uint8) if x.element_size() == 1 else x
    g = host(byte_view(inp["g"])[et].view(inp["g"].dtype), cfg)
    d = host(byte_view(inp["d"])[et].view(inp["d"].dtype), cfg)
    tt = torch.as_tensor(tokens, device=inp["a"].device).long()
    a = host(byte_view(inp["a"])[tt].view(inp["a"].dtype), cfg)
    sc = lambda k, idx: None if inp[k] is None else inp[k][idx].cpu().numpy()
    s = oracle.moe_sorting(ids_c, w, len(experts), cfg.unit)
    dt = DT[cfg.dtype]
    o = oracle.fused_moe(a, dt, g, dt, d, dt, *s, cfg.unit, len(tokens), len(experts), cfg.hidden, cfg.inter,
                         cfg.topk, a_scale=sc("a_scale", tt), g_scale=sc("g_scale", et), d_scale=sc("d_scale", et))
    return oracle.bf16_to_f32(o)


@pytest.mark.parametrize("name", list(mi.CONFIGS))
def test_full_size_workload(name):
    from tests.gpu_util import rel_l2
    cfg = mi.CONFIGS[name]
    print(f"full-size {cfg}", flush=True)
    inp = mi.make_inputs_torch(cfg, "cuda", seed=0)
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, "cuda")
    args = ta.make_args(traits, buf, inp["a"], inp["g"], inp["d"], inp["topk_ids"], inp["topk_weight"],
                        a_scale=inp["a_scale"], g_scale=inp["g_scale"], d_scale=inp["d_scale"])
    assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    out1 = buf.out.clone()

    # sorting: bit-exact on the full routing
    s = oracle.moe_sorting(inp["topk_ids"].cpu().numpy(), inp["topk_weight"].cpu().numpy(), cfg.experts, cfg.unit)
    pp = s[3]
    assert int(buf.total[0]) == pp and int(buf.total[1]) == cfg.tokens
    assert np.array_equal(buf.sorted_ids[:pp].cpu().numpy(), s[0][:pp])
    assert np.array_equal(buf.sorted_w[:pp].cpu().numpy(), s[1][:pp])
    assert np.array_equal(buf.sorted_eid[:pp // cfg.unit].cpu().numpy(), s[2][:pp // cfg.unit])

    # sampled tokens against the oracle
    rng = np.random.default_rng(1)
    n = 6 if cfg.hidden * cfg.inter > 2e7 else 16
    tokens = np.sort(rng.choice(cfg.tokens, size=min(n, cfg.tokens), replace=False))
    ref = sampled_oracle(cfg, inp, tokens)
    got = out1[torch.as_tensor(tokens, device="cuda").long()].float().cpu().numpy()
    err = rel_l2(got, ref)
    print(f"  {name}: sampled-token rel-L2 = {err:.3e} (tolerance {TOL[cfg.dtype]:.0e})", flush=True)
    assert torch.isfinite(out1.float()).all()
    assert err <= TOL[cfg.dtype]

    # determinism: same bits on a second run
    assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    assert torch.equal(out1.view(torch.uint16), buf.out.view(torch.uint16))

    # linearity in the top-k weights: x2 is exact in every rounding on the path
    w2 = (inp["topk_weight"] * 2).contiguous()
    args.topk_weight_ptr = w2
    assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    assert torch.equal((out1.float() * 2).to(torch.bfloat16).view(torch.uint16), buf.out.view(torch.uint16))
