"""The fused path inside a captured HIP graph: launches only (no allocation, no host synchronisation, no
memset node), so serving loops can capture it.  Every replay is checked against the eager result, with
eager work and synchronisations between the replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,scale,fused_quant", [
    ("cfg4_decode_int8_t64", dict(hidden=1024, inter=512), 0),
    ("cfg1_cpu_ref_bf16", {}, 0),
    ("cfg3_dsv3_fp8", dict(tokens=2048, hidden=512, inter=256, experts=8), 0),
    # fp8 with skewed routing: two kernel families per GEMM, the sort decides on the device which one has work
    ("cfg3_dsv3_fp8", dict(tokens=256, hidden=512, inter=2048, experts=64, topk=4, router="zipf"), 0),
    # the decode kernel with two token blocks per tile (40 rows per expert)
    ("cfg4_decode_int8_t64", dict(tokens=160, hidden=1024, inter=512, experts=32), 0),
    # with the re-quantisation pass between the GEMMs (decode kernel / large-tile kernel)
    ("cfg4_decode_int8_t64", dict(hidden=1024, inter=512), 2),
    ("cfg4_decode_int8_t64", dict(tokens=2048, hidden=512, inter=256, experts=8), 2),
    # fp8 with re-quantised rows: the pass between the GEMMs, the fill of the unit block scales, row scales in the combine
    ("cfg3_dsv3_fp8", dict(tokens=64, hidden=512, inter=256, experts=16, topk=4), 2),
    ("cfg3_dsv3_fp8", dict(tokens=2048, hidden=512, inter=256, experts=8), 2)])
def test_capture_and_replay(name, scale, fused_quant):
    import torch

    import therock_amd as ta
    from therock_amd import inputs as mi

    cfg = mi.CONFIGS[name].scaled(**scale) if scale else mi.CONFIGS[name]
    dev = torch.device("cuda:0")
    inp = mi.make_inputs_torch(cfg, dev, 0)
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit, fused_quant=fused_quant)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, dev)
    args = ta.make_args(traits, buf, inp["a"], inp["g"], inp["d"], inp["topk_ids"], inp["topk_weight"],
                        a_scale=inp["a_scale"], g_scale=inp["g_scale"], d_scale=inp["d_scale"])
    assert ta.fused_moe(traits, args) == 0.0  # first call outside the capture (per-kernel attributes are set once)
    torch.cuda.synchronize()
    ref = buf.out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    scratch = torch.empty((1 << 20,), device=dev)
    for r in range(4):
        buf.out.fill_(float("nan"))
        scratch.normal_()          # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(buf.out.view(torch.int16), ref.view(torch.int16)), f"replay {r} differs from the eager result"
