"""mi355_fused_moe_static_ws, the entry point that allocates nothing (library-owned workspace), against
mi355_fused_moe with a caller workspace: bit-identical outputs and sort results, two calls in a row with the
second on a smaller input (the shared buffer keeps the first call's contents)."""
import numpy as np
import pytest

from therock_amd import inputs as mi
from tests.gpu_util import TORCH_DT, dev

pytestmark = pytest.mark.gpu


def _run(cfg, seed, static):
    import torch
    import therock_amd as ta

    inp = mi.make_inputs_np(cfg, seed)
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, "cuda")
    buf.sorted_ids.fill_(-1)
    buf.sorted_w.fill_(-1.0)
    buf.sorted_eid.fill_(-1)
    view = TORCH_DT[cfg.dtype]
    sc = {k: (None if inp[k] is None else dev(inp[k])) for k in ("a_scale", "g_scale", "d_scale")}
    args = ta.make_args(traits, buf, dev(inp["a"]).view(view), dev(inp["g"]).view(view), dev(inp["d"]).view(view),
                        dev(inp["topk_ids"]), dev(inp["topk_weight"]), a_scale=sc["a_scale"], g_scale=sc["g_scale"],
                        d_scale=sc["d_scale"])
    if static:
        args.workspace = None  # nothing of the caller's is used as scratch
        assert ta.fused_moe_static_ws(traits, args) == 0.0
    else:
        assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    return (buf.out.view(torch.uint16).cpu().numpy(), buf.sorted_ids.cpu().numpy(), buf.sorted_w.cpu().numpy(),
            buf.sorted_eid.cpu().numpy(), buf.total.cpu().numpy())


@pytest.mark.parametrize("dtype", ["int8", "bf16", "fp8"])
def test_static_workspace_entry_point_matches_the_caller_workspace_one(dtype):
    import therock_amd as ta

    big = mi.MoeConfig("n", 64, 1024, 512, 32, 4, dtype, "softmax")        # decode-sized: decode kernels
    small = mi.MoeConfig("n", 9, 512, 256, 8, 2, dtype, "softmax_renorm")  # smaller, other shapes: stale contents around
    mid = mi.MoeConfig("n", 700, 256, 128, 4, 2, dtype, "softmax_renorm")  # large-tile kernels, still within capacity
    for cfg, seed in ((big, 1), (small, 2), (mid, 3)):
        traits = ta.fused_moe_traits(prec_i=dtype, prec_w=dtype, block_m=cfg.unit)
        need = ta.fused_moe_get_workspace_size(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter)
        assert 0 < need <= ta.fused_moe_static_ws_capacity()
        ref = _run(cfg, seed, static=False)
        got = _run(cfg, seed, static=True)
        for r, g, name in zip(ref, got, ("out", "sorted_ids", "sorted_w", "sorted_eid", "total")):
            assert np.array_equal(r, g), f"{dtype} {cfg}: {name} differs"


def _prepared(cfg, seed):
    import therock_amd as ta

    inp = mi.make_inputs_np(cfg, seed)
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, block_m=cfg.unit)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, "cuda")
    view = TORCH_DT[cfg.dtype]
    sc = {k: (None if inp[k] is None else dev(inp[k])) for k in ("a_scale", "g_scale", "d_scale")}
    args = ta.make_args(traits, buf, dev(inp["a"]).view(view), dev(inp["g"]).view(view), dev(inp["d"]).view(view),
                        dev(inp["topk_ids"]), dev(inp["topk_weight"]), a_scale=sc["a_scale"], g_scale=sc["g_scale"],
                        d_scale=sc["d_scale"])
    args.workspace = None
    return traits, buf, args


def test_static_workspace_calls_allocate_no_device_memory():
    """The contract of the entry point: after the first call on a device (which looks up the address of the library's
    array) no call changes the amount of free device memory - neither the driver's figure nor torch's allocator."""
    import torch
    import therock_amd as ta

    traits, buf, args = _prepared(mi.MoeConfig("n", 64, 1024, 512, 32, 4, "int8", "softmax"), 4)
    assert ta.fused_moe_static_ws(traits, args) == 0.0   # warm-up: symbol lookup, per-kernel attributes
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0, allocated0 = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
    for _ in range(5):
        assert ta.fused_moe_static_ws(traits, args) == 0.0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"free device memory went from {free0} to {free1} bytes"
    assert (torch.cuda.memory_reserved(), torch.cuda.memory_allocated()) == (reserved0, allocated0)


def test_static_workspace_call_inside_a_captured_graph():
    """What the entry point is for: a capture, where nothing may be allocated.  The first call on the device comes
    before the capture (the address lookup is not a stream operation); every replay is checked against the eager
    result, with eager work and synchronisations between the replays."""
    import torch
    import therock_amd as ta

    traits, buf, args = _prepared(mi.MoeConfig("n", 48, 512, 256, 16, 4, "fp8", "softmax_renorm"), 5)
    assert ta.fused_moe_static_ws(traits, args) == 0.0
    torch.cuda.synchronize()
    ref = buf.out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert ta.fused_moe_static_ws(traits, args) == 0.0
    torch.cuda.synchronize()
    scratch = torch.empty((1 << 18,), device="cuda")
    for r in range(3):
        buf.out.fill_(float("nan"))
        scratch.normal_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(buf.out.view(torch.int16), ref.view(torch.int16)), f"replay {r} differs from the eager result"


def test_static_workspace_rejects_what_does_not_fit():
    import therock_amd as ta

    t = ta.fused_moe_traits(prec_i="fp8", prec_w="fp8")
    assert ta.fused_moe_get_workspace_size(t, 8192, 256, 8, 7168, 2048) > ta.fused_moe_static_ws_capacity()
    args = ta.fused_moe_args(block_m=32, hidden_size=7168, intermediate_size=2048, num_tokens=8192, num_experts=256,
                             topk=8, stride_token=7168)
    with pytest.raises(RuntimeError, match="library-owned"):
        ta.fused_moe_static_ws(t, args)
