"""GPU parity of the stand-alone grouped GEMMs (mi355_moe_flatmm) against the oracle, through the C ABI."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _bits(t):
    import torch
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _rel(a, b):
    a, b = a.astype(np.float64), b.astype(np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


# (tokens, experts, topk, hidden, inter, unit): decode kernel, 128-row tiles, decode kernel with two token blocks
# per tile (fp8: 64-row tiles), large-tile kernel
SHAPES = [(24, 16, 4, 512, 256, 32), (300, 8, 2, 256, 384, 32), (130, 6, 2, 1152, 256, 64), (1024, 4, 2, 512, 384, 32)]


def _c_types(kind):
    """C's torch dtype, the oracle's code for it and the rel-L2 tolerance: fp16 operands give an fp16 C."""
    import torch
    if kind == "fp16":
        return torch.float16, oracle.DT_F16, 2e-3
    return torch.bfloat16, oracle.DT_BF16, (1e-2 if kind == "bf16" else 3e-2)


@pytest.mark.parametrize("T,E,K,H,I,unit", SHAPES)
@pytest.mark.parametrize("kind", ["bf16", "fp16", "int8", "fp8"])
def test_gate_up_then_down(T, E, K, H, I, unit, kind):
    import torch
    import therock_amd as ta
    from tests.gpu_util import run_sorting

    rng = np.random.default_rng(T + H)
    cdt, odt, tol = _c_types(kind)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32)
    s_ids, s_w, s_eid, total = run_sorting(ids, w, E, unit, fill=True)
    pp = int(total[0])
    ref_sort = oracle.moe_sorting(ids, w, E, unit)
    assert pp == ref_sort[3]
    dev = lambda a: torch.from_numpy(a).cuda()
    bf = lambda a: torch.from_numpy(a).cuda().to(cdt)
    x32 = rng.standard_normal((T, H)).astype(np.float32)
    g32 = (rng.standard_normal((E, 2 * I, H)) * 0.05).astype(np.float32)
    d32 = (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32)
    d_ids, d_w, d_eid, d_tot = dev(s_ids), dev(s_w), dev(s_eid), dev(total.astype(np.int32))
    if kind in ("bf16", "fp16"):
        x, g, d = bf(x32), bf(g32), bf(d32)
        xr, gr, dr = x.float().cpu().numpy(), g.float().cpu().numpy(), d.float().cpu().numpy()
        sa = sg = sd = None
        d_sa = d_sg = d_sd = None
    else:
        qdt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
        kw = dict(nearest=True) if kind == "int8" else {}
        xq, sa = oracle.rowwise_quant(x32, qdt, **kw)
        gq, sg = oracle.rowwise_quant(g32.reshape(E * 2 * I, H), qdt, **kw)
        dq, sd = oracle.rowwise_quant(d32.reshape(E * H, I), qdt, **kw)
        x, g, d = dev(xq), dev(gq.reshape(E, 2 * I, H)), dev(dq.reshape(E, H, I))
        xr, gr, dr = (oracle.to_f32(xq, qdt), oracle.to_f32(gq.reshape(E, 2 * I, H), qdt),
                      oracle.to_f32(dq.reshape(E, H, I), qdt))
        sg, sd = sg.reshape(E, 2 * I), sd.reshape(E, H)
        d_sa, d_sg, d_sd = dev(sa), dev(sg), dev(sd)

    # gate+up: every (token, slot) row written exactly, nothing else touched
    y = torch.full((T * K + 3, I), float("nan"), dtype=cdt, device="cuda")
    assert ta.moe_flatmm(ta.GEMM1_GATE_UP, x, g, y, d_ids, d_eid, d_tot, T, K, unit, scale_m=d_sa, scale_n=d_sg) == 0.0
    torch.cuda.synchronize()
    y_ref = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, xr, gr, np.zeros((T * K, I), np.uint16), T, K, sa, sg,
                            c_dtype=odt)
    yg = y.float().cpu().numpy()
    assert np.isnan(yg[T * K:]).all() and not np.isnan(yg[:T * K]).any()
    assert _rel(yg[:T * K], oracle.to_f32(y_ref, odt)) <= tol

    # the same with B as ck_tile::shuffle_b hands it to a flatmm kernel (16-row warp tiles): read in place, same bits
    y2 = torch.full_like(y, float("nan"))
    assert ta.moe_flatmm(ta.GEMM1_GATE_UP, x, ta.permute_weights(g), y2, d_ids, d_eid, d_tot, T, K, unit, scale_m=d_sa,
                         scale_n=d_sg, b_shuffle=1) == 0.0
    torch.cuda.synchronize()
    assert torch.equal(y[:T * K].view(torch.int16), y2[:T * K].view(torch.int16))

    # gate only: the gate half of the same weights on their own, c = silu(a b^T)
    g_only = g[:, :I].contiguous()
    yo = torch.full((T * K + 3, I), float("nan"), dtype=cdt, device="cuda")
    assert ta.moe_flatmm(ta.GEMM1_GATE_ONLY, x, g_only, yo, d_ids, d_eid, d_tot, T, K, unit, scale_m=d_sa,
                         scale_n=None if d_sg is None else d_sg[:, :I].contiguous()) == 0.0
    torch.cuda.synchronize()
    yo_ref = oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, xr, np.ascontiguousarray(gr[:, :I]),
                             np.zeros((T * K, I), np.uint16), T, K, sa, None if sg is None else np.ascontiguousarray(sg[:, :I]),
                             c_dtype=odt)
    yog = yo.float().cpu().numpy()
    assert np.isnan(yog[T * K:]).all() and not np.isnan(yog[:T * K]).any()
    assert _rel(yog[:T * K], oracle.to_f32(yo_ref, odt)) <= tol

    # down: added to what c holds; a takes the reference's 16-bit Y so that the two GEMMs are checked apart
    # (fp8: that Y quantised per row, the row scales going in as scale_m)
    y_f32 = oracle.to_f32(y_ref, odt)
    if kind == "fp8":
        yq, sy = oracle.rowwise_quant(y_f32, oracle.DT_E4M3)
        y_in, a_ref, s_m, d_sm = dev(yq), oracle.to_f32(yq, oracle.DT_E4M3), sy, dev(sy)
    else:
        y_in, a_ref, s_m, d_sm = torch.from_numpy(y_ref.view(np.int16)).cuda().view(cdt), y_f32, None, None
    c0 = (rng.standard_normal((T, H)) * 0.1).astype(np.float32)
    c = bf(c0)
    c_ref = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, a_ref, dr, _bits(c).copy(), T, K, s_m, sd, c_dtype=odt)
    c2 = c.clone()
    assert ta.moe_flatmm(ta.GEMM2, y_in, d, c, d_ids, d_eid, d_tot, T, K, unit, sorted_weights=d_w, scale_m=d_sm,
                         scale_n=d_sd) == 0.0
    torch.cuda.synchronize()
    assert _rel(c.float().cpu().numpy(), oracle.to_f32(c_ref, odt)) <= tol
    assert ta.moe_flatmm(ta.GEMM2, y_in, ta.permute_weights(d), c2, d_ids, d_eid, d_tot, T, K, unit, sorted_weights=d_w,
                         scale_m=d_sm, scale_n=d_sd, b_shuffle=1) == 0.0
    torch.cuda.synchronize()
    assert torch.equal(c.view(torch.int16), c2.view(torch.int16))


def test_skewed_fp8_batch_takes_the_large_tiles_on_the_device():
    """A decode-sized fp8 batch with Zipf routing: the host's average says 32-row tiles, the tile-list pass sees few
    active experts with many rows each and builds the list for 320-row tiles (its choice is word 1 of the workspace);
    a uniformly routed batch of the same size keeps the decode tiles.  Both against the oracle."""
    import torch
    import therock_amd as ta
    from tests.gpu_util import run_sorting
    from therock_amd import inputs as mi

    T, E, K, H, I, unit = 256, 64, 4, 512, 2048, 32
    for router, want in (("zipf", 320), ("softmax_renorm", 32)):
        rng = np.random.default_rng(11)
        ids, w = mi.route_np(rng.standard_normal((T, E), dtype=np.float32), K, router)
        s_ids, s_w, s_eid, total = run_sorting(ids, w, E, unit, fill=True)
        pp = int(total[0])
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        x32 = rng.standard_normal((T, H)).astype(np.float32)
        g32 = (rng.standard_normal((E, 2 * I, H)) * 0.05).astype(np.float32)
        d32 = (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32)
        xq, sa = oracle.rowwise_quant(x32, oracle.DT_E4M3)
        gq, sg = oracle.rowwise_quant(g32.reshape(E * 2 * I, H), oracle.DT_E4M3)
        dq, sd = oracle.rowwise_quant(d32.reshape(E * H, I), oracle.DT_E4M3)
        gq, dq, sg, sd = gq.reshape(E, 2 * I, H), dq.reshape(E, H, I), sg.reshape(E, 2 * I), sd.reshape(E, H)
        d_ids, d_w, d_eid, d_tot = dev(s_ids), dev(s_w), dev(s_eid), dev(total.astype(np.int32))
        x, g, d = dev(xq), dev(gq), dev(dq)
        y = torch.full((T * K, I), float("nan"), dtype=torch.bfloat16, device="cuda")
        ws = torch.empty((ta.moe_flatmm_get_workspace_size(ta.GEMM1_GATE_UP, x, g, y, d_ids, d_eid, d_tot, T, K, unit),),
                         dtype=torch.uint8, device="cuda")
        assert ta.moe_flatmm(ta.GEMM1_GATE_UP, x, g, y, d_ids, d_eid, d_tot, T, K, unit, scale_m=dev(sa), scale_n=dev(sg),
                             workspace=ws) == 0.0
        torch.cuda.synchronize()
        assert int(ws.view(torch.int32)[1]) == want, router
        y_ref = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, oracle.to_f32(xq, oracle.DT_E4M3),
                                oracle.to_f32(gq, oracle.DT_E4M3), np.zeros((T * K, I), np.uint16), T, K, sa, sg)
        yg = y.float().cpu().numpy()
        assert not np.isnan(yg).any() and _rel(yg, oracle.to_f32(y_ref, oracle.DT_BF16)) <= 3e-2
        yq, sy = oracle.rowwise_quant(oracle.to_f32(y_ref, oracle.DT_BF16), oracle.DT_E4M3)
        c = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
        c_ref = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, oracle.to_f32(yq, oracle.DT_E4M3),
                                oracle.to_f32(dq, oracle.DT_E4M3), _bits(c).copy(), T, K, sy, sd)
        ws2 = torch.empty((ta.moe_flatmm_get_workspace_size(ta.GEMM2, dev(yq), d, c, d_ids, d_eid, d_tot, T, K, unit),),
                          dtype=torch.uint8, device="cuda")
        assert ta.moe_flatmm(ta.GEMM2, dev(yq), d, c, d_ids, d_eid, d_tot, T, K, unit, sorted_weights=d_w, scale_m=dev(sy),
                             scale_n=dev(sd), workspace=ws2) == 0.0
        torch.cuda.synchronize()
        # the down GEMM has two column tiles per expert here: too few active experts to fill the chip, decode tiles
        assert int(ws2.view(torch.int32)[1]) == 32
        assert _rel(c.float().cpu().numpy(), oracle.to_f32(c_ref, oracle.DT_BF16)) <= 3e-2


@pytest.mark.parametrize("T,E,K,H,I,unit", [(24, 16, 4, 512, 256, 32), (300, 8, 2, 256, 384, 32), (1024, 4, 2, 512, 384, 32)])
@pytest.mark.parametrize("kind", ["bf16", "fp16", "int8", "fp8"])
@pytest.mark.parametrize("act,with_bias", [("silu", True), ("swiglu", False), ("swiglu", True)])  # (silu, no bias) is the test above
def test_bias_and_swiglu(T, E, K, H, I, unit, kind, act, with_bias):
    """Expert bias and ck_tile's clamped SwiGLU (moe::Swiglu{alpha, limit}) on all three GEMM kinds, every kernel
    family (decode, small tiles, large tiles) and every operand type."""
    import torch
    import therock_amd as ta
    from tests.gpu_util import run_sorting

    rng = np.random.default_rng(T + H + with_bias)
    cdt, odt, tol = _c_types(kind)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32)
    s_ids, s_w, s_eid, total = run_sorting(ids, w, E, unit, fill=True)
    pp = int(total[0])
    dev = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()
    bf = lambda a: torch.from_numpy(a).cuda().to(cdt)
    x32 = (rng.standard_normal((T, H)) * 2).astype(np.float32)
    g32 = (rng.standard_normal((E, 2 * I, H)) * 0.1).astype(np.float32)   # gate / up values reach past the limit
    d32 = (rng.standard_normal((E, H, I)) * 0.05).astype(np.float32)
    bias_g = (rng.standard_normal((E, 2 * I)) * 1.5).astype(np.float32) if with_bias else None
    bias_d = (rng.standard_normal((E, H)) * 0.5).astype(np.float32) if with_bias else None
    d_ids, d_w, d_eid, d_tot = dev(s_ids), dev(s_w), dev(s_eid), dev(total.astype(np.int32))
    if kind in ("bf16", "fp16"):
        x, g, d = bf(x32), bf(g32), bf(d32)
        xr, gr, dr = x.float().cpu().numpy(), g.float().cpu().numpy(), d.float().cpu().numpy()
        sa = sg = sd = None
    else:
        qdt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
        kw = dict(nearest=True) if kind == "int8" else {}
        xq, sa = oracle.rowwise_quant(x32, qdt, **kw)
        gq, sg = oracle.rowwise_quant(g32.reshape(E * 2 * I, H), qdt, **kw)
        dq, sd = oracle.rowwise_quant(d32.reshape(E * H, I), qdt, **kw)
        x, g, d = dev(xq), dev(gq.reshape(E, 2 * I, H)), dev(dq.reshape(E, H, I))
        xr, gr, dr = (oracle.to_f32(xq, qdt), oracle.to_f32(gq.reshape(E, 2 * I, H), qdt),
                      oracle.to_f32(dq.reshape(E, H, I), qdt))
        sg, sd = sg.reshape(E, 2 * I), sd.reshape(E, H)
    a_code = ta.ACT_SWIGLU if act == "swiglu" else ta.ACT_SILU
    o_code = oracle.ACT_SWIGLU if act == "swiglu" else oracle.ACT_SILU
    alpha, limit = 1.702, 7.0

    y = torch.full((T * K, I), float("nan"), dtype=cdt, device="cuda")
    assert ta.moe_flatmm(ta.GEMM1_GATE_UP, x, g, y, d_ids, d_eid, d_tot, T, K, unit, scale_m=dev(sa), scale_n=dev(sg),
                         exp_bias=dev(bias_g), activation=a_code, swiglu_alpha=alpha, swiglu_limit=limit) == 0.0
    torch.cuda.synchronize()
    y_ref = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, xr, gr, np.zeros((T * K, I), np.uint16), T, K, sa, sg,
                            exp_bias=bias_g, act=o_code, alpha=alpha, limit=limit, c_dtype=odt)
    yg = y.float().cpu().numpy()
    assert not np.isnan(yg).any()
    assert _rel(yg, oracle.to_f32(y_ref, odt)) <= tol

    g_only = g[:, :I].contiguous()
    b_only = None if bias_g is None else np.ascontiguousarray(bias_g[:, :I])
    s_only = None if sg is None else np.ascontiguousarray(sg[:, :I])
    yo = torch.full((T * K, I), float("nan"), dtype=cdt, device="cuda")
    assert ta.moe_flatmm(ta.GEMM1_GATE_ONLY, x, g_only, yo, d_ids, d_eid, d_tot, T, K, unit, scale_m=dev(sa), scale_n=dev(s_only),
                         exp_bias=dev(b_only), activation=a_code, swiglu_alpha=alpha, swiglu_limit=limit) == 0.0
    torch.cuda.synchronize()
    yo_ref = oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, xr, np.ascontiguousarray(gr[:, :I]),
                             np.zeros((T * K, I), np.uint16), T, K, sa, s_only, exp_bias=b_only, act=o_code, alpha=alpha,
                             limit=limit, c_dtype=odt)
    assert _rel(yo.float().cpu().numpy(), oracle.to_f32(yo_ref, odt)) <= tol

    if not with_bias:
        return  # the down GEMM has no activation
    y_f32 = oracle.to_f32(y_ref, odt)
    if kind == "fp8":
        yq, sy = oracle.rowwise_quant(y_f32, oracle.DT_E4M3)
        y_in, a_ref, s_m = dev(yq), oracle.to_f32(yq, oracle.DT_E4M3), sy
    else:
        y_in, a_ref, s_m = torch.from_numpy(y_ref.view(np.int16)).cuda().view(cdt), y_f32, None
    c = bf((rng.standard_normal((T, H)) * 0.1).astype(np.float32))
    c_ref = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, a_ref, dr, _bits(c).copy(), T, K, s_m, sd, exp_bias=bias_d,
                            c_dtype=odt)
    assert ta.moe_flatmm(ta.GEMM2, y_in, d, c, d_ids, d_eid, d_tot, T, K, unit, sorted_weights=d_w, scale_m=dev(s_m),
                         scale_n=dev(sd), exp_bias=dev(bias_d)) == 0.0
    torch.cuda.synchronize()
    assert _rel(c.float().cpu().numpy(), oracle.to_f32(c_ref, odt)) <= tol


@pytest.mark.parametrize("T,E,K,H,I,unit", [(24, 16, 4, 512, 256, 32), (300, 8, 2, 256, 384, 32), (1024, 4, 2, 512, 384, 32)])
@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_padded_zeros(T, E, K, H, I, unit, kind):
    """n_padded_zeros / k_padded_zeros of MoeFlatmmHostArgs: the last weight rows, respectively the last K columns,
    hold garbage that must not reach the result."""
    import torch
    import therock_amd as ta
    from tests.gpu_util import run_sorting

    rng = np.random.default_rng(T + I)
    tol = 1e-2 if kind == "bf16" else 3e-2
    npad, kpad = 48, 64
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32)
    s_ids, s_w, s_eid, total = run_sorting(ids, w, E, unit, fill=True)
    pp = int(total[0])
    dev = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()
    x32 = rng.standard_normal((T, H)).astype(np.float32)
    g32 = (rng.standard_normal((E, 2 * I, H)) * 0.05).astype(np.float32)
    x32[:, H - kpad:] = 3.0          # what sits in the padding is large ...
    g32[:, :, H - kpad:] = 1.0
    g32[:, 2 * I - npad:, :] = 1.0   # ... and would dominate the result if it were read
    bias = (rng.standard_normal((E, 2 * I))).astype(np.float32)
    if kind == "bf16":
        x, g = dev(x32).to(torch.bfloat16), dev(g32).to(torch.bfloat16)
        xr, gr, sa, sg = x.float().cpu().numpy(), g.float().cpu().numpy(), None, None
    else:
        xq, sa = oracle.rowwise_quant(x32, oracle.DT_I8, nearest=True)
        gq, sg = oracle.rowwise_quant(g32.reshape(E * 2 * I, H), oracle.DT_I8, nearest=True)
        x, g = dev(xq), dev(gq.reshape(E, 2 * I, H))
        xr, gr, sg = oracle.to_f32(xq, oracle.DT_I8), oracle.to_f32(gq.reshape(E, 2 * I, H), oracle.DT_I8), sg.reshape(E, 2 * I)
    y = torch.full((T * K, I), float("nan"), dtype=torch.bfloat16, device="cuda")
    d_ids, d_eid, d_tot = dev(s_ids), dev(s_eid), dev(total.astype(np.int32))
    assert ta.moe_flatmm(ta.GEMM1_GATE_UP, x, g, y, d_ids, d_eid, d_tot, T, K, unit, scale_m=dev(sa), scale_n=dev(sg),
                         exp_bias=dev(bias), n_padded_zeros=npad, k_padded_zeros=kpad) == 0.0
    torch.cuda.synchronize()
    y_ref = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, xr, gr, np.zeros((T * K, I), np.uint16), T, K, sa, sg,
                            exp_bias=bias, n_padded_zeros=npad, k_padded_zeros=kpad)
    assert _rel(y.float().cpu().numpy(), oracle.to_f32(y_ref, oracle.DT_BF16)) <= tol


def test_unsupported_and_errors():
    import torch
    import therock_amd as ta

    z = lambda *s, dt=torch.bfloat16: torch.zeros(s, dtype=dt, device="cuda")
    ids, eid, tot = z(64, dt=torch.int32), z(2, dt=torch.int32), z(2, dt=torch.int32)
    # an unknown kind has no kernel: -1 like ck_tile's dispatcher
    assert ta.moe_flatmm(3, z(4, 64), z(2, 128, 64), z(8, 64), ids, eid, tot, 4, 2, 32) == -1.0
    with pytest.raises(RuntimeError):
        ta.moe_flatmm(ta.GEMM2, z(8, 64), z(2, 64, 64), z(4, 64), ids, eid, tot, 4, 2, 32)  # no sorted weights
    # an empty batch is a no-op, whatever storage its tensors have
    assert ta.moe_flatmm(ta.GEMM1_GATE_UP, z(0, 64), z(2, 128, 64), z(0, 64), ids, eid, tot, 0, 2, 32) == 0.0


@pytest.mark.parametrize("T,E,K,H,I,unit", [(40, 6, 3, 64, 96, 32), (130, 8, 2, 256, 128, 16)])
def test_oracle_against_ck_tile_device_reference(T, E, K, H, I, unit):
    """Pins moe_oracle_moe_gemm on ck_tile::reference_moe_gemm_gpu, which only runs on a GPU.  The gate+up
    kind accumulates in the same order: equal up to the device's exp in SiLU (one bf16 ulp at most, rarely).
    The down kind adds bf16 partial sums with atomics in ck_tile: compared to a bf16-rounding tolerance."""
    import torch

    torch.cuda.init()  # this process's HIP runtime first, then the reference library with its device code
    if oracle.ck_ref_gpu() is None:
        pytest.skip("oracle/_ref/libck_ref_gpu.so not built")
    rng = np.random.default_rng(T)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    x, g, d = bf(rng.standard_normal((T, H))), bf(rng.standard_normal((E, 2 * I, H)) * 0.1), bf(rng.standard_normal((E, H, I)) * 0.1)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32)
    s_ids, s_w, s_eid, pp = oracle.moe_sorting(ids, w, E, unit)
    sa, sg = (0.5 + rng.random(T)).astype(np.float32), (0.5 + rng.random((E, 2 * I))).astype(np.float32)
    f32 = lambda a: oracle.to_f32(a, oracle.DT_BF16)

    y_ck = oracle.ck_moe_gemm_gpu(1, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, I), np.uint16), T, K, sa, sg)
    y_or = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, f32(x), f32(g), np.zeros((T * K, I), np.uint16), T, K, sa, sg)
    diff = np.abs(y_ck.astype(np.int32) - y_or.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01

    g1 = np.ascontiguousarray(g[:, :I])
    s1 = np.ascontiguousarray(sg[:, :I])
    z_ck = oracle.ck_moe_gemm_gpu(0, s_ids, s_eid, s_w, pp, unit, x, g1, np.zeros((T * K, I), np.uint16), T, K, sa, s1)
    z_or = oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, f32(x), f32(g1), np.zeros((T * K, I), np.uint16), T, K, sa, s1)
    diff = np.abs(z_ck.astype(np.int32) - z_or.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01

    c0 = bf(rng.standard_normal((T, H)) * 0.1)
    o_ck = oracle.ck_moe_gemm_gpu(2, s_ids, s_eid, s_w, pp, unit, y_or, d, c0.copy(), T, K)
    o_or = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, f32(y_or), f32(d), c0.copy(), T, K)
    assert _rel(f32(o_ck), f32(o_or)) < 8e-3

    # expert bias and ck_tile's own moe::Swiglu functor (default alpha 1.702, limit 7), inputs scaled so that the
    # clamps bite; the device functor uses exp and an approximate reciprocal: a few bf16 ulps on a few elements
    bias = (rng.standard_normal((E, 2 * I)) * 2).astype(np.float32)
    x4 = bf(f32(x) * 4)
    for act in (oracle.ACT_SILU, oracle.ACT_SWIGLU):
        y_ck = oracle.ck_moe_gemm_gpu(1, s_ids, s_eid, s_w, pp, unit, x4, g, np.zeros((T * K, I), np.uint16), T, K, sa, sg,
                                      exp_bias=bias, act=act)
        y_or = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, f32(x4), f32(g), np.zeros((T * K, I), np.uint16), T, K, sa, sg,
                               exp_bias=bias, act=act)
        assert (np.abs(f32(y_or)) >= 7.0).any() or act == oracle.ACT_SILU
        diff = np.abs(y_ck.astype(np.int32) - y_or.astype(np.int32))
        assert diff.max() <= 2 and (diff != 0).mean() < 0.02, (act, diff.max(), (diff != 0).mean())
        z_ck = oracle.ck_moe_gemm_gpu(0, s_ids, s_eid, s_w, pp, unit, x4, g, np.zeros((T * K, 2 * I), np.uint16), T, K, sa, sg,
                                      exp_bias=bias, act=act)
        z_or = oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, f32(x4), f32(g), np.zeros((T * K, 2 * I), np.uint16), T, K, sa,
                               sg, exp_bias=bias, act=act)
        diff = np.abs(z_ck.astype(np.int32) - z_or.astype(np.int32))
        assert diff.max() <= 2 and (diff != 0).mean() < 0.02, (act, diff.max(), (diff != 0).mean())
    bias_d = (rng.standard_normal((E, H)) * 0.5).astype(np.float32)
    o_ck = oracle.ck_moe_gemm_gpu(2, s_ids, s_eid, s_w, pp, unit, y_or, d, c0.copy(), T, K, exp_bias=bias_d)
    o_or = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, f32(y_or), f32(d), c0.copy(), T, K, exp_bias=bias_d)
    assert _rel(f32(o_ck), f32(o_or)) < 8e-3
