"""GPU parity of the activation quantisers (mi355_moe_rowwise_quant, mi355_moe_smoothquant) against the
oracle, through the C ABI.  Bit-exact: scales are a maximum and one division, values one division and
one conversion."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _bf16(a):
    import torch
    return torch.from_numpy(a).cuda().to(torch.bfloat16)


def _raw(t):
    import torch
    return t.view(torch.uint8).cpu().numpy() if t.element_size() == 1 and t.dtype != torch.int8 else t.cpu().numpy()


# 7168: 16-byte pieces kept in registers; 12288: more pieces than the register cache holds; 1004, 100: scalar path
@pytest.mark.parametrize("rows,cols", [(1, 32), (64, 4096), (513, 7168), (7, 1000), (33, 12288), (5, 1004), (3, 100)])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_rowwise_quant(rows, cols, kind):
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(rows + cols)
    x = _bf16((rng.standard_normal((rows, cols)) * rng.choice([1e-2, 1, 30], size=(rows, 1))).astype(np.float32))
    x[rows // 2] = 0  # an all-zero row: scale 1, zeros
    q, s = ta.rowwise_quant(x, kind)
    torch.cuda.synchronize()
    dt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
    rq, rs = oracle.rowwise_quant(x.float().cpu().numpy(), dt)
    assert np.array_equal(s.cpu().numpy(), rs)
    assert np.array_equal(_raw(q), rq)
    # the same rows 2 bytes off a 16-byte boundary: the scalar path
    flat = torch.zeros((rows * cols + 8,), dtype=torch.bfloat16, device="cuda")
    shifted = flat[1:1 + rows * cols].view(rows, cols)
    shifted.copy_(x)
    assert shifted.data_ptr() % 16 == 2
    q2, s2 = ta.rowwise_quant(shifted, kind)
    torch.cuda.synchronize()
    assert np.array_equal(s2.cpu().numpy(), rs) and np.array_equal(_raw(q2), rq)


# second line: scale tables larger than an XCD's L2, short and long rows, many slots
@pytest.mark.parametrize("tokens,hidden,experts,topk", [(1, 64, 4, 2), (64, 4096, 128, 8), (300, 1024, 8, 2), (17, 7168, 256, 8),
                                                         (9, 10240, 4, 3), (5, 100, 3, 2),
                                                         (33, 2048, 512, 5), (5, 16400, 64, 3), (40, 7184, 128, 64),
                                                         (3, 7168, 128, 65)])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_moe_smoothquant(tokens, hidden, experts, topk, kind):
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(tokens * 7 + hidden)
    x = _bf16((rng.standard_normal((tokens, hidden)) * rng.choice([1e-2, 1, 30], size=(tokens, 1))).astype(np.float32))
    if tokens > 2:
        x[tokens // 2] = 0  # a row of zeros: scale 0, codes 0
    sm = torch.from_numpy((0.25 + rng.random((experts, hidden)) * 2).astype(np.float32)).cuda()
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    qy, ys = ta.moe_smoothquant(x, sm, torch.from_numpy(ids).cuda(), kind)
    torch.cuda.synchronize()
    dt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
    rq, rs = oracle.smoothquant(x.float().cpu().numpy(), sm.cpu().numpy(), ids, dt)
    assert np.array_equal(ys.cpu().numpy(), rs)
    assert np.array_equal(_raw(qy), rq)
    # a second call into the same outputs
    ta.moe_smoothquant(x, sm, torch.from_numpy(ids).cuda(), kind, out=(qy, ys))
    torch.cuda.synchronize()
    assert np.array_equal(ys.cpu().numpy(), rs) and np.array_equal(_raw(qy), rq)


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("hidden", [100, 4096])  # the scalar and the 16-byte kernel
def test_rows_of_zeros_quantise_to_zero(kind, hidden):
    """Padded batches hold rows of zeros: their codes are 0 (not the 0 / 0 of the plain formula), the scale is 0
    from smooth-quant (amax / qmax) and 1 from the row-wise quantiser."""
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(hidden)
    x = _bf16(rng.standard_normal((6, hidden)).astype(np.float32))
    x[1] = 0
    x[4] = 0
    sm = torch.from_numpy((0.25 + rng.random((4, hidden)) * 2).astype(np.float32)).cuda()
    ids = np.stack([rng.permutation(4)[:2] for _ in range(6)]).astype(np.int32)
    qy, ys = ta.moe_smoothquant(x, sm, torch.from_numpy(ids).cuda(), kind)
    q, s = ta.rowwise_quant(x, kind)
    torch.cuda.synchronize()
    dt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
    rq, rs = oracle.smoothquant(x.float().cpu().numpy(), sm.cpu().numpy(), ids, dt)
    assert np.array_equal(ys.cpu().numpy(), rs) and np.array_equal(_raw(qy), rq)
    for r in (1, 4):
        assert not _raw(qy)[:, r].any() and not ys.cpu().numpy()[:, r].any()
        assert not _raw(q)[r].any() and float(s[r]) == 1.0


@pytest.mark.parametrize("shape,dtype,nw,kw,kv", [((4, 256, 512), "bf16", 16, 4, 8), ((3, 64, 256), "int8", 16, 4, 16),
                                                   ((2, 64, 64), "bf16", 32, 2, 8), ((8, 4096, 1024), "fp8", 16, 4, 16)])
def test_permute_weights(shape, dtype, nw, kw, kv):
    """ck_tile's pre-shuffled weight layout and back: exact data movement."""
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(shape[1])
    npdt = np.uint16 if dtype == "bf16" else np.uint8
    w_np = rng.integers(0, 255, size=shape).astype(npdt)
    tdt = {"bf16": torch.bfloat16, "int8": torch.int8, "fp8": torch.float8_e4m3fn}[dtype]
    w = torch.from_numpy(w_np.view(np.int16) if dtype == "bf16" else w_np.view(np.int8)).cuda().view(tdt)
    p = ta.permute_weights(w, nw, kw, kv)
    back = ta.permute_weights(p, nw, kw, kv, inverse=True)
    torch.cuda.synchronize()
    as_np = lambda t: t.view(torch.int16 if dtype == "bf16" else torch.int8).cpu().numpy().view(npdt)
    assert np.array_equal(as_np(p), oracle.permute_weights(w_np, nw, kw, kv))
    assert np.array_equal(as_np(back), w_np)
