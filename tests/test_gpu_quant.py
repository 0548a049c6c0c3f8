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


@pytest.mark.parametrize("rows,cols", [(1, 32), (64, 4096), (513, 7168), (7, 1000)])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_rowwise_quant(rows, cols, kind):
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(rows + cols)
    x = _bf16((rng.standard_normal((rows, cols)) * rng.choice([1e-2, 1, 30], size=(rows, 1))).astype(np.float32))
    q, s = ta.rowwise_quant(x, kind)
    torch.cuda.synchronize()
    dt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
    rq, rs = oracle.rowwise_quant(x.float().cpu().numpy(), dt)
    assert np.array_equal(s.cpu().numpy(), rs)
    assert np.array_equal(_raw(q), rq)


@pytest.mark.parametrize("tokens,hidden,experts,topk", [(1, 64, 4, 2), (64, 4096, 128, 8), (300, 1024, 8, 2), (17, 7168, 256, 8)])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_moe_smoothquant(tokens, hidden, experts, topk, kind):
    import torch
    import therock_amd as ta

    rng = np.random.default_rng(tokens * 7 + hidden)
    x = _bf16(rng.standard_normal((tokens, hidden)).astype(np.float32))
    sm = torch.from_numpy((0.25 + rng.random((experts, hidden)) * 2).astype(np.float32)).cuda()
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    qy, ys = ta.moe_smoothquant(x, sm, torch.from_numpy(ids).cuda(), kind)
    torch.cuda.synchronize()
    dt = oracle.DT_I8 if kind == "int8" else oracle.DT_E4M3
    rq, rs = oracle.smoothquant(x.float().cpu().numpy(), sm.cpu().numpy(), ids, dt)
    assert np.array_equal(ys.cpu().numpy(), rs)
    assert np.array_equal(_raw(qy), rq)
