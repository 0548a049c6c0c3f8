"""GPU parity of the router front-end (mi355_topk_softmax) against the oracle, through the C ABI."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

RTOL = 1e-5  # fp32 weights: the wave reductions sum in another order than the reference
FLT_MIN = 1.1754944e-38


def _run(x_np, topk, dtype="fp32", **kw):
    import torch

    import therock_amd as ta

    x = torch.from_numpy(x_np).cuda()
    if dtype != "fp32":
        x = x.to({"bf16": torch.bfloat16, "fp16": torch.float16}[dtype])
    w, ids = ta.topk_softmax(x, topk, **kw)
    torch.cuda.synchronize()
    return w.cpu().numpy(), ids.cpu().numpy(), x.float().cpu().numpy()


def _check(w, ids, ref_w, ref_ids, probs_of):
    np.testing.assert_allclose(w, ref_w, rtol=RTOL, atol=1e-9)
    same = ids == ref_ids
    if not same.all():
        # a different expert is acceptable only where the two candidates are tied within tolerance
        r, c = np.nonzero(~same)
        # (atol: the device's exp flushes a subnormal probability to zero, so below FLT_MIN its ranking may differ
        # from the reference's, which keeps 1e-45 apart from 0)
        np.testing.assert_allclose(probs_of(r, ids[r, c]), probs_of(r, ref_ids[r, c]), rtol=RTOL, atol=FLT_MIN)


@pytest.mark.parametrize("rows,experts,topk", [(1, 8, 2), (128, 8, 2), (4096, 8, 2), (8192, 256, 8), (64, 128, 8),
                                               (257, 64, 6), (33, 1000, 17), (5, 3, 3), (100, 65, 64)])
@pytest.mark.parametrize("activation,renorm", [("softmax", False), ("sigmoid", True)])
def test_matches_oracle(rows, experts, topk, activation, renorm):
    rng = np.random.default_rng(rows * 31 + experts)
    x = (rng.standard_normal((rows, experts)) * 2.5).astype(np.float32)
    w, ids, xin = _run(x, topk, activation=activation, renormalize=renorm)
    ref_w, ref_ids = oracle.topk_softmax(xin, topk, sigmoid=activation == "sigmoid", renorm=renorm)
    full_w, full_ids = oracle.topk_softmax(xin, experts, sigmoid=activation == "sigmoid")
    dense = np.zeros_like(xin)
    np.put_along_axis(dense, full_ids, full_w, axis=1)
    if renorm:
        _check(w, ids, ref_w, ref_ids, lambda r, e: dense[r, e])
        np.testing.assert_allclose(w.sum(axis=1), 1.0, rtol=1e-5)
    else:
        _check(w, ids, ref_w, ref_ids, lambda r, e: dense[r, e])
    assert np.all(np.diff(w, axis=1) <= 0)
    for r in range(min(rows, 64)):
        assert len(set(ids[r].tolist())) == topk  # distinct experts per token, as moe_sorting requires


def test_bf16_logits_and_ties():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((300, 128)).astype(np.float32)
    w, ids, xin = _run(x, 8, dtype="bf16")  # bf16 logits collide often: ties go to the lower expert id
    ref_w, ref_ids = oracle.topk_softmax(xin, 8)
    assert np.array_equal(ids, ref_ids)
    np.testing.assert_allclose(w, ref_w, rtol=RTOL)
    w, ids, _ = _run(np.zeros((4, 32), np.float32), 5)
    assert np.array_equal(ids, np.tile(np.arange(5, dtype=np.int32), (4, 1)))
    np.testing.assert_allclose(w, 1 / 32, rtol=1e-6)


def test_fp16_logits():
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((300, 256)) * 3).astype(np.float32)
    for act, renorm in (("softmax", False), ("sigmoid", True)):
        w, ids, xin = _run(x, 8, dtype="fp16", activation=act, renormalize=renorm)
        ref_w, ref_ids = oracle.topk_softmax(xin, 8, sigmoid=act == "sigmoid", renorm=renorm)
        assert np.array_equal(ids, ref_ids)
        np.testing.assert_allclose(w, ref_w, rtol=RTOL)


def test_subnormal_tail_probabilities():
    """Rows whose softmax tail lies below FLT_MIN: the reference ranks 1e-45 above 0, the device may see both as 0
    and then takes the lower expert id.  The chosen probabilities agree to FLT_MIN either way, the leading ones
    exactly like everywhere else."""
    rng = np.random.default_rng(4002)
    x = np.full((64, 96), -104.0, dtype=np.float32)
    x[:, 0] = 0.0
    x[:, 1:40] = -103.0 - rng.random((64, 39), dtype=np.float32)  # exp() between 1e-45 and 2e-45
    x[:, 50] = -2.0
    w, ids, xin = _run(x, 6)
    ref_w, ref_ids = oracle.topk_softmax(xin, 6)
    assert np.array_equal(ids[:, :2], ref_ids[:, :2]) and np.all(ids[:, 0] == 0) and np.all(ids[:, 1] == 50)
    np.testing.assert_allclose(w, ref_w, rtol=RTOL, atol=FLT_MIN)
    assert np.all(w[:, 2:] <= FLT_MIN)
    for r in range(64):
        assert len(set(ids[r].tolist())) == 6


def test_feeds_the_sort():
    """router -> moe_sorting on device equals the oracle pipeline on the same logits."""
    import torch

    import therock_amd as ta
    from tests.gpu_util import run_sorting

    rng = np.random.default_rng(9)
    T, E, K, U = 512, 64, 6, 32
    x = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    w, ids = ta.topk_softmax(torch.from_numpy(x).cuda(), K)
    ref_w, ref_ids = oracle.topk_softmax(x, K)
    assert np.array_equal(ids.cpu().numpy(), ref_ids)
    got = run_sorting(ids.cpu().numpy(), w.cpu().numpy(), E, U)
    exp = oracle.moe_sorting(ids.cpu().numpy(), w.cpu().numpy(), E, U)
    pp = exp[3]
    assert got[3][0] == pp and np.array_equal(got[0][:pp], exp[0][:pp]) and np.array_equal(got[1][:pp], exp[1][:pp])


def test_errors():
    import torch

    import therock_amd as ta

    x = torch.zeros((4, 16), device="cuda")
    with pytest.raises(Exception):
        ta.topk_softmax(x, 17)
    with pytest.raises(Exception):
        ta.topk_softmax(torch.zeros((4, 2048), device="cuda"), 2)
