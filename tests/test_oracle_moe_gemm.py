"""Pins the oracle of the unfused grouped GEMMs (ck_tile's MoeFlatmm conventions).  ck_tile's own
reference for them is a device kernel, so the pins are mathematical: a dense float64 formulation that
never looks at the sorted arrays, the composition against the fused oracle, and a triple loop."""
import numpy as np
import pytest

import oracle
from therock_amd import inputs as mi


def _problem(seed, T, E, K, H, I, unit):
    rng = np.random.default_rng(seed)
    x = oracle.to_f32(oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)), oracle.DT_BF16)
    g = oracle.to_f32(oracle.f32_to_bf16((rng.standard_normal((E, 2 * I, H)) * 0.1).astype(np.float32)), oracle.DT_BF16)
    d = oracle.to_f32(oracle.f32_to_bf16((rng.standard_normal((E, H, I)) * 0.1).astype(np.float32)), oracle.DT_BF16)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32)
    s_ids, s_w, s_eid, pp = oracle.moe_sorting(ids, w, E, unit)
    return x, g, d, ids, w, s_ids, s_w, s_eid, pp


def _silu(v):
    return v / (1.0 + np.exp(-v))


@pytest.mark.parametrize("T,E,K,H,I,unit", [(5, 3, 2, 32, 32, 4), (40, 6, 3, 64, 96, 32), (1, 4, 4, 32, 64, 16)])
def test_against_dense_float64(T, E, K, H, I, unit):
    x, g, d, ids, w, s_ids, s_w, s_eid, pp = _problem(T + H, T, E, K, H, I, unit)
    y = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, I), np.uint16), T, K)
    yf = oracle.to_f32(y, oracle.DT_BF16)
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            ref = _silu(x[t].astype(np.float64) @ g[e, :I].T.astype(np.float64)) * (x[t].astype(np.float64) @ g[e, I:].T)
            np.testing.assert_allclose(yf[t * K + k], ref, rtol=1.2e-2, atol=1e-6)  # one bf16 rounding
    # gate only: silu(a b^T) over all rows of b; with b = the full gate+up matrix its first half is the gate part
    z = oracle.to_f32(oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, 2 * I), np.uint16), T, K),
                      oracle.DT_BF16)
    for t in range(T):
        for k in range(K):
            ref = _silu(x[t].astype(np.float64) @ g[ids[t, k]].T.astype(np.float64))
            np.testing.assert_allclose(z[t * K + k], ref, rtol=1.2e-2, atol=1e-6)
    c0 = oracle.f32_to_bf16(np.full((T, H), 0.25, np.float32))
    o = oracle.to_f32(oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, yf, d, c0.copy(), T, K), oracle.DT_BF16)
    for t in range(T):
        ref = 0.25 + sum(w[t, k] * (yf[t * K + k].astype(np.float64) @ d[ids[t, k]].T.astype(np.float64)) for k in range(K))
        np.testing.assert_allclose(o[t], ref, rtol=1.2e-2, atol=1e-5)


def test_composition_matches_fused_oracle():
    T, E, K, H, I, unit = 48, 8, 2, 128, 64, 32
    x, g, d, ids, w, s_ids, s_w, s_eid, pp = _problem(3, T, E, K, H, I, unit)
    y = oracle.to_f32(oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, I), np.uint16), T, K),
                      oracle.DT_BF16)
    o = oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, y, d, np.zeros((T, H), np.uint16), T, K)
    fused = oracle.fused_moe(x, oracle.DT_F32, g, oracle.DT_F32, d, oracle.DT_F32, s_ids, s_w, s_eid, pp, unit, T, E, H, I, K)
    a, b = oracle.to_f32(o, oracle.DT_BF16).astype(np.float64), oracle.to_f32(fused, oracle.DT_BF16).astype(np.float64)
    # the only difference is the bf16 rounding of Y between the two GEMMs
    assert np.linalg.norm(a - b) / np.linalg.norm(b) < 6e-3


def test_scales_and_padding_rows():
    """Scales factor out of the dot products; padding ids and rows past post_pad write nothing."""
    T, E, K, H, I, unit = 9, 4, 2, 32, 32, 8
    x, g, d, ids, w, s_ids, s_w, s_eid, pp = _problem(11, T, E, K, H, I, unit)
    rng = np.random.default_rng(0)
    sa, sb = (0.5 + rng.random(T)).astype(np.float32), (0.5 + rng.random((E, 2 * I))).astype(np.float32)
    y_s = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x, g, np.full((T * K, I), 0x7fc0, np.uint16), T, K, sa, sb)
    y_f = oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x * sa[:, None], g * sb[:, :, None],
                          np.full((T * K, I), 0x7fc0, np.uint16), T, K)
    a, b = oracle.to_f32(y_s, oracle.DT_BF16), oracle.to_f32(y_f, oracle.DT_BF16)
    assert not np.isnan(a).any()  # every (token, slot) row was written exactly once
    np.testing.assert_allclose(a, b, rtol=2e-2, atol=1e-6)
