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


def test_fp16_output_is_the_same_sums_rounded_to_fp16():
    """c_dtype=DT_F16: the fp32 results before the final rounding are those of the bf16 variant (checked through the
    dense float64 formulation at fp16's tighter precision), and the down kind starts from the fp16 value c holds."""
    T, E, K, H, I, unit = 40, 6, 3, 64, 96, 32
    x, g, d, ids, w, s_ids, s_w, s_eid, pp = _problem(11, T, E, K, H, I, unit)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)
    x, g, d = f16(x), f16(g), f16(d)
    y = oracle.to_f32(oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, I), np.uint16), T, K,
                                      c_dtype=oracle.DT_F16), oracle.DT_F16)
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            ref = _silu(x[t].astype(np.float64) @ g[e, :I].T.astype(np.float64)) * (x[t].astype(np.float64) @ g[e, I:].T)
            np.testing.assert_allclose(y[t * K + k], ref, rtol=1.5e-3, atol=1e-6)  # one fp16 rounding (2^-11) + fp32 sums
    c0 = np.full((T, H), 0.3, np.float32).astype(np.float16)
    o = oracle.to_f32(oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, y, d, c0.view(np.uint16).copy(), T, K,
                                      c_dtype=oracle.DT_F16), oracle.DT_F16)
    for t in range(T):
        ref = float(c0[0, 0]) + sum(w[t, k] * (y[t * K + k].astype(np.float64) @ d[ids[t, k]].T.astype(np.float64))
                                    for k in range(K))
        np.testing.assert_allclose(o[t], ref, rtol=1.5e-3, atol=2e-5)
    # the bf16 variant of the same call differs only by the coarser rounding
    ob = oracle.to_f32(oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, y, d, np.zeros((T, H), np.uint16), T, K), oracle.DT_BF16)
    of = oracle.to_f32(oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, y, d, np.zeros((T, H), np.uint16), T, K,
                                       c_dtype=oracle.DT_F16), oracle.DT_F16)
    assert np.array_equal(oracle.f32_to_bf16(of) , oracle.f32_to_bf16(ob)) or \
        np.abs(of - ob).max() <= np.abs(ob).max() * 2.0 ** -8


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


def test_swiglu_closed_forms():
    """ck_tile::moe::Swiglu (moe_flatmm_kernel.hpp:149-183): gate clamps from above only, linear from both sides,
    the sigmoid takes alpha * gate, the linear branch gets + 1."""
    a, lim = 1.702, 7.0
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    f = lambda g, l, alpha=a, limit=lim: oracle.moe_act(oracle.ACT_SWIGLU, g, l, alpha, limit)
    assert f(0.0, 3.0) == 0.0                                          # gate 0 -> 0
    np.testing.assert_allclose(f(1.0, 0.0), 1.0 * sig(a), rtol=1e-6)   # linear 0 -> gate * sigmoid(alpha gate)
    np.testing.assert_allclose(f(1.0, -1.0), 0.0, atol=1e-7)           # linear -1 -> factor (linear + 1) = 0
    np.testing.assert_allclose(f(100.0, 2.0), lim * sig(a * lim) * 3.0, rtol=1e-6)      # gate above the limit is the limit
    np.testing.assert_allclose(f(-100.0, 2.0), -100.0 * sig(-a * 100.0) * 3.0, rtol=1e-6, atol=1e-30)  # not clamped from below
    np.testing.assert_allclose(f(2.0, 50.0), 2.0 * sig(2 * a) * (lim + 1.0), rtol=1e-6)   # linear clamps at +limit
    np.testing.assert_allclose(f(2.0, -50.0), 2.0 * sig(2 * a) * (-lim + 1.0), rtol=1e-6) # ... and at -limit
    np.testing.assert_allclose(f(2.0, 1.0, alpha=1.0, limit=100.0), 2.0 * sig(2.0) * 2.0, rtol=1e-6)  # alpha 1: silu(gate) * (l + 1)
    # MoeSilu: silu(gate) * linear
    np.testing.assert_allclose(oracle.moe_act(oracle.ACT_SILU, 1.5, -2.0), 1.5 * sig(1.5) * -2.0, rtol=1e-6)


@pytest.mark.parametrize("act", [oracle.ACT_SILU, oracle.ACT_SWIGLU])
def test_bias_activation_and_padding_against_dense_float64(act):
    """Expert bias is added after the scales and before the activation (gate and up halves of the bias row), the
    down kind multiplies (dot + bias) by the top-k weight; padded weight rows and padded K columns count as zeros."""
    T, E, K, H, I, unit = 12, 4, 2, 64, 32, 8
    x, g, d, ids, w, s_ids, s_w, s_eid, pp = _problem(5, T, E, K, H, I, unit)
    rng = np.random.default_rng(2)
    x = x * 4.0  # large enough for the clamps of the swiglu to bite
    bias = (rng.standard_normal((E, 2 * I)) * 2).astype(np.float32)
    sa, sb = (0.5 + rng.random(T)).astype(np.float32), (0.5 + rng.random((E, 2 * I))).astype(np.float32)
    npad, kpad = 8, 16
    a, lim = 1.3, 2.5
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))

    def act_ref(gate, lin):
        if act == oracle.ACT_SILU:
            return gate * sig(gate) * lin
        gate, lin = np.minimum(gate, lim), np.clip(lin, -lim, lim)
        return gate * sig(a * gate) * (lin + 1.0)

    y = oracle.to_f32(oracle.moe_gemm(1, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, I), np.uint16), T, K, sa, sb,
                                      exp_bias=bias, act=act, alpha=a, limit=lim, n_padded_zeros=npad, k_padded_zeros=kpad),
                      oracle.DT_BF16)
    z = oracle.to_f32(oracle.moe_gemm(0, s_ids, s_eid, s_w, pp, unit, x, g, np.zeros((T * K, 2 * I), np.uint16), T, K, sa, sb,
                                      exp_bias=bias, act=act, alpha=a, limit=lim, n_padded_zeros=npad, k_padded_zeros=kpad),
                      oracle.DT_BF16)
    x64, g64 = x.astype(np.float64), g.astype(np.float64)
    x64[:, H - kpad:] = 0
    gz = g64.copy()
    gz[:, 2 * I - npad:] = 0
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            dots = (x64[t] @ gz[e].T) * sa[t] * sb[e] + bias[e]
            np.testing.assert_allclose(y[t * K + k], act_ref(dots[:I], dots[I:]), rtol=1.2e-2, atol=1e-5)
            np.testing.assert_allclose(z[t * K + k], act_ref(dots, 1.0), rtol=1.2e-2, atol=1e-5)
    # down: (dot * scales + bias) * weight, summed over the slots on top of what C holds
    bias_d = (rng.standard_normal((E, H)) * 0.5).astype(np.float32)
    sm, sn = (0.5 + rng.random(T * K)).astype(np.float32), (0.5 + rng.random((E, H))).astype(np.float32)
    yin = oracle.to_f32(oracle.f32_to_bf16(rng.standard_normal((T * K, I)).astype(np.float32)), oracle.DT_BF16)
    c0 = oracle.f32_to_bf16(np.full((T, H), -0.5, np.float32))
    o = oracle.to_f32(oracle.moe_gemm(2, s_ids, s_eid, s_w, pp, unit, yin, d, c0.copy(), T, K, sm, sn, exp_bias=bias_d,
                                      n_padded_zeros=npad, k_padded_zeros=8), oracle.DT_BF16)
    y64, d64 = yin.astype(np.float64), d.astype(np.float64)
    y64[:, I - 8:] = 0
    dz = d64.copy()
    dz[:, H - npad:] = 0
    for t in range(T):
        ref = -0.5 + sum(w[t, k] * ((y64[t * K + k] @ dz[ids[t, k]].T) * sm[t * K + k] * sn[ids[t, k]] + bias_d[ids[t, k]])
                         for k in range(K))
        np.testing.assert_allclose(o[t], ref, rtol=1.2e-2, atol=1e-4)
