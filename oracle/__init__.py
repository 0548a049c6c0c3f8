"""ctypes bindings of the CPU oracle (test infrastructure only).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package.  ``libmoe_oracle.so`` is the plain-C restatement in ``moe_oracle.c``;
``_ref/libck_ref.so`` is Composable Kernel's own host reference compiled from the ck_tile headers
that ship with ROCm (``ck_ref.cpp``).  Both are built by ``oracle/Makefile``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

DT_F32, DT_BF16, DT_E4M3, DT_I8, DT_F16 = 0, 1, 2, 3, 4
_NP_OF_DT = {DT_F32: np.float32, DT_BF16: np.uint16, DT_E4M3: np.uint8, DT_I8: np.int8}


def build(force: bool = False) -> None:
    """Compile the oracle libraries (gcc, and hipcc for the ck_tile reference)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load(path: str):
    return C.CDLL(path) if os.path.exists(path) else None


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        p = os.path.join(_HERE, "libmoe_oracle.so")
        if not os.path.exists(p):
            build()
        _lib = C.CDLL(p)
        _lib.moe_oracle_bf16_to_f32.restype = C.c_float
        _lib.moe_oracle_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.moe_oracle_f32_to_bf16.restype = C.c_uint16
        _lib.moe_oracle_f32_to_bf16.argtypes = [C.c_float]
        _lib.moe_oracle_e4m3_to_f32.restype = C.c_float
        _lib.moe_oracle_e4m3_to_f32.argtypes = [C.c_uint8]
        _lib.moe_oracle_f32_to_e4m3.restype = C.c_uint8
        _lib.moe_oracle_f32_to_e4m3.argtypes = [C.c_float]
        _lib.moe_oracle_silu.restype = C.c_float
        _lib.moe_oracle_silu.argtypes = [C.c_float]
        _lib.moe_oracle_gelu.restype = C.c_float
        _lib.moe_oracle_gelu.argtypes = [C.c_float]
        _lib.moe_oracle_num_threads.restype = C.c_int
        _lib.moe_oracle_set_num_threads.argtypes = [C.c_int]
    return _lib


def ck_ref():
    """ck_tile's own reference, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is None:
        _ref = _load(os.path.join(_HERE, "_ref", "libck_ref.so"))
        if _ref is not None:
            _ref.ck_ref_f32_to_bf16.restype = C.c_uint16
            _ref.ck_ref_f32_to_bf16.argtypes = [C.c_float]
            _ref.ck_ref_f32_to_fp8.restype = C.c_uint8
            _ref.ck_ref_f32_to_fp8.argtypes = [C.c_float]
            _ref.ck_ref_fp8_to_f32.restype = C.c_float
            _ref.ck_ref_fp8_to_f32.argtypes = [C.c_uint8]
            _ref.ck_ref_silu.restype = C.c_float
            _ref.ck_ref_silu.argtypes = [C.c_float]
            _ref.ck_ref_gelu.restype = C.c_float
            _ref.ck_ref_gelu.argtypes = [C.c_float]
    return _ref


_ref_gpu = None


def ck_ref_gpu():
    """ck_tile's device reference (needs a GPU), or None when not built.  Load it only after the process
    has initialised its own HIP runtime: the library carries device code."""
    global _ref_gpu
    if _ref_gpu is None:
        _ref_gpu = _load(os.path.join(_HERE, "_ref", "libck_ref_gpu.so"))
    return _ref_gpu


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def max_num_tokens_padded(tokens: int, topk: int, experts: int, unit: int) -> int:
    return topk * tokens + experts * unit - topk


# --------------------------------------------------------------------------- conversions
def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Vectorised RNE float32 -> bf16 bit pattern (same rule as moe_oracle_f32_to_bf16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


_E4M3_TABLE = None


def e4m3_table() -> np.ndarray:
    """256-entry decode table produced by the C oracle."""
    global _E4M3_TABLE
    if _E4M3_TABLE is None:
        l = lib()
        _E4M3_TABLE = np.array([l.moe_oracle_e4m3_to_f32(i) for i in range(256)], dtype=np.float32)
    return _E4M3_TABLE


def e4m3_to_f32(q: np.ndarray) -> np.ndarray:
    return e4m3_table()[np.ascontiguousarray(q, dtype=np.uint8)]


def to_f32(x: np.ndarray, dt: int) -> np.ndarray:
    if dt == DT_F32:
        return np.asarray(x, dtype=np.float32)
    if dt == DT_BF16:
        return bf16_to_f32(x)
    if dt == DT_E4M3:
        return e4m3_to_f32(x)
    if dt == DT_F16:
        return np.ascontiguousarray(x, dtype=np.uint16).view(np.float16).astype(np.float32)
    return np.asarray(x, dtype=np.int8).astype(np.float32)


def rowwise_quant(x: np.ndarray, dt: int, nearest: bool = False):
    """Per-row dynamic quantisation of a float32 [M,N] matrix -> (q, scale[M]).  int8 values are
    converted as ck_tile does (truncation toward zero) unless nearest=True (round to nearest even, the
    quantiser of the synthetic benchmark inputs)."""
    x = _c(x, np.float32)
    M, N = x.shape
    q = np.empty((M, N), dtype=_NP_OF_DT[dt])
    s = np.empty((M,), dtype=np.float32)
    rc = lib().moe_oracle_rowwise_quant2(_p(x), C.c_int64(M), C.c_int64(N), C.c_int(dt), C.c_int(int(nearest)),
                                         _p(q), _p(s))
    if rc != 0:
        raise ValueError("rowwise_quant: unsupported dtype")
    return q, s


def ck_rowwise_quant(x: np.ndarray, scale: np.ndarray, dt: int):
    """ck_tile::reference_rowwise_quantization2d on fp32 rows with the given per-row scales."""
    r = ck_ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    x, scale = _c(x, np.float32), _c(scale, np.float32)
    M, N = x.shape
    q = np.empty((M, N), dtype=_NP_OF_DT[dt])
    r.ck_ref_rowwise_quant(_p(x), _p(scale), C.c_int32(M), C.c_int32(N), C.c_int32(int(dt == DT_E4M3)), _p(q))
    return q


def permute_weights(w: np.ndarray, nw: int, kw: int, kv: int, inverse: bool = False) -> np.ndarray:
    """ck_tile's b_nr_kr_kw_nw_kv pre-shuffle of [experts, n, k] weights (any dtype), or its inverse:
    view [e, n/nw, nw, k/(kw*kv), kw, kv], permute (0, 1, 3, 4, 2, 5) (reference_permute.hpp:20-57)."""
    e, n, k = w.shape
    if inverse:
        v = np.ascontiguousarray(w).reshape(e, n // nw, k // (kw * kv), kw, nw, kv)
        return np.ascontiguousarray(v.transpose(0, 1, 4, 2, 3, 5)).reshape(e, n, k)
    v = np.ascontiguousarray(w).reshape(e, n // nw, nw, k // (kw * kv), kw, kv)
    return np.ascontiguousarray(v.transpose(0, 1, 3, 4, 2, 5)).reshape(e, n, k)


def ck_permute_weights(w: np.ndarray, nw: int, kw: int, kv: int) -> np.ndarray:
    """The same permutation computed by ck_tile::reference_permute on the byte view."""
    r = ck_ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    e, n, k = w.shape
    b = np.ascontiguousarray(w).view(np.uint8)
    out = np.empty_like(b)
    r.ck_ref_permute_b_nr_kr_kw_nw_kv(_p(b), C.c_int32(e), C.c_int32(n // nw), C.c_int32(nw), C.c_int32(k // (kw * kv)),
                                      C.c_int32(kw), C.c_int32(kv * w.itemsize), _p(out))
    return out.view(w.dtype).reshape(e, n, k)


def ck_shuffle_b(w, n_warp, k_warp):
    """ck_tile::shuffle_b on every expert of w [e, n, k] (1- or 2-byte elements) for a GemmConfig with the warp tile
    n_warp x k_warp (elements); None when oracle/_ref is not built."""
    r = ck_ref()
    if r is None:
        return None
    e, n, k = w.shape
    b = np.ascontiguousarray(w)
    out = np.empty_like(b)
    for i in range(e):
        src, dst = b[i], out[i]
        rc = r.ck_ref_shuffle_b(_p(src), C.c_int32(n), C.c_int32(k), C.c_int32(w.itemsize), C.c_int32(n_warp),
                                C.c_int32(k_warp), _p(dst))
        if rc != 0:
            raise ValueError("ck_ref_shuffle_b: no instance for this warp tile")
    return out


def smoothquant(x, smscale, topk_ids, dt):
    """MoE smooth-quant oracle: fp32 x [T,H], smscale [E,H], topk_ids [T,K] -> (qy [K,T,H], yscale [K,T])."""
    x, smscale, topk_ids = _c(x, np.float32), _c(smscale, np.float32), _c(topk_ids, np.int32)
    T, H = x.shape
    E = smscale.shape[0]
    K = topk_ids.shape[1]
    qy = np.empty((K, T, H), dtype=_NP_OF_DT[dt])
    ys = np.empty((K, T), dtype=np.float32)
    rc = lib().moe_oracle_smoothquant(_p(x), _p(smscale), _p(topk_ids), C.c_int32(T), C.c_int32(H), C.c_int32(E),
                                      C.c_int32(K), C.c_int(dt), _p(qy), _p(ys))
    if rc != 0:
        raise ValueError(f"moe_oracle_smoothquant failed ({rc})")
    return qy, ys


# ------------------------------------------------------------------------------- sorting
def moe_sorting(topk_ids, weights, experts, unit, local_expert_mask=None, skip_empty=True,
                fill_id=-1, fill_w=-1.0, fill_eid=-1):
    """Returns (sorted_ids[max_pad], sorted_w[max_pad], sorted_eid[tiles_max], post_pad).
    Cells past the written prefix keep the fill values."""
    topk_ids = _c(topk_ids, np.int32)
    weights = _c(weights, np.float32)
    T, K = topk_ids.shape
    mp = max_num_tokens_padded(T, K, experts, unit)
    if not skip_empty:  # every expert owns a tile: with fewer than K distinct experts in use the bound above is short
        mp = max(mp, experts * unit)
    ids = np.full((mp,), fill_id, dtype=np.int32)
    w = np.full((mp,), fill_w, dtype=np.float32)
    eid = np.full(((mp + unit - 1) // unit,), fill_eid, dtype=np.int32)
    pp = C.c_int32(0)
    mask = _c(local_expert_mask, np.int32)
    rc = lib().moe_oracle_sorting(_p(topk_ids), _p(weights), _p(mask), T, K, experts, unit,
                                  int(bool(skip_empty)), _p(ids), _p(w), _p(eid), C.byref(pp))
    if rc < 0:
        raise ValueError(f"moe_oracle_sorting failed ({rc})")
    return ids, w, eid, int(pp.value)


def ck_moe_sorting(topk_ids, weights, experts, unit, local_expert_mask=None, skip_empty=True,
                   fill_id=-1, fill_w=-1.0, fill_eid=-1):
    """Same contract as moe_sorting, computed by ck_tile::reference_moe_sorting."""
    r = ck_ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    topk_ids = _c(topk_ids, np.int32)
    weights = _c(weights, np.float32)
    T, K = topk_ids.shape
    mp = max_num_tokens_padded(T, K, experts, unit)
    if not skip_empty:  # every expert owns a tile: with fewer than K distinct experts in use the bound above is short
        mp = max(mp, experts * unit)
    ids = np.full((mp,), fill_id, dtype=np.int32)
    w = np.full((mp,), fill_w, dtype=np.float32)
    eid = np.full(((mp + unit - 1) // unit,), fill_eid, dtype=np.int32)
    mask = _c(local_expert_mask, np.int32)
    pp = r.ck_ref_moe_sorting(_p(topk_ids), _p(weights), _p(mask), T, K, experts, unit,
                              int(mask is not None), int(bool(skip_empty)), _p(ids), _p(w), _p(eid))
    return ids, w, eid, int(pp)


# ------------------------------------------------------------------- unfused grouped GEMMs
ACT_SILU, ACT_SWIGLU = 0, 1


def moe_act(act, gate, linear, alpha=1.702, limit=7.0):
    """The oracle's scalar activation (ck_tile::moe::MoeSilu / Swiglu, host branch)."""
    f = lib().moe_oracle_moe_act
    f.restype = C.c_float
    return float(f(C.c_int(act), C.c_float(gate), C.c_float(linear), C.c_float(alpha), C.c_float(limit)))


def moe_gemm(kind, sorted_ids, sorted_eid, sorted_w, post_pad, block_m, a, b, c, num_tokens, topk,
             scale_a=None, scale_b=None, exp_bias=None, act=ACT_SILU, alpha=1.702, limit=7.0, n_padded_zeros=0,
             k_padded_zeros=0, c_dtype=DT_BF16):
    """Oracle of ck_tile's unfused MoE GEMMs (kind 0 = gate only, 1 = gate+up with act(gate, up), 2 = down with
    weights, added to c).  a, b fp32; c bf16 bits (fp16 bits with c_dtype=DT_F16) [rows, >= N or N/2], updated in
    place and returned."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    c = np.ascontiguousarray(c, dtype=np.uint16)
    E, N, K = b.shape
    ids, eid = _c(sorted_ids, np.int32), _c(sorted_eid, np.int32)
    w = _c(sorted_w, np.float32)
    f = lib().moe_oracle_moe_gemm_dt
    f.restype = C.c_int
    rc = f(C.c_int(kind), _p(ids), _p(eid), _p(w), C.c_int32(int(post_pad)), C.c_int32(block_m), _p(a), _p(b), _p(c),
           C.c_int32(num_tokens), C.c_int32(topk), C.c_int32(N), C.c_int32(K), C.c_int32(a.shape[1]),
           C.c_int32(c.shape[1]), _p(_c(scale_a, np.float32)), _p(_c(scale_b, np.float32)),
           _p(_c(exp_bias, np.float32)), C.c_int32(act), C.c_float(alpha), C.c_float(limit), C.c_int32(n_padded_zeros),
           C.c_int32(k_padded_zeros), C.c_int32(c_dtype))
    if rc != 0:
        raise ValueError(f"moe_oracle_moe_gemm failed ({rc})")
    return c


def ck_moe_gemm_gpu(kind, sorted_ids, sorted_eid, sorted_w, post_pad, block_m, a_bf16, b_bf16, c_bf16, num_tokens, topk,
                    scale_a=None, scale_b=None, exp_bias=None, act=ACT_SILU):
    """ck_tile::reference_moe_gemm_gpu (a device kernel: needs a GPU) on bf16 operands given as bf16 bits, with
    ck_tile's own activation functor (MoeSilu, or Swiglu with its default alpha 1.702 and limit 7).
    c is updated in place (the down kind adds to it) and returned."""
    r = ck_ref_gpu()
    if r is None:
        raise RuntimeError("oracle/_ref/libck_ref_gpu.so is not built")
    a, b = _c(a_bf16, np.uint16), _c(b_bf16, np.uint16)
    c = np.ascontiguousarray(c_bf16, dtype=np.uint16)
    E, N, K = b.shape
    ids, eid, w = _c(sorted_ids, np.int32), _c(sorted_eid, np.int32), _c(sorted_w, np.float32)
    sa = _c(scale_a if scale_a is not None else np.ones(a.shape[0], np.float32), np.float32)
    sb = _c(scale_b if scale_b is not None else np.ones((E, N), np.float32), np.float32)
    r.ck_ref_moe_gemm_gpu.restype = C.c_int
    rc = r.ck_ref_moe_gemm_gpu(C.c_int32(kind), _p(ids), _p(eid), C.c_int32(int(post_pad)), _p(a), _p(b), _p(c), _p(w),
                               C.c_int32(num_tokens), C.c_int32(block_m), C.c_int32(topk), C.c_int32(ids.size),
                               C.c_int32(E), C.c_int32(N), C.c_int32(K), _p(sa), _p(sb), _p(_c(exp_bias, np.float32)),
                               C.c_int32(act))
    if rc != 0:
        raise RuntimeError(f"ck_ref_moe_gemm_gpu failed ({rc})")
    return c


# ----------------------------------------------------------------------------- router
def topk_softmax(logits, topk, sigmoid=False, renorm=False):
    """Oracle router: softmax (or sigmoid) over the last axis of fp32 `logits` [rows, experts], then the
    top-k values (descending; ties to the lower expert id) and expert ids."""
    x = _c(logits, np.float32)
    rows, experts = x.shape
    w = np.empty((rows, topk), dtype=np.float32)
    idx = np.empty((rows, topk), dtype=np.int32)
    f = lib().moe_oracle_topk_softmax
    f.restype = C.c_int
    rc = f(_p(x), C.c_int32(rows), C.c_int32(experts), C.c_int32(topk), C.c_int32(int(bool(sigmoid))),
           C.c_int32(int(bool(renorm))), _p(w), _p(idx))
    if rc != 0:
        raise ValueError(f"moe_oracle_topk_softmax failed ({rc})")
    return w, idx


def ck_topk_softmax(logits, topk):
    """ck_tile::reference_softmax + reference_topk on fp32 logits."""
    r = ck_ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    x = _c(logits, np.float32)
    rows, experts = x.shape
    w = np.empty((rows, topk), dtype=np.float32)
    idx = np.empty((rows, topk), dtype=np.int32)
    r.ck_ref_topk_softmax(_p(x), C.c_int32(rows), C.c_int32(experts), C.c_int32(topk), _p(w), _p(idx))
    return w, idx


# ----------------------------------------------------------------------------- fused MoE
def fused_moe(a, a_dt, g, g_dt, d, d_dt, sorted_ids, sorted_w, sorted_eid, post_pad, block_m,
              tokens, experts, hidden, inter, topk, a_scale=None, g_scale=None, d_scale=None,
              gate_only=False, out_dt=DT_BF16, strict=False, want_partials=False, activation=1):
    """Oracle forward.  Operands are numpy arrays holding the raw storage type of their dtype
    code (uint16 for bf16, uint8 for e4m3, int8, float32).  Returns o[tokens, hidden] (uint16 bf16
    bits or float32) and, if asked, the fp32 per-slot partials [tokens, topk, hidden]."""
    a = _c(a, _NP_OF_DT[a_dt])
    g = _c(g, _NP_OF_DT[g_dt])
    d = _c(d, _NP_OF_DT[d_dt])
    n0 = inter * (1 if gate_only else 2)
    assert a.size == tokens * hidden and g.size == experts * n0 * hidden and d.size == experts * hidden * inter
    a_scale, g_scale, d_scale = _c(a_scale, np.float32), _c(g_scale, np.float32), _c(d_scale, np.float32)
    o = np.empty((tokens, hidden), dtype=_NP_OF_DT[out_dt])
    part = np.empty((tokens, topk, hidden), dtype=np.float32) if want_partials else None
    ids, w, eid = _c(sorted_ids, np.int32), _c(sorted_w, np.float32), _c(sorted_eid, np.int32)
    rc = lib().moe_oracle_fused_moe(_p(a), a_dt, _p(a_scale), _p(g), g_dt, _p(g_scale), _p(d), d_dt,
                                    _p(d_scale), _p(o), out_dt, _p(ids), _p(w), _p(eid),
                                    int(post_pad), block_m, tokens, experts, hidden, inter, topk,
                                    int(bool(gate_only)), int(bool(strict)), _p(part), int(activation))
    if rc != 0:
        raise MemoryError("moe_oracle_fused_moe failed")
    return (o, part) if want_partials else o


def fused_moe_f16(a, g, d, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, tokens, experts, hidden, inter, topk,
                  **kw):
    """The oracle for fp16 operands (numpy float16 arrays) and fp16 output: every fp16 value is an fp32 value, so the
    operands go in as float32 and the fp32 result is rounded to fp16 once (numpy's cast: IEEE round to nearest even),
    which is what reference_fused_moe does when instantiated with half_t (reference_fused_moe.hpp:186-197)."""
    f = lambda x: np.ascontiguousarray(np.asarray(x, dtype=np.float16).astype(np.float32))
    o = fused_moe(f(a), DT_F32, f(g), DT_F32, f(d), DT_F32, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, tokens,
                  experts, hidden, inter, topk, out_dt=DT_F32, **kw)
    return o.astype(np.float16)


def ck_fused_moe(a, g, d, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, tokens, experts,
                 hidden, inter, topk, gate_only=False, f32_inputs=False, activation=1, f16=False):
    """ck_tile::reference_fused_moe on bf16 (uint16 bits), fp16 (f16: float16 bits in and out) or float32 operands
    -> bf16 bits (fp16 bits with f16)."""
    r = ck_ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    dt = np.float32 if f32_inputs else np.uint16
    a, g, d = _c(a, dt), _c(g, dt), _c(d, dt)
    o = np.empty((tokens, hidden), dtype=np.uint16)
    fn = r.ck_ref_fused_moe_f32 if f32_inputs else (r.ck_ref_fused_moe_f16 if f16 else r.ck_ref_fused_moe_bf16)
    ids, w, eid = _c(sorted_ids, np.int32), _c(sorted_w, np.float32), _c(sorted_eid, np.int32)
    fn(_p(a), _p(g), _p(d), _p(o), _p(ids), _p(w), _p(eid), int(post_pad), block_m, tokens, experts,
       hidden, inter, topk, int(bool(gate_only)), int(activation))
    return o


def num_threads() -> int:
    return int(lib().moe_oracle_num_threads())
