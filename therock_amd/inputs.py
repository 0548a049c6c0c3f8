"""Seeded synthetic inputs for the fused-MoE workloads.

The five workloads are the benchmark configurations of this build: a small bf16 case the CPU
reference can run, a Mixtral-style bf16 layer, a DeepSeek-V3-shaped fp8 layer, an int8 decode
regime and a Zipf-skewed bf16 stress case.  Generation runs on whatever device it is given (numpy
Philox on the host for oracle-sized cases, torch's generator on the GPU for full-size ones) and
produces raw storage tensors: bf16 bit patterns, e4m3 (OCP) bytes or int8, plus fp32 scales.

Quantisation follows ck_tile's row-wise rule (host/reference/reference_rowwise_quantization2d.hpp:
12-31): scale = amax / qmax per output channel (weights) or per token (activations),
q = convert(saturate(x / scale)).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace

import numpy as np


@dataclass(frozen=True)
class MoeConfig:
    name: str
    tokens: int
    hidden: int
    inter: int
    experts: int
    topk: int
    dtype: str = "bf16"  # "bf16" | "fp16" | "fp8" | "int8": storage type of activations and weights
    router: str = "softmax_renorm"  # softmax_renorm | softmax | sigmoid_renorm | zipf
    unit: int = 32  # block_m / unit_size used by moe_sorting

    @property
    def flops(self) -> float:
        return 6.0 * self.tokens * self.topk * self.hidden * self.inter

    @property
    def max_pad(self) -> int:
        return self.topk * self.tokens + self.experts * self.unit - self.topk

    def scaled(self, **kw) -> "MoeConfig":
        return replace(self, **kw)


CONFIGS = {
    "cfg1_cpu_ref_bf16": MoeConfig("cfg1_cpu_ref_bf16", 128, 1024, 1024, 8, 2, "bf16", "softmax_renorm"),
    "cfg2_mixtral_bf16": MoeConfig("cfg2_mixtral_bf16", 4096, 4096, 14336, 8, 2, "bf16", "softmax_renorm"),
    "cfg3_dsv3_fp8": MoeConfig("cfg3_dsv3_fp8", 8192, 7168, 2048, 256, 8, "fp8", "sigmoid_renorm"),
    "cfg4_decode_int8_t16": MoeConfig("cfg4_decode_int8_t16", 16, 4096, 1536, 128, 8, "int8", "softmax"),
    "cfg4_decode_int8_t64": MoeConfig("cfg4_decode_int8_t64", 64, 4096, 1536, 128, 8, "int8", "softmax"),
    "cfg4_decode_int8_t256": MoeConfig("cfg4_decode_int8_t256", 256, 4096, 1536, 128, 8, "int8", "softmax"),
    "cfg5_zipf_bf16": MoeConfig("cfg5_zipf_bf16", 32768, 2048, 1408, 64, 6, "bf16", "zipf"),
}

ZIPF_S = 1.2
ZIPF_BETA = 1.5  # logit bias = beta * ln(zipf probability): a handful of tail experts get no token


def zipf_bias(experts: int) -> np.ndarray:
    p = np.arange(1, experts + 1, dtype=np.float64) ** (-ZIPF_S)
    p /= p.sum()
    return (ZIPF_BETA * np.log(p)).astype(np.float32)


# ------------------------------------------------------------------------------ numpy
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_e4m3_bits(x: np.ndarray) -> np.ndarray:
    """Saturating round-to-nearest-even float32 -> OCP e4m3 byte (vectorised)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.minimum(np.abs(x), np.float32(448.0))
    _, e = np.frexp(a)
    ex = np.maximum(e.astype(np.int32) - 1, -6)
    q = np.rint(np.ldexp(a, 3 - ex)).astype(np.int32)  # rint = round half to even
    carry = q == 16
    q = np.where(carry, 8, q)
    ex = np.where(carry, ex + 1, ex)
    sub = (ex == -6) & (q < 8)
    biased = np.where(sub, 0, ex + 7)
    man = np.where(sub, q, q - 8)
    out = (sign | (biased.astype(np.uint8) << 3) | man.astype(np.uint8)).astype(np.uint8)
    out = np.where(a == 0, sign, out).astype(np.uint8)
    out = np.where(np.isnan(x), np.uint8(0x7F), out).astype(np.uint8)
    return out


def rowwise_quant_np(x: np.ndarray, dtype: str):
    """x float32 [..., N] -> (q, scale[...]) with scale = amax/qmax along the last axis."""
    qmax = 448.0 if dtype == "fp8" else 127.0
    amax = np.abs(x).max(axis=-1)
    scale = np.where(amax > 0, amax / np.float32(qmax), np.float32(1.0)).astype(np.float32)
    v = x / scale[..., None]
    if dtype == "fp8":
        q = f32_to_e4m3_bits(v)
    else:
        q = np.rint(np.clip(v, -128.0, 127.0)).astype(np.int8)
    return q, scale


def route_np(logits: np.ndarray, topk: int, router: str):
    """Router front-end used to *generate* topk_ids / topk_weight (input to the path)."""
    logits = logits.astype(np.float32)
    if router == "zipf":
        logits = logits + zipf_bias(logits.shape[1])[None, :]
    if router in ("softmax_renorm", "softmax", "zipf"):
        z = logits - logits.max(axis=1, keepdims=True)
        p = np.exp(z)
        p /= p.sum(axis=1, keepdims=True)
    else:  # sigmoid_renorm
        p = 1.0 / (1.0 + np.exp(-logits))
    ids = np.argsort(-p, axis=1, kind="stable")[:, :topk].astype(np.int32)
    w = np.take_along_axis(p, ids, axis=1).astype(np.float32)
    if router != "softmax":
        w = w / w.sum(axis=1, keepdims=True)
    return np.ascontiguousarray(ids), np.ascontiguousarray(w.astype(np.float32))


def make_inputs_np(cfg: MoeConfig, seed: int = 0) -> dict:
    """Host-side inputs (numpy).  Keys: a, g, d (raw storage), a_scale, g_scale, d_scale (or None),
    topk_ids [T,K] int32, topk_weight [T,K] float32."""
    rng = np.random.Generator(np.random.Philox(seed))
    T, H, I, E, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.topk
    x = rng.standard_normal((T, H), dtype=np.float32)
    g = rng.standard_normal((E, 2 * I, H), dtype=np.float32) * np.float32(0.02)
    d = rng.standard_normal((E, H, I), dtype=np.float32) * np.float32(0.02)
    logits = rng.standard_normal((T, E), dtype=np.float32)
    ids, w = route_np(logits, K, cfg.router)
    out = {"topk_ids": ids, "topk_weight": w, "a_scale": None, "g_scale": None, "d_scale": None}
    if cfg.dtype == "bf16":
        out["a"], out["g"], out["d"] = f32_to_bf16_bits(x), f32_to_bf16_bits(g), f32_to_bf16_bits(d)
    elif cfg.dtype == "fp16":  # fp16 bits
        out["a"], out["g"], out["d"] = (v.astype(np.float16).view(np.uint16) for v in (x, g, d))
    else:
        xb = bf16_bits_to_f32(f32_to_bf16_bits(x))  # activations start life as bf16
        out["a_bf16"] = f32_to_bf16_bits(x)
        out["a"], out["a_scale"] = rowwise_quant_np(xb, cfg.dtype)
        out["g"], out["g_scale"] = rowwise_quant_np(g, cfg.dtype)
        out["d"], out["d_scale"] = rowwise_quant_np(d, cfg.dtype)
    return out


# ------------------------------------------------------------------------------ torch
def make_inputs_torch(cfg: MoeConfig, device, seed: int = 0, expert_chunk: int = 8) -> dict:
    """Device-side inputs (torch tensors of raw storage dtype) for full-size workloads."""
    import torch

    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    T, H, I, E, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.topk
    st = {"bf16": torch.bfloat16, "fp8": torch.float8_e4m3fn, "int8": torch.int8}[cfg.dtype]
    qmax = {"fp8": 448.0, "int8": 127.0}.get(cfg.dtype)

    def quant(v):  # v float32 [..., N]
        amax = v.abs().amax(dim=-1)
        scale = torch.where(amax > 0, amax / qmax, torch.ones_like(amax))
        q = v / scale[..., None]
        if cfg.dtype == "fp8":
            q = q.clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
        else:
            q = q.clamp(-128.0, 127.0).round().to(torch.int8)
        return q, scale.float()

    def weights(n, k):
        w = torch.empty((E, n, k), dtype=st, device=device)
        s = torch.empty((E, n), dtype=torch.float32, device=device) if qmax else None
        for e0 in range(0, E, expert_chunk):
            e1 = min(E, e0 + expert_chunk)
            v = torch.randn((e1 - e0, n, k), generator=gen, device=device, dtype=torch.float32) * 0.02
            if qmax:
                w[e0:e1], s[e0:e1] = quant(v)
            else:
                w[e0:e1] = v.to(st)
            del v
        return w, s

    x = torch.randn((T, H), generator=gen, device=device, dtype=torch.float32).to(torch.bfloat16)
    g, g_scale = weights(2 * I, H)
    d, d_scale = weights(H, I)
    logits = torch.randn((T, E), generator=gen, device=device, dtype=torch.float32)
    if cfg.router == "zipf":
        logits = logits + torch.from_numpy(zipf_bias(E)).to(device)[None, :]
    p = torch.sigmoid(logits) if cfg.router == "sigmoid_renorm" else torch.softmax(logits, dim=1)
    w, ids = torch.topk(p, K, dim=1)
    if cfg.router != "softmax":
        w = w / w.sum(dim=1, keepdim=True)
    out = {"topk_ids": ids.to(torch.int32).contiguous(), "topk_weight": w.float().contiguous(),
           "g": g, "d": d, "g_scale": g_scale, "d_scale": d_scale, "a_scale": None, "a_bf16": x}
    if qmax:
        out["a"], out["a_scale"] = quant(x.float())
    else:
        out["a"] = x
    return out


def decode_bytes(cfg: MoeConfig, active_experts: int, post_pad: int) -> float:
    """Algorithmic HBM bytes of one pass in the bandwidth-bound (decode) regime: weights and
    scales of the experts that received a token, activations in, output out, routing metadata."""
    b = {"bf16": 2, "fp8": 1, "int8": 1}[cfg.dtype]
    T, H, I, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.topk
    byt = active_experts * 3 * H * I * b
    if cfg.dtype != "bf16":
        byt += active_experts * (2 * I + H) * 4 + T * 4
    byt += T * H * b + T * H * 2 + T * K * 8 + post_pad * 8 + math.ceil(post_pad / cfg.unit) * 4
    return float(byt)
