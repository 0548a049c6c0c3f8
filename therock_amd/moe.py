"""Host-side mirror of Composable Kernel's fused-MoE example API on top of the C ABI.

Same names, argument meaning and error behaviour as CK's example/ck_tile/15_fused_moe and
13_moe_sorting (``fused_moe_traits`` / ``fused_moe_args`` / ``fused_moe()``, ``moe_sorting_trait`` /
``moe_sorting_args`` / ``moe_sorting()``): tensors are caller-owned device tensors, the calls are
asynchronous on a stream, ``fused_moe`` returns a float (0 when not timing, -1 when no kernel
matches the traits) and HIP / argument errors raise ``RuntimeError``.  torch is used only to hold
device memory and streams; all compute happens in libmi355_moe.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

from . import _lib


@dataclass
class fused_moe_traits:
    prec_i: str = "bf16"   # input (activation) precision
    prec_w: str = "bf16"   # weight precision
    prec_o: str = "bf16"   # output precision
    prec_st: str = "fp32"  # token scale
    prec_sw: str = "fp32"  # weight scale
    prec_sq: str = "fp32"  # smooth-quant scale
    prec_kw: str = "fp32"  # top-k weight
    block_m: int = 32
    activation: int = 1    # 0 gelu, 1 silu
    gate_only: int = 0
    fused_quant: int = 0
    local_expert_masking: bool = False
    weight_permute: int = 0  # 1: g and d in ck_tile's pre-shuffled layout b_nr_kr_kw_nw_kv

    def pod(self) -> _lib.FusedMoeTraits:
        d = _lib.DTYPES
        for k in ("prec_i", "prec_w", "prec_o", "prec_st", "prec_sw", "prec_sq", "prec_kw"):
            if getattr(self, k) not in d:
                raise ValueError(f"unknown precision {getattr(self, k)!r} for {k}")
        return _lib.FusedMoeTraits(d[self.prec_i], d[self.prec_w], d[self.prec_o], d[self.prec_st], d[self.prec_sw],
                                   d[self.prec_sq], d[self.prec_kw], self.block_m, self.activation, self.gate_only,
                                   self.fused_quant, int(self.local_expert_masking), int(self.weight_permute))


@dataclass
class moe_sorting_trait:
    index_type: str = "int32"
    weight_type: str = "fp32"
    local_expert_masking: bool = False
    clear_workspace_inside_api: bool = False   # accepted: the workspace never needs clearing
    dispatch_policy: int = 0                   # 0 the library picks, 1 single kernel, 2 multi-launch passes
    # MoeSortingProblemEx::SkipExpertsWithZeroTokens (a template argument in ck_tile): False gives every expert of
    # this rank that no token chose one unit of padding
    skip_experts_with_zero_tokens: bool = True


def _ptr(t) -> Optional[int]:
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if not t.is_cuda:
        raise ValueError("tensors handed to the MoE path must live on the GPU")
    if not t.is_contiguous():
        raise ValueError("tensors handed to the MoE path must be contiguous")
    return t.data_ptr()


def _stream(stream) -> Optional[int]:
    import torch

    if stream is None:
        stream = torch.cuda.current_stream()
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream)


@dataclass
class moe_sorting_args:
    p_topk_ids: object = None
    p_weights: object = None
    p_local_expert_mask: object = None
    p_local_tokens: object = None
    p_sorted_token_ids: object = None
    p_sorted_weights: object = None
    p_sorted_expert_ids: object = None
    p_total_tokens_post_pad: object = None
    p_moe_buf: object = None
    p_ws: object = None
    tokens: int = 0
    unit_size: int = 32
    num_experts: int = 0
    topk: int = 0
    moe_buf_interm_dim: int = 0
    moe_buf_elem_bytes: int = 0


@dataclass
class fused_moe_args:
    a_ptr: object = None
    a_scale_ptr: object = None
    g_ptr: object = None
    d_ptr: object = None
    g_scale_ptr: object = None
    d_scale_ptr: object = None
    y_smooth_scale_ptr: object = None
    local_expert_mask_ptr: object = None
    o_ptr: object = None
    ws_ptr: object = None       # CK's example: the sort's workspace; may stay None (the library workspace holds it)
    workspace: object = None    # device tensor of fused_moe_get_workspace_size() bytes, passed beside the arguments
    topk_ids_ptr: object = None
    topk_weight_ptr: object = None
    sorted_token_ids_ptr: object = None
    sorted_weight_ptr: object = None
    sorted_expert_ids_ptr: object = None
    num_sorted_tiles_ptr: object = None
    block_m: int = 32
    hidden_size: int = 0
    intermediate_size: int = 0
    num_tokens: int = 0
    num_experts: int = 0
    topk: int = 0
    stride_token: int = 0


def _check(rc: int, what: str) -> None:
    if rc != _lib.OK:
        raise RuntimeError(f"{what} failed ({rc}): {_lib.last_error()}")


def moe_max_num_tokens_padded(tokens: int, num_experts: int, topk: int, unit_size: int) -> int:
    return int(_lib.load().mi355_moe_max_num_tokens_padded(tokens, num_experts, topk, unit_size))


def moe_sorting_get_workspace_size(tokens: int, num_experts: int, topk: int, dispatch_policy: int = 0) -> int:
    return int(_lib.load().mi355_moe_sorting_workspace_size2(tokens, num_experts, topk, dispatch_policy))


def moe_sorting(trait: moe_sorting_trait, a: moe_sorting_args, stream=None) -> float:
    """Returns 0.0 on success, -1.0 when the trait has no kernel (as CK's dispatcher does)."""
    if trait.index_type != "int32" or trait.weight_type != "fp32":
        return -1.0
    t = _lib.SortingTraits(_lib.DTYPES["int32"], _lib.DTYPES["fp32"], int(trait.local_expert_masking),
                           int(trait.clear_workspace_inside_api), int(trait.dispatch_policy),
                           int(trait.skip_experts_with_zero_tokens))
    s = _lib.SortingArgs(_ptr(a.p_topk_ids), _ptr(a.p_weights), _ptr(a.p_local_expert_mask), _ptr(a.p_local_tokens),
                         _ptr(a.p_sorted_token_ids), _ptr(a.p_sorted_weights), _ptr(a.p_sorted_expert_ids),
                         _ptr(a.p_total_tokens_post_pad), _ptr(a.p_moe_buf), _ptr(a.p_ws), a.tokens, a.unit_size,
                         a.num_experts, a.topk, a.moe_buf_interm_dim, a.moe_buf_elem_bytes)
    _check(_lib.load().mi355_moe_sorting2(C.byref(t), C.byref(s), _stream(stream)), "moe_sorting")
    return 0.0


def fused_moe_get_workspace_size(traits: fused_moe_traits, tokens, num_experts, topk, hidden_size,
                                 intermediate_size) -> int:
    t = traits.pod()
    return int(_lib.load().mi355_fused_moe_workspace_size(C.byref(t), tokens, num_experts, topk, hidden_size,
                                                          intermediate_size))


def _workspace(ws) -> "_lib.Workspace":
    return _lib.Workspace(_ptr(ws), 0 if ws is None else ws.numel() * ws.element_size())


def _fused_args(a: fused_moe_args) -> "_lib.FusedMoeArgs":
    return _lib.FusedMoeArgs(_ptr(a.a_ptr), _ptr(a.a_scale_ptr), _ptr(a.g_ptr), _ptr(a.d_ptr), _ptr(a.g_scale_ptr),
                             _ptr(a.d_scale_ptr), _ptr(a.y_smooth_scale_ptr), _ptr(a.local_expert_mask_ptr),
                             _ptr(a.o_ptr), _ptr(a.ws_ptr), _ptr(a.topk_ids_ptr),
                             _ptr(a.topk_weight_ptr), _ptr(a.sorted_token_ids_ptr), _ptr(a.sorted_weight_ptr),
                             _ptr(a.sorted_expert_ids_ptr), _ptr(a.num_sorted_tiles_ptr), a.block_m, a.hidden_size,
                             a.intermediate_size, a.num_tokens, a.num_experts, a.topk, a.stride_token)


def fused_moe(traits: fused_moe_traits, a: fused_moe_args, stream=None) -> float:
    """Sort + gate/up GEMM + SiLU*up + down GEMM + top-k combine.  0.0 on success, -1.0 when no
    kernel matches the traits."""
    lib = _lib.load()
    t = traits.pod()
    if not lib.mi355_fused_moe_supported(C.byref(t)):
        return -1.0
    f = _fused_args(a)
    ws = _workspace(a.workspace)
    rc = lib.mi355_fused_moe(C.byref(t), C.byref(f), C.byref(ws), _stream(stream))
    if rc == _lib.E_UNSUPPORTED:
        return -1.0
    _check(rc, "fused_moe")
    return 0.0


def fused_moe_static_ws_capacity() -> int:
    return int(_lib.load().mi355_fused_moe_static_ws_capacity())


def fused_moe_static_ws(traits: fused_moe_traits, a: fused_moe_args, stream=None) -> float:
    """fused_moe() on the library-owned workspace: allocates nothing, a.workspace is ignored.  Problems that need
    more than fused_moe_static_ws_capacity() bytes raise; calls that overlap on one GPU race."""
    lib = _lib.load()
    t = traits.pod()
    if not lib.mi355_fused_moe_supported(C.byref(t)):
        return -1.0
    rc = lib.mi355_fused_moe_static_ws(C.byref(t), C.byref(_fused_args(a)), _stream(stream))
    if rc == _lib.E_UNSUPPORTED:
        return -1.0
    _check(rc, "fused_moe_static_ws")
    return 0.0


def fused_moegemm(traits: fused_moe_traits, a: fused_moe_args, stream=None) -> float:
    """GEMM half only: consumes sorted_* / num_sorted_tiles already written by moe_sorting."""
    lib = _lib.load()
    t = traits.pod()
    if not lib.mi355_fused_moe_supported(C.byref(t)):
        return -1.0
    g = _lib.FusedMoeGemmArgs(_ptr(a.a_ptr), _ptr(a.a_scale_ptr), _ptr(a.g_ptr), _ptr(a.d_ptr), _ptr(a.g_scale_ptr),
                              _ptr(a.d_scale_ptr), _ptr(a.y_smooth_scale_ptr), _ptr(a.o_ptr),
                              _ptr(a.sorted_token_ids_ptr), _ptr(a.sorted_weight_ptr), _ptr(a.sorted_expert_ids_ptr),
                              _ptr(a.num_sorted_tiles_ptr), a.hidden_size,
                              a.intermediate_size, a.num_tokens, a.num_experts, a.topk, a.stride_token)
    ws = _workspace(a.workspace)
    rc = lib.mi355_fused_moegemm(C.byref(t), C.byref(g), C.byref(ws), _stream(stream))
    if rc == _lib.E_UNSUPPORTED:
        return -1.0
    _check(rc, "fused_moegemm")
    return 0.0


def rowwise_quant(x, q_dtype: str, stream=None):
    """Per-token dynamic quantisation of a bf16 [rows, cols] tensor -> (q, scale[rows] fp32)."""
    import torch

    rows, cols = x.shape
    st = {"fp8": torch.float8_e4m3fn, "int8": torch.int8}[q_dtype]
    q = torch.empty((rows, cols), dtype=st, device=x.device)
    scale = torch.empty((rows,), dtype=torch.float32, device=x.device)
    _check(_lib.load().mi355_moe_rowwise_quant(_ptr(x), rows, cols, x.stride(0), _lib.DTYPES[q_dtype], _ptr(q),
                                               _ptr(scale), _stream(stream)), "rowwise_quant")
    return q, scale


GEMM1_GATE_ONLY, GEMM1_GATE_UP, GEMM2 = 0, 1, 2


ACT_SILU, ACT_SWIGLU = 0, 1


def _flatmm_args(kind, a, b, c, sorted_ids, sorted_eid, max_token_id, num_tokens, topk, block_m, sorted_weights,
                 scale_m, scale_n, exp_bias, activation, swiglu_alpha, swiglu_limit, n_padded_zeros, k_padded_zeros,
                 b_shuffle=0):
    import torch

    experts, n, k = b.shape
    dt = {torch.bfloat16: "bf16", torch.float16: "fp16", torch.int8: "int8", torch.float8_e4m3fn: "fp8", torch.uint8: "fp8"}
    return _lib.FlatmmArgs(_ptr(sorted_ids), _ptr(sorted_weights), _ptr(sorted_eid), _ptr(max_token_id), _ptr(a), _ptr(b),
                           _ptr(c), num_tokens, experts, topk, 1, sorted_ids.numel(), n, k, a.stride(0), k, c.stride(0),
                           n_padded_zeros, k_padded_zeros, _ptr(scale_m), _ptr(scale_n), _ptr(exp_bias),
                           _lib.DTYPES[dt[a.dtype]], _lib.DTYPES[dt[b.dtype]], block_m, activation, swiglu_alpha,
                           swiglu_limit, b_shuffle)


def moe_flatmm_get_workspace_size(kind: int, a, b, c, sorted_ids, sorted_eid, max_token_id, num_tokens: int, topk: int,
                                  block_m: int, **kw) -> int:
    """Bytes of the workspace tensor moe_flatmm needs for these arguments (0: no kernel)."""
    args = _flatmm_args(kind, a, b, c, sorted_ids, sorted_eid, max_token_id, num_tokens, topk, block_m, None, None, None,
                        None, ACT_SILU, 1.702, 7.0, kw.get("n_padded_zeros", 0), kw.get("k_padded_zeros", 0))
    return int(_lib.load().mi355_moe_flatmm_workspace_size(kind, C.byref(args)))


def moe_flatmm(kind: int, a, b, c, sorted_ids, sorted_eid, max_token_id, num_tokens: int, topk: int, block_m: int,
               sorted_weights=None, scale_m=None, scale_n=None, exp_bias=None, activation: int = ACT_SILU,
               swiglu_alpha: float = 1.702, swiglu_limit: float = 7.0, n_padded_zeros: int = 0, k_padded_zeros: int = 0,
               workspace=None, stream=None, b_shuffle: int = 0):
    """One grouped GEMM of the MoE layer as its own launch (ck_tile's MoeFlatmm conventions): kind
    GEMM1_GATE_UP writes c[token * topk + slot, :N/2] = act(gate, up), GEMM1_GATE_ONLY c[.., :N] = act(a b^T),
    kind GEMM2 adds the weighted down projection of a[token * topk + slot] to c[token].  b is [experts, N, K].
    workspace: a device tensor of moe_flatmm_get_workspace_size() bytes owned by the caller (it must stay alive
    until the launches have run); when None one is allocated here on torch's current stream, which is then the
    only stream the call may use."""
    import torch

    args = _flatmm_args(kind, a, b, c, sorted_ids, sorted_eid, max_token_id, num_tokens, topk, block_m, sorted_weights,
                        scale_m, scale_n, exp_bias, activation, swiglu_alpha, swiglu_limit, n_padded_zeros, k_padded_zeros,
                        b_shuffle)
    lib = _lib.load()
    if workspace is None:
        if stream is not None and _stream(stream) != _stream(None):
            raise ValueError("moe_flatmm: pass a caller-owned workspace when launching on a stream other than the current one")
        ws_bytes = int(lib.mi355_moe_flatmm_workspace_size(kind, C.byref(args)))
        workspace = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=a.device)
    ws = _workspace(workspace)
    rc = lib.mi355_moe_flatmm(kind, C.byref(args), C.byref(ws), _stream(stream))
    if rc == _lib.E_UNSUPPORTED:
        return -1.0
    _check(rc, "moe_flatmm")
    return 0.0


def permute_weights(w, nw: int = 16, kw: int = 4, kv: int | None = None, inverse: bool = False, stream=None):
    """[experts, n, k] weights to (inverse=False) or from (inverse=True) ck_tile's pre-shuffled layout
    b_nr_kr_kw_nw_kv.  kv defaults to 16 bytes worth of elements (CK's example: 8 for bf16, 16 for 8-bit)."""
    import torch

    experts, n, k = w.shape
    eb = w.element_size()
    kv = kv if kv is not None else 16 // eb
    out = torch.empty_like(w)
    _check(_lib.load().mi355_moe_permute_weights(_ptr(w), _ptr(out), experts, n, k, eb, nw, kw, kv, int(bool(inverse)),
                                                 _stream(stream)), "permute_weights")
    return out


def moe_smoothquant(x, smscale, topk_ids, q_dtype: str = "int8", stream=None, out=None):
    """CK's moe_smoothquant(traits, args, stream): x [tokens, hidden] bf16, smscale [experts, hidden] fp32,
    topk_ids [tokens, topk] int32 -> (qy [topk, tokens, hidden] int8 / e4m3, yscale [topk, tokens] fp32).
    out: a (qy, yscale) pair of contiguous tensors to write into instead of new ones."""
    import torch

    tokens, hidden = x.shape
    experts, topk = smscale.shape[0], topk_ids.shape[1]
    st = {"fp8": torch.float8_e4m3fn, "int8": torch.int8}[q_dtype]
    if out is not None:
        qy, ys = out
        assert qy.shape == (topk, tokens, hidden) and qy.dtype == st and qy.is_contiguous()
        assert ys.shape == (topk, tokens) and ys.dtype == torch.float32 and ys.is_contiguous()
    else:
        qy = torch.empty((topk, tokens, hidden), dtype=st, device=x.device)
        ys = torch.empty((topk, tokens), dtype=torch.float32, device=x.device)
    a = _lib.SmoothquantArgs(_ptr(x), _ptr(smscale), _ptr(topk_ids), _ptr(ys), _ptr(qy), tokens, hidden, experts, topk,
                             x.stride(0) if tokens else hidden, hidden)
    _check(_lib.load().mi355_moe_smoothquant(C.byref(a), _lib.DTYPES[q_dtype], _stream(stream)), "moe_smoothquant")
    return qy, ys


def topk_softmax(logits, topk: int, activation: str = "softmax", renormalize: bool = False, stream=None):
    """Router front-end (CK's topk_softmax(trait, kargs, stream)): softmax or sigmoid over the experts of
    each row of `logits` [rows, experts] (fp32, bf16 or fp16), then the top-k weights (fp32, descending) and
    expert ids (int32).  Returns (weights[rows, topk], ids[rows, topk])."""
    import torch

    rows, experts = logits.shape
    assert logits.stride(1) == 1
    kind = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}[logits.dtype]
    w = torch.empty((rows, topk), dtype=torch.float32, device=logits.device)
    ids = torch.empty((rows, topk), dtype=torch.int32, device=logits.device)
    t = _lib.TopkSoftmaxTraits(_lib.DTYPES[kind], _lib.DTYPES["fp32"], experts,
                               {"softmax": 0, "sigmoid": 1}[activation], int(bool(renormalize)))
    a = _lib.TopkSoftmaxArgs(_ptr(logits), _ptr(w), _ptr(ids), rows, experts, topk, logits.stride(0) if rows else experts, topk)
    _check(_lib.load().mi355_topk_softmax(C.byref(t), C.byref(a), _stream(stream)), "topk_softmax")
    return w, ids


# ------------------------------------------------------------------ convenience for harnesses
def fused_moe_tile_rows(traits: fused_moe_traits, tokens, num_experts, topk, hidden_size, intermediate_size) -> int:
    """Sorted rows one GEMM workgroup owns at this problem size (320 selects the large-tile kernel)."""
    t = traits.pod()
    return int(_lib.load().mi355_fused_moe_tile_rows(C.byref(t), tokens, num_experts, topk, hidden_size,
                                                     intermediate_size))


def fused_moe_chosen_tile_rows(traits: fused_moe_traits, buf, tokens, num_experts, topk, hidden_size, intermediate_size,
                               stream=None) -> int:
    """The tile height the last fused_moe call on buf's workspace ran with (where the routing decides, the sort's
    choice on the device, read back after a stream synchronisation; else fused_moe_tile_rows)."""
    t = traits.pod()
    ws = _workspace(buf.ws)
    return int(_lib.load().mi355_fused_moe_chosen_tile_rows(C.byref(t), tokens, num_experts, topk, hidden_size,
                                                            intermediate_size, C.byref(ws), _stream(stream)))


class MoeBuffers:
    """Caller-side allocation of everything fused_moe needs (what CK's example main does with
    DeviceMem): sort outputs, workspace and the output tensor."""

    def __init__(self, traits: fused_moe_traits, tokens, experts, topk, hidden, inter, device):
        import torch

        self.max_pad = moe_max_num_tokens_padded(tokens, experts, topk, traits.block_m)
        self.max_tiles = (self.max_pad + traits.block_m - 1) // traits.block_m
        self.sorted_ids = torch.empty((self.max_pad,), dtype=torch.int32, device=device)
        self.sorted_w = torch.empty((self.max_pad,), dtype=torch.float32, device=device)
        self.sorted_eid = torch.empty((self.max_tiles,), dtype=torch.int32, device=device)
        self.total = torch.zeros((2,), dtype=torch.int32, device=device)
        ws = fused_moe_get_workspace_size(traits, tokens, experts, topk, hidden, inter)
        self.ws = torch.empty((max(ws, 256),), dtype=torch.uint8, device=device)
        self.out = torch.empty((tokens, hidden), dtype=torch.float16 if traits.prec_o == "fp16" else torch.bfloat16,
                               device=device)


def make_args(traits: fused_moe_traits, buf: MoeBuffers, a, g, d, topk_ids, topk_weight, a_scale=None,
              g_scale=None, d_scale=None, local_expert_mask=None, num_experts=None) -> fused_moe_args:
    T, H = a.shape
    E, n0, _ = g.shape
    if num_experts is not None:  # with a local expert mask g/d hold the local experts only
        E = num_experts
    return fused_moe_args(
        a_ptr=a, a_scale_ptr=a_scale, g_ptr=g, d_ptr=d, g_scale_ptr=g_scale, d_scale_ptr=d_scale,
        local_expert_mask_ptr=local_expert_mask, o_ptr=buf.out, workspace=buf.ws, topk_ids_ptr=topk_ids,
        topk_weight_ptr=topk_weight, sorted_token_ids_ptr=buf.sorted_ids, sorted_weight_ptr=buf.sorted_w,
        sorted_expert_ids_ptr=buf.sorted_eid, num_sorted_tiles_ptr=buf.total, block_m=traits.block_m,
        hidden_size=H, intermediate_size=n0 if traits.gate_only else n0 // 2, num_tokens=T, num_experts=E, topk=topk_ids.shape[1],
        stride_token=a.stride(0))
