"""Helpers shared by the GPU parity tests: move oracle-sized numpy inputs to the device, run the
HIP path through the C ABI (therock_amd.moe is a ctypes veneer) and bring results back."""
import numpy as np
import torch

import therock_amd as ta

TORCH_DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp8": torch.float8_e4m3fn, "int8": torch.int8}
NP_VIEW = {"bf16": torch.uint16, "fp8": torch.uint8, "int8": torch.int8}


def dev(x, view=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t.view(view) if view is not None else t


def run_sorting(topk_ids, weights, experts, unit, mask=None, local_tokens=None, moe_buf=None,
                fill=True, skip_empty=True, dispatch_policy=0):
    """Returns numpy (ids, w, eid, total[2]) with untouched cells holding -1 (when fill)."""
    T, K = topk_ids.shape
    mp = ta.moe_max_num_tokens_padded(T, experts, K, unit)
    if not skip_empty:  # every expert owns a unit even when no token chose it
        mp = T * K + experts * unit
    ids = torch.full((mp,), -1, dtype=torch.int32, device="cuda")
    w = torch.full((mp,), -1.0, dtype=torch.float32, device="cuda")
    eid = torch.full(((mp + unit - 1) // unit,), -1, dtype=torch.int32, device="cuda")
    total = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    ws_bytes = ta.moe_sorting_get_workspace_size(T, experts, K, dispatch_policy)
    ws = torch.full((max(ws_bytes, 4),), 0x5A, dtype=torch.uint8, device="cuda")  # deliberately dirty
    args = ta.moe_sorting_args(
        p_topk_ids=dev(topk_ids.astype(np.int32)), p_weights=dev(weights.astype(np.float32)),
        p_local_expert_mask=None if mask is None else dev(mask.astype(np.int32)),
        p_local_tokens=None if local_tokens is None else dev(np.array([local_tokens], dtype=np.int32)),
        p_sorted_token_ids=ids, p_sorted_weights=w, p_sorted_expert_ids=eid, p_total_tokens_post_pad=total,
        p_moe_buf=moe_buf, p_ws=ws if ws_bytes else None, tokens=T, unit_size=unit, num_experts=experts, topk=K,
        moe_buf_interm_dim=0 if moe_buf is None else moe_buf.shape[1],
        moe_buf_elem_bytes=0 if moe_buf is None else moe_buf.element_size())
    rc = ta.moe_sorting(ta.moe_sorting_trait(local_expert_masking=mask is not None, dispatch_policy=dispatch_policy,
                                             skip_experts_with_zero_tokens=skip_empty), args)
    assert rc == 0.0
    torch.cuda.synchronize()
    return ids.cpu().numpy(), w.cpu().numpy(), eid.cpu().numpy(), total.cpu().numpy()


def run_fused_moe(cfg, inp, mask=None, unfused=False, stride_pad=0, activation=1, gate_only=0, weight_permute=0,
                  fused_quant=0):
    """Runs mi355_fused_moe (or sorting + mi355_fused_moegemm) on numpy inputs of
    therock_amd.inputs.make_inputs_np.  Returns (out bf16 bits (fp16 bits for fp16 operands) [T,H] numpy, buffers)."""
    traits = ta.fused_moe_traits(prec_i=cfg.dtype, prec_w=cfg.dtype, prec_o="fp16" if cfg.dtype == "fp16" else "bf16",
                                 block_m=cfg.unit, local_expert_masking=mask is not None, activation=activation,
                                 gate_only=gate_only, weight_permute=weight_permute, fused_quant=fused_quant)
    buf = ta.MoeBuffers(traits, cfg.tokens, cfg.experts, cfg.topk, cfg.hidden, cfg.inter, "cuda")
    view = TORCH_DT[cfg.dtype]
    a = dev(inp["a"]).view(view)
    if stride_pad:
        wide = torch.zeros((cfg.tokens, cfg.hidden + stride_pad), dtype=view, device="cuda")
        wide[:, :cfg.hidden] = a
        a = wide[:, :cfg.hidden]
        buf.out = torch.zeros((cfg.tokens, cfg.hidden + stride_pad), dtype=buf.out.dtype, device="cuda")[:, :cfg.hidden]
    g, d = dev(inp["g"]).view(view), dev(inp["d"]).view(view)
    if weight_permute:  # what ck_tile's example does before the call (b_nr_kr_kw_nw_kv, 16-byte kv)
        g, d = ta.permute_weights(g), ta.permute_weights(d)
    sc = {k: (None if inp[k] is None else dev(inp[k])) for k in ("a_scale", "g_scale", "d_scale")}
    args = ta.make_args(traits, buf, a, g, d, dev(inp["topk_ids"]), dev(inp["topk_weight"]), a_scale=sc["a_scale"],
                        g_scale=sc["g_scale"], d_scale=sc["d_scale"],
                        local_expert_mask=None if mask is None else dev(mask.astype(np.int32)),
                        num_experts=cfg.experts)
    if stride_pad:  # non-contiguous views: hand over raw pointers
        args.a_ptr, args.o_ptr = a.data_ptr(), buf.out.data_ptr()
    if unfused:
        sargs = ta.moe_sorting_args(
            p_topk_ids=args.topk_ids_ptr, p_weights=args.topk_weight_ptr, p_local_expert_mask=args.local_expert_mask_ptr,
            p_sorted_token_ids=buf.sorted_ids, p_sorted_weights=buf.sorted_w, p_sorted_expert_ids=buf.sorted_eid,
            p_total_tokens_post_pad=buf.total, p_moe_buf=None, tokens=cfg.tokens, unit_size=cfg.unit,
            num_experts=cfg.experts, topk=cfg.topk)
        ws_sort = ta.moe_sorting_get_workspace_size(cfg.tokens, cfg.experts, cfg.topk)
        if ws_sort:
            sargs.p_ws = torch.empty((ws_sort,), dtype=torch.uint8, device="cuda")
        assert ta.moe_sorting(ta.moe_sorting_trait(local_expert_masking=mask is not None), sargs) == 0.0
        assert ta.fused_moegemm(traits, args) == 0.0
    else:
        assert ta.fused_moe(traits, args) == 0.0
    torch.cuda.synchronize()
    return buf.out.contiguous().view(torch.uint16).cpu().numpy(), buf


def rel_l2(x, ref):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    return float(np.linalg.norm(x - ref) / max(np.linalg.norm(ref), 1e-30))
