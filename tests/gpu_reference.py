"""A full-size GPU reference for the fused-MoE output: per-expert fp32 matmuls in torch on de-quantised operands
(the textbook dense-MoE formula, no sorting, y kept in fp32 like ck_tile's host reference).  It is not the oracle:
tests check it against the oracle on sampled tokens first and only then use it to compare EVERY element of the
HIP path's output - every expert, every column tile, every XCD chunk boundary."""
import torch


def _deq(x, scale):
    x = x.float()
    return x if scale is None else x * scale[..., None]


def fused_moe_fp32(cfg, inp, activation=1):
    """[tokens, hidden] float32 (not rounded to bf16) = sum_k w[t,k] * FFN_{e(t,k)}(x_t), fp32 throughout."""
    T, H, I, E, K = cfg.tokens, cfg.hidden, cfg.inter, cfg.experts, cfg.topk
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        x = _deq(inp["a"], inp["a_scale"])
        out = torch.zeros((T, K, H), dtype=torch.float32, device=x.device)
        ids = inp["topk_ids"].long()
        for e in range(E):
            t_idx, k_idx = torch.nonzero(ids == e, as_tuple=True)
            if t_idx.numel() == 0:
                continue
            g = _deq(inp["g"][e], None if inp["g_scale"] is None else inp["g_scale"][e])
            d = _deq(inp["d"][e], None if inp["d_scale"] is None else inp["d_scale"][e])
            acc = x[t_idx] @ g.T
            gate, up = acc[:, :I], acc[:, I:]
            y = (torch.nn.functional.silu(gate) if activation == 1 else torch.nn.functional.gelu(gate)) * up
            out[t_idx, k_idx] = (y @ d.T) * inp["topk_weight"][t_idx, k_idx][:, None]
        # slots summed in slot order, as the reference's reduction does
        o = out[:, 0].clone()
        for k in range(1, K):
            o += out[:, k]
        return o
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


def error_profile(got_bf16, ref_f32, col_block=256):
    """rel-L2 over everything, the worst single token, and the worst (token, col_block columns) cell relative to the
    RMS cell norm of the reference (cells of near-zero reference norm would otherwise dominate)."""
    diff = got_bf16.float() - ref_f32
    total = float(diff.norm() / ref_f32.norm())
    per_tok = diff.norm(dim=1) / ref_f32.norm(dim=1).clamp_min(1e-30)
    T, H = ref_f32.shape
    nb = H // col_block
    dc = diff[:, :nb * col_block].reshape(T, nb, col_block).norm(dim=2)
    rc = ref_f32[:, :nb * col_block].reshape(T, nb, col_block).norm(dim=2)
    cell = dc / rc.pow(2).mean().sqrt()
    return total, float(per_tok.max()), float(cell.max())
