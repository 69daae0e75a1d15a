"""fp32 dense-mask attention: O = softmax(scale * Q K^T + mask) V.

Restates masked_attention of intra_attn/reference.py:78-83 (which is one call of
torch.nn.functional.scaled_dot_product_attention on fp32 copies with a boolean attn_mask and
enable_gqa) with explicit matmul / softmax, processed in chunks of query rows so that the
S x S score matrix never exists for all heads at once.  Works on CPU and GPU tensors alike.
"""
import torch


def masked_attention_rows(q, k, v, mask_rows, rows=None, softmax_scale=None, chunk=1024, out_dtype=None):
    """Attention output for a subset of query positions.

    q: (B, S, H, D); k, v: (B, S, Hkv, D), H % Hkv == 0; query head h uses kv head h // (H/Hkv).
    mask_rows: (len(rows), S) bool, row r belongs to query position rows[r] (all positions in
    order if rows is None).  Returns (B, len(rows), H, D) in q.dtype like the reference's
    masked_attention, or in `out_dtype` (torch.float32: the result before that final rounding).
    """
    B, S, H, D = q.shape
    Hkv = k.shape[2]
    rep = H // Hkv
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    if rows is None:
        rows = torch.arange(S, device=q.device)
    rows = torch.as_tensor(rows, device=q.device, dtype=torch.long)
    kf = k.float().permute(0, 2, 3, 1)  # B, Hkv, D, S
    vf = v.float().permute(0, 2, 1, 3)  # B, Hkv, S, D
    out_dtype = q.dtype if out_dtype is None else out_dtype
    out = torch.empty(B, rows.numel(), H, D, dtype=out_dtype, device=q.device)
    for r0 in range(0, rows.numel(), chunk):
        idx = rows[r0:r0 + chunk]
        qf = q[:, idx].float().permute(0, 2, 1, 3)  # B, H, R, D
        qf = qf.reshape(B, Hkv, rep, idx.numel(), D)
        s = torch.matmul(qf, kf[:, :, None]) * scale  # B, Hkv, rep, R, S
        s = s.masked_fill(~mask_rows[r0:r0 + chunk].to(q.device)[None, None, None], float("-inf"))
        p = torch.softmax(s, dim=-1)
        o = torch.matmul(p, vf[:, :, None])  # B, Hkv, rep, R, D
        out[:, r0:r0 + chunk] = o.reshape(B, H, idx.numel(), D).permute(0, 2, 1, 3).to(out_dtype)
    return out


def masked_lse_rows(q, k, mask_rows, rows=None, softmax_scale=None, chunk=1024):
    """Natural log of the softmax denominator, log(sum_j exp(scale * q_i . k_j)) over the keys the
    mask shows to row i: (B, H, len(rows)) fp32.  The reference's kernels compute this value as
    `softmax_lse` (csrc/flash_attn/flash_api.cpp:470,670) and its Python layer drops it
    (intra_attn/interface.py:44,65); it is one library routine, torch.logsumexp."""
    B, S, H, D = q.shape
    Hkv = k.shape[2]
    rep = H // Hkv
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    if rows is None:
        rows = torch.arange(S, device=q.device)
    rows = torch.as_tensor(rows, device=q.device, dtype=torch.long)
    kf = k.float().permute(0, 2, 3, 1)
    out = torch.empty(B, H, rows.numel(), dtype=torch.float32, device=q.device)
    for r0 in range(0, rows.numel(), chunk):
        idx = rows[r0:r0 + chunk]
        qf = q[:, idx].float().permute(0, 2, 1, 3).reshape(B, Hkv, rep, idx.numel(), D)
        s = torch.matmul(qf, kf[:, :, None]) * scale
        s = s.masked_fill(~mask_rows[r0:r0 + chunk].to(q.device)[None, None, None], float("-inf"))
        out[:, :, r0:r0 + chunk] = torch.logsumexp(s, dim=-1).reshape(B, H, idx.numel())
    return out


def masked_attention(q, k, v, mask, softmax_scale=None, chunk=1024):
    """reference.py:78-83: q, k, v (B, S, H, D) with H % Hkv == 0; mask (S, S) bool."""
    return masked_attention_rows(q, k, v, mask, None, softmax_scale, chunk)


def masked_attention_grads(q, k, v, dout, mask, softmax_scale=None, dtype=torch.float32):
    """Gradients (dq, dk, dv) of sum(masked_attention(q, k, v, mask) * dout) with respect to q, k
    and v, by automatic differentiation of the explicit matmul / softmax formulation in `dtype`.
    The reference differentiates the same dense-mask attention in its training experiments
    (experiments/llm/llama_intra.py:26: masked SDPA under autograd); it has no backward kernels.
    q, dout: (B, S, H, D); k, v: (B, S, Hkv, D); mask: (S, S) bool.  Results in `dtype`."""
    B, S, H, D = q.shape
    Hkv = k.shape[2]
    rep = H // Hkv
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    with torch.enable_grad():
        qf, kf, vf = (t.detach().to(dtype).requires_grad_(True) for t in (q, k, v))
        qh = qf.permute(0, 2, 1, 3).reshape(B, Hkv, rep, S, D)
        s = torch.matmul(qh, kf.permute(0, 2, 3, 1)[:, :, None]) * scale
        s = s.masked_fill(~mask.to(q.device)[None, None, None], float("-inf"))
        o = torch.matmul(torch.softmax(s, dim=-1), vf.permute(0, 2, 1, 3)[:, :, None])
        o = o.reshape(B, H, S, D).permute(0, 2, 1, 3)
        return torch.autograd.grad(o, (qf, kf, vf), dout.detach().to(dtype))
