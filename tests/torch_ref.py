"""Independent fp64 statement of the SFT step built from library routines
(torch matmul, F.rms_norm, F.scaled_dot_product_attention, F.silu, F.gelu,
F.cross_entropy, autograd, torch.optim.AdamW).  Used only to pin the oracle:
the backward here comes from autograd, not from hand-written formulas."""
import math

import numpy as np
import torch
import torch.nn.functional as F

from llm_metal_amd.configs import GEMMA3
from llm_metal_amd.synth import lora_views


def _t(a):
    return torch.tensor(np.asarray(a, dtype=np.float64), dtype=torch.float64)


def rope_hf(x, theta):
    """HF-style half-split rotary embedding on [B, H, N, hd]: x*cos + rotate_half(x)*sin."""
    hd, N = x.shape[-1], x.shape[-2]
    inv = 1.0 / (theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd))
    ang = torch.arange(N, dtype=torch.float64)[:, None] * inv[None, :]
    cos = torch.cat([ang.cos(), ang.cos()], -1)
    sin = torch.cat([ang.sin(), ang.sin()], -1)
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    return x * cos + torch.cat([-x2, x1], -1) * sin


class _LinearUpdatedFirst(torch.autograd.Function):
    """y = x W^T whose backward first forms dW, applies W' = half(W - lr dW) and only then
    propagates dx = dy W' — the order in which the reference's full-parameter SGD mode treats
    the Q, K and V projections (src/nn/fast_sft.c:922-946)."""

    @staticmethod
    def forward(ctx, x, W, lr):
        ctx.save_for_backward(x, W)
        ctx.lr = lr
        return x @ W.T

    @staticmethod
    def backward(ctx, dy):
        x, W = ctx.saved_tensors
        dW = dy.reshape(-1, dy.shape[-1]).T @ x.reshape(-1, x.shape[-1])
        W_new = (W.float() - torch.tensor(ctx.lr, dtype=torch.float32) * dW.float()).half().double()
        return dy @ W_new, dW, None


def forward_loss(c, used, lora_flat, tok, tgt, x_embed=None, params=None, qkv_lr=None):
    """lora_flat: torch fp64 leaf tensor.  Returns (mean CE loss, logits).
    params (optional): {name: [per-layer leaf tensors]} + "lm_head" used in place of `used`'s matrices;
    qkv_lr: route the Q/K/V projections through _LinearUpdatedFirst with this learning rate."""
    B, N, D, Hq, Hkv, hd = c.batch, c.seq, c.D, c.Hq, c.Hkv, c.hd
    lv = lora_views(c, lora_flat) if c.R else None
    thetas = c.rope_thetas()
    if x_embed is None:
        x = _t(used["token_emb"])[torch.as_tensor(tok.astype(np.int64))]
        if c.model_type == GEMMA3:
            x = x * float(np.float32(c.emb_scale))
    else:
        x = x_embed
    x = x.reshape(B, N, D)
    sc = c.lora_scaling if c.R else 0.0
    for L in range(c.NL):
        g = lambda k: params[k][L] if (params is not None and k in params) else _t(used[k][L])
        ln = F.rms_norm(x, (D,), g("g_in"), c.eps)
        if qkv_lr is None:
            q = ln @ g("wq").T
            k = ln @ g("wk").T
            v = ln @ g("wv").T
        else:
            q = _LinearUpdatedFirst.apply(ln, g("wq"), qkv_lr)
            k = _LinearUpdatedFirst.apply(ln, g("wk"), qkv_lr)
            v = _LinearUpdatedFirst.apply(ln, g("wv"), qkv_lr)
        if c.R:
            q = q + sc * (ln @ lv[L]["A_q"].T) @ lv[L]["B_q"].T
            v = v + sc * (ln @ lv[L]["A_v"].T) @ lv[L]["B_v"].T
        q = q.reshape(B, N, Hq, hd).transpose(1, 2)
        k = k.reshape(B, N, Hkv, hd).transpose(1, 2)
        v = v.reshape(B, N, Hkv, hd).transpose(1, 2)
        q = rope_hf(F.rms_norm(q, (hd,), g("g_q"), c.eps), thetas[L])
        k = rope_hf(F.rms_norm(k, (hd,), g("g_k"), c.eps), thetas[L])
        if getattr(c, "window", 0) and c.local_layers()[L]:
            # sliding window as a boolean mask for the library routine: query i attends keys i - window + 1 .. i
            i, j = torch.arange(N)[:, None], torch.arange(N)[None, :]
            o = F.scaled_dot_product_attention(q, k, v, attn_mask=(j <= i) & (i - j < c.window), enable_gqa=True)
        else:
            o = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        o = o.transpose(1, 2).reshape(B, N, Hq * hd) @ g("wo").T
        if c.model_type == GEMMA3:
            x = x + F.rms_norm(o, (D,), g("g_post_attn"), c.eps)
            ln = F.rms_norm(x, (D,), g("g_pre_ff"), c.eps)
            a = F.gelu(ln @ g("wg").T, approximate="tanh") * (ln @ g("wu").T)
            x = x + F.rms_norm(a @ g("wd").T, (D,), g("g_post_ff"), c.eps)
        else:
            x = x + o
            ln = F.rms_norm(x, (D,), g("g_post_attn"), c.eps)
            a = F.silu(ln @ g("wg").T) * (ln @ g("wu").T)
            x = x + a @ g("wd").T
    ln = F.rms_norm(x, (D,), _t(used["g_final"]), c.eps)
    lm = params["lm_head"] if params is not None else _t(used["lm_head"])
    logits = ln.reshape(B * N, D) @ lm.T
    loss = F.cross_entropy(logits, torch.as_tensor(tgt.astype(np.int64)), reduction="mean")
    return loss, logits


def train_steps(c, used, lora0, batches, lr, clip=True):
    """Runs len(batches) steps with torch.optim.AdamW + clip_grad_norm_.  Returns
    per-step dicts (loss, grad (pre-clip), lora after the update)."""
    p = torch.nn.Parameter(_t(lora0).clone())
    opt = torch.optim.AdamW([p], lr=lr, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    out = []
    for tok, tgt in batches:
        opt.zero_grad()
        loss, logits = forward_loss(c, used, p, tok, tgt)
        loss.backward()
        g = p.grad.detach().clone()
        gn = float(g.norm())
        if clip and gn > 1.0:
            p.grad.mul_(1.0 / gn)      # the reference's rule: scale by max_norm/norm, no epsilon
        opt.step()
        out.append({"loss": float(loss.detach()), "grad": g.numpy().copy(), "grad_norm": gn,
                    "lora": p.detach().numpy().copy(), "logits": logits.detach().numpy().copy()})
    return out


MATS = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")


def full_param_grads(c, used, tok, tgt, qkv_lr=None):
    """Autograd gradients of the mean CE loss w.r.t. every frozen matrix (R = 0).
    Returns ({name: [per-layer arrays]} + "lm_head", loss, logits)."""
    params = {k: [_t(w).requires_grad_(True) for w in used[k]] for k in MATS}
    params["lm_head"] = _t(used["lm_head"]).requires_grad_(True)
    loss, logits = forward_loss(c, used, None, tok, tgt, params=params, qkv_lr=qkv_lr)
    loss.backward()
    grads = {k: [p.grad.numpy().copy() for p in params[k]] for k in MATS}
    grads["lm_head"] = params["lm_head"].grad.numpy().copy()
    return grads, float(loss.detach()), logits.detach().numpy().copy()
