"""One decode step per token through the inference ops, in the order of the reference's forward_token
(src/nn/fast_inference.c:376-467): once on the CPU oracle's ops and once through the C ABI on the GPU.
Both return the logits of every position, so they can be compared with each other and with the rows of the
training forward (causal attention: position t only sees tokens 0..t)."""
import numpy as np

from llm_metal_amd.configs import GEMMA3
from llm_metal_amd.synth import MATS, lora_views, mat_shapes
from oracle import oracle
from oracle.oracle import SZ, op


def _pack(w, fmt):
    """Weight bytes as the reference's WMat holds them (src/nn/wmat.c:46-75)."""
    if fmt == "q8_0":
        return oracle.q8_quantize(w)
    return np.ascontiguousarray(w.astype(np.float16)).view(np.uint16)


def oracle_decode(c, model, fmt, tokens, max_seq, precision="f32", lora=None):
    dt = oracle.real_dtype(precision)
    shp = mat_shapes(c)
    W = {k: [_pack(model[k][L], fmt) for L in range(c.NL)] for k in MATS}
    lm = _pack(model["lm_head"], fmt)
    lv = lora_views(c, np.asarray(lora, dtype=dt)) if lora is not None else None
    thetas = c.rope_thetas()
    qd, kd = c.Hq * c.hd, c.Hkv * c.hd

    def matvec(w, rows, cols, x):
        y = np.zeros(rows, dt)
        if fmt == "q8_0":
            op(precision, "or_q8_matvec", w, x, y, rows, cols // 32)
        else:
            op(precision, "or_f16_batch_matvec", w, x, y, rows, cols, 1)
        return y

    def norm(x, g):
        out = np.zeros_like(x)
        op(precision, "or_rms_norm", x, np.asarray(g, np.float32), out, x.size, c.eps, 1)
        return out

    kc = [np.zeros((c.Hkv, max_seq, c.hd), dt) for _ in range(c.NL)]
    vc = [np.zeros((c.Hkv, max_seq, c.hd), dt) for _ in range(c.NL)]
    logits = np.zeros((len(tokens), c.V), dt)
    for pos, tok in enumerate(tokens):
        x = model["token_emb"][tok].astype(dt) * dt(c.emb_scale)
        for L in range(c.NL):
            ln = norm(x, model["g_in"][L])
            q = matvec(W["wq"][L], *shp["wq"], ln)
            k = matvec(W["wk"][L], *shp["wk"], ln)
            v = matvec(W["wv"][L], *shp["wv"], ln)
            if lv is not None:
                for dst, A, B, n in ((q, lv[L]["A_q"], lv[L]["B_q"], qd), (v, lv[L]["A_v"], lv[L]["B_v"], kd)):
                    tmp, out = np.zeros(c.R, dt), np.zeros(n, dt)
                    op(precision, "or_matmul", ln, np.ascontiguousarray(A), tmp, 1, c.R, c.D)
                    op(precision, "or_matmul", tmp, np.ascontiguousarray(B), out, 1, n, c.R)
                    op(precision, "or_add_scaled", dst, out, c.lora_scaling, SZ(n))
            op(precision, "or_rms_norm", q, model["g_q"][L], q, c.hd, c.eps, c.Hq)          # per head, in place
            op(precision, "or_rms_norm", k, model["g_k"][L], k, c.hd, c.eps, c.Hkv)
            op(precision, "or_rope", q, k, c.Hq, c.Hkv, c.hd, pos, float(thetas[L]))
            op(precision, "or_kv_cache_store", k, v, kc[L], vc[L], c.Hkv, max_seq, c.hd, pos)
            att = np.zeros(qd, dt)
            op(precision, "or_attention", q, kc[L], vc[L], att, pos + 1, c.hd, max_seq, c.Hq, c.Hq // c.Hkv)
            x2 = matvec(W["wo"][L], *shp["wo"], att)
            if c.model_type == GEMMA3:
                x2 = norm(x2, model["g_post_attn"][L])
            x = x + x2
            ln = norm(x, model["g_pre_ff"][L] if c.model_type == GEMMA3 else model["g_post_attn"][L])
            gate = matvec(W["wg"][L], *shp["wg"], ln)
            up = matvec(W["wu"][L], *shp["wu"], ln)
            op(precision, "or_gelu_mul" if c.model_type == GEMMA3 else "or_silu_mul", gate, up, SZ(c.IS))
            ff = matvec(W["wd"][L], *shp["wd"], gate)
            if c.model_type == GEMMA3:
                ff = norm(ff, model["g_post_ff"][L])
            x = x + ff
        logits[pos] = matvec(lm, c.V, c.D, norm(x, model["g_final"]))
    return logits


def device_decode(dev, c, model, fmt, tokens, max_seq, lora=None, use_off=False):
    """The same walk through metal_enqueue_*; use_off: q, k, v, attention output live in one buffer and the
    per-item ops get byte offsets (the reference's batched-inference variants)."""
    L_, F = dev.L, np.float32
    shp = mat_shapes(c)
    W = {k: [dev.up(_pack(model[k][L], fmt)) for L in range(c.NL)] for k in MATS}
    lm = dev.up(_pack(model["lm_head"], fmt))
    G = {k: [dev.up(np.asarray(g, F)) if g is not None else None for g in model[k]]
         for k in ("g_in", "g_post_attn", "g_pre_ff", "g_post_ff", "g_q", "g_k")}
    g_final = dev.up(np.asarray(model["g_final"], F))
    lv = lora_views(c, np.asarray(lora, dtype=F)) if lora is not None else None
    lb = [{k: dev.up(np.ascontiguousarray(v)) for k, v in d.items()} for d in lv] if lv is not None else None
    thetas = c.rope_thetas()
    qd, kd = c.Hq * c.hd, c.Hkv * c.hd
    kc = [dev.up(np.zeros((c.Hkv, max_seq, c.hd), F)) for _ in range(c.NL)]
    vc = [dev.up(np.zeros((c.Hkv, max_seq, c.hd), F)) for _ in range(c.NL)]
    x, x2, ln = dev.empty(c.D * 4), dev.empty(c.D * 4), dev.empty(c.D * 4)
    gate, up, ff = dev.empty(c.IS * 4), dev.empty(c.IS * 4), dev.empty(c.D * 4)
    lg = dev.empty(c.V * 4)
    tmp, lout = dev.empty(max(c.R, 1) * 4), dev.empty(qd * 4)
    if use_off:
        arena = dev.empty((2 * qd + 2 * kd) * 4)
        q_off, k_off, v_off, a_off = 0, qd * 4, (qd + kd) * 4, (qd + 2 * kd) * 4
        q = dev.view(arena, q_off, qd * 4); k = dev.view(arena, k_off, kd * 4)
        v = dev.view(arena, v_off, kd * 4); att = dev.view(arena, a_off, qd * 4)
    else:
        q, k, v, att = dev.empty(qd * 4), dev.empty(kd * 4), dev.empty(kd * 4), dev.empty(qd * 4)

    def matvec(w, rows, cols, xin, yout):
        if fmt == "q8_0":
            L_.metal_enqueue_q8_matvec(w.h, xin.h, yout.h, rows, cols // 32)
        else:
            L_.metal_enqueue_f16_matvec(w.h, xin.h, yout.h, rows, cols)

    logits = np.zeros((len(tokens), c.V), F)
    for pos, tok in enumerate(tokens):
        x.write((model["token_emb"][tok].astype(F) * F(c.emb_scale)).astype(F))
        for L in range(c.NL):
            L_.metal_enqueue_rms_norm(x.h, G["g_in"][L].h, ln.h, c.D, c.eps)
            matvec(W["wq"][L], *shp["wq"], ln, q)
            matvec(W["wk"][L], *shp["wk"], ln, k)
            matvec(W["wv"][L], *shp["wv"], ln, v)
            if lb is not None:
                for dst, A, B, n in ((q, lb[L]["A_q"], lb[L]["B_q"], qd), (v, lb[L]["A_v"], lb[L]["B_v"], kd)):
                    L_.metal_enqueue_float_matmul(ln.h, A.h, tmp.h, 1, c.R, c.D)
                    L_.metal_enqueue_float_matmul(tmp.h, B.h, lout.h, 1, n, c.R)
                    L_.metal_enqueue_add_scaled(dst.h, lout.h, c.lora_scaling, n)
            th = float(thetas[L])
            if use_off:
                L_.metal_enqueue_per_head_rms_norm_off(arena.h, q_off, G["g_q"][L].h, c.Hq, c.hd, c.eps)
                L_.metal_enqueue_per_head_rms_norm_off(arena.h, k_off, G["g_k"][L].h, c.Hkv, c.hd, c.eps)
                L_.metal_enqueue_rope_off(arena.h, q_off, arena.h, k_off, c.Hq, c.Hkv, c.hd, pos, th)
                L_.metal_enqueue_kv_cache_store_off(arena.h, k_off, arena.h, v_off, kc[L].h, vc[L].h, c.Hkv, max_seq, c.hd, pos)
                L_.metal_enqueue_attention_off(arena.h, q_off, kc[L].h, vc[L].h, arena.h, a_off, pos + 1, c.hd, max_seq, c.Hq,
                                               c.Hq // c.Hkv)
            else:
                L_.metal_enqueue_per_head_rms_norm(q.h, G["g_q"][L].h, c.Hq, c.hd, c.eps)
                L_.metal_enqueue_per_head_rms_norm(k.h, G["g_k"][L].h, c.Hkv, c.hd, c.eps)
                L_.metal_enqueue_rope(q.h, k.h, c.Hq, c.Hkv, c.hd, pos, th)
                L_.metal_enqueue_kv_cache_store(k.h, v.h, kc[L].h, vc[L].h, c.Hkv, max_seq, c.hd, pos)
                L_.metal_enqueue_attention(q.h, kc[L].h, vc[L].h, att.h, pos + 1, c.hd, max_seq, c.Hq, c.Hq // c.Hkv)
            matvec(W["wo"][L], *shp["wo"], att, x2)
            if c.model_type == GEMMA3:
                L_.metal_enqueue_rms_norm(x2.h, G["g_post_attn"][L].h, ln.h, c.D, c.eps)
                L_.metal_enqueue_residual_add(x.h, ln.h, c.D)
            else:
                L_.metal_enqueue_residual_add(x.h, x2.h, c.D)
            g_ff = G["g_pre_ff"][L] if c.model_type == GEMMA3 else G["g_post_attn"][L]
            L_.metal_enqueue_rms_norm(x.h, g_ff.h, ln.h, c.D, c.eps)
            matvec(W["wg"][L], *shp["wg"], ln, gate)
            matvec(W["wu"][L], *shp["wu"], ln, up)
            if c.model_type == GEMMA3:
                L_.metal_enqueue_gelu_mul(gate.h, up.h, c.IS)
            else:
                L_.metal_enqueue_silu_mul(gate.h, up.h, c.IS)
            matvec(W["wd"][L], *shp["wd"], gate, ff)
            if c.model_type == GEMMA3:
                L_.metal_enqueue_rms_norm(ff.h, G["g_post_ff"][L].h, x2.h, c.D, c.eps)
                L_.metal_enqueue_residual_add(x.h, x2.h, c.D)
            else:
                L_.metal_enqueue_residual_add(x.h, ff.h, c.D)
        L_.metal_enqueue_rms_norm(x.h, g_final.h, ln.h, c.D, c.eps)
        matvec(lm, c.V, c.D, ln, lg)
        L_.metal_flush()
        logits[pos] = lg.read(F)
    return logits
