"""ctypes binding of the CPU oracle (oracle/sft_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the product package.
"""
import ctypes as C
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}


def build(force=False):
    """Compile liboracle_f32.so / liboracle_f64.so with the Makefile next to this file."""
    have = all(os.path.exists(os.path.join(_HERE, f"liboracle_{p}.so")) for p in ("f32", "f64"))
    if force or not have:
        if force:
            subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
        subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


class OrCfg(C.Structure):
    _fields_ = [("model_type", C.c_int), ("NL", C.c_int), ("D", C.c_int), ("Hq", C.c_int),
                ("Hkv", C.c_int), ("hd", C.c_int), ("IS", C.c_int), ("V", C.c_int),
                ("batch", C.c_int), ("seq", C.c_int), ("R", C.c_int),
                ("lora_scaling", C.c_float), ("eps", C.c_float), ("emb_scale", C.c_float), ("window", C.c_int)]


_PP = C.POINTER(C.POINTER(C.c_float))


class OrWeights(C.Structure):
    _fields_ = [(k, _PP) for k in ("wq", "wk", "wv", "wo", "wg", "wu", "wd",
                                   "g_in", "g_post_attn", "g_pre_ff", "g_post_ff", "g_q", "g_k")] + \
               [("g_final", C.POINTER(C.c_float)), ("lm_head", C.POINTER(C.c_float)),
                ("token_emb", C.POINTER(C.c_float)), ("rope_theta", C.POINTER(C.c_float))]


_PU16 = C.POINTER(C.POINTER(C.c_uint16))


class OrFull(C.Structure):
    _fields_ = [("accum", C.c_int), ("lr", C.c_float)] + \
               [(k, _PU16) for k in ("gq", "gk", "gv", "go", "gg", "gu", "gd")] + \
               [("glm", C.POINTER(C.c_uint16))]


def lib(precision="f32"):
    if precision not in _LIBS:
        path = os.path.join(_HERE, f"liboracle_{precision}.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.or_sft_loss.restype = C.c_double
        L.or_sft_train_step.restype = C.c_double
        L.or_full_param_pass.restype = C.c_double
        L.or_clip_grad_norm.restype = C.c_double
        L.or_lora_layer_size.restype = C.c_size_t
        L.or_f32_to_f16_bits.restype = C.c_uint16
        L.or_f32_to_f16_bits.argtypes = [C.c_float]
        L.or_f16_bits_to_f32.restype = C.c_float
        L.or_f16_bits_to_f32.argtypes = [C.c_uint16]
        _LIBS[precision] = L
    return _LIBS[precision]


def real_dtype(precision):
    return np.float32 if precision == "f32" else np.float64


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


# ---------------------------------------------------------------- formats

def f32_to_f16_bits(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().or_f32_to_f16_array(_p(a), _p(out), C.c_size_t(a.size))
    return out


def f16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().or_f16_to_f32_array(_p(b), _p(out), C.c_size_t(b.size))
    return out


def round_f16(a):
    """fp32 values after a round trip through F16 (what an F16 WMat holds)."""
    return f16_bits_to_f32(f32_to_f16_bits(a))


def q8_quantize(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = a.shape
    out = np.zeros(rows * (cols // 32) * 34, dtype=np.uint8)
    lib().or_q8_quantize(_p(a), _p(out), C.c_int(rows), C.c_int(cols))
    return out


def q8_dequant(blocks, rows, cols):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    out = np.zeros((rows, cols), dtype=np.float32)
    lib().or_q8_dequant(_p(blocks), _p(out), C.c_int(rows), C.c_int(cols))
    return out


def weights_as_used(model, fmt="f16"):
    """The fp32 values the step multiplies with: frozen matrices and lm_head
    after F16 rounding (or a Q8_0 round trip); gammas and the embedding table
    stay fp32 (src/nn/fast_sft.c:231-239)."""
    conv = round_f16 if fmt == "f16" else (lambda a: q8_dequant(q8_quantize(a), *a.shape))
    used = dict(model)
    for k in ("wq", "wk", "wv", "wo", "wg", "wu", "wd"):
        used[k] = [conv(w) for w in model[k]]
    used["lm_head"] = conv(model["lm_head"])
    return used


# ---------------------------------------------------------------- the step

def _cfg(c):
    return OrCfg(c.model_type, c.NL, c.D, c.Hq, c.Hkv, c.hd, c.IS, c.V, c.batch, c.seq, c.R,
                 c.lora_scaling if c.R else 0.0, c.eps, c.emb_scale, getattr(c, "window", 0))


class _Packed:
    """Keeps the pointer tables alive for the duration of a call."""

    def __init__(self, c, used):
        self.keep = []
        self.w = OrWeights()
        ones_d = np.ones(c.D, dtype=np.float32)
        for k in ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "g_in", "g_post_attn", "g_pre_ff",
                  "g_post_ff", "g_q", "g_k"):
            arrs = [np.ascontiguousarray(a if a is not None else ones_d, dtype=np.float32) for a in used[k]]
            tbl = (C.POINTER(C.c_float) * c.NL)(*[_fp(a) for a in arrs])
            self.keep += [arrs, tbl]
            setattr(self.w, k, C.cast(tbl, _PP))
        for k in ("g_final", "lm_head", "token_emb"):
            a = np.ascontiguousarray(used[k], dtype=np.float32)
            self.keep.append(a)
            setattr(self.w, k, _fp(a))
        th = np.asarray(c.rope_thetas(), dtype=np.float32)
        self.keep.append(th)
        self.w.rope_theta = _fp(th)


def sft_loss(c, used, lora, tok, tgt, precision="f32", want_logits=False):
    L = lib(precision)
    dt = real_dtype(precision)
    pk = _Packed(c, used)
    lora = np.ascontiguousarray(lora, dtype=dt)
    logits = np.zeros((c.BN, c.V), dtype=dt) if want_logits else None
    loss = L.or_sft_loss(C.byref(_cfg(c)), C.byref(pk.w), _p(lora),
                         _p(np.ascontiguousarray(tok, dtype=np.uint32)),
                         _p(np.ascontiguousarray(tgt, dtype=np.uint32)),
                         _p(logits) if want_logits else None)
    return (loss, logits) if want_logits else loss


def sft_train_step(c, used, lora, m, v, step, tok, tgt, lr, do_update=True, precision="f32",
                   want_logits=False, want_dx=False):
    """One step.  lora/m/v are updated in place when do_update (arrays must be of
    the precision's dtype).  Returns dict(loss, grad, step, grad_norm[, logits, dx])."""
    L = lib(precision)
    dt = real_dtype(precision)
    assert lora.dtype == dt and m.dtype == dt and v.dtype == dt
    pk = _Packed(c, used)
    grad = np.zeros_like(lora)
    logits = np.zeros((c.BN, c.V), dtype=dt) if want_logits else None
    dx = np.zeros((c.BN, c.D), dtype=dt) if want_dx else None
    sc = C.c_int(step)
    gn = C.c_double(0)
    tok = np.ascontiguousarray(tok, dtype=np.uint32)
    tgt = np.ascontiguousarray(tgt, dtype=np.uint32)
    loss = L.or_sft_train_step(C.byref(_cfg(c)), C.byref(pk.w), _p(lora), _p(grad), _p(m), _p(v),
                               C.byref(sc), _p(tok), _p(tgt), C.c_float(lr), C.c_int(1 if do_update else 0),
                               _p(logits) if want_logits else None, _p(dx) if want_dx else None,
                               C.byref(gn))
    out = {"loss": loss, "grad": grad, "step": sc.value, "grad_norm": gn.value}
    if want_logits:
        out["logits"] = logits
    if want_dx:
        out["dx"] = dx
    return out


# ---------------------------------------------------------------- full-parameter mode

_GA_KEYS = (("gq", "wq"), ("gk", "wk"), ("gv", "wv"), ("go", "wo"), ("gg", "wg"), ("gu", "wu"), ("gd", "wd"))


def new_grad_accum(used):
    """Zeroed F16 (bit pattern) accumulators shaped like the matrices of `used`
    (sft_alloc_grad_accum, src/nn/fast_sft.c:996-1019)."""
    ga = {g: [np.zeros(w.shape, dtype=np.uint16) for w in used[k]] for g, k in _GA_KEYS}
    ga["glm"] = np.zeros(used["lm_head"].shape, dtype=np.uint16)
    return ga


def _full(c, ga, lr):
    f = OrFull()
    keep = []
    f.accum = 1 if ga is not None else 0
    f.lr = lr
    if ga is not None:
        for g, _ in _GA_KEYS:
            tbl = (C.POINTER(C.c_uint16) * c.NL)(*[a.ctypes.data_as(C.POINTER(C.c_uint16)) for a in ga[g]])
            keep.append(tbl)
            setattr(f, g, C.cast(tbl, _PU16))
        f.glm = ga["glm"].ctypes.data_as(C.POINTER(C.c_uint16))
    return f, keep


def full_param_pass(c, used, ga, lr=0.0, tok=None, x_rows=None, tgt=None, grpo=None, precision="f32",
                    want_logits=False, want_dx=False, lora=None):
    """Forward + full-parameter backward.  ga = accumulators (sft_backward_accum) or
    None (sft_backward_sgd with lr: the float32 matrices of `used` are updated in
    place).  grpo = dict(actions, old_lp, advs, clip_eps, dl_scale) switches the
    loss to the policy gradient.  With lora (flat adapters, c.R > 0) the backward is the
    LoRA one instead and the result carries "grad".  Returns dict(loss[, logits, new_lp, dx, grad])."""
    assert (c.R == 0) == (lora is None)
    L = lib(precision)
    dt = real_dtype(precision)
    pk = _Packed(c, used)
    full, keep = _full(c, ga, lr)
    fullp = C.byref(full) if lora is None else None
    lora_a = np.ascontiguousarray(lora, dtype=dt) if lora is not None else None
    grad = np.zeros_like(lora_a) if lora is not None else None
    lp, gp = (_p(lora_a), _p(grad)) if lora is not None else (None, None)
    logits = np.zeros((c.BN, c.V), dtype=dt) if want_logits else None
    dx = np.zeros((c.BN, c.D), dtype=dt) if want_dx else None
    new_lp = np.zeros(c.BN, dtype=dt)
    tokp = _p(np.ascontiguousarray(tok, dtype=np.uint32)) if tok is not None else None
    xr = np.ascontiguousarray(x_rows, dtype=dt) if x_rows is not None else None
    if grpo is None:
        tg = np.ascontiguousarray(tgt, dtype=np.uint32)
        loss = L.or_full_param_pass(C.byref(_cfg(c)), C.byref(pk.w), fullp, lp, gp, tokp, _p(xr) if xr is not None else None,
                                    C.c_int(0), _p(tg), None, None, C.c_float(0), C.c_float(0),
                                    _p(logits) if want_logits else None, None, _p(dx) if want_dx else None)
    else:
        act = np.ascontiguousarray(grpo["actions"], dtype=np.uint32)
        olp = np.ascontiguousarray(grpo["old_lp"], dtype=dt)
        adv = np.ascontiguousarray(grpo["advs"], dtype=dt)
        loss = L.or_full_param_pass(C.byref(_cfg(c)), C.byref(pk.w), fullp, lp, gp, tokp, _p(xr) if xr is not None else None,
                                    C.c_int(1), _p(act), _p(olp), _p(adv), C.c_float(grpo["clip_eps"]),
                                    C.c_float(grpo["dl_scale"]),
                                    _p(logits) if want_logits else None, _p(new_lp), _p(dx) if want_dx else None)
    out = {"loss": loss, "new_lp": new_lp}
    if want_logits:
        out["logits"] = logits
    if want_dx:
        out["dx"] = dx
    if grad is not None:
        out["grad"] = grad
    return out


def apply_grad_sgd(c, used, ga, lr):
    """W = half(W - lr G), G = 0 on every matrix (sft_apply_grad_sgd)."""
    pk = _Packed(c, used)
    full, keep = _full(c, ga, lr)
    lib().or_apply_grad_sgd(C.byref(_cfg(c)), C.byref(pk.w), C.byref(full), C.c_float(lr))


# ---------------------------------------------------------------- single ops

class SZ(int):
    """Marks an integer argument that the C side takes as size_t."""


def op(precision, name, *args):
    """Call an oracle op by name: numpy arrays go as pointers, SZ as size_t,
    int as int, float as float.  Returns the C return value (int by default)."""
    conv = []
    for a in args:
        if isinstance(a, np.ndarray):
            assert a.flags["C_CONTIGUOUS"]
            conv.append(_p(a))
        elif isinstance(a, SZ):
            conv.append(C.c_size_t(int(a)))
        elif isinstance(a, (int, np.integer)):
            conv.append(C.c_int(int(a)))
        elif isinstance(a, (float, np.floating)):
            conv.append(C.c_float(float(a)))
        elif a is None:
            conv.append(None)
        else:
            raise TypeError(type(a))
    return getattr(lib(precision), name)(*conv)
