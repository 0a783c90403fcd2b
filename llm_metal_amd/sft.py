"""Python mirror of the C host API of the SFT step (include/sft_hip.h), used by
tests and bench.py: device buffers as thin handles, the SFT state as a class.
Every method is one call into libllm_metal_hip.so."""
import ctypes as C

import numpy as np

from . import lib as _lib
from .configs import SFTConfig


def _vp(a):
    return a.ctypes.data_as(C.c_void_p)


class Backend:
    """fast_metal_init / fast_metal_shutdown as a context manager."""

    def __init__(self):
        self.L = _lib.load()
        if self.L.fast_metal_init() != 0:
            raise RuntimeError("fast_metal_init failed: no gfx950 device (this library has no CPU path)")

    def close(self):
        if self.L is not None:
            self.L.fast_metal_shutdown()
            self.L = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- buffers
    def buf(self, arr):
        arr = np.ascontiguousarray(arr)
        return Buf(self.L, self.L.metal_buf_from_data(_vp(arr), arr.nbytes), arr.nbytes)

    def empty(self, nbytes):
        return Buf(self.L, self.L.metal_buf_create(nbytes), nbytes)

    def flush(self):
        self.L.metal_flush()


class Buf:
    def __init__(self, L, handle, nbytes, owned=True):
        if not handle:
            raise RuntimeError("buffer creation failed")
        self.L, self.h, self.nbytes, self.owned = L, handle, nbytes, owned

    def read(self, dtype, shape=None):
        out = np.empty(self.nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        self.L.metal_buf_read(self.h, 0, _vp(out), out.nbytes)
        return out.reshape(shape) if shape is not None else out

    def write(self, arr):
        arr = np.ascontiguousarray(arr)
        self.L.metal_buf_write(self.h, 0, _vp(arr), arr.nbytes)

    def free(self):
        if self.owned and self.h:
            self.L.metal_buf_free(self.h)
        self.h = None


def _layer_refs(c: SFTConfig, model, keep):
    refs = (_lib.LayerWeightRef * c.NL)()
    names = {"q_proj": "wq", "k_proj": "wk", "v_proj": "wv", "o_proj": "wo",
             "gate_proj": "wg", "up_proj": "wu", "down_proj": "wd"}
    gam = {"input_norm_g": "g_in", "post_attn_norm_g": "g_post_attn", "pre_ff_norm_g": "g_pre_ff",
           "post_ff_norm_g": "g_post_ff", "q_norm_g": "g_q", "k_norm_g": "g_k"}
    for L in range(c.NL):
        for field, key in names.items():
            a = np.ascontiguousarray(model[key][L], dtype=np.float32)
            keep.append(a)
            setattr(refs[L], field, _lib.WeightRef(a.ctypes.data, a.shape[0], a.shape[1]))
        for field, key in gam.items():
            g = model[key][L]
            if g is None:
                setattr(refs[L], field, None)
            else:
                a = np.ascontiguousarray(g, dtype=np.float32)
                keep.append(a)
                setattr(refs[L], field, a.ctypes.data)
        refs[L].d_model = c.D
        refs[L].head_dim = c.hd
    return refs


def model_ref(c: SFTConfig, model, lora_init=True):
    """SFTModelRef over the numpy arrays of a synthetic model; returns (ref, arrays the ref points into, embedding
    table).  The arrays must live until the create call returns; the SFT state also borrows the embedding table for
    its lifetime (sft_get_token_emb hands it out)."""
    keep = []
    refs = _layer_refs(c, model, keep)
    thetas = np.asarray(c.rope_thetas(), dtype=np.float32)
    emb = np.ascontiguousarray(model["token_emb"], dtype=np.float32)
    head = emb if model["lm_head"] is model["token_emb"] else np.ascontiguousarray(model["lm_head"], dtype=np.float32)
    gf = np.ascontiguousarray(model["g_final"], dtype=np.float32)
    lora = np.ascontiguousarray(model["lora"], dtype=np.float32) if (lora_init and c.R) else None
    m = _lib.SFTModelRef(c.model_type, c.NL, c.D, c.Hq, c.Hkv, c.hd, c.IS, c.V, thetas.ctypes.data, refs,
                         emb.ctypes.data, head.ctypes.data, gf.ctypes.data,
                         lora.ctypes.data if lora is not None else None)
    keep += [refs, thetas, emb, head, gf, lora]
    return m, keep, emb


class SFTState:
    """sft_state_create_from_ref ... sft_state_free."""

    def __init__(self, c: SFTConfig, model, lora_init=True):
        self.L = _lib.load()
        self.c = c
        m, keep, self._emb = model_ref(c, model, lora_init)
        self.h = self.L.sft_state_create_from_ref(C.byref(m), c.batch, c.seq, c.R, c.alpha,
                                                  1 if c.weight_format == "f16" else 0)
        if not self.h:
            raise RuntimeError("sft_state_create_from_ref failed (no gfx950 device or unsupported dims)")
        if c.window:
            self.L.sft_set_sliding_window(self.h, c.window, None)

    def train_step(self, tok, tgt, lr):
        tok = np.ascontiguousarray(tok, dtype=np.uint32)
        tgt = np.ascontiguousarray(tgt, dtype=np.uint32)
        return float(self.L.sft_train_step(self.h, _vp(tok), _vp(tgt), lr))

    def enqueue_train_step(self, tok, tgt, lr):
        self.L.sft_enqueue_train_step(self.h, _vp(tok), _vp(tgt), lr)

    def finish_train_step(self):
        return float(self.L.sft_finish_train_step(self.h))

    def lora(self):
        out = np.empty(self.L.sft_lora_numel(self.h), dtype=np.float32)
        self.L.sft_copy_lora(self.h, _vp(out))
        return out

    def lora_grads(self):
        out = np.empty(self.L.sft_lora_numel(self.h), dtype=np.float32)
        self.L.sft_copy_lora_grads(self.h, _vp(out))
        return out

    def set_lora(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        assert arr.size == self.L.sft_lora_numel(self.h)
        self.L.sft_set_lora(self.h, _vp(arr))

    def logits(self):
        b = Buf(self.L, self.L.sft_get_logits(self.h), self.c.BN * self.c.V * 4, owned=False)
        return b.read(np.float32, (self.c.BN, self.c.V))

    def losses(self):
        p = self.L.sft_get_losses_cpu(self.h)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(self.c.BN,)).copy()

    def grad_norm(self):
        return float(self.L.sft_get_last_grad_norm(self.h))

    def step_count(self):
        return self.L.sft_get_step_count(self.h)

    def x_cpu(self):
        p = self.L.sft_get_x_cpu(self.h)
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(self.c.BN, self.c.D))

    def dlogits_buf(self):
        return Buf(self.L, self.L.sft_get_dlogits(self.h), self.c.BN * self.c.V * 4, owned=False)

    def forward_to_logits(self):
        self.L.forward_to_logits(self.h)

    def backward(self):
        self.L.sft_backward(self.h)

    # -- full-parameter mode (lora_rank 0)
    MATRICES = ("wq", "wk", "wv", "wo", "wg", "wu", "wd", "lm_head")

    def matrix_shape(self, which):
        c = self.c
        return {"wq": (c.Hq * c.hd, c.D), "wk": (c.Hkv * c.hd, c.D), "wv": (c.Hkv * c.hd, c.D), "wo": (c.D, c.Hq * c.hd),
                "wg": (c.IS, c.D), "wu": (c.IS, c.D), "wd": (c.D, c.IS), "lm_head": (c.V, c.D)}[which]

    def matrix_f16(self, layer, which, source=0):
        """F16 bit pattern (uint16, row-major) of one matrix: source 0 = weight, 1 = its transposed image,
        2 = gradient accumulator."""
        out = np.zeros(self.matrix_shape(which), dtype=np.uint16)
        self.L.sft_copy_matrix_f16(self.h, layer, self.MATRICES.index(which), source, _vp(out))
        return out

    def is_full_param(self):
        return bool(self.L.sft_is_full_param(self.h))

    def alloc_grad_accum(self):
        self.L.sft_alloc_grad_accum(self.h)

    def backward_accum(self):
        self.L.sft_backward_accum(self.h)

    def backward_sgd(self, lr):
        self.L.sft_backward_sgd(self.h, lr)

    def apply_grad_sgd(self, lr):
        self.L.sft_apply_grad_sgd(self.h, lr)

    def save_full_checkpoint(self, path):
        self.L.sft_save_full_checkpoint(self.h, path.encode())

    def grpo_apply_completions(self, prompt, gen_tokens, gen_logprobs, advantages, clip_eps, lr, accurate=True):
        """Phases 3-4 of a GRPO step over already sampled completions.  Returns the policy's
        log-probabilities of the actions, [G, seq].  A state built with batch B runs B completions per pass."""
        G = len(gen_tokens)
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        toks = [np.ascontiguousarray(t, dtype=np.uint32) for t in gen_tokens]
        lps = [np.ascontiguousarray(p, dtype=np.float32) for p in gen_logprobs]
        lens = np.asarray([len(t) for t in toks], dtype=np.int32)
        adv = np.ascontiguousarray(advantages, dtype=np.float32)
        tp = (C.c_void_p * G)(*[t.ctypes.data for t in toks])
        lp = (C.c_void_p * G)(*[p.ctypes.data for p in lps])
        c = _lib.GRPOCompletions(prompt.ctypes.data, len(prompt), G, tp, lens.ctypes.data, lp, adv.ctypes.data,
                                 clip_eps, 1 if accurate else 0)
        new_lp = np.zeros((G, self.c.seq), dtype=np.float32)
        self.L.grpo_apply_completions(self.h, C.byref(c), lr, _vp(new_lp))
        return new_lp

    def free(self):
        if self.h:
            self.L.sft_state_free(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()


class InferenceState:
    """inference_state_create_from_ref / _from_sft ... inference_state_free (include/inference_hip.h)."""

    def __init__(self, c: SFTConfig = None, model=None, max_seq=256, use_fp16=True, sft: "SFTState" = None, path=None,
                 model_type=0):
        self.L = _lib.load()
        if path is not None:                               # inference_state_create_from_file
            self.c, self._keep = c, []
            self.h = self.L.inference_state_create_from_file(str(path).encode(), model_type, max_seq, 1 if use_fp16 else 0)
        elif sft is not None:
            self.c, self._keep = sft.c, [sft]
            self.h = self.L.inference_state_create_from_sft(sft.h, max_seq)
        else:
            self.c = c
            m, keep, _ = model_ref(c, model, lora_init=False)
            self._keep = []
            self.h = self.L.inference_state_create_from_ref(C.byref(m), max_seq, 1 if use_fp16 else 0)
            del keep
        if not self.h:
            raise RuntimeError("inference state creation failed (no gfx950 device or unsupported dims)")
        self.V = self.L.inference_state_vocab_size(self.h)

    def reset(self):
        self.L.inference_state_reset(self.h)

    def forward_token(self, token):
        p = self.L.inference_forward_token(self.h, int(token))
        if not p:
            raise RuntimeError("inference_forward_token refused the token (outside the vocabulary or cache full)")
        return np.ctypeslib.as_array(p, shape=(self.V,)).copy()

    def forward_token_argmax(self, token):
        return int(self.L.inference_forward_token_argmax(self.h, int(token)))

    def generate(self, prompt, max_gen_len):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max_gen_len, dtype=np.uint32)
        n = self.L.inference_generate(self.h, _vp(prompt), len(prompt), _vp(out), max_gen_len)
        return out[:n]

    def generate_batch(self, prompt, max_gen_len, batch):
        """[batch, n] tokens: the same prompt decoded greedily `batch` times in lock step."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros((batch, max_gen_len), dtype=np.uint32)
        n = self.L.inference_generate_batch(self.h, _vp(prompt), len(prompt), _vp(out), max_gen_len, batch)
        return out[:, :n]

    def step_batch(self, tokens, pos, want_logits=True):
        """One lock-step step with a token per sequence at position `pos`; [batch, V] logits (None if not asked for)."""
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        out = np.empty((len(t), self.V), dtype=np.float32) if want_logits else None
        if self.L.inference_step_batch(self.h, _vp(t), len(t), int(pos), _vp(out) if want_logits else None) != 0:
            raise RuntimeError("inference_step_batch refused its arguments")
        return out

    def set_eos(self, ids):
        a = np.ascontiguousarray(ids, dtype=np.int32)
        self.L.inference_state_set_eos(self.h, _vp(a), len(a))

    def load_eos(self, path):
        self.L.inference_state_load_eos(self.h, str(path).encode())

    def attach_lora(self, sft):
        """inference_state_set_lora: a state with its own weights reads the training state's adapters from then on."""
        self.L.inference_state_set_lora(self.h, sft.h)
        self._keep.append(sft)

    def refresh_from_sft(self):
        self.L.inference_state_refresh_from_sft(self.h)

    def position(self):
        return int(self.L.inference_state_position(self.h))

    def free(self):
        if self.h:
            self.L.inference_state_free(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()
