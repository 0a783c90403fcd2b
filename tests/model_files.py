"""Writers of small checkpoint files for the loader tests: safetensors (the HuggingFace layout: 8-byte header
length, JSON header, raw little-endian data) and GGUF v3 (magic, counts, metadata key/values, tensor infos, data
aligned to 32 bytes), and the tensor names the reference's model loaders look for
(src/nn/qwen3.c:211-371, src/nn/gemma3.c:176-285)."""
import json
import struct

import numpy as np

from llm_metal_amd.configs import GEMMA3
from oracle import oracle

GGML_F32, GGML_F16, GGML_Q8_0 = 0, 1, 8


def bf16_round(a):
    """fp32 values rounded to the nearest bfloat16 (ties to even), still as fp32."""
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
    return b.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def _raw(arr, dtype):
    arr = np.ascontiguousarray(arr, np.float32)
    if dtype == "F32":
        return arr.tobytes()
    if dtype == "F16":
        return arr.astype(np.float16).tobytes()
    if dtype == "BF16":
        return (arr.view(np.uint32) >> 16).astype(np.uint16).tobytes()         # exact for bf16-rounded input
    raise ValueError(dtype)


def write_safetensors(path, tensors, metadata=None):
    """tensors: {name: (fp32 array, "F32" | "F16" | "BF16")}"""
    header, blobs, off = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, (arr, dtype) in tensors.items():
        raw = _raw(arr, dtype)
        header[name] = {"dtype": dtype, "shape": list(np.shape(arr)), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    text = json.dumps(header).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text + b"".join(blobs))


def _gg_str(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, tensors, kv=None, version=3):
    """tensors: {name: (fp32 array, GGML type)}; 2-D shapes are stored innermost first, as GGUF does.
    kv: list of (key, type id, packed value bytes) written verbatim."""
    kv = kv or []
    infos, blobs, off = b"", [], 0
    for name, (arr, typ) in tensors.items():
        arr = np.ascontiguousarray(arr, np.float32)
        raw = (arr.tobytes() if typ == GGML_F32 else arr.astype(np.float16).tobytes() if typ == GGML_F16
               else oracle.q8_quantize(arr.reshape(-1, arr.shape[-1])).tobytes())
        dims = list(arr.shape)[::-1]
        infos += _gg_str(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", typ, off)
        raw += b"\0" * (-len(raw) % 32)
        blobs.append(raw)
        off += len(raw)
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kv))
    for key, typ, val in kv:
        head += _gg_str(key) + struct.pack("<I", typ) + val
    head += infos
    head += b"\0" * (-len(head) % 32)
    with open(path, "wb") as f:
        f.write(head + b"".join(blobs))


SAMPLE_KV = [("general.architecture", 8, _gg_str("qwen3")), ("general.file_type", 4, struct.pack("<I", 7)),
             ("qwen3.rope.freq_base", 6, struct.pack("<f", 1e6)), ("flag", 7, b"\1"), ("big", 10, struct.pack("<Q", 1 << 40)),
             ("tokenizer.ggml.tokens", 9, struct.pack("<IQ", 8, 3) + _gg_str("a") + _gg_str("bc") + _gg_str("")),
             ("tokenizer.ggml.scores", 9, struct.pack("<IQ", 6, 3) + struct.pack("<3f", 0, 1, 2))]


def model_tensors(c, model, gguf=False):
    """{tensor name: fp32 array} of a synthetic model under the names the loaders read.  Gemma3 files hold norm
    weights minus one; `model` must then hold gammas of the form float32(w + 1)."""
    gemma = c.model_type == GEMMA3
    t = {}

    def norm(g):
        return (np.asarray(g, np.float32) - np.float32(1.0)).astype(np.float32) if gemma else np.asarray(g, np.float32)

    t["token_embd.weight" if gguf else "model.embed_tokens.weight"] = model["token_emb"]
    hf = {"g_in": "input_layernorm", "wq": "self_attn.q_proj", "wk": "self_attn.k_proj", "wv": "self_attn.v_proj",
          "g_q": "self_attn.q_norm", "g_k": "self_attn.k_norm", "wo": "self_attn.o_proj", "g_post_attn": "post_attention_layernorm",
          "g_pre_ff": "pre_feedforward_layernorm", "wg": "mlp.gate_proj", "wu": "mlp.up_proj", "wd": "mlp.down_proj",
          "g_post_ff": "post_feedforward_layernorm"}
    gg = {"g_in": "attn_norm", "wq": "attn_q", "wk": "attn_k", "wv": "attn_v", "g_q": "attn_q_norm", "g_k": "attn_k_norm",
          "wo": "attn_output", "g_post_attn": "ffn_norm", "wg": "ffn_gate", "wu": "ffn_up", "wd": "ffn_down"}
    for L in range(c.NL):
        for key, name in (gg if gguf else hf).items():
            a = model[key][L]
            if a is None:
                continue
            full = f"blk.{L}.{name}.weight" if gguf else f"model.layers.{L}.{name}.weight"
            t[full] = norm(a) if key.startswith("g_") else a
    t["output_norm.weight" if gguf else "model.norm.weight"] = norm(model["g_final"])
    if model["lm_head"] is not model["token_emb"]:
        t["output.weight" if gguf else "lm_head.weight"] = model["lm_head"]
    return t
