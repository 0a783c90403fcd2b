"""CPU tests of the checkpoint readers (include/loader_hip.h): safetensors and GGUF files written by
tests/model_files.py are parsed through the C ABI and every tensor is compared with what was written; the widening
rules are the reference's (src/data/safetensors.c:315-341, src/data/gguf.c:188-253): F16 / BF16 exact, Q8_0 =
float(code) * float(scale).  No GPU is needed for these functions."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

from llm_metal_amd import lib
from llm_metal_amd.configs import C1, GEMMA3, SFTConfig
from llm_metal_amd.synth import make_model
from oracle import oracle
from tests import model_files as mf

F = np.float32


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(lib.LIB_PATH):
        lib.build()
    return lib.load()


def load_f32(L, h, name):
    n = C.c_size_t(0)
    p = L.model_file_load_f32(h, name.encode(), C.byref(n))
    assert p, name
    out = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=(n.value,)).copy()
    C.CDLL(None).free(C.c_void_p(p))
    return out


def info(L, h, name):
    dt, nd, shape = C.c_int(-9), C.c_int(0), (C.c_uint64 * 4)()
    if not L.model_file_find(h, name.encode(), C.byref(dt), C.byref(nd), shape):
        return None
    return dt.value, [int(shape[i]) for i in range(nd.value)]


def test_safetensors_single_file(L, tmp_path):
    rng = np.random.default_rng(0)
    a = rng.standard_normal((5, 8)).astype(F)
    b = rng.standard_normal((3, 4)).astype(F)
    c = mf.bf16_round(rng.standard_normal((2, 3, 4)).astype(F))
    d = np.array([0.0, -0.0, 6e-8, 6.1e-5, 65504.0, np.inf, -1.5], F)          # F16 subnormals, the largest normal, inf
    path = tmp_path / "m.safetensors"
    mf.write_safetensors(path, {"a.weight": (a, "F32"), "b": (b, "F16"), "c \"q\"": (c, "BF16"), "d": (d, "F16")},
                         metadata={"format": "pt", "note": "x{y}[z]\"w"})
    h = L.model_file_open(str(path).encode())
    assert h and not L.model_file_is_gguf(h) and L.model_file_count(h) == 4
    assert [L.model_file_name(h, i).decode() for i in range(4)] == ["a.weight", "b", 'c "q"', "d"]
    assert info(L, h, "a.weight") == (0, [5, 8]) and info(L, h, "b") == (1, [3, 4]) and info(L, h, 'c "q"') == (30, [2, 3, 4])
    assert info(L, h, "nope") is None
    assert np.array_equal(load_f32(L, h, "a.weight"), a.ravel())
    assert np.array_equal(load_f32(L, h, "b"), b.astype(np.float16).astype(F).ravel())
    assert np.array_equal(load_f32(L, h, 'c "q"'), c.ravel())
    assert np.array_equal(load_f32(L, h, "d").view(np.uint32), d.astype(np.float16).astype(F).view(np.uint32))
    r, cc = C.c_int(0), C.c_int(0)
    assert L.model_file_matrix_shape(h, b"a.weight", C.byref(r), C.byref(cc)) and (r.value, cc.value) == (5, 8)
    assert L.model_file_matrix_shape(h, b"d", C.byref(r), C.byref(cc)) and (r.value, cc.value) == (1, 7)
    assert not L.model_file_matrix_shape(h, b'c "q"', C.byref(r), C.byref(cc))            # rank 3
    nb = C.c_size_t(0)
    p = L.model_file_data(h, b"b", C.byref(nb))
    assert nb.value == 24 and C.string_at(p, 24) == b.astype(np.float16).tobytes()
    L.model_file_close(h)


def test_safetensors_shard_directory(L, tmp_path):
    d = tmp_path / "ckpt"
    d.mkdir()
    x, y, z = (np.full((2, 2), v, F) for v in (1, 2, 3))
    mf.write_safetensors(d / "model-00002-of-00002.safetensors", {"y": (y, "F32"), "z": (z, "BF16")})
    mf.write_safetensors(d / "model-00001-of-00002.safetensors", {"x": (x, "F16")})
    (d / "config.json").write_text("{}")
    (d / "model.safetensors.index.json").write_text("{}")                      # does not end in .safetensors
    h = L.model_file_open(str(d).encode())
    assert h and L.model_file_count(h) == 3
    assert [L.model_file_name(h, i).decode() for i in range(3)] == ["x", "y", "z"]   # shards in alphabetical order
    for name, want in (("x", x), ("y", y), ("z", z)):
        assert np.array_equal(load_f32(L, h, name), want.ravel())
    L.model_file_close(h)


def test_gguf_types_shapes_and_metadata_skipping(L, tmp_path):
    rng = np.random.default_rng(1)
    w = rng.standard_normal((6, 64)).astype(F)
    e = rng.standard_normal((10, 32)).astype(F)
    g = rng.standard_normal(32).astype(F)
    path = tmp_path / "m.gguf"
    mf.write_gguf(path, {"blk.0.attn_q.weight": (w, mf.GGML_Q8_0), "token_embd.weight": (e, mf.GGML_F16),
                         "output_norm.weight": (g, mf.GGML_F32)}, kv=mf.SAMPLE_KV)
    h = L.model_file_open(str(path).encode())
    assert h and L.model_file_is_gguf(h) and L.model_file_count(h) == 3
    assert info(L, h, "blk.0.attn_q.weight") == (8, [64, 6])                   # innermost dimension first
    r, c = C.c_int(0), C.c_int(0)
    assert L.model_file_matrix_shape(h, b"blk.0.attn_q.weight", C.byref(r), C.byref(c)) and (r.value, c.value) == (6, 64)
    blocks = oracle.q8_quantize(w)
    assert np.array_equal(load_f32(L, h, "blk.0.attn_q.weight"), oracle.q8_dequant(blocks, 6, 64).ravel())
    nb = C.c_size_t(0)
    p = L.model_file_data(h, b"blk.0.attn_q.weight", C.byref(nb))
    assert nb.value == 6 * 2 * 34 and C.string_at(p, nb.value) == blocks.tobytes()
    assert np.array_equal(load_f32(L, h, "token_embd.weight"), e.astype(np.float16).astype(F).ravel())
    assert np.array_equal(load_f32(L, h, "output_norm.weight"), g)
    L.model_file_close(h)
    # version 2 and a custom alignment
    mf.write_gguf(path, {"t": (g, mf.GGML_F32)}, kv=[("general.alignment", 4, struct.pack("<I", 32))], version=2)
    h = L.model_file_open(str(path).encode())
    assert h and np.array_equal(load_f32(L, h, "t"), g)
    L.model_file_close(h)


def test_unreadable_files_are_refused(L, tmp_path, capfd):
    assert not L.model_file_open(str(tmp_path / "absent.gguf").encode())
    good = tmp_path / "g.gguf"
    mf.write_gguf(good, {"t": (np.ones((4, 32), F), mf.GGML_F32)}, kv=mf.SAMPLE_KV)
    raw = good.read_bytes()
    (tmp_path / "cut.gguf").write_bytes(raw[:len(raw) - 100])                  # tensor data beyond the end
    assert not L.model_file_open(str(tmp_path / "cut.gguf").encode())
    (tmp_path / "hdr.gguf").write_bytes(raw[:60])                              # header cut inside the metadata
    assert not L.model_file_open(str(tmp_path / "hdr.gguf").encode())
    (tmp_path / "v9.gguf").write_bytes(raw[:4] + struct.pack("<I", 9) + raw[8:])
    assert not L.model_file_open(str(tmp_path / "v9.gguf").encode())
    st = tmp_path / "s.safetensors"
    mf.write_safetensors(st, {"t": (np.ones((2, 2), F), "F32")})
    raw = st.read_bytes()
    (tmp_path / "s_cut.safetensors").write_bytes(raw[:-4])
    assert not L.model_file_open(str(tmp_path / "s_cut.safetensors").encode())
    (tmp_path / "s_bad.safetensors").write_bytes(struct.pack("<Q", 5) + b"{nope")
    assert not L.model_file_open(str(tmp_path / "s_bad.safetensors").encode())
    empty = tmp_path / "empty"
    empty.mkdir()
    assert not L.model_file_open(str(empty).encode())
    assert "[Loader]" in capfd.readouterr().err


def _safetensors_raw(path, header: str, data: bytes):
    h = header.encode()
    path.write_bytes(struct.pack("<Q", len(h)) + h + data)


def test_crafted_offsets_and_shapes_are_refused(L, tmp_path, capfd):
    """Headers whose sums would wrap 64 bits, reversed offsets and dimension products that overflow must be refused at
    open time: later reads trust the shape."""
    data = b"\0" * 64
    big = (1 << 64) - 8
    cases = {
        "reversed": '{"t":{"dtype":"F32","shape":[2,2],"data_offsets":[16,0]}}',
        "wrapping_begin": '{"t":{"dtype":"F32","shape":[2,2],"data_offsets":[%d,%d]}}' % (big, big + 4),
        "huge_end": '{"t":{"dtype":"F32","shape":[2,2],"data_offsets":[0,%d]}}' % big,
        "overflowing_shape": '{"t":{"dtype":"F32","shape":[4294967296,4294967296],"data_offsets":[0,0]}}',
        "shape_mismatch": '{"t":{"dtype":"F32","shape":[4,5],"data_offsets":[0,16]}}',
    }
    for name, hdr in cases.items():
        f = tmp_path / f"{name}.safetensors"
        _safetensors_raw(f, hdr, data)
        assert not L.model_file_open(str(f).encode()), name
    ok = tmp_path / "ok.safetensors"
    _safetensors_raw(ok, '{"t":{"dtype":"F32","shape":[2,2],"data_offsets":[0,16]}}', data)
    h = L.model_file_open(str(ok).encode())
    assert h
    L.model_file_close(h)

    def gguf(dims, typ, off, n_data=64):
        info = mf._gg_str("t") + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", typ, off)
        head = struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + info
        head += b"\0" * (-len(head) % 32)
        return head + b"\0" * n_data
    bad = {
        "dims_overflow_to_zero": gguf([1 << 32, 1 << 32], mf.GGML_F32, 0),          # product 2^64 wraps to 0 bytes
        "dims_overflow_q8": gguf([1 << 40, 1 << 30], mf.GGML_Q8_0, 0),
        "wrapping_offset": gguf([4, 4], mf.GGML_F32, (1 << 64) - 32),
        "array_count_overflow": struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + mf._gg_str("k") + struct.pack("<IIQ", 9, 10, (1 << 62) + 1) + b"\0" * 64,
    }
    for name, raw in bad.items():
        f = tmp_path / f"{name}.gguf"
        f.write_bytes(raw)
        assert not L.model_file_open(str(f).encode()), name
    f = tmp_path / "fine.gguf"
    f.write_bytes(gguf([4, 4], mf.GGML_F32, 0))
    h = L.model_file_open(str(f).encode())
    assert h
    L.model_file_close(h)
    assert "[Loader]" in capfd.readouterr().err


TINY_GEMMA = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=256, V=512, seq=5, tied=True)


def arr(p, *shape):
    return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_float)), shape=shape)


def check_ref(c, model, ref, thetas):
    m = ref.contents
    assert (m.model_type, m.n_layers, m.d_model, m.n_q_heads, m.n_kv_heads, m.head_dim, m.intermediate_size, m.vocab_size) == \
           (c.model_type, c.NL, c.D, c.Hq, c.Hkv, c.hd, c.IS, c.V)
    assert np.array_equal(arr(m.rope_thetas, c.NL), np.asarray(thetas, F))
    assert np.array_equal(arr(m.token_emb, c.V, c.D), model["token_emb"])
    assert np.array_equal(arr(m.lm_head, c.V, c.D), model["lm_head"])
    assert (m.lm_head == m.token_emb) == (model["lm_head"] is model["token_emb"])
    assert np.array_equal(arr(m.final_norm_g, c.D), model["g_final"])
    for Li in range(c.NL):
        r = m.layers[Li]
        for field, key in (("q_proj", "wq"), ("k_proj", "wk"), ("v_proj", "wv"), ("o_proj", "wo"), ("gate_proj", "wg"),
                           ("up_proj", "wu"), ("down_proj", "wd")):
            w = getattr(r, field)
            assert (w.rows, w.cols) == model[key][Li].shape and np.array_equal(arr(w.data, w.rows, w.cols), model[key][Li])
        for field, key in (("input_norm_g", "g_in"), ("post_attn_norm_g", "g_post_attn"), ("pre_ff_norm_g", "g_pre_ff"),
                           ("post_ff_norm_g", "g_post_ff"), ("q_norm_g", "g_q"), ("k_norm_g", "g_k")):
            g = model[key][Li]
            if g is None:
                assert not getattr(r, field)
            else:
                assert np.array_equal(arr(getattr(r, field), len(g)), g), (Li, field)
        assert (r.d_model, r.head_dim) == (c.D, c.hd)


def test_model_ref_load_qwen3_and_gemma3(L, tmp_path, capfd):
    # Qwen3, safetensors BF16 with its own LM head
    c = C1.with_(tied=False)
    model = make_model(c, seed=3, gamma_jitter=0.1)
    for k in ("wq", "wk", "wv", "wo", "wg", "wu", "wd"):
        model[k] = [mf.bf16_round(w) for w in model[k]]
    model["token_emb"], model["lm_head"] = mf.bf16_round(model["token_emb"]), mf.bf16_round(model["lm_head"])
    t = mf.model_tensors(c, model)
    mf.write_safetensors(tmp_path / "q.safetensors", {n: (a, "BF16" if a.ndim == 2 else "F32") for n, a in t.items()})
    ref = L.model_ref_load(str(tmp_path / "q.safetensors").encode(), 0)
    assert ref
    check_ref(c, model, ref, [1e6] * c.NL)
    L.model_ref_free(ref)
    # Qwen3, GGUF without output.weight: the LM head is the embedding
    c = C1
    model = make_model(c, seed=4, gamma_jitter=0.1)
    t = mf.model_tensors(c, model, gguf=True)
    mf.write_gguf(tmp_path / "q.gguf", {n: (a, mf.GGML_F32) for n, a in t.items()}, kv=mf.SAMPLE_KV)
    ref = L.model_ref_load(str(tmp_path / "q.gguf").encode(), 0)
    assert ref
    check_ref(c, model, ref, [1e6] * c.NL)
    L.model_ref_free(ref)
    # Gemma3: the file holds norm weights minus one, seven layers show both RoPE bases
    c = TINY_GEMMA
    model = make_model(c, seed=5, gamma_jitter=0.1)
    for k in ("g_in", "g_post_attn", "g_pre_ff", "g_post_ff", "g_q", "g_k"):
        model[k] = [((g - F(1)).astype(F) + F(1)).astype(F) for g in model[k]]
    model["g_final"] = ((model["g_final"] - F(1)).astype(F) + F(1)).astype(F)
    t = mf.model_tensors(c, model)
    mf.write_safetensors(tmp_path / "g.safetensors", {n: (a, "F32") for n, a in t.items()})
    ref = L.model_ref_load(str(tmp_path / "g.safetensors").encode(), 1)
    assert ref
    check_ref(c, model, ref, [1e6 if Li % 6 == 0 else 1e4 for Li in range(c.NL)])
    L.model_ref_free(ref)
    # a missing tensor fails the load
    del t["model.layers.3.mlp.up_proj.weight"]
    mf.write_safetensors(tmp_path / "bad.safetensors", {n: (a, "F32") for n, a in t.items()})
    assert not L.model_ref_load(str(tmp_path / "bad.safetensors").encode(), 1)
    assert "model.layers.3.mlp.up_proj.weight" in capfd.readouterr().err
