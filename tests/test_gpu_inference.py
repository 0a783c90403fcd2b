"""GPU parity of the pipeline-level generation API (include/inference_hip.h) against the CPU oracle's decode chain:
logits of every position, greedy generation, EOS handling, and a state that shares weights and adapters with an
SFT state (the GRPO sampling set-up of the reference, src/nn/fast_grpo.c:192-345)."""
import json
import sys

import numpy as np
import pytest

from llm_metal_amd.configs import C1, C3, GEMMA3, SFTConfig
from llm_metal_amd import lib as _lib
from llm_metal_amd.sft import InferenceState, SFTState
from llm_metal_amd.synth import make_batch, make_model
from tests.decode_chain import oracle_decode
from tests.gpu_util import maxrel

pytestmark = pytest.mark.gpu
F = np.float32
TINY_GEMMA = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=256, V=512, seq=6, tied=True)


def _free_bytes(L):
    import ctypes
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    L.hip_mem_info(ctypes.byref(free), ctypes.byref(total))
    return free.value


def say(*a):
    print(*a, flush=True, file=sys.stderr)


@pytest.mark.parametrize("cfg,fmt", [(C1.with_(seq=8), "f16"), (C1.with_(seq=8), "q8_0"), (TINY_GEMMA, "f16"), (TINY_GEMMA, "q8_0")])
def test_forward_token_logits_and_greedy_generation(cfg, fmt):
    say("inference", cfg.name, fmt)
    c = cfg.with_(weight_format=fmt)
    model = make_model(c, seed=7, gamma_jitter=0.1)
    tok, _ = make_batch(c, seed=8)
    toks = [int(t) for t in tok]
    ref = oracle_decode(c, model, fmt, toks, max_seq=32, precision="f32")
    with InferenceState(c, model, max_seq=32, use_fp16=(fmt == "f16")) as inf:
        assert inf.V == c.V
        got = np.stack([inf.forward_token(t) for t in toks])
        assert inf.position() == len(toks)
        assert maxrel(got, ref) < 2e-4
        # the same positions again after a reset, through the GPU argmax
        inf.reset()
        best = [inf.forward_token_argmax(t) for t in toks]
        assert best == [int(a) for a in got.argmax(1)]
        # greedy generation = feeding back the argmax, one token at a time
        prompt = toks[:3]
        gen = inf.generate(prompt, 10)
        assert len(gen) == 10
        inf.reset()
        for t in prompt[:-1]:
            inf.forward_token_argmax(t)
        nxt, want = inf.forward_token_argmax(prompt[-1]), []
        for _ in range(10):
            want.append(nxt)
            nxt = inf.forward_token_argmax(nxt)
        assert [int(g) for g in gen] == want
        # the oracle run on prompt + generated tokens agrees with every choice that was not a near-tie
        full = prompt + want[:-1]
        lo = oracle_decode(c, model, fmt, full, max_seq=32, precision="f32")[len(prompt) - 1:]
        srt = np.sort(lo, axis=1)
        clear = (srt[:, -1] - srt[:, -2]) > 1e-3 * np.abs(lo).max()
        assert clear.sum() >= 5 and (lo.argmax(1)[clear] == np.asarray(want)[clear]).all()
        # an EOS token ends the generation after it has been emitted
        inf.set_eos([want[2]])
        gen2 = inf.generate(prompt, 10)
        stop = want.index(want[2])
        assert [int(g) for g in gen2] == want[:stop + 1]
        # the cache is full after max_seq positions; a token outside the vocabulary is refused
        inf.reset()
        for _ in range(32):
            inf.forward_token_argmax(1)
        assert inf.forward_token_argmax(1) == -1
        inf.reset()
        assert inf.forward_token_argmax(c.V) == -1 and inf.position() == 0


@pytest.mark.parametrize("cfg,with_lora,n_prompt", [(C1.with_(seq=8), False, 4), (TINY_GEMMA, False, 4), (C1.with_(seq=8), True, 4),
                                                    (C1.with_(seq=8), True, 270)],
                         ids=["qwen3", "gemma3", "qwen3_adapters", "qwen3_adapters_two_key_slices"])
def test_batched_generation_decodes_every_copy_like_the_single_sequence(cfg, with_lora, n_prompt):
    """inference_generate_batch (qwen3_generate_fast_batch, src/nn/fast_inference.c:895-1000): B copies of one prompt
    in lock step, weights read once per step.  Every copy must produce the single-sequence greedy tokens (wherever the
    choice was not a near-tie: the batched products keep 22 bits of the activations, the single ones all 24), the
    oracle's decode chain must agree with them, and an end token stops the loop once all copies have emitted it.
    The 270-token prompt puts the context beyond one slice of keys, where every copy's slice results are merged."""
    say("batched generation", cfg.name, with_lora, n_prompt)
    c = cfg
    model = make_model(c, seed=17, gamma_jitter=0.1)
    if n_prompt <= 8:
        tok, _ = make_batch(c, seed=18)
        prompt = [int(t) for t in tok[:n_prompt]]
    else:
        prompt = [int(t) for t in np.random.default_rng(18).integers(1, c.V, n_prompt)]
    B, n = 5, 12
    max_seq = 32 if n_prompt <= 8 else n_prompt + n + 6

    def check(inf, lora):
        single = [int(g) for g in inf.generate(prompt, n)]
        assert len(single) == n
        pos = inf.position()
        got = inf.generate_batch(prompt, n, B)
        assert got.shape == (B, n) and inf.position() == pos          # its own caches: the state's are left alone
        lo = oracle_decode(c, model, "f16", prompt + single[:-1], max_seq=max_seq, precision="f32", lora=lora)[len(prompt) - 1:]
        srt = np.sort(lo, axis=1)
        clear = (srt[:, -1] - srt[:, -2]) > 1e-3 * np.abs(lo).max()
        first_tie = n if clear.all() else int(np.argmin(clear))        # after a near-tie the sequences may part ways
        assert first_tie >= 4
        for b in range(B):
            assert [int(t) for t in got[b, :first_tie]] == single[:first_tie], b
            assert np.array_equal(got[b], got[0])                      # identical inputs, identical arithmetic
        assert (lo.argmax(1)[:first_tie] == np.asarray(single)[:first_tie]).all()
        # an end token: every copy emits it at the same step, and the loop stops after it
        inf.set_eos([single[2]])
        stop = single.index(single[2])
        got2 = inf.generate_batch(prompt, n, 3)
        assert got2.shape == (3, stop + 1) and [int(t) for t in got2[1]] == single[:stop + 1]
        # refused: too many copies, a token outside the vocabulary
        assert inf.generate_batch(prompt, n, 33).shape[1] == 0
        assert inf.generate_batch([c.V], n, 2).shape[1] == 0

    if with_lora:
        with SFTState(c, model) as sft:
            with InferenceState(sft=sft, max_seq=max_seq) as inf:
                check(inf, model["lora"])
    else:
        with InferenceState(c, model, max_seq=max_seq, use_fp16=True) as inf:
            check(inf, None)
        with InferenceState(c, model, max_seq=max_seq, use_fp16=False) as q8:
            assert q8.generate_batch(prompt, n, 2).shape[1] == 0       # F16 weights only, as in the reference


@pytest.mark.parametrize("with_lora", [False, True], ids=["plain", "adapters"])
def test_batch_steps_with_a_token_of_their_own_per_sequence(with_lora):
    """inference_step_batch: sequence b of a lock-step batch is fed its own tokens (forward_token_batch with distinct
    tokens_b, src/nn/fast_inference.c:808-893).  Each sequence's logits must match the single-sequence path run on that
    sequence alone, to the 22 bits the batched products keep of the activations; the batch's caches survive from call to
    call, and a greedy batch run afterwards reuses them without disturbing its result."""
    say("batch steps with distinct tokens", with_lora)
    c = C1.with_(seq=8)
    model = make_model(c, seed=31, gamma_jitter=0.1)
    B, n = 4, 9
    seqs = np.random.default_rng(32).integers(1, c.V, (B, n))

    def check(inf):
        greedy_before = inf.generate_batch([int(t) for t in seqs[0, :3]], 5, B)
        batch_logits = np.stack([inf.step_batch(seqs[:, i], i) for i in range(n)], axis=1)      # [B, n, V]
        for b in range(B):
            inf.reset()
            single = np.stack([inf.forward_token(int(t)) for t in seqs[b]])
            assert maxrel(batch_logits[b], single) < 1e-4, b
        # a step that does not follow the one before is refused; pos = 0 restarts
        with pytest.raises(RuntimeError):
            inf.step_batch(seqs[:, 0], n + 3)
        again = inf.step_batch(seqs[:, 0], 0)
        assert np.array_equal(again, batch_logits[:, 0])
        with pytest.raises(RuntimeError):
            inf.step_batch([c.V] * B, 1)
        assert np.array_equal(inf.generate_batch([int(t) for t in seqs[0, :3]], 5, B), greedy_before)
        # another batch size takes new caches
        two = inf.step_batch(seqs[:2, 0], 0)
        assert maxrel(two, batch_logits[:2, 0]) < 1e-4

    if with_lora:
        with SFTState(c, model) as sft:
            with InferenceState(sft=sft, max_seq=32) as inf:
                check(inf)
    else:
        with InferenceState(c, model, max_seq=32, use_fp16=True) as inf:
            check(inf)


# Qwen3-4B's widths (hidden 2560, 32 / 8 heads of 128, FFN 9728): the instantiations that `bench.py --decode` launches --
# two weight rows per wave with the SiLU gate and the norm inside the launch at 19456 x 2560, the norm-fused Q|K|V
# product at 6144 x 2560, the attention kernel with four-key steps, the fused per-head prologue and the O weights asked
# for ahead at 32 / 8 heads of 128, and, for the batch, the matrix-core products on split rows.  Two layers, vocabulary cut.
C3_DECODE = C3.with_(name="c3_decode_widths", NL=2, V=8192, seq=24)


@pytest.mark.parametrize("fmt,with_lora,from_sft", [("f16", False, False), ("q8_0", False, False), ("f16", True, False),
                                                    ("f16", True, True), ("q8_0", True, True)],
                         ids=["f16", "q8_0", "f16_adapters", "f16_on_training_tiles", "q8_0_on_training_tiles"])
def test_decode_at_the_benchmarked_widths(fmt, with_lora, from_sft):
    say("decode at config 3's widths", fmt, with_lora, from_sft)
    c = C3_DECODE.with_(weight_format=fmt)
    model = make_model(c, seed=27, gamma_jitter=0.1)
    toks = [int(t) for t in np.random.default_rng(28).integers(1, c.V, 16)]
    lora = model["lora"] if with_lora else None
    ref = oracle_decode(c, model, fmt, toks, max_seq=64, precision="f32", lora=lora)

    def check(inf):
        got = np.stack([inf.forward_token(t) for t in toks])
        # Q8_0 tiles of a training state enter its products as half(d * q), one rounding to 11 bits per weight that the
        # matrix-vector kernels (and the oracle), which multiply by d in fp32, do not make
        assert maxrel(got, ref) < (2e-3 if from_sft and fmt == "q8_0" else 5e-4), maxrel(got, ref)
        # greedy generation from a prompt: the tokens are the argmax of the oracle's logits wherever that is not a near-tie
        prompt = toks[:5]
        gen = [int(g) for g in inf.generate(prompt, 8)]
        lo = oracle_decode(c, model, fmt, prompt + gen[:-1], max_seq=64, precision="f32", lora=lora)[len(prompt) - 1:]
        srt = np.sort(lo, axis=1)
        clear = (srt[:, -1] - srt[:, -2]) > 1e-3 * np.abs(lo).max()
        first_tie = len(gen) if clear.all() else int(np.argmin(clear))
        assert first_tie >= 3 and (lo.argmax(1)[:first_tie] == np.asarray(gen)[:first_tie]).all()
        if fmt == "f16" or from_sft:
            # eight copies in lock step (the products on the matrix cores): every copy the single-sequence tokens
            got8 = inf.generate_batch(prompt, 8, 8)
            assert got8.shape == (8, 8)
            for b in range(8):
                assert np.array_equal(got8[b], got8[0])
                assert [int(t) for t in got8[b, :first_tie]] == gen[:first_tie], b
            # twenty copies: 40 split rows, where the wide products of the streaming kernel take 128 weight rows per
            # workgroup (gate|up, and down at twice the K chunks)
            got20 = inf.generate_batch(prompt, 8, 20)
            assert got20.shape == (20, 8)
            for b in range(20):
                assert np.array_equal(got20[b], got20[0])
                assert [int(t) for t in got20[b, :first_tie]] == gen[:first_tie], b

    if from_sft:
        # the state reads the training state's tiles in place: it allocates caches, scratch and planes, nothing weight-sized
        L = _lib.load()
        weight_count = c.NL * (c.D * (c.Hq + 2 * c.Hkv) * c.hd + c.D * c.Hq * c.hd + 3 * c.D * c.IS) + c.V * c.D
        with SFTState(c, model) as sft:
            free0 = _free_bytes(L)
            with InferenceState(sft=sft, max_seq=64) as inf:
                check(inf)
                assert free0 - _free_bytes(L) < weight_count // 2, (free0 - _free_bytes(L), weight_count)
    elif with_lora:
        with SFTState(c, model) as sft:
            with InferenceState(c, model, max_seq=64, use_fp16=True) as inf:
                inf.attach_lora(sft)
                check(inf)
    else:
        with InferenceState(c, model, max_seq=64, use_fp16=(fmt == "f16")) as inf:
            check(inf)


def test_eos_ids_from_config_json(tmp_path, capfd):
    c = C1.with_(seq=4)
    model = make_model(c, seed=9)
    with InferenceState(c, model, max_seq=8) as inf:
        d = tmp_path / "m"; d.mkdir()
        (d / "config.json").write_text(json.dumps({"architectures": ["X"], "eos_token_id": [5, 9, 11], "pad": 0}))
        inf.load_eos(d)                                   # a directory
        assert "EOS tokens (3): 5 9 11" in capfd.readouterr().err
        (d / "config.json").write_text('{"bos_token_id": 2,\n  "eos_token_id" : 77}')
        inf.load_eos(d / "model.safetensors")             # a file next to config.json
        assert "EOS tokens (1): 77" in capfd.readouterr().err
        inf.load_eos(tmp_path / "nowhere" / "x.bin")      # nothing there: the reference's Qwen3 defaults
        assert "EOS tokens (2): 151645 151643" in capfd.readouterr().err


@pytest.mark.parametrize("cfg,fmt", [(C1.with_(seq=8), "f16"), (TINY_GEMMA, "f16"), (C1.with_(seq=8), "q8_0")],
                         ids=["qwen3", "gemma3", "qwen3_q8_0"])
def test_state_sharing_weights_and_adapters_with_sft(cfg, fmt):
    """inference_state_create_from_sft (src/nn/fast_inference.c:596-603, owns_weights = 0): the generation state reads the
    training state's own tiles and adapter buffers in place."""
    say("inference from sft", cfg.name, fmt)
    c = cfg.with_(weight_format=fmt)
    model = make_model(c, seed=11, gamma_jitter=0.1)
    tok, tgt = make_batch(c, seed=12)
    toks = [int(t) for t in tok]
    tol = 2e-3 if fmt == "q8_0" else 2e-4      # a training state's Q8_0 tiles enter its products as half(d * q)
    with SFTState(c, model) as sft:
        with InferenceState(sft=sft, max_seq=16) as inf:
            ref = oracle_decode(c, model, fmt, toks, max_seq=16, precision="f32", lora=model["lora"])
            got = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got, ref) < tol
            # greedy generation and the lock-step batch agree with the token-by-token argmax
            inf.reset()
            want = []
            for t in toks[:4]:
                nxt = inf.forward_token_argmax(t)
            for _ in range(5):
                want.append(nxt)
                nxt = inf.forward_token_argmax(nxt)
            assert [int(g) for g in inf.generate(toks[:4], 5)] == want
            assert [int(g) for g in inf.generate_batch(toks[:4], 5, 3)[2]] == want
            # the training forward of the same state gives the same rows (its GEMMs round activations to fp16)
            loss = sft.train_step(tok, tgt, 1e-2)
            assert np.isfinite(loss)
            assert maxrel(sft.logits(), got) < 5e-3
            # the adapters are shared buffers: the step that just ran moved the logits
            lora_new = sft.lora()
            ref2 = oracle_decode(c, model, fmt, toks, max_seq=16, precision="f32", lora=lora_new)
            inf.reset()
            got2 = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got2, ref2) < tol
            assert maxrel(got2, got) > 1e-4


@pytest.mark.parametrize("cfg", [C1.with_(seq=8, R=0), TINY_GEMMA.with_(R=0)], ids=["qwen3", "gemma3"])
def test_state_from_sft_sees_full_parameter_updates_without_a_refresh(cfg):
    """The weights of a state made from a training state are that state's: after a full-parameter SGD step the next
    token is computed with the updated matrices, with no call in between."""
    say("inference from a full-parameter sft state", cfg.name)
    c = cfg
    model = make_model(c, seed=13, gamma_jitter=0.1)
    tok, tgt = make_batch(c, seed=14)
    toks = [int(t) for t in tok]

    def current(sft):
        m = dict(model)
        names = ("wq", "wk", "wv", "wo", "wg", "wu", "wd")
        for k in names:
            m[k] = [sft.matrix_f16(L, k, 0).view(np.float16).astype(np.float32) for L in range(c.NL)]
        m["lm_head"] = sft.matrix_f16(0, "lm_head", 0).view(np.float16).astype(np.float32)
        return m

    with SFTState(c, model) as sft:
        assert sft.is_full_param()
        with InferenceState(sft=sft, max_seq=16) as inf:
            got = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got, oracle_decode(c, current(sft), "f16", toks, max_seq=16, precision="f32")) < 2e-4
            assert np.isfinite(sft.train_step(tok, tgt, 0.2))          # fused SGD: every matrix moves
            inf.reset()
            got2 = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got2, oracle_decode(c, current(sft), "f16", toks, max_seq=16, precision="f32")) < 2e-4
            assert maxrel(got2, got) > 1e-3


def test_own_weights_with_a_training_states_adapters():
    """inference_state_set_lora (src/nn/fast_inference.h:46) on a state with its own row-major weights: the
    matrix-vector pipeline with the adapter terms, reading the training state's adapter buffers."""
    say("own weights + attached adapters")
    c = C1.with_(seq=8)
    model = make_model(c, seed=15, gamma_jitter=0.1)
    tok, _ = make_batch(c, seed=16)
    toks = [int(t) for t in tok]
    with SFTState(c, model) as sft:
        with InferenceState(c, model, max_seq=16, use_fp16=True) as inf:
            inf.attach_lora(sft)
            ref = oracle_decode(c, model, "f16", toks, max_seq=16, precision="f32", lora=model["lora"])
            got = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got, ref) < 2e-5
            plain = oracle_decode(c, model, "f16", toks, max_seq=16, precision="f32")
            assert maxrel(got, plain) > 1e-4


# ---------------------------------------------------------------- checkpoint files (include/loader_hip.h)

def _as_used(model, conv):
    m = dict(model)
    for k in ("wq", "wk", "wv", "wo", "wg", "wu", "wd"):
        m[k] = [conv(w) for w in model[k]]
    return m


def test_weights_from_files_are_bit_exact_in_every_format_pair(tmp_path):
    import ctypes as C
    from llm_metal_amd.sft import Backend, Buf
    from oracle import oracle
    from tests import model_files as mf
    rng = np.random.default_rng(21)
    w = (rng.standard_normal((48, 96)) * 0.05).astype(F)
    wb = mf.bf16_round(w)
    mf.write_safetensors(tmp_path / "t.safetensors", {"f32": (w, "F32"), "f16": (w, "F16"), "bf16": (wb, "BF16")})
    mf.write_gguf(tmp_path / "t.gguf", {"q8": (w, mf.GGML_Q8_0), "f16": (w, mf.GGML_F16), "f32": (w, mf.GGML_F32)})
    h16 = w.astype(np.float16)
    blocks = oracle.q8_quantize(w)
    deq = oracle.q8_dequant(blocks, 48, 96)
    want = {("f32", 1): h16.tobytes(), ("f16", 1): h16.tobytes(), ("bf16", 1): wb.astype(np.float16).tobytes(),
            ("f32", 0): blocks.tobytes(), ("f16", 0): oracle.q8_quantize(h16.astype(F)).tobytes(),
            ("bf16", 0): oracle.q8_quantize(wb).tobytes(), ("q8", 0): blocks.tobytes(), ("q8", 1): deq.astype(np.float16).tobytes()}
    with Backend() as be:
        for fname, names in (("t.safetensors", ("f32", "f16", "bf16")), ("t.gguf", ("q8", "f16", "f32"))):
            fh = be.L.model_file_open(str(tmp_path / fname).encode())
            assert fh
            for name in names:
                for use_fp16 in (1, 0):
                    wm = be.L.model_file_load_wmat(fh, name.encode(), use_fp16)
                    assert wm and (wm.contents.rows, wm.contents.cols) == (48, 96)
                    nbytes = 48 * 96 * 2 if use_fp16 else 48 * 3 * 34
                    got = Buf(be.L, wm.contents.mbuf, nbytes, owned=False).read(np.uint8).tobytes()
                    assert got == want[(name, use_fp16)], (fname, name, use_fp16)
                    be.L.wmat_free(wm)
            be.L.model_file_close(fh)


@pytest.mark.parametrize("case", ["qwen_bf16_to_f16", "qwen_gguf_q8_as_is", "qwen_gguf_q8_to_f16", "gemma_f16_to_q8"])
def test_generation_state_straight_from_a_checkpoint_file(case, tmp_path):
    from oracle import oracle
    from tests import model_files as mf
    say("inference from file", case)
    gemma = case.startswith("gemma")
    c = TINY_GEMMA if gemma else C1.with_(seq=6, tied=case != "qwen_bf16_to_f16")
    model = make_model(c, seed=13, gamma_jitter=0.1)
    if gemma:
        for k in ("g_in", "g_post_attn", "g_pre_ff", "g_post_ff", "g_q", "g_k"):
            model[k] = [((g - F(1)).astype(F) + F(1)).astype(F) for g in model[k]]
        model["g_final"] = ((model["g_final"] - F(1)).astype(F) + F(1)).astype(F)
    tied = model["lm_head"] is model["token_emb"]
    if case == "qwen_bf16_to_f16":
        model = _as_used(model, mf.bf16_round)
        model["token_emb"], model["lm_head"] = mf.bf16_round(model["token_emb"]), mf.bf16_round(model["lm_head"])
        t = mf.model_tensors(c, model)
        path = tmp_path / "m.safetensors"
        mf.write_safetensors(path, {n: (a, "BF16" if a.ndim == 2 else "F32") for n, a in t.items()})
        used, fmt, fp16 = model, "f16", True
    elif case.startswith("qwen_gguf"):
        emb16 = model["token_emb"].astype(np.float16).astype(F)                # the file stores the table as F16
        model["token_emb"] = model["lm_head"] = emb16
        t = mf.model_tensors(c, model, gguf=True)
        path = tmp_path / "m.gguf"
        mf.write_gguf(path, {n: (a, mf.GGML_F32 if a.ndim == 1 else mf.GGML_F16 if n == "token_embd.weight" else mf.GGML_Q8_0)
                             for n, a in t.items()}, kv=mf.SAMPLE_KV)
        if case == "qwen_gguf_q8_as_is":
            used, fmt, fp16 = model, "q8_0", False                             # the oracle quantises the same fp32 values
        else:
            used = _as_used(model, lambda w: oracle.q8_dequant(oracle.q8_quantize(w), *w.shape))
            used["token_emb"] = used["lm_head"] = emb16
            fmt, fp16 = "f16", True
    else:
        model = _as_used(model, lambda w: w.astype(np.float16).astype(F))
        model["token_emb"] = model["lm_head"] = model["token_emb"].astype(np.float16).astype(F)
        t = mf.model_tensors(c, model)
        path = tmp_path / "g.safetensors"
        mf.write_safetensors(path, {n: (a, "F16" if a.ndim == 2 else "F32") for n, a in t.items()})
        used, fmt, fp16 = model, "q8_0", False
    assert tied == (used["lm_head"] is used["token_emb"])
    tok, _ = make_batch(c, seed=14)
    toks = [int(x) for x in tok]
    ref = oracle_decode(c, used, fmt, toks, max_seq=16, precision="f32")
    with InferenceState(c, path=path, model_type=c.model_type, max_seq=16, use_fp16=fp16) as inf:
        assert inf.V == c.V
        got = np.stack([inf.forward_token(x) for x in toks])
        assert maxrel(got, ref) < 2e-4


def test_sft_state_from_a_loaded_model_description(tmp_path):
    import ctypes as C
    from llm_metal_amd import lib as _lib
    from tests import model_files as mf
    c = C1.with_(seq=16)
    model = make_model(c, seed=15, gamma_jitter=0.1)
    t = mf.model_tensors(c, model)
    mf.write_safetensors(tmp_path / "m.safetensors", {n: (a, "F32") for n, a in t.items()})
    tok, tgt = make_batch(c, seed=16)
    with SFTState(c, model) as a:
        la = a.train_step(tok, tgt, 1e-3)
    L = _lib.load()
    ref = L.model_ref_load(str(tmp_path / "m.safetensors").encode(), 0)
    assert ref
    lora = np.ascontiguousarray(model["lora"], F)
    ref.contents.lora_init = lora.ctypes.data
    h = L.sft_state_create_from_ref(ref, c.batch, c.seq, c.R, c.alpha, 1)
    assert h
    lb = float(L.sft_train_step(h, np.ascontiguousarray(tok, np.uint32).ctypes.data, np.ascontiguousarray(tgt, np.uint32).ctypes.data, 1e-3))
    L.sft_state_free(h)
    L.model_ref_free(ref)
    assert la == lb                                                            # the same weights, the same arithmetic
