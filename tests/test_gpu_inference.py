"""GPU parity of the pipeline-level generation API (include/inference_hip.h) against the CPU oracle's decode chain:
logits of every position, greedy generation, EOS handling, and a state that shares weights and adapters with an
SFT state (the GRPO sampling set-up of the reference, src/nn/fast_grpo.c:192-345)."""
import json
import sys

import numpy as np
import pytest

from llm_metal_amd.configs import C1, GEMMA3, SFTConfig
from llm_metal_amd.sft import InferenceState, SFTState
from llm_metal_amd.synth import make_batch, make_model
from tests.decode_chain import oracle_decode
from tests.gpu_util import maxrel

pytestmark = pytest.mark.gpu
F = np.float32
TINY_GEMMA = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=256, V=512, seq=6, tied=True)


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


@pytest.mark.parametrize("cfg", [C1.with_(seq=8), TINY_GEMMA])
def test_state_sharing_weights_and_adapters_with_sft(cfg):
    say("inference from sft", cfg.name)
    c = cfg
    model = make_model(c, seed=11, gamma_jitter=0.1)
    tok, tgt = make_batch(c, seed=12)
    toks = [int(t) for t in tok]
    with SFTState(c, model) as sft:
        with InferenceState(sft=sft, max_seq=16) as inf:
            ref = oracle_decode(c, model, "f16", toks, max_seq=16, precision="f32", lora=model["lora"])
            got = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got, ref) < 2e-4
            # the training forward of the same state gives the same rows (its GEMMs round activations to fp16)
            loss = sft.train_step(tok, tgt, 1e-2)
            assert np.isfinite(loss)
            assert maxrel(sft.logits(), got) < 5e-3
            # the adapters are shared buffers: the step that just ran moved the logits
            lora_new = sft.lora()
            ref2 = oracle_decode(c, model, "f16", toks, max_seq=16, precision="f32", lora=lora_new)
            inf.reset()
            got2 = np.stack([inf.forward_token(t) for t in toks])
            assert maxrel(got2, ref2) < 2e-4
            assert maxrel(got2, got) > 1e-4
