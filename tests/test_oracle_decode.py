"""Pins the oracle's decode-step ops as a chain: the logits of token t decoded one token at a time
(src/nn/fast_inference.c:376-467) must be row t of the training forward (src/nn/fast_sft.c:616-752) on the same
weights, adapters and tokens, because attention is causal.  The training forward is pinned in test_oracle_step.py
(against the compiled reference's logits and torch autograd); the two walks share no code above the elementwise ops."""
import numpy as np
import pytest

from llm_metal_amd.configs import C1, GEMMA3, SFTConfig
from llm_metal_amd.synth import make_batch, make_model
from oracle import oracle
from tests.decode_chain import oracle_decode

TINY_GEMMA = SFTConfig("tiny_gemma3", GEMMA3, NL=7, D=128, Hq=4, Hkv=1, hd=32, IS=256, V=512, seq=5, tied=True)


@pytest.mark.parametrize("cfg,fmt", [(C1.with_(seq=6), "f16"), (C1.with_(seq=6), "q8_0"), (TINY_GEMMA, "f16")])
def test_decoded_logits_are_the_rows_of_the_training_forward(cfg, fmt):
    c = cfg.with_(weight_format=fmt)
    model = make_model(c, seed=5, gamma_jitter=0.1)
    tok, tgt = make_batch(c, seed=6)
    used = oracle.weights_as_used(model, fmt)
    _, ref = oracle.sft_loss(c, used, model["lora"], tok, tgt, precision="f64", want_logits=True)
    got = oracle_decode(c, model, fmt, [int(t) for t in tok], max_seq=c.seq + 3, precision="f64", lora=model["lora"])
    assert np.abs(got - ref).max() / np.abs(ref).max() < 1e-11
    # and the adapters matter: without them the logits move
    base = oracle_decode(c, model, fmt, [int(t) for t in tok[:2]], max_seq=4, precision="f64")
    assert np.abs(base - ref[:2]).max() / np.abs(ref).max() > 1e-6
