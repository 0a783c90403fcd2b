"""Pins the oracle's F16 rounding and Q8_0 quantise/dequantise.

Pins: the hand-derived known answers in tests/golden/q8_0_kat.json (made by
tests/golden/make_q8_kat.py without the oracle), numpy's IEEE float16 casts as
the library routine for round-to-nearest-even over every half bit pattern and
over adversarial floats, and an exhaustive numpy float32 restatement of the
quantiser on random and boundary blocks."""
import json
import os

import numpy as np

from oracle import oracle

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "q8_0_kat.json")))


def test_f16_known_answers():
    for case in KAT["f16"]:
        f = np.array([case["f32_bits"]], dtype=np.uint32).view(np.float32)
        assert int(oracle.f32_to_f16_bits(f)[0]) == case["f16_bits"], hex(case["f32_bits"])


def test_f16_every_half_round_trips_and_matches_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    assert np.isnan(f[nan]).all()
    back = oracle.f32_to_f16_bits(f)
    assert np.array_equal(back[~nan], bits[~nan])


def test_f16_rounding_matches_numpy_on_midpoints_and_random():
    rng = np.random.default_rng(0)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)       # exact ties (representable in fp32)
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    rnd = rng.standard_normal(200000).astype(np.float32) * np.float32(0.02)
    wide = (rng.standard_normal(200000) * np.exp(rng.uniform(-20, 12, 200000))).astype(np.float32)
    allv = np.concatenate([mids, -mids, near, rnd, wide, np.float32([65519.99, 65520.0, 1e9, -1e9])])
    with np.errstate(over="ignore"):
        ref = allv.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(allv), ref)


def test_q8_known_answer_blocks():
    for case in KAT["q8_blocks"]:
        x = np.array(case["x_bits"], dtype=np.uint32).view(np.float32).reshape(1, 32)
        got = oracle.q8_quantize(x)
        assert got.tolist() == case["bytes"], case["name"]


def _q8_numpy(x):
    """IEEE fp32 restatement with numpy scalars (round half away from zero)."""
    rows, cols = x.shape
    nb = cols // 32
    out = np.zeros((rows, nb, 34), dtype=np.uint8)
    xb = x[:, :nb * 32].reshape(rows, nb, 32)
    amax = np.abs(xb).max(axis=2)
    scale = (amax / np.float32(127.0)).astype(np.float32)
    out[:, :, 0:2] = scale.astype(np.float16).view(np.uint8).reshape(rows, nb, 2)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = (np.float32(1.0) / scale).astype(np.float32)
        t = (xb * inv[:, :, None]).astype(np.float32)
    q = np.where(t >= 0, np.floor(t + np.float32(0.5)), -np.floor(-t + np.float32(0.5)))
    # floor(t + 0.5) in fp32 can differ from roundf when t + 0.5 rounds up: redo those in float64
    t64 = t.astype(np.float64)
    q = np.where(t64 >= 0, np.floor(t64 + 0.5), -np.floor(-t64 + 0.5))
    q = np.clip(q, -128, 127)
    q = np.where(scale[:, :, None] == 0, 0, q).astype(np.int8)
    out[:, :, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def test_q8_matches_numpy_restatement_and_truncates_ragged_cols():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((37, 96 + 7)) * 0.02).astype(np.float32)      # 7 ragged columns are dropped
    x[3, 32:64] = 0                                                         # a zero block
    x[5, :32] = np.float32(1e-30)                                           # scale underflows fp16 but not fp32
    x[6, :32] *= np.float32(1e6)                                            # scale overflows fp16 -> inf bits
    got = oracle.q8_quantize(x)
    assert got.size == 37 * 3 * 34
    assert np.array_equal(got, _q8_numpy(x))


def test_q8_dequant_is_scale_times_code_in_fp32():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((8, 128)) * 0.02).astype(np.float32)
    blocks = oracle.q8_quantize(x)
    deq = oracle.q8_dequant(blocks, 8, 128)
    b = blocks.reshape(8, 4, 34)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float32).reshape(8, 4, 1)
    q = b[:, :, 2:].view(np.int8).astype(np.float32)
    assert np.array_equal(deq.reshape(8, 4, 32), d * q)
    # error bound of the format: half a code step of the UN-rounded scale + fp16 rounding of the scale
    amax = np.abs(x.reshape(8, 4, 32)).max(axis=2, keepdims=True)
    assert np.all(np.abs(deq.reshape(8, 4, 32) - x.reshape(8, 4, 32)) <= amax / 127 * (0.5 + 127 * 2.0 ** -11) + 1e-12)
    # idempotence: a dequantised block re-quantises to the same 34 bytes
    assert np.array_equal(oracle.q8_quantize(oracle.q8_dequant(blocks, 8, 128)), blocks)
