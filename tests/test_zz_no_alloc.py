"""hip_attention_noalloc (the one entry point that allocates nothing) against metal_enqueue_attention, through the C ABI.

Both run the same kernels, so the outputs must be bit-identical; the entry point under test keeps its slice results in
a fixed per-device array instead of the library's grow-only arena.  Two calls in a row share that array, the second
with a smaller input, and both are also checked against the CPU oracle's attention."""
import numpy as np
import pytest

from oracle.oracle import op
from tests.gpu_util import Dev, rel

pytestmark = pytest.mark.gpu
F = np.float32


def _case(dev, rng, Hq, G, hd, n_attend, max_seq):
    Hkv = Hq // G
    q = rng.standard_normal(Hq * hd).astype(F)
    kc = rng.standard_normal((Hkv, max_seq, hd)).astype(F)
    vc = rng.standard_normal((Hkv, max_seq, hd)).astype(F)
    Q, Kc, Vc = dev.up(q), dev.up(kc), dev.up(vc)
    out_a, out_b = dev.empty(Hq * hd * 4), dev.empty(Hq * hd * 4)
    L = dev.L
    L.metal_enqueue_attention(Q.h, Kc.h, Vc.h, out_a.h, n_attend, hd, max_seq, Hq, G)
    rc = L.hip_attention_noalloc(L.hip_buf_device_ptr(Q.h), L.hip_buf_device_ptr(Kc.h), L.hip_buf_device_ptr(Vc.h),
                                 L.hip_buf_device_ptr(out_b.h), n_attend, hd, max_seq, Hq, G)
    assert rc == 0
    a, b = out_a.read(F), out_b.read(F)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (Hq, G, hd, n_attend)
    ref = np.zeros(Hq * hd, F)
    op("f32", "or_attention", q, kc, vc, ref, n_attend, hd, max_seq, Hq, G)
    assert rel(b, ref) < 1e-5, rel(b, ref)


def test_no_alloc_attention_matches_the_allocating_entry_point_on_consecutive_calls():
    dev = Dev()
    try:
        rng = np.random.default_rng(11)
        _case(dev, rng, Hq=32, G=4, hd=128, n_attend=3000, max_seq=3072)     # 12 slices: the fixed array is used
        _case(dev, rng, Hq=8, G=8, hd=64, n_attend=700, max_seq=1024)        # smaller, right after: stale contents beside it
        _case(dev, rng, Hq=4, G=1, hd=256, n_attend=100, max_seq=128)        # one slice: no partials at all
        _case(dev, rng, Hq=64, G=16, hd=256, n_attend=8192, max_seq=8192)    # every limit at once
    finally:
        dev.close()


def test_no_alloc_attention_refuses_what_does_not_fit(capfd):
    dev = Dev()
    try:
        L = dev.L
        buf = dev.empty(1 << 20)
        p = L.hip_buf_device_ptr(buf.h)
        assert L.hip_attention_noalloc(p, p, p, p, 8193, 128, 16384, 32, 4) == -1       # too many keys
        assert L.hip_attention_noalloc(p, p, p, p, 512, 512, 1024, 32, 4) == -1         # head too wide
        assert L.hip_attention_noalloc(p, p, p, p, 512, 128, 1024, 128, 4) == -1        # too many heads
        assert L.hip_attention_noalloc(p, p, p, p, 512, 128, 256, 32, 4) == -1          # more keys than the cache holds
        assert L.hip_attention_noalloc(None, p, p, p, 512, 128, 1024, 32, 4) == -1
        assert "attention_noalloc" in capfd.readouterr().err
    finally:
        dev.close()
