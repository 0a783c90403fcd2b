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


def test_no_alloc_attention_leaves_device_memory_as_it_was():
    """What the entry point exists for: between two readings of the device's free memory, calls at several sizes (with and
    without slice partials) allocate nothing.  fast_metal_init has resolved the fixed array's address on this device
    before, so the calls themselves resolve nothing either (a caller under graph capture must have initialised the
    library on its device first)."""
    import ctypes as C
    dev = Dev()
    try:
        L = dev.L
        rng = np.random.default_rng(12)
        Hq, G, hd, max_seq = 32, 4, 128, 4096
        Q = dev.up(rng.standard_normal(Hq * hd).astype(F))
        Kc = dev.up(rng.standard_normal((Hq // G, max_seq, hd)).astype(F))
        Vc = dev.up(rng.standard_normal((Hq // G, max_seq, hd)).astype(F))
        out = dev.empty(Hq * hd * 4)
        ptrs = [L.hip_buf_device_ptr(b.h) for b in (Q, Kc, Vc, out)]
        L.metal_flush()
        free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
        L.hip_mem_info(C.byref(free0), C.byref(total))
        for n_attend in (4096, 100, 2500, 257):
            assert L.hip_attention_noalloc(*ptrs, n_attend, hd, max_seq, Hq, G) == 0
        L.metal_flush()
        L.hip_mem_info(C.byref(free1), C.byref(total))
        assert free1.value == free0.value, (free0.value, free1.value)
        assert np.isfinite(out.read(F)).all()
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
