"""CPU tests of the token-file batcher (include/data_hip.h) against the batching rule of the reference's
dataloader_next_batch (src/data/dataloader.c:97-141), restated with numpy slicing."""
import os

import numpy as np
import pytest

from llm_metal_amd import lib


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(lib.LIB_PATH):
        lib.build()
    return lib.load()


def test_batches_targets_epoch_end_and_shuffle(L, tmp_path):
    ids = np.arange(100, 100 + 41, dtype=np.int32)
    path = tmp_path / "tokens.bin"
    ids.tofile(path)
    B, S = 2, 5
    dl = L.token_loader_open(str(path).encode(), B, S)
    assert dl and L.token_loader_n_tokens(dl) == 41 and L.token_loader_n_batches(dl) == 4     # (41 - 1) / 10
    inp, tgt = np.zeros(B * S, np.uint32), np.zeros(B * S, np.uint32)
    for k in range(4):
        assert L.token_loader_next(dl, inp.ctypes.data, tgt.ctypes.data) == 0
        assert np.array_equal(inp, ids[10 * k:10 * k + 10]) and np.array_equal(tgt, ids[10 * k + 1:10 * k + 11])
        assert L.token_loader_position(dl) == 10 * (k + 1)
    before = inp.copy()
    assert L.token_loader_next(dl, inp.ctypes.data, tgt.ctypes.data) == -1                   # 40 + 10 + 1 > 41
    assert L.token_loader_position(dl) == 0 and np.array_equal(inp, before)
    assert L.token_loader_next(dl, inp.ctypes.data, tgt.ctypes.data) == 0 and inp[0] == 100
    for _ in range(20):
        L.token_loader_shuffle(dl)
        assert L.token_loader_position(dl) < 20                                             # rand() % (n_tokens / 2)
    L.token_loader_reset(dl)
    assert L.token_loader_position(dl) == 0
    L.token_loader_free(dl)
    # a file shorter than one batch never yields one; a missing file is refused
    ids[:7].tofile(path)
    dl = L.token_loader_open(str(path).encode(), B, S)
    assert L.token_loader_n_batches(dl) == 0 and L.token_loader_next(dl, inp.ctypes.data, tgt.ctypes.data) == -1
    L.token_loader_free(dl)
    assert not L.token_loader_open(str(tmp_path / "absent.bin").encode(), B, S)
