"""Helpers for the GPU parity tests: numpy <-> device buffers through the C ABI."""
import numpy as np

from llm_metal_amd.sft import Backend


def rel(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-300))


def maxrel(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / (np.abs(b).max() + 1e-300))


class Dev:
    """Backend plus bookkeeping of the buffers a test created."""

    def __init__(self):
        self.be = Backend()
        self.L = self.be.L
        self.bufs = []

    def up(self, arr):
        b = self.be.buf(arr)
        self.bufs.append(b)
        return b

    def empty(self, nbytes):
        b = self.be.empty(nbytes)
        self.bufs.append(b)
        return b

    def view(self, parent, offset, nbytes):
        from llm_metal_amd.sft import Buf
        b = Buf(self.L, self.L.metal_buf_view(parent.h, offset, nbytes), nbytes)
        self.bufs.insert(0, b)                      # freed before its parent
        return b

    def close(self):
        for b in self.bufs:
            b.free()
        self.be.close()
