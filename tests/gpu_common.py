"""Helpers for the GPU parity tests (they call the HIP library through its C ABI binding)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

LOWEST = np.finfo(np.float32).min


def pkg():
    import __graft_entry__ as ge
    return ge.ensure_built()


def say(*a):
    """Names the case before each GPU step, so a faulting run still shows what it was doing."""
    print("[gpu-case]", *a, flush=True)


def make_mask(rng, rows, vocab, frac):
    words = (vocab - 1) // 32 + 1
    bits = rng.random((rows, words * 32)) < frac
    bits[:, vocab:] = False
    for r in range(rows):
        if not bits[r, :vocab].any():
            bits[r, rng.integers(0, vocab)] = True
    packed = np.packbits(bits.reshape(rows, words, 32), axis=-1, bitorder="little").view(np.uint32).reshape(rows, words)
    return np.ascontiguousarray(packed)
