"""Loader of tests/golden/sampler_golden.npz: vectors recorded from the reference library by
tests/golden/make_golden.py (inputs and expected outputs only)."""
import hashlib
import os

import numpy as np

GOLDEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sampler_golden.npz")

# 1 + ErrorCode::InvalidArgument in the recorded return codes
REF_ERROR_INVALID_ARGUMENT = 1


def load():
    return np.load(GOLDEN_PATH, allow_pickle=False)


def sha256(array):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(array).tobytes()).digest(), dtype=np.uint8)


def float32_to_bf16_bits(values):
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounding = np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    return ((bits + rounding) >> np.uint32(16)).astype(np.uint16)


def large_row(seed, vocab, scale, bf16):
    """The generator of the benchmark-sized golden rows (must stay identical to make_golden.py)."""
    rng = np.random.Generator(np.random.PCG64(int(seed)))
    logits = rng.standard_normal(int(vocab), dtype=np.float32) * np.float32(scale)
    spikes = rng.integers(0, int(vocab), size=3)
    logits[spikes] += np.float32(6.0)
    if bf16:
        logits = (float32_to_bf16_bits(logits).astype(np.uint32) << np.uint32(16)).view(np.float32)
    return np.ascontiguousarray(logits, dtype=np.float32)


def options_of(row):
    return dict(temperature=float(np.float32(row[0])), top_k=int(row[1]), top_p=float(np.float32(row[2])),
                min_p=float(np.float32(row[3])))
