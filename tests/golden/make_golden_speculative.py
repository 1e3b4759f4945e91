#!/usr/bin/env python3
"""Writes tests/golden/speculative_golden.npz from the REFERENCE library (oracle/_ref/libref_sampler.so).

Run in the build container only, where the reference checkout exists:

    make -C oracle && python tests/golden/make_golden_speculative.py

The file holds inputs and expected outputs only (data, no reference code): pairs of filtered
distributions (target, draft), the seed and position of the mt19937_64 draw, the canonical uniform a
shadow generator produced for it, and what the reference's own sample_residual_distribution
(src/engine/session.cpp:150-202) returned: code, token, probability, draws consumed.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402

CASES = 160
CAP = 64


def main():
    if not ol.reference_available():
        sys.exit("the reference library is not built: run `make -C oracle` where /root/reference exists")
    rng = np.random.default_rng(515151)
    out = {name: np.zeros((CASES, CAP), dtype=dtype) for name, dtype in (
        ("target_ids", np.int32), ("target_probabilities", np.float32),
        ("draft_ids", np.int32), ("draft_probabilities", np.float32))}
    counts = np.zeros((CASES, 2), dtype=np.uint32)
    vocab = np.zeros(CASES, dtype=np.uint32)
    seeds = np.zeros((CASES, 2), dtype=np.uint64)
    uniforms = np.zeros(CASES, dtype=np.float32)
    rc = np.zeros(CASES, dtype=np.int32)
    tokens = np.zeros(CASES, dtype=np.int32)
    probabilities = np.zeros(CASES, dtype=np.float32)
    draws = np.zeros(CASES, dtype=np.uint32)
    for case in range(CASES):
        size = int(rng.choice([2, 5, 17, 64, 300, 152000]))
        logits = (rng.standard_normal((2, size)) * rng.uniform(0.5, 4)).astype(np.float32)
        logits[1] = logits[0] + rng.standard_normal(size).astype(np.float32) * np.float32(rng.choice([0.0, 0.2, 1.0, 3.0], p=[0.1, 0.3, 0.3, 0.3]))
        options = dict(temperature=float(rng.choice([0.5, 0.8, 1.0, 1.5])), top_k=int(rng.choice([1, 2, 8, 20, 64], p=[0.05, 0.15, 0.3, 0.3, 0.2])),
                       top_p=float(rng.choice([1.0, 0.9, 0.6])), min_p=float(rng.choice([0.0, 0.05])))
        _, target_ids, target_p, _ = ol.reference_distribution(logits[0], **options)
        _, draft_ids, draft_p, _ = ol.reference_distribution(logits[1], **options)
        seed, discard = int(rng.integers(0, 2 ** 40)), int(rng.integers(0, 4))
        shadow = ol.OracleRng(seed)
        for _ in range(discard):
            shadow.uniform()
        uniforms[case] = shadow.uniform()
        rc[case], tokens[case], probabilities[case], draws[case], _ = ol.reference_sample_residual(
            target_ids, target_p, draft_ids, draft_p, size, seed, discard)
        counts[case] = (target_ids.size, draft_ids.size)
        out["target_ids"][case, :target_ids.size] = target_ids
        out["target_probabilities"][case, :target_ids.size] = target_p
        out["draft_ids"][case, :draft_ids.size] = draft_ids
        out["draft_probabilities"][case, :draft_ids.size] = draft_p
        vocab[case] = size
        seeds[case] = (seed, discard)
    np.savez_compressed(os.path.join(HERE, "speculative_golden.npz"), counts=counts, vocab=vocab, seeds=seeds,
                        uniforms=uniforms, rc=rc, tokens=tokens, probabilities=probabilities, draws=draws, **out)
    print("wrote %d cases: %d empty residuals, %d sampled" % (CASES, int((rc != 0).sum()), int((rc == 0).sum())))


if __name__ == "__main__":
    main()
