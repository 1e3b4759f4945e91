#!/usr/bin/env python3
"""Writes tests/golden/sampler_golden.npz from the REFERENCE library (oracle/_ref/libref_sampler.so).

Run in the build container only, where the reference checkout exists:

    make -C oracle && python tests/golden/make_golden.py

The file holds inputs and expected outputs only (data, no reference code):
  small_*    rows of at most 64 logits stored verbatim, with the reference's filtered distribution;
  session_*  one reference Session (seed 20240917) sampled 300 times, with the uniforms a shadow
             mt19937_64 produced for it, the tokens and probabilities it returned;
  large_*    rows at the benchmark vocabulary sizes regenerated from a seed (a SHA-256 of the bytes
             guards the regeneration), with the reference's kept count, the head of its
             distribution, a SHA-256 of the whole distribution, and sampled tokens.
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402

HEAD = 64


def large_row(seed, vocab, scale, bf16):
    """The generator the golden tests re-run: PCG64(seed) standard normals times scale (+3 spikes)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    logits = rng.standard_normal(vocab, dtype=np.float32) * np.float32(scale)
    spikes = rng.integers(0, vocab, size=3)
    logits[spikes] += np.float32(6.0)
    if bf16:
        logits = ol.widen_bf16(ol.quantize_bf16(logits))
    return np.ascontiguousarray(logits, dtype=np.float32)


LARGE_CASES = [
    # seed, vocab, scale, bf16, temperature, top_k, top_p, min_p
    (101, 32000, 2.5, False, 0.8, 50, 0.9, 0.0),
    (102, 151936, 3.0, False, 0.7, 20, 0.8, 0.0),
    (103, 201088, 1.4, True, 1.0, 0, 0.95, 0.0),
    (104, 129280, 2.0, False, 1.3, 0, 0.9, 0.05),
    (105, 129280, 2.0, False, 0.9, 1000, 0.97, 0.01),
    (106, 262144, 1.5, True, 0.6, 64, 0.9, 0.02),
    (107, 129280, 0.05, False, 1.0, 0, 0.5, 0.0),   # flat row: the cut depends on sequential fp32 sums
]


def digest(array):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(array).tobytes()).digest(), dtype=np.uint8)


def main():
    if not ol.reference_available():
        sys.exit("the reference library is not built: run `make -C oracle` where /root/reference exists")
    out = {}
    rng = np.random.default_rng(424242)

    # ---- small rows
    small_logits = np.full((96, 64), np.nan, dtype=np.float32)
    small_vocab = np.zeros(96, dtype=np.uint32)
    small_options = np.zeros((96, 4), dtype=np.float64)
    small_rc = np.zeros(96, dtype=np.int32)
    small_count = np.zeros(96, dtype=np.uint32)
    small_ids = np.full((96, 64), -1, dtype=np.int32)
    small_probabilities = np.zeros((96, 64), dtype=np.float32)
    for case in range(96):
        vocab = int(rng.integers(1, 65))
        logits = (rng.standard_normal(vocab) * rng.uniform(0.2, 4)).astype(np.float32)
        if case % 4 == 1:
            logits = np.round(logits)
        if case % 7 == 3:
            logits[rng.integers(0, vocab)] = -np.inf
        if case % 23 == 5:
            logits[rng.integers(0, vocab)] = np.inf
        options = (float(rng.choice([0.1, 0.5, 0.8, 1.0, 2.0])), int(rng.choice([0, 1, 3, 10, 64, 100])),
                   float(rng.choice([1.0, 0.95, 0.7, 0.3])), float(rng.choice([0.0, 0.05, 0.3])))
        rc, ids, probabilities, _ = ol.reference_distribution(logits, *options)
        small_logits[case, :vocab] = logits
        small_vocab[case] = vocab
        small_options[case] = options
        small_rc[case] = rc
        small_count[case] = len(ids)
        small_ids[case, :len(ids)] = ids
        small_probabilities[case, :len(ids)] = probabilities
    out.update(small_logits=small_logits, small_vocab=small_vocab, small_options=small_options, small_rc=small_rc,
               small_count=small_count, small_ids=small_ids, small_probabilities=small_probabilities)

    # ---- one Session in RNG lock-step
    seed = 20240917
    session = ol.ReferenceSession(seed)
    shadow = ol.OracleRng(seed)
    steps = 300
    session_logits = np.zeros((steps, 48), dtype=np.float32)
    session_options = np.zeros((steps, 4), dtype=np.float64)
    session_uniform = np.zeros(steps, dtype=np.float32)
    session_drew = np.zeros(steps, dtype=np.uint8)
    session_rc = np.zeros(steps, dtype=np.int32)
    session_token = np.zeros(steps, dtype=np.int32)
    session_probability = np.zeros(steps, dtype=np.float32)
    for step in range(steps):
        logits = (rng.standard_normal(48) * 2).astype(np.float32)
        options = (float(rng.choice([0.0, 0.6, 1.0, 1.4])), int(rng.choice([0, 1, 5, 40])),
                   float(rng.choice([1.0, 0.9, 0.5, 1e-4])), float(rng.choice([0.0, 0.1])))
        # whether the reference draws is what the oracle says; the next steps would diverge otherwise
        drew = int(ol.oracle_sample(logits, 0.0, *options)["draw_consumed"])
        uniform = shadow.uniform() if drew else 0.0
        rc, token, probability, _ = session.sample(logits, *options)
        session_logits[step] = logits
        session_options[step] = options
        session_uniform[step] = uniform
        session_drew[step] = drew
        session_rc[step] = rc
        session_token[step] = token
        session_probability[step] = probability
    out.update(session_seed=np.array([seed], dtype=np.uint64), session_logits=session_logits,
               session_options=session_options, session_uniform=session_uniform, session_drew=session_drew,
               session_rc=session_rc, session_token=session_token, session_probability=session_probability)

    # ---- benchmark-sized rows
    count = len(LARGE_CASES)
    large_spec = np.zeros((count, 8), dtype=np.float64)
    large_logits_sha = np.zeros((count, 32), dtype=np.uint8)
    large_kept = np.zeros(count, dtype=np.uint32)
    large_head_ids = np.full((count, HEAD), -1, dtype=np.int32)
    large_head_probabilities = np.zeros((count, HEAD), dtype=np.float32)
    large_ids_sha = np.zeros((count, 32), dtype=np.uint8)
    large_probabilities_sha = np.zeros((count, 32), dtype=np.uint8)
    large_uniform = np.zeros((count, 8), dtype=np.float32)
    large_token = np.zeros((count, 8), dtype=np.int32)
    large_probability = np.zeros((count, 8), dtype=np.float32)
    for case, (row_seed, vocab, scale, bf16, temperature, top_k, top_p, min_p) in enumerate(LARGE_CASES):
        logits = large_row(row_seed, vocab, scale, bf16)
        rc, ids, probabilities, _ = ol.reference_distribution(logits, temperature, top_k, top_p, min_p)
        assert rc == 0
        large_spec[case] = (row_seed, vocab, scale, int(bf16), temperature, top_k, top_p, min_p)
        large_logits_sha[case] = digest(logits)
        large_kept[case] = len(ids)
        head = min(HEAD, len(ids))
        large_head_ids[case, :head] = ids[:head]
        large_head_probabilities[case, :head] = probabilities[:head]
        large_ids_sha[case] = digest(ids)
        large_probabilities_sha[case] = digest(probabilities)
        row_session = ol.ReferenceSession(row_seed)
        row_shadow = ol.OracleRng(row_seed)
        for draw in range(8):
            large_uniform[case, draw] = row_shadow.uniform() if len(ids) > 1 else 0.0
            rc, token, probability, _ = row_session.sample(logits, temperature, top_k, top_p, min_p)
            assert rc == 0
            large_token[case, draw] = token
            large_probability[case, draw] = probability
    out.update(large_spec=large_spec, large_logits_sha=large_logits_sha, large_kept=large_kept,
               large_head_ids=large_head_ids, large_head_probabilities=large_head_probabilities,
               large_ids_sha=large_ids_sha, large_probabilities_sha=large_probabilities_sha,
               large_uniform=large_uniform, large_token=large_token, large_probability=large_probability)

    path = os.path.join(HERE, "sampler_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote %s (%d bytes)" % (path, os.path.getsize(path)))


if __name__ == "__main__":
    main()
