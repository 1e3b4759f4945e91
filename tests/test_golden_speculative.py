"""The oracle's residual sampling against vectors recorded from the reference's own
sample_residual_distribution (tests/golden/speculative_golden.npz, written by
tests/golden/make_golden_speculative.py where the reference builds).  Runs wherever the repository is."""
import os

import numpy as np

import oracle_lib as ol

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "speculative_golden.npz")


def test_residual_golden_vectors():
    golden = np.load(GOLDEN)
    sampled = 0
    for case in range(golden["rc"].size):
        target_count, draft_count = golden["counts"][case]
        status, token, probability = ol.oracle_sample_residual(
            golden["target_ids"][case, :target_count], golden["target_probabilities"][case, :target_count],
            golden["draft_ids"][case, :draft_count], golden["draft_probabilities"][case, :draft_count],
            int(golden["vocab"][case]), float(golden["uniforms"][case]))
        if golden["rc"][case] != 0:
            assert status == 3 and golden["draws"][case] == 0  # "speculative residual distribution is empty"
            continue
        sampled += 1
        assert status == 0 and golden["draws"][case] == 1
        assert token == golden["tokens"][case]
        assert np.float32(probability).view(np.uint32) == golden["probabilities"][case].view(np.uint32)
    assert sampled > 100


def test_golden_uniforms_are_the_generator_draws():
    golden = np.load(GOLDEN)
    for case in range(0, golden["rc"].size, 7):
        seed, discard = (int(v) for v in golden["seeds"][case])
        shadow = ol.OracleRng(seed)
        for _ in range(discard):
            shadow.uniform()
        assert np.float32(shadow.uniform()) == golden["uniforms"][case]
