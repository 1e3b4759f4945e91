"""The CPU oracle against the REFERENCE library itself (oracle/_ref/libref_sampler.so, built from the
reference checkout where that is present).  Skipped where the library has not been built."""
import numpy as np
import pytest

import oracle_lib as ol

pytestmark = [pytest.mark.reference,
              pytest.mark.skipif(not ol.reference_available(), reason="reference library not built here")]

REF_ERROR_INVALID_ARGUMENT = 1  # 1 + ErrorCode::InvalidArgument


def random_options(rng, vocab):
    return dict(
        temperature=float(rng.choice([0.05, 0.3, 0.7, 1.0, 1.5, 4.0])),
        top_k=int(rng.choice([0, 0, 1, 2, 20, 50, 64, 65, 1000, vocab, vocab + 1])),
        top_p=float(rng.choice([1.0, 0.99, 0.95, 0.9, 0.8, 0.5, 0.1, 1e-3])),
        min_p=float(rng.choice([0.0, 0.0, 0.01, 0.02, 0.1, 0.5, 1.0])),
    )


def random_logits(rng, vocab):
    kind = rng.integers(0, 6)
    logits = (rng.standard_normal(vocab) * rng.uniform(0.3, 5.0)).astype(np.float32)
    if kind == 1:
        logits = np.round(logits * 2) / 2            # heavy ties
    elif kind == 2:
        logits = ol.widen_bf16(ol.quantize_bf16(logits))
    elif kind == 3:
        logits[rng.integers(0, vocab, max(1, vocab // 10))] = -np.inf
    elif kind == 4:
        logits[:] = logits[0]                        # all equal
    elif kind == 5:
        logits[rng.integers(0, vocab, 3)] += 15.0    # spikes
    return logits.astype(np.float32)


@pytest.mark.parametrize("seed", range(40))
def test_distribution_bit_exact(seed):
    rng = np.random.default_rng(1000 + seed)
    vocab = int(rng.choice([1, 2, 3, 7, 64, 65, 500, 4097, 20000]))
    logits = random_logits(rng, vocab)
    for _ in range(6):
        options = random_options(rng, vocab)
        rc, ref_ids, ref_probabilities, message = ol.reference_distribution(logits, **options)
        status, ids, probabilities = ol.oracle_distribution(logits, **options)
        if rc != 0:
            assert rc == REF_ERROR_INVALID_ARGUMENT
            assert status != 0 and ol.STATUS_MESSAGES[status] == message
            continue
        assert status == 0
        assert np.array_equal(ids, ref_ids)
        assert np.array_equal(probabilities.view(np.uint32), ref_probabilities.view(np.uint32))


@pytest.mark.parametrize("vocab,options", [
    (32000, dict(temperature=0.8, top_k=50, top_p=0.9)),
    (151936, dict(temperature=0.7, top_k=20, top_p=0.8)),
    (201088, dict(temperature=1.0, top_k=0, top_p=0.95)),
    (129280, dict(temperature=1.4, top_k=0, top_p=0.97, min_p=0.01)),
    (129280, dict(temperature=0.9, top_k=1000, top_p=0.8, min_p=0.05)),
    (262144, dict(temperature=0.6, top_k=64, top_p=0.9, min_p=0.02)),
])
def test_benchmark_shapes_bit_exact(vocab, options):
    rng = np.random.default_rng(vocab)
    logits = (rng.standard_normal(vocab) * 2.5).astype(np.float32)
    if vocab in (201088, 262144):
        logits = ol.widen_bf16(ol.quantize_bf16(logits))
    rc, ref_ids, ref_probabilities, _ = ol.reference_distribution(logits, **options)
    status, ids, probabilities = ol.oracle_distribution(logits, **options)
    assert rc == 0 and status == 0
    assert np.array_equal(ids, ref_ids)
    assert np.array_equal(probabilities.view(np.uint32), ref_probabilities.view(np.uint32))


def test_flat_row_top_p_cut_depends_on_sequential_sums():
    """A long flat row: the sequential fp32 normaliser absorbs small terms, which moves the Top-P cut.
    The oracle must land on the reference's cut exactly."""
    rng = np.random.default_rng(77)
    logits = (rng.standard_normal(129280) * 0.05).astype(np.float32)
    for top_p in (0.5, 0.9, 0.999):
        rc, ref_ids, ref_probabilities, _ = ol.reference_distribution(logits, 1.0, 0, top_p, 0.0)
        status, ids, probabilities = ol.oracle_distribution(logits, 1.0, 0, top_p, 0.0)
        assert rc == 0 and status == 0 and len(ids) == len(ref_ids)
        assert np.array_equal(ids, ref_ids)
        assert np.array_equal(probabilities.view(np.uint32), ref_probabilities.view(np.uint32))


def test_session_sample_in_rng_lockstep():
    """A real reference Session against the oracle fed by a shadow mt19937_64: tokens, probabilities,
    errors and -- through the next draw -- whether each call consumed a draw."""
    rng = np.random.default_rng(5)
    session = ol.ReferenceSession(987654321)
    shadow = ol.OracleRng(987654321)
    for step in range(400):
        vocab = int(rng.choice([2, 3, 5, 100, 3000]))
        logits = random_logits(rng, vocab)
        if step % 17 == 0:
            logits[rng.integers(0, vocab)] = np.inf
        options = random_options(rng, vocab)
        if step % 5 == 0:
            options["temperature"] = 0.0
        if step % 29 == 0:
            options["top_p"] = 0.0
        # the oracle tells whether this call draws; only then is the shadow generator advanced
        probe = ol.oracle_sample(logits, 0.0, **options)
        uniform = shadow.uniform() if probe["draw_consumed"] else 0.0
        mine = ol.oracle_sample(logits, uniform, **options)
        rc, token, probability, message = session.sample(logits, **options)
        if rc != 0:
            assert rc == REF_ERROR_INVALID_ARGUMENT
            assert mine["status"] != 0 and ol.STATUS_MESSAGES[int(mine["status"])] == message
            continue
        assert mine["status"] == 0
        assert token == mine["token_id"], (step, options)
        assert np.float32(probability) == mine["probability"]


def test_fall_through_returns_last_candidate():
    """u above every running sum (the sums end slightly below 1): the reference returns the last candidate."""
    logits = np.array([1.0, 1.0, 1.0], dtype=np.float32)
    status, ids, probabilities = ol.oracle_distribution(logits)
    cumulative = np.float32(0)
    for p in probabilities:
        cumulative = np.float32(cumulative + p)
    u = float(np.nextafter(np.float32(1.0), np.float32(0.0)))
    mine = ol.oracle_sample(logits, u)
    assert mine["token_id"] == 2
    # find a seed whose first draw is >= the final running sum, if the sums fall short of 1
    if cumulative < 1.0:
        for seed in range(20000):
            if ol.OracleRng(seed).uniform() >= cumulative:
                rc, token, probability, _ = ol.ReferenceSession(seed).sample(logits)
                assert rc == 0 and token == 2
                break


def test_bf16_helpers_match_reference_exhaustively():
    lib, ref = ol.oracle(), ol.reference()
    for bits in range(0, 65536):
        a, b = lib.oracle_bfloat16_to_float(bits), ref.ref_bfloat16_to_float(bits)
        assert (np.isnan(a) and np.isnan(b)) or a == b
    rng = np.random.default_rng(9)
    values = np.concatenate([
        (rng.standard_normal(20000) * 10).astype(np.float32),
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    values = values[~np.isnan(values)]
    for v in values:
        assert lib.oracle_float_to_bfloat16(float(v)) == ref.ref_float_to_bfloat16(float(v))
