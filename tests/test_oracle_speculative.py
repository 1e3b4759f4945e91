"""The oracle's speculative-verification step (src/engine/session.cpp:138-202, 776-874).

candidate_probability and sample_residual_distribution are file-static functions of the reference and
are compared with the reference library itself where it has been built.  The accept loop is inline in
the reference's generate(); it is pinned by those two functions plus what the mathematics fixes: the
token a verification step emits first follows the TARGET distribution whatever the draft distribution
is (integrated here over a grid of uniforms), and greedy verification is arg-max equality."""
import numpy as np
import pytest

import oracle_lib as ol

needs_reference = pytest.mark.skipif(not ol.reference_available(), reason="reference library not built here")
REF_INTERNAL_ERROR = 1 + 4  # 1 + ErrorCode::InternalError (include/ncnn/moe/result.h:12-19)


def random_distribution(rng, vocab, count):
    ids = rng.choice(vocab, size=count, replace=False).astype(np.int32)
    weights = rng.random(count).astype(np.float32) ** 3 + np.float32(1e-4)
    probabilities = np.sort((weights / weights.sum(dtype=np.float32)).astype(np.float32))[::-1].copy()
    return ids, probabilities


def test_candidate_probability_definition():
    ids = np.array([7, 3, 9], dtype=np.int32)
    probabilities = np.array([0.5, 0.3, 0.2], dtype=np.float32)
    assert ol.oracle_candidate_probability(ids, probabilities, 3) == np.float32(0.3)
    assert ol.oracle_candidate_probability(ids, probabilities, 4) == 0.0
    assert ol.oracle_candidate_probability(ids[:0], probabilities[:0], 4) == 0.0


def test_residual_brute_force():
    """max(0, p - q) normalised, walked in token-id order: checked against a float64 model."""
    rng = np.random.default_rng(5)
    for _ in range(200):
        vocab = int(rng.integers(2, 40))
        target_ids, target_p = random_distribution(rng, vocab, int(rng.integers(1, vocab + 1)))
        draft_ids, draft_p = random_distribution(rng, vocab, int(rng.integers(1, vocab + 1)))
        dense = np.zeros(vocab)
        dense[target_ids] = target_p
        dense_draft = np.zeros(vocab)
        dense_draft[draft_ids] = draft_p
        residual = np.maximum(0.0, dense - dense_draft)
        u = float(rng.random())
        status, token, probability = ol.oracle_sample_residual(target_ids, target_p, draft_ids, draft_p, vocab, u)
        if residual.sum() <= 1e-7:
            continue  # too close to the empty case for a float64 model to decide
        assert status == 0
        cdf = np.cumsum(residual) / residual.sum()
        gap = np.min(np.abs(cdf - u))
        if gap > 1e-5:
            assert token == int(np.searchsorted(cdf, u, side="right"))
        assert residual[token] > 0
        assert abs(probability - residual[token] / residual.sum()) < 1e-5


def test_residual_empty_and_fall_through():
    ids = np.array([1, 2], dtype=np.int32)
    p = np.array([0.5, 0.5], dtype=np.float32)
    status, token, _ = ol.oracle_sample_residual(ids, p, ids, p, 4, 0.3)
    assert status == 3 and token == -1  # "speculative residual distribution is empty"
    # canonical draws just below 1 still land on a token that has residual mass
    target_ids = np.array([0, 1, 2, 3], dtype=np.int32)
    target_p = np.array([0.4, 0.3, 0.2, 0.1], dtype=np.float32)
    draft_ids = np.array([3], dtype=np.int32)
    draft_p = np.array([1.0], dtype=np.float32)
    status, token, probability = ol.oracle_sample_residual(
        target_ids, target_p, draft_ids, draft_p, 4, float(np.float32(1.0) - np.float32(2.0 ** -24)))
    assert status == 0 and token == 2 and probability > 0


@needs_reference
@pytest.mark.reference
def test_residual_matches_reference_function():
    rng = np.random.default_rng(6)
    for case in range(300):
        vocab = int(rng.choice([2, 5, 17, 64, 300, 5000]))
        target_ids, target_p = random_distribution(rng, vocab, int(rng.integers(1, min(vocab, 64) + 1)))
        draft_ids, draft_p = random_distribution(rng, vocab, int(rng.integers(1, min(vocab, 64) + 1)))
        if case % 5 == 0:
            draft_ids = target_ids.copy()  # full overlap: many exact zeros
            draft_p = np.roll(target_p, 1)
        seed, discard = int(rng.integers(0, 2 ** 40)), int(rng.integers(0, 5))
        shadow = ol.OracleRng(seed)
        for _ in range(discard):
            shadow.uniform()
        canonical = shadow.uniform()
        rc, ref_token, ref_probability, draws, message = ol.reference_sample_residual(
            target_ids, target_p, draft_ids, draft_p, vocab, seed, discard)
        status, token, probability = ol.oracle_sample_residual(target_ids, target_p, draft_ids, draft_p, vocab, canonical)
        if rc != 0:
            assert rc == REF_INTERNAL_ERROR and status in (3, 4) and ol.VERIFY_MESSAGES[status] == message
            assert draws == (0 if status == 3 else 1)
            continue
        assert status == 0 and draws == 1
        assert token == ref_token
        assert np.float32(probability).view(np.uint32) == np.float32(ref_probability).view(np.uint32)


@needs_reference
@pytest.mark.reference
def test_candidate_probability_matches_reference_function():
    rng = np.random.default_rng(7)
    for _ in range(100):
        ids, probabilities = random_distribution(rng, 100, int(rng.integers(1, 50)))
        for token in list(ids[:3]) + [int(rng.integers(0, 100))]:
            assert ol.oracle_candidate_probability(ids, probabilities, token) == \
                ol.reference_candidate_probability(ids, probabilities, token)


def test_greedy_verification_is_argmax_equality():
    rng = np.random.default_rng(8)
    for _ in range(50):
        drafts, vocab = int(rng.integers(1, 9)), 50
        target = rng.standard_normal((drafts + 1, vocab)).astype(np.float32)
        draft = rng.standard_normal((drafts, vocab)).astype(np.float32)
        best = np.argmax(target, axis=1)
        proposed = best[:drafts].copy()
        wrong = int(rng.integers(0, drafts + 1))
        if wrong < drafts:
            proposed[wrong] = (proposed[wrong] + 1) % vocab
        result, accepted = ol.oracle_speculative_verify(target, draft, proposed, np.zeros(drafts + 1), temperature=0.0)
        assert result["status"] == 0 and result["accepted"] == wrong
        assert result["next_token_id"] == best[wrong] and result["next_probability"] == 1.0
        assert result["accept_draws"] == 0 and result["final_draw_consumed"] == 0 and result["next_is_residual"] == 0
        assert (accepted[:wrong] == 1.0).all()


@pytest.mark.parametrize("options", [dict(temperature=1.0), dict(temperature=0.7, top_k=4),
                                     dict(temperature=1.3, top_p=0.8), dict(temperature=0.9, min_p=0.15)])
def test_first_emitted_token_follows_the_target_distribution(options):
    """Speculative sampling is exact: whatever the draft proposes, the first token that leaves the
    verification step is distributed as the target's filtered distribution.  A swapped ratio, a wrong
    comparison direction or a residual taken the other way round all break this identity."""
    rng = np.random.default_rng(9)
    vocab, grid = 6, 96
    target = (rng.standard_normal((2, vocab)) * 1.5).astype(np.float32)
    draft = (rng.standard_normal((1, vocab)) * 1.5).astype(np.float32)
    status, target_ids, target_p = ol.oracle_distribution(target[0], **options)
    status_draft, draft_ids, draft_p = ol.oracle_distribution(draft[0], **options)
    assert status == 0 and status_draft == 0
    expected = np.zeros(vocab)
    expected[target_ids] = target_p
    measured = np.zeros(vocab)
    points = (np.arange(grid) + 0.5) / grid
    for proposed, weight in zip(draft_ids, draft_p):
        for u_accept in points:
            for u_final in points:
                result, _ = ol.oracle_speculative_verify(target, draft, [proposed], [u_accept, u_final], **options)
                assert result["status"] == 0
                first = proposed if result["accepted"] == 1 else result["next_token_id"]
                measured[first] += float(weight) / (grid * grid)
    assert np.abs(measured - expected).max() < 2.5 / grid, (measured, expected)


def test_accept_loop_consumes_uniforms_in_order():
    """Position i is tested against uniforms[i]; the token after a rejection draws uniforms[accept_draws];
    with everything accepted the extra target row is sampled with uniforms[D]."""
    rng = np.random.default_rng(10)
    vocab, drafts = 40, 4
    options = dict(temperature=0.8, top_k=12, top_p=0.95)
    for _ in range(200):
        target = (rng.standard_normal((drafts + 1, vocab)) * 2).astype(np.float32)
        draft = (target[:drafts] + rng.standard_normal((drafts, vocab)).astype(np.float32) * 0.7).astype(np.float32)
        proposed = []
        for row in draft:
            _, ids, p = ol.oracle_distribution(row, **options)
            proposed.append(int(rng.choice(ids, p=p.astype(np.float64) / p.astype(np.float64).sum())))
        uniforms = rng.random(drafts + 1).astype(np.float32)
        result, accepted = ol.oracle_speculative_verify(target, draft, proposed, uniforms, **options)
        assert result["status"] == 0
        k = int(result["accepted"])
        for i in range(k):
            _, t_ids, t_p = ol.oracle_distribution(target[i], **options)
            assert accepted[i] == ol.oracle_candidate_probability(t_ids, t_p, proposed[i])
        if k == drafts:
            assert result["accept_draws"] == drafts and result["next_is_residual"] == 0
            row = ol.oracle_sample(target[drafts], uniforms[drafts], **options)
            assert result["next_token_id"] == row["token_id"] and result["next_probability"] == row["probability"]
            assert result["final_draw_consumed"] == row["draw_consumed"]
        else:
            assert result["accept_draws"] == k + 1 and result["next_is_residual"] == 1
            _, t_ids, t_p = ol.oracle_distribution(target[k], **options)
            _, d_ids, d_p = ol.oracle_distribution(draft[k], **options)
            status, token, probability = ol.oracle_sample_residual(t_ids, t_p, d_ids, d_p, vocab, uniforms[k + 1])
            assert status == 0 and result["next_token_id"] == token and result["next_probability"] == np.float32(probability)


def test_error_statuses():
    vocab = 8
    target = np.zeros((2, vocab), dtype=np.float32)
    draft = np.zeros((1, vocab), dtype=np.float32)
    draft[0, :4] = 5.0
    # the proposed token is outside the draft's Top-K window
    result, _ = ol.oracle_speculative_verify(target, draft, [6], [0.5, 0.5], temperature=1.0, top_k=4)
    assert result["status"] == 2 and result["next_token_id"] == -1
    # identical distributions and a draw of exactly the acceptance bound: ratio 1, u < 1 always accepts
    result, _ = ol.oracle_speculative_verify(target, target[:1], [0], [0.999999, 0.5], temperature=1.0)
    assert result["status"] == 0 and result["accepted"] == 1
    # a target row without a finite logit fails as the sampler does
    broken = target.copy()
    broken[0, :] = -np.inf
    result, _ = ol.oracle_speculative_verify(broken, draft, [0], [0.5, 0.5], temperature=1.0)
    assert result["status"] == 1 and result["row_status"] == ol.STATUS_NO_FINITE_LOGIT
    # rows behind the rejection are never looked at
    later = np.zeros((3, vocab), dtype=np.float32)
    later[2, :] = np.nan
    result, _ = ol.oracle_speculative_verify(later, np.zeros((2, vocab), dtype=np.float32), [1, 1], [0.2, 0.2, 0.2],
                                             temperature=0.0)
    assert result["status"] == 0 and result["accepted"] == 0 and result["next_token_id"] == 0
