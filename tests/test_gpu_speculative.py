"""GPU parity of the speculative-verification entry (ncnn_moe_hip_sampler_speculative_verify, called
through the C ABI) against the CPU oracle on identical seeded inputs: accepted count, emitted token,
probabilities (bit for bit), statuses and the number of draws consumed."""
import numpy as np
import pytest

import oracle_lib
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu


def _announce(text):
    print("[case] " + text, flush=True)


@pytest.fixture(scope="module")
def sampler():
    handle = hip_sampler.HipSampler(2 * hip_sampler.MAX_DRAFT_TOKENS + 1, 152000)
    yield handle
    handle.close()


def _bits(value):
    return np.float32(value).view(np.uint32)


def _compare(sampler, target, draft, proposed, uniforms, context, bf16=False, **options):
    _announce(context)
    rows = np.concatenate([target, draft], axis=0)
    if bf16:
        bits = workloads.float32_to_bf16_bits(rows)
        sampler.upload_logits(bits)
        widened = workloads.bf16_bits_to_float32(bits)
        target, draft = widened[:target.shape[0]], widened[target.shape[0]:]
    else:
        sampler.upload_logits(rows)
    gpu, gpu_accepted = sampler.speculative_verify(proposed, uniforms, **options)
    cpu, cpu_accepted = oracle_lib.oracle_speculative_verify(target, draft, proposed, uniforms, **options)
    for field in ("status", "row_status", "accepted", "next_token_id", "accept_draws", "final_draw_consumed",
                  "next_is_residual"):
        assert gpu[field] == cpu[field], "%s: %s gpu %s cpu %s" % (context, field, gpu, cpu)
    assert _bits(gpu["next_probability"]) == _bits(cpu["next_probability"]), (context, gpu, cpu)
    accepted = int(cpu["accepted"])
    assert np.array_equal(gpu_accepted[:accepted].view(np.uint32), cpu_accepted[:accepted].view(np.uint32)), context
    return gpu


def _propose(rng, draft, options):
    proposed = []
    for row in draft:
        status, ids, p = oracle_lib.oracle_distribution(row, **options)
        assert status == 0
        p = p.astype(np.float64)
        proposed.append(int(rng.choice(ids, p=p / p.sum())))
    return proposed


@pytest.mark.parametrize("vocab,drafts,options", [
    (50, 1, dict(temperature=1.0, top_k=8)),
    (1000, 4, dict(temperature=0.8, top_k=20, top_p=0.9)),
    (32000, 8, dict(temperature=0.7, top_k=64, top_p=0.95, min_p=0.01)),
    (151936, 5, dict(temperature=1.2, top_k=40)),
    (151936, 16, dict(temperature=0.6, top_k=20, top_p=0.8)),
    (32000, 3, dict(temperature=0.9, top_k=300, top_p=0.98)),        # the wide select kernel
    (50000, 4, dict(temperature=1.0, top_k=1024)),
    (20000, 2, dict(temperature=0.5, top_p=0.9)),                    # no Top-K window: sort + replay, short nucleus
    (3000, 3, dict(temperature=0.8, top_k=2000, top_p=0.7, min_p=0.001)),
])
def test_random_steps_match_oracle(sampler, vocab, drafts, options):
    rng = np.random.default_rng(vocab + drafts)
    outcomes = set()
    for case in range(12):
        target = (rng.standard_normal((drafts + 1, vocab)) * 2.5).astype(np.float32)
        noise = rng.standard_normal((drafts, vocab)).astype(np.float32) * np.float32(rng.choice([0.1, 0.5, 1.5]))
        draft = (target[:drafts] + noise).astype(np.float32)
        proposed = _propose(rng, draft, options)
        uniforms = rng.random(drafts + 1).astype(np.float32)
        if case % 4 == 3:
            uniforms[:] = 0.0  # everything accepted: the row after the last drafted token is sampled
        gpu = _compare(sampler, target, draft, proposed, uniforms,
                       "V=%d D=%d case %d %s" % (vocab, drafts, case, options), **options)
        outcomes.add((int(gpu["accepted"]) == drafts, int(gpu["next_is_residual"])))
    assert (True, 0) in outcomes, "no case accepted every drafted token"
    if drafts > 1:
        assert (False, 1) in outcomes, "no case was rejected"


def test_bf16_rows(sampler):
    rng = np.random.default_rng(21)
    options = dict(temperature=0.9, top_k=32, top_p=0.9)
    for case in range(6):
        target = (rng.standard_normal((5, 30011)) * 2).astype(np.float32)
        draft = (target[:4] + rng.standard_normal((4, 30011)).astype(np.float32) * 0.5).astype(np.float32)
        widened_draft = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(draft))
        proposed = _propose(rng, widened_draft, options)
        _compare(sampler, target, draft, proposed, rng.random(5).astype(np.float32), "bf16 case %d" % case,
                 bf16=True, **options)


def test_greedy_steps(sampler):
    rng = np.random.default_rng(22)
    for wrong in range(0, 5):
        drafts, vocab = 4, 20000
        target = rng.standard_normal((drafts + 1, vocab)).astype(np.float32)
        draft = rng.standard_normal((drafts, vocab)).astype(np.float32)
        proposed = np.argmax(target[:drafts], axis=1).astype(np.int32)
        if wrong < drafts:
            proposed[wrong] = (proposed[wrong] + 7) % vocab
        gpu = _compare(sampler, target, draft, proposed, np.zeros(drafts + 1, dtype=np.float32),
                       "greedy, first mismatch at %d" % wrong, temperature=0.0)
        assert gpu["accepted"] == wrong and gpu["accept_draws"] == 0


def test_residual_edge_cases(sampler):
    vocab = 64
    base = np.zeros((2, vocab), dtype=np.float32)
    base[0, :8] = np.linspace(3.0, 1.0, 8, dtype=np.float32)
    base[1, :8] = 2.0
    draft = base[:1].copy()
    # identical distributions: the ratio is 1 and every canonical draw accepts
    _compare(sampler, base, draft, [3], [np.float32(1.0) - np.float32(2.0 ** -24), 0.3], "identical distributions",
             temperature=1.0, top_k=8)
    # the draft puts everything on one token the target rates lower: rejected, residual over the others
    sharp = base[:1].copy()
    sharp[0, 5] = 30.0
    gpu = _compare(sampler, base, sharp, [5], [0.99, 0.999999], "sharp draft, late residual draw", temperature=1.0, top_k=8)
    assert gpu["next_is_residual"] == 1 and gpu["next_token_id"] != 5
    _compare(sampler, base, sharp, [5], [0.99, 0.0], "sharp draft, first residual token", temperature=1.0, top_k=8)
    # the proposed token is not among the draft's candidates
    gpu = _compare(sampler, base, draft, [40], [0.5, 0.5], "token outside the draft window", temperature=1.0, top_k=8)
    assert gpu["status"] == hip_sampler.VERIFY_ZERO_DRAFT_PROBABILITY
    assert hip_sampler.verify_status_message(gpu["status"]) == oracle_lib.VERIFY_MESSAGES[2]
    # a target row the sampler rejects
    broken = base.copy()
    broken[0, :] = -np.inf
    gpu = _compare(sampler, broken, draft, [3], [0.5, 0.5], "target row without a finite logit", temperature=1.0, top_k=8)
    assert gpu["status"] == hip_sampler.VERIFY_ROW_ERROR and gpu["row_status"] == hip_sampler.ROW_NO_FINITE_LOGIT
    # rows behind the rejection are not looked at
    later = np.zeros((3, vocab), dtype=np.float32)
    later[0, 1] = 1.0
    later[2, :] = np.nan
    _compare(sampler, later, np.zeros((2, vocab), dtype=np.float32), [0, 0], [0.5, 0.5, 0.5],
             "NaN row behind a greedy mismatch", temperature=0.0)
    # heavy ties at the Top-K boundary (the select lists overflow and the full-order kernels serve the rows)
    tied = np.ones((3, 20000), dtype=np.float32)
    _compare(sampler, tied, tied[:2], [3, 9], [0.4, 0.6, 0.2], "all logits tied", temperature=1.0, top_k=16)


def test_long_distributions_and_argument_errors(sampler):
    """Filtered distributions of more than 1024 candidates take the dense residual; wrong shapes are refused."""
    flat = np.zeros((3, 5000), dtype=np.float32)
    for options in (dict(temperature=1.0, top_k=0), dict(temperature=1.0, top_k=1025), dict(temperature=1.0, top_p=0.2)):
        for uniforms in ([0.5, 0.5], [0.999, 0.7]):
            _compare(sampler, flat[:2], flat[2:], [1], uniforms, "flat rows %s %s" % (options, uniforms), **options)
    sampler.upload_logits(flat)
    with pytest.raises(hip_sampler.SamplerError):
        sampler.speculative_verify([1, 2], [0.5, 0.5, 0.5], temperature=1.0, top_k=8)  # 3 rows hold one drafted token


@pytest.mark.parametrize("vocab,drafts,bf16,options", [
    (5000, 2, False, dict(temperature=1.0)),
    (40000, 3, False, dict(temperature=1.0, top_p=0.95)),
    (40000, 3, True, dict(temperature=0.9, top_p=0.98, min_p=0.00001)),
    (33333, 4, False, dict(temperature=1.3, top_k=3000)),
    (151936, 5, False, dict(temperature=1.0, top_p=0.9)),
    (151936, 2, False, dict(temperature=1.5)),
])
def test_long_distributions_match_the_oracle(sampler, vocab, drafts, bf16, options):
    """Rows whose filtered distributions hold thousands of tokens: accepted prefixes of every length, the
    residual draw early and late in the vocabulary, and the draw that follows a fully accepted draft."""
    rng = np.random.default_rng(4242 + vocab + drafts)
    for trial in range(4):
        target = (rng.standard_normal((drafts + 1, vocab)) * 1.5).astype(np.float32)
        draft = (target[:drafts] + rng.standard_normal((drafts, vocab)).astype(np.float32) * (0.2 + 0.4 * trial)).astype(np.float32)
        if bf16:
            target = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(target))
            draft = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(draft))
        proposed = _propose(rng, draft, options)
        uniforms = rng.random(drafts + 1).astype(np.float32)
        if trial == 1:
            uniforms[0] = np.float32(0.9999)    # reject the first drafted token
        if trial == 2:
            uniforms[:drafts] = np.float32(0.0)  # accept everything
        if trial == 3:
            uniforms[drafts - 1] = np.float32(0.9999)
            uniforms[drafts] = np.float32(0.99999)  # a residual draw near the end of the vocabulary
        _compare(sampler, target, draft, proposed, uniforms,
                 "long lists: vocab %d drafts %d trial %d %s" % (vocab, drafts, trial, options), bf16=bf16, **options)
