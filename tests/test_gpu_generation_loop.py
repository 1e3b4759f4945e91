"""The batched generation loop of the C++ host mirror (BatchGenerationLoop::generate: prefill, then per
token index one device call that samples every active Session from device-resident logits, stop
handling, decode of the survivors) against the CPU oracle.

The C++ test program runs the loop on a synthetic model whose logits are an integer hash of (session,
position, token fed), exact in fp32, and prints every emitted token.  This test rebuilds the same logits
in numpy and replays each Session alone in the order of Session::generate
(src/engine/session.cpp:978-1020): sample with the Session's own mt19937_64 (a draw is consumed only when
more than one candidate survives), stop on a stop token or at max_new_tokens, feed the token back."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as ol
from ncnn_moe_runtime_amd import workloads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TEST_PROGRAM = os.path.join(ROOT, "ncnn-moe-runtime_amd", "test_session_sampler")


synthetic_logits = workloads.synthetic_model_logits


def test_synthetic_logits_are_exact_multiples():
    row = synthetic_logits(3000, 3, 5, 1234)
    assert row.dtype == np.float32 and row.min() >= -8.0 and row.max() < 14.0
    scaled = row.astype(np.float64) * 1048576.0
    assert np.array_equal(scaled, np.round(scaled))
    assert not np.array_equal(row, synthetic_logits(3000, 3, 6, 1234))
    assert not np.array_equal(row, synthetic_logits(3000, 3, 5, -1))


def _bits_to_float(bits):
    return float(np.array([bits], dtype=np.uint32).view(np.float32)[0])


def _parse(trace):
    sessions, tokens, results, vocab = {}, {}, {}, None
    extra = {}
    for line in trace.splitlines():
        fields = line.split()
        if not fields:
            continue
        if fields[0] == "session":
            stops = [int(v) for v in fields[fields.index("stops") + 1:]]
            sessions[int(fields[1])] = dict(
                seed=int(fields[3]), max_new_tokens=int(fields[5]), temperature=_bits_to_float(int(fields[7])),
                top_k=int(fields[9]), top_p=_bits_to_float(int(fields[11])), min_p=_bits_to_float(int(fields[13])), stops=stops)
            if "speculative" in fields:
                at = fields.index("speculative")
                sessions[int(fields[1])].update(speculative=int(fields[at + 1]), confidence=_bits_to_float(int(fields[at + 3])),
                                                max_draft=int(fields[at + 5]))
        elif fields[0] == "token":
            tokens.setdefault(int(fields[1]), []).append(
                dict(index=int(fields[2]), token_id=int(fields[3]), probability_bits=int(fields[4]), is_stop=int(fields[5])))
        elif fields[0] == "result":
            results[int(fields[1])] = dict(tokens=int(fields[3]), stopped_by_stop_token=int(fields[5]), stopped_by_callback=int(fields[7]))
        elif fields[0] == "vocab":
            vocab = int(fields[1])
        elif fields[0] in ("block", "transactions"):
            extra[fields[0]] = int(fields[1])
    if extra:
        return sessions, tokens, results, vocab, extra
    return sessions, tokens, results, vocab


@pytest.mark.gpu
def test_generation_loop_matches_the_oracle_session_by_session():
    print("[case] C++ batched generation loop, trace against the oracle", flush=True)
    assert os.path.exists(TEST_PROGRAM), "build it with make -C ncnn-moe-runtime_amd"
    done = subprocess.run([TEST_PROGRAM, "--generation-trace"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    sessions, tokens, results, vocab = _parse(done.stdout)
    assert vocab == 3000 and len(sessions) == 8 and set(results) == set(sessions)
    stopped_early = 0
    for index, session in sessions.items():
        generator = ol.OracleRng(session["seed"])
        pending = None  # the generator's next draw, kept while no sample has consumed it
        fed = -1
        expected = []
        stopped = False
        for position in range(session["max_new_tokens"]):
            if pending is None:
                pending = generator.uniform()
            row = synthetic_logits(vocab, index, position, fed)
            sampled = ol.oracle_sample(row, pending, session["temperature"], session["top_k"], session["top_p"], session["min_p"])
            assert sampled["status"] == 0
            if sampled["draw_consumed"]:
                pending = None
            token = int(sampled["token_id"])
            is_stop = token in session["stops"]
            expected.append((position, token, int(np.float32(sampled["probability"]).view(np.uint32)), int(is_stop)))
            if is_stop:
                stopped = True
                break
            fed = token
        got = [(t["index"], t["token_id"], t["probability_bits"], t["is_stop"]) for t in tokens[index]]
        assert got == expected, "session %d: %s vs %s" % (index, got[:6], expected[:6])
        assert results[index] == dict(tokens=len(expected), stopped_by_stop_token=int(stopped), stopped_by_callback=0)
        stopped_early += int(stopped)
    assert stopped_early >= 1
    assert len({t["token_id"] for t in tokens[1]}) > 3  # the sampled Sessions do not sit on one token


def _draft_logits(vocab, session, position, fed, draft_index):
    """synthetic_draft_logits of tests/cpp/test_session_sampler.cpp: the target's row there, + 0.75 at every fifth token."""
    row = synthetic_logits(vocab, session, position, fed).copy()
    row[(session + draft_index) % 5::5] += np.float32(0.75)
    return row


def _confidence_logit(session, position):
    return -0.5 if (session * 7 + position * 3) % 11 == 0 else 2.0


class _Draws:
    """The Session's generator with the draws that were looked at and not consumed kept in front."""

    def __init__(self, seed):
        self._generator = ol.OracleRng(seed)
        self._ahead = []

    def ahead(self, position):
        while len(self._ahead) <= position:
            self._ahead.append(self._generator.uniform())
        return self._ahead[position]

    def consume(self, count):
        del self._ahead[:count]


def _replay_speculative_session(index, session, vocab, block, transactions):
    """Session::generate's speculative loop (src/engine/session.cpp:522-977) for one Session, with the CPU oracle:
    first token, then propose (every draft sampled with the Session's generator) - cut - verify - emit, a plain
    step where one token is left or speculative mode was left."""
    sampling = dict(temperature=session["temperature"], top_k=session["top_k"], top_p=session["top_p"], min_p=session["min_p"])
    draws = _Draws(session["seed"])
    emitted = []  # (token, probability bits, is_stop)
    stopped = False

    def sample(row):
        sampled = ol.oracle_sample(row, draws.ahead(0), **sampling)
        assert sampled["status"] == 0
        if sampled["draw_consumed"]:
            draws.consume(1)
        return int(sampled["token_id"]), int(np.float32(sampled["probability"]).view(np.uint32))

    def emit(token, probability_bits):
        nonlocal stopped
        is_stop = token in session["stops"]
        emitted.append((token, probability_bits, int(is_stop)))
        stopped = stopped or is_stop
        return not is_stop and len(emitted) < session["max_new_tokens"]

    position = 0  # of the model state: index of the last token whose logits exist
    going = emit(*sample(synthetic_logits(vocab, index, 0, -1)))
    active = bool(session["speculative"]) and block > 0
    while going:
        anchor = emitted[-1][0]
        remaining = session["max_new_tokens"] - len(emitted)
        if remaining == 1 or not active:
            position += 1
            going = emit(*sample(synthetic_logits(vocab, index, position, anchor)))
            continue
        proposed, draft_rows = [], []
        fed = anchor
        for k in range(block):
            draft_rows.append(_draft_logits(vocab, index, position + 1 + k, fed, k))
            fed = sample(draft_rows[-1])[0]
            proposed.append(fed)
        draft_count = min(len(proposed), remaining - 1)
        if session["max_draft"]:
            draft_count = min(draft_count, session["max_draft"])
        if session["confidence"] > 0.0:
            for k in range(draft_count):
                confidence = np.float32(1.0) / (np.float32(1.0) + np.exp(np.float32(-_confidence_logit(index, position + 1 + k)), dtype=np.float32))
                if confidence < np.float32(session["confidence"]):
                    draft_count = k
                    break
        if draft_count == 0:
            active = False
            continue
        target_rows = [synthetic_logits(vocab, index, position + 1 + k, anchor if k == 0 else proposed[k - 1]) for k in range(draft_count + 1)]
        uniforms = [draws.ahead(k) for k in range(draft_count + 1)]
        verified, accepted_probabilities = ol.oracle_speculative_verify(
            np.stack(target_rows), np.stack(draft_rows[:draft_count]), proposed[:draft_count], uniforms, **sampling)
        assert verified["status"] == 0
        if int(verified["accepted"]) == 0 and not transactions:
            draws.consume(int(verified["accept_draws"]))
            active = False
            continue
        draws.consume(int(verified["accept_draws"]) + int(verified["final_draw_consumed"]))
        step = [(proposed[k], int(np.float32(accepted_probabilities[k]).view(np.uint32))) for k in range(int(verified["accepted"]))]
        step.append((int(verified["next_token_id"]), int(np.float32(verified["next_probability"]).view(np.uint32))))
        for token, probability_bits in step:
            position += 1
            going = emit(token, probability_bits)
            if not going:
                break
    return emitted, stopped


@pytest.mark.gpu
@pytest.mark.parametrize("transactions", [1, 0])
def test_speculative_generation_loop_matches_the_oracle(transactions):
    """BatchGenerationLoop::generate over a source with a draft head: eight Sessions with different options
    (greedy, sampled, speculation off, a draft limit, stop tokens, a two-token budget, a single survivor, a
    threshold nothing passes), with and without state cache transactions, each replayed alone by the oracle."""
    print("[case] C++ speculative generation loop (transactions %d), trace against the oracle" % transactions, flush=True)
    done = subprocess.run([TEST_PROGRAM, "--speculative-trace", str(transactions)], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    sessions, tokens, results, vocab, extra = _parse(done.stdout)
    assert vocab == 3000 and extra == dict(block=4, transactions=transactions) and len(sessions) == 8
    accepted_somewhere = False
    for index, session in sessions.items():
        expected, stopped = _replay_speculative_session(index, session, vocab, extra["block"], bool(transactions))
        got = [(t["token_id"], t["probability_bits"], t["is_stop"]) for t in tokens[index]]
        assert [t["index"] for t in tokens[index]] == list(range(len(got)))
        assert got == expected, "session %d: %s vs %s" % (index, got[:8], expected[:8])
        assert results[index] == dict(tokens=len(expected), stopped_by_stop_token=int(stopped), stopped_by_callback=0)
        accepted_somewhere = accepted_somewhere or any(bits == 0x3F800000 for _, bits, _ in expected[1:]) or session["temperature"] > 0
    assert accepted_somewhere
