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
    for line in trace.splitlines():
        fields = line.split()
        if not fields:
            continue
        if fields[0] == "session":
            stops = [int(v) for v in fields[fields.index("stops") + 1:]]
            sessions[int(fields[1])] = dict(
                seed=int(fields[3]), max_new_tokens=int(fields[5]), temperature=_bits_to_float(int(fields[7])),
                top_k=int(fields[9]), top_p=_bits_to_float(int(fields[11])), min_p=_bits_to_float(int(fields[13])), stops=stops)
        elif fields[0] == "token":
            tokens.setdefault(int(fields[1]), []).append(
                dict(index=int(fields[2]), token_id=int(fields[3]), probability_bits=int(fields[4]), is_stop=int(fields[5])))
        elif fields[0] == "result":
            results[int(fields[1])] = dict(tokens=int(fields[3]), stopped_by_stop_token=int(fields[5]), stopped_by_callback=int(fields[7]))
        elif fields[0] == "vocab":
            vocab = int(fields[1])
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
