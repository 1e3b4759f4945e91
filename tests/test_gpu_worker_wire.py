"""The sampling slice of the worker's JSON-lines protocol, end to end on the GPU: the test worker
(tests/cpp/sampling_worker.cpp: the HIP sampler behind the request and event lines of
examples/ncnn_moe_worker.cpp:870-905, 1031-1058) is driven with the requests tools/ncnn_moe_protocol.py
sends, and every `token` event is checked against the CPU oracle replaying the same Session on the same
synthetic logits; the text of each number is checked against the worker's formatting rule
(std::setprecision(10) on the double value)."""
import json
import os
import re
import subprocess

import numpy as np
import pytest

import oracle_lib as ol
from ncnn_moe_runtime_amd import workloads

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
WORKER = os.path.join(ROOT, "ncnn-moe-runtime_amd", "test_sampling_worker")
VOCAB = 4096


class Worker:
    def __init__(self):
        self.process = subprocess.Popen([WORKER], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
        self.ready = self.read()

    def send(self, request):
        self.process.stdin.write(json.dumps(request) + "\n")
        self.process.stdin.flush()

    def read(self):
        line = self.process.stdout.readline()
        assert line, "the worker closed its output"
        self.last_line = line.rstrip("\n")
        return json.loads(line)

    def generate(self, **request):
        """The request of WorkerClient.generate (tools/ncnn_moe_protocol.py:140-176); returns (events, lines)."""
        message = {"op": "generate", "request_id": "generate", "max_new_tokens": 1024, "temperature": 0.0, "top_k": 0,
                   "top_p": 1.0, "min_p": 0.0, "stop_tokens": [], "enable_speculative": True, "speculative_confidence": 0.5,
                   "speculative_max_draft": 0, "metrics_enabled": True, "metrics_interval_ms": 1000}
        message.update(request)
        self.send(message)
        events, lines = [], []
        while True:
            event = self.read()
            events.append(event)
            lines.append(self.last_line)
            if event["event"] in ("done", "error"):
                return events, lines

    def close(self):
        self.send({"op": "shutdown"})
        assert self.read()["event"] == "shutdown"
        self.process.wait(timeout=30)


@pytest.fixture(scope="module")
def worker():
    assert os.path.exists(WORKER), "build it with make -C ncnn-moe-runtime_amd"
    print("[case] test worker over the JSON-lines protocol", flush=True)
    handle = Worker()
    assert handle.ready == {"event": "ready", "vocabulary_size": VOCAB}
    yield handle
    handle.close()


class OracleSession:
    """One Session replayed on the CPU: its generator, its position, the worker's synthetic model."""

    def __init__(self, number, seed):
        self.number, self.generator, self.pending, self.sequence_length = number, ol.OracleRng(seed), None, 0

    def generate(self, prompt, max_new_tokens, temperature, top_k, top_p, min_p, stops):
        self.sequence_length += len(prompt)
        fed, tokens = prompt[-1], []
        for index in range(max_new_tokens):
            if self.pending is None:
                self.pending = self.generator.uniform()
            row = workloads.synthetic_model_logits(VOCAB, self.number, self.sequence_length - 1, fed)
            sampled = ol.oracle_sample(row, self.pending, temperature, top_k, top_p, min_p)
            assert sampled["status"] == 0
            if sampled["draw_consumed"]:
                self.pending = None
            token = int(sampled["token_id"])
            tokens.append((index, token, float(np.float32(sampled["probability"])), token in stops))
            if token in stops or index + 1 == max_new_tokens:
                break
            fed = token
            self.sequence_length += 1
        return tokens


def _check_generation(events, lines, expected, session_id, request_id="generate"):
    assert [e["event"] for e in events] == ["token"] * len(expected) + ["done"]
    for event, line, (index, token, probability, is_stop) in zip(events, lines, expected):
        assert event["request_id"] == request_id and event["session_id"] == session_id
        assert (event["index"], event["token_id"], event["is_stop_token"]) == (index, token, is_stop)
        # the text on the wire is the double of the fp32 probability with ten significant digits
        assert re.search(r'"probability":([^,]+),', line).group(1) == "%.10g" % probability
        assert list(event) == ["event", "request_id", "session_id", "index", "token_id", "probability", "is_stop_token",
                               "elapsed_seconds"]
    done = events[-1]
    assert done["ok"] is True and done["generated_tokens"] == len(expected)
    assert done["stopped_by_stop_token"] == bool(expected[-1][3]) and done["stopped_by_callback"] is False
    return done


def test_sessions_generate_like_the_cpu_sampler(worker):
    worker.send({"op": "create_session", "session_id": "a", "seed": 7, "prefill_chunk_size": 64, "enable_speculative_context": True})
    assert worker.read() == {"event": "session_created", "session_id": "a", "sequence_length": 0}
    worker.send({"op": "create_session", "session_id": "b", "seed": 8})
    assert worker.read()["event"] == "session_created"
    a, b = OracleSession(0, 7), OracleSession(1, 8)

    # greedy by default: a request without a temperature
    worker.send({"op": "generate", "session_id": "a", "prompt_tokens": [11, 12, 13], "max_new_tokens": 5})
    events, lines = [], []
    while not events or events[-1]["event"] != "done":
        events.append(worker.read())
        lines.append(worker.last_line)
    expected = a.generate([11, 12, 13], 5, 0.0, 0, 1.0, 0.0, [])
    done = _check_generation(events, lines, expected, "a")
    assert all(probability == 1.0 for _, _, probability, _ in expected)
    assert done["sequence_length"] == a.sequence_length == 3 + 4

    # the client's full request: temperature + Top-K + Top-P, continuing the same Session and generator
    events, lines = worker.generate(session_id="a", request_id="r2", prompt_tokens=[40], max_new_tokens=12,
                                    temperature=0.7, top_k=20, top_p=0.8)
    expected = a.generate([40], 12, 0.7, 20, 0.8, 0.0, [])
    done = _check_generation(events, lines, expected, "a", "r2")
    assert done["sequence_length"] == a.sequence_length
    assert done["sampling"]["sampled_tokens"] == 5 + 12 and done["sampling"]["sample_time_microseconds"] > 0

    # another Session, stop tokens: every seventh id stops it
    stops = list(range(0, VOCAB, 7))
    events, lines = worker.generate(session_id="b", prompt_tokens=[1, 2], max_new_tokens=64, temperature=1.1, top_k=0,
                                    top_p=0.95, min_p=0.001, stop_tokens=stops)
    expected = b.generate([1, 2], 64, 1.1, 0, 0.95, 0.001, stops)
    done = _check_generation(events, lines, expected, "b")
    assert done["stopped_by_stop_token"] is True and len(expected) < 64

    worker.send({"op": "stats", "session_id": "b"})
    stats = worker.read()
    assert stats["event"] == "stats" and stats["sampled_tokens"] == len(expected) and stats["sequence_length"] == b.sequence_length


def test_errors_are_reported_as_the_worker_reports_them(worker):
    events, _ = worker.generate(session_id="nobody", prompt_tokens=[1])
    assert events == [{"event": "error", "request_id": "generate", "code": "invalid_request", "message": "unknown session: nobody"}]
    worker.send({"op": "create_session", "session_id": "c", "seed": 1})
    assert worker.read()["event"] == "session_created"
    events, _ = worker.generate(session_id="c", prompt_tokens=[1], temperature=0.5, top_p=0.0)
    assert events == [{"event": "error", "request_id": "generate", "code": "invalid_argument",
                       "message": "top_p must be in the range (0, 1]"}]
    events, _ = worker.generate(session_id="c", prompt_tokens=[1], temperature=-1.0)
    assert events[0]["message"] == "temperature must be finite and non-negative" and events[0]["code"] == "invalid_argument"
    events, _ = worker.generate(session_id="c", prompt_tokens=[1], max_new_tokens=0)
    assert events[0]["message"] == "max_new_tokens must be non-zero"
    events, _ = worker.generate(session_id="c", prompt_tokens=[])
    assert events[0] == {"event": "error", "request_id": "generate", "code": "invalid_request", "message": "prompt_tokens must not be empty"}
    worker.send({"op": "create_session", "session_id": "c"})
    assert worker.read() == {"event": "error", "code": "invalid_request", "message": "session already exists: c"}
    # the Session still works after the rejected requests
    events, lines = worker.generate(session_id="c", prompt_tokens=[9], max_new_tokens=3, temperature=0.9, top_k=50)
    _check_generation(events, lines, OracleSession(2, 1).generate([9], 3, 0.9, 50, 1.0, 0.0, []), "c")
