"""The CPU oracle against the golden vectors recorded from the reference library."""
import numpy as np

import golden_util
import oracle_lib as ol


def test_small_rows():
    g = golden_util.load()
    for case in range(g["small_vocab"].size):
        vocab = int(g["small_vocab"][case])
        logits = g["small_logits"][case, :vocab]
        options = golden_util.options_of(g["small_options"][case])
        status, ids, probabilities = ol.oracle_distribution(logits, **options)
        if g["small_rc"][case] != 0:
            assert g["small_rc"][case] == golden_util.REF_ERROR_INVALID_ARGUMENT and status != 0
            continue
        count = int(g["small_count"][case])
        assert status == 0 and len(ids) == count, case
        assert np.array_equal(ids, g["small_ids"][case, :count])
        assert np.array_equal(probabilities.view(np.uint32), g["small_probabilities"][case, :count].view(np.uint32))


def test_session_in_lockstep():
    g = golden_util.load()
    shadow = ol.OracleRng(int(g["session_seed"][0]))
    for step in range(g["session_token"].size):
        logits = g["session_logits"][step]
        options = golden_util.options_of(g["session_options"][step])
        probe = ol.oracle_sample(logits, 0.0, **options)
        assert int(probe["draw_consumed"]) == int(g["session_drew"][step])
        uniform = shadow.uniform() if probe["draw_consumed"] else 0.0
        assert np.float32(uniform) == g["session_uniform"][step]
        mine = ol.oracle_sample(logits, uniform, **options)
        if g["session_rc"][step] != 0:
            assert mine["status"] != 0
            continue
        assert mine["status"] == 0
        assert mine["token_id"] == g["session_token"][step]
        assert mine["probability"] == g["session_probability"][step]


def test_benchmark_sized_rows():
    g = golden_util.load()
    for case in range(g["large_kept"].size):
        seed, vocab, scale, bf16, temperature, top_k, top_p, min_p = g["large_spec"][case]
        logits = golden_util.large_row(seed, vocab, scale, bool(bf16))
        assert np.array_equal(golden_util.sha256(logits), g["large_logits_sha"][case]), "row generator drifted"
        options = golden_util.options_of((temperature, top_k, top_p, min_p))
        status, ids, probabilities = ol.oracle_distribution(logits, **options)
        assert status == 0 and len(ids) == int(g["large_kept"][case])
        head = min(64, len(ids))
        assert np.array_equal(ids[:head], g["large_head_ids"][case, :head])
        assert np.array_equal(probabilities[:head].view(np.uint32),
                              g["large_head_probabilities"][case, :head].view(np.uint32))
        assert np.array_equal(golden_util.sha256(ids), g["large_ids_sha"][case])
        assert np.array_equal(golden_util.sha256(probabilities), g["large_probabilities_sha"][case])
        for draw in range(8):
            mine = ol.oracle_sample(logits, float(g["large_uniform"][case, draw]), **options)
            assert mine["token_id"] == g["large_token"][case, draw]
            assert mine["probability"] == g["large_probability"][case, draw]
