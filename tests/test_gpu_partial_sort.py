"""Full-order fp32 rows that are sorted only in part (GPU): a kernel guesses how far down the sorted row a term
can still move one of the sampler's sums, only that much of the row is sorted, and the walk checks the guess
against its exact sums.  The results must be the oracle's, byte for byte those of the whole sort, and a row whose
guess turns out too short must come back from the second launch that sorts it whole."""
import numpy as np
import pytest

import parity_util
from ncnn_moe_runtime_amd import hip_sampler, workloads

pytestmark = pytest.mark.gpu

ROWS, VOCAB = 40, 70001  # nine tiles of 8,192 keys: the sort is spread over several workgroups


def _announce(text):
    print("[case] " + text, flush=True)


@pytest.fixture(scope="module")
def sampler():
    handle = hip_sampler.HipSampler(ROWS, VOCAB, testing=True)
    yield handle
    handle.close()


def _rows(seed, spread=2.0):
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((ROWS, VOCAB)) * spread).astype(np.float32)
    params = hip_sampler.make_params(ROWS, 1.0, 0, 1.0, 0.0)
    params["temperature"] = np.linspace(0.05, 1.5, ROWS).astype(np.float32)
    return rng, logits, params


def _sample_both_ways(sampler, logits, params, uniforms, context):
    """The oracle's results, from the partial sort and from the whole sort; returns the partial sort's results and
    how many elements of each row it sorted in the end."""
    _announce(context)
    sampler.upload_logits(logits)
    partial = sampler.sample(params, uniforms, None)
    lengths = sampler.sort_lengths(ROWS)
    sampler.partial_sort(False)
    try:
        whole = sampler.sample(params, uniforms, None)
    finally:
        sampler.partial_sort(True)
    cpu = parity_util.run_oracle(logits, params, uniforms)
    parity_util.assert_results_match(partial, cpu, "f32", context)
    assert partial.tobytes() == whole.tobytes(), context
    return partial, lengths


def test_rows_are_sorted_as_far_as_their_terms_matter(sampler):
    """Temperatures from 0.05 to 1.5 over N(0, 4) logits: the cold rows are sorted a few thousand elements deep, the
    warm ones whole; Top-P and Min-P cuts on some rows, a wide Top-K on others."""
    rng, logits, params = _rows(4100)
    params["top_p"] = np.where(np.arange(ROWS) % 3 == 0, 1.0, rng.uniform(0.5, 0.999, size=ROWS)).astype(np.float32)
    params["min_p"] = np.where(np.arange(ROWS) % 4 == 1, rng.uniform(0.0, 0.05, size=ROWS), 0.0).astype(np.float32)
    params["top_k"][6::9] = 3000  # wider than the select kernels take, narrower than some rows' sorted part
    for trial in range(3):
        uniforms = rng.random(ROWS, dtype=np.float32)
        gpu, lengths = _sample_both_ways(sampler, logits, params, uniforms, "partial sort, draw %d" % trial)
        assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
    shortened = lengths < VOCAB
    assert shortened[:ROWS // 3].all(), lengths        # cold rows: a small part
    assert (lengths[:ROWS // 4] < VOCAB // 4).all(), lengths
    assert (lengths[-3:] > VOCAB - 16).all(), lengths  # T around 1.5 over N(0, 4): every term matters, but for the last few
    assert (lengths[shortened] >= 4096).all(), lengths


def test_rows_whose_guess_is_too_short_are_sorted_whole(sampler):
    """A draw that no partial sum exceeds takes the row's last element, and a Min-P threshold below every term
    keeps the whole row: neither can be served from the sorted part, and the rows come back from the second
    launch."""
    rng, logits, params = _rows(4200)
    ordinary = rng.random(ROWS, dtype=np.float32)
    _, lengths_before = _sample_both_ways(sampler, logits, params, ordinary, "partial sort, ordinary draws")
    shortened = lengths_before < VOCAB
    assert shortened.sum() >= ROWS // 2
    # the largest uniform below one: the renormalised probabilities of about half the rows add up to no more
    last = np.full(ROWS, np.float32(1.0) - np.float32(2.0 ** -24), dtype=np.float32)
    gpu, lengths = _sample_both_ways(sampler, logits, params, last, "partial sort, draws at the top of [0, 1)")
    sent_back = shortened & (lengths == hip_sampler.SORT_WHOLE_ROW)
    assert sent_back.any(), lengths
    assert (gpu["kept_count"][sent_back] == VOCAB).all()
    # a Min-P threshold far below the smallest probability
    params["min_p"] = np.float32(1e-30)
    _, lengths = _sample_both_ways(sampler, logits, params, ordinary, "partial sort, Min-P below every probability")
    # (but for the coldest rows, whose smallest terms are zero and stay below any threshold)
    assert (lengths[shortened][-5:] == hip_sampler.SORT_WHOLE_ROW).all(), lengths


def test_rows_with_logits_that_are_not_finite(sampler):
    """-inf and NaN lie behind the sorted part of a row (they are counted, and NaN is flagged); +inf rejects the
    row; a row of few finite logits is sorted whole."""
    rng, logits, params = _rows(4300)
    params["temperature"] = np.float32(0.4)
    logits[0, 100:5000] = -np.inf
    logits[1, ::7] = np.nan
    logits[2, 17] = np.inf
    logits[3, :] = -np.inf
    logits[3, 5:2000] = rng.standard_normal(1995).astype(np.float32)
    logits[4, 9::2] = np.nan
    logits[4, 8::2] = -np.inf
    logits[5, :] = -np.inf
    logits[6, :] = np.nan
    params["top_p"][7:] = rng.uniform(0.7, 1.0, size=ROWS - 7).astype(np.float32)
    uniforms = rng.random(ROWS, dtype=np.float32)
    gpu, lengths = _sample_both_ways(sampler, logits, params, uniforms, "partial sort, infinities and NaN")
    assert gpu["status"][2] != 0 and gpu["status"][5] != 0 and gpu["status"][6] != 0
    assert lengths[0] < VOCAB and lengths[1] < VOCAB
    assert (gpu["flags"][1] & hip_sampler.FLAG_HAS_NAN) != 0


def test_heavy_ties_and_narrow_rows(sampler):
    """Rows of a few dozen distinct values (a bucket of the guess holds thousands of equal keys), rows whose logits
    all lie in one bucket, and rows at a temperature so low that the sorted part is the minimum."""
    rng, logits, params = _rows(4400)
    logits[0:8] = np.round(logits[0:8])
    logits[8:12] = (1.0 + rng.random((4, VOCAB)) * 0.05).astype(np.float32)  # one bucket holds the row
    logits[12:16] = (rng.integers(0, 3, size=(4, VOCAB)) * 8.0).astype(np.float32)
    params["temperature"][16:20] = np.float32(0.01)
    params["top_p"] = rng.uniform(0.6, 1.0, size=ROWS).astype(np.float32)
    for trial in range(2):
        uniforms = rng.random(ROWS, dtype=np.float32)
        _sample_both_ways(sampler, logits, params, uniforms, "partial sort, ties and narrow rows, draw %d" % trial)


def _sample_with_three_passes_and_four(sampler, logits, params, uniforms, context):
    """The oracle's results from the sort in three passes (with the lowest byte put in order on the way to the
    terms) and from the sort in four; returns the former's results and which rows it handed to the second launch."""
    _announce(context)
    sampler.upload_logits(logits)
    three = sampler.sample(params, uniforms, None)
    disordered = sampler.disordered_rows(ROWS)
    sampler.skip_low_digit(False)
    try:
        four = sampler.sample(params, uniforms, None)
    finally:
        sampler.skip_low_digit(True)
    cpu = parity_util.run_oracle(logits, params, uniforms)
    parity_util.assert_results_match(three, cpu, "f32", context)
    assert three.tobytes() == four.tobytes(), context
    return three, disordered


def test_three_passes_leave_the_lowest_byte_to_the_terms_kernel(sampler):
    """Logits spread over the floats: keys that agree in their upper 24 bits are one to three neighbours, which the
    terms kernel orders; no row goes to the second launch for it.  Cold rows (sorted in part) and warm ones (whole)."""
    rng, logits, params = _rows(4500)
    params["top_p"] = rng.uniform(0.5, 1.0, size=ROWS).astype(np.float32)
    logits[5] = (4.0 + rng.random(VOCAB) * 4.0).astype(np.float32)  # every 256 floats of [4, 8) hold two of these
    logits[6] = (2.0 + rng.random(VOCAB)).astype(np.float32)        # ... and of [2, 3) four
    params["temperature"][5:7] = np.float32(1.0)
    for trial in range(2):
        uniforms = rng.random(ROWS, dtype=np.float32)
        gpu, disordered = _sample_with_three_passes_and_four(sampler, logits, params, uniforms, "three passes, draw %d" % trial)
        assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()
        assert not disordered.any(), np.nonzero(disordered)[0]


def _grouped_row(rng, group, vocab=VOCAB):
    """A row of positive logits in groups of `group` keys that share their upper 24 bits and differ in the lowest byte
    (drawn without replacement where 256 values allow it), in random places of the row."""
    groups = (vocab + group - 1) // group
    cells = rng.choice(np.arange(0x3F8000, 0x410000, dtype=np.uint32), size=groups, replace=False)  # floats in [1, 8)
    low = np.concatenate([rng.permutation(256)[:group] if group <= 256 else rng.integers(0, 256, size=group) for _ in range(groups)])
    bits = (np.repeat(cells, group).astype(np.uint32) << np.uint32(8)) | low.astype(np.uint32)
    return rng.permutation(bits[:vocab]).view(np.float32)


def test_groups_of_keys_that_differ_in_the_lowest_byte_only(sampler):
    """Groups of up to 16 such keys are within the terms kernel's reach and come out in order; longer ones that are
    not in order send the row to the second launch; long runs of equal keys (and a row of few distinct values)
    are in order as they are."""
    rng, logits, params = _rows(4600)
    params["temperature"] = np.float32(1.0)
    params["top_p"] = rng.uniform(0.3, 1.0, size=ROWS).astype(np.float32)
    sizes = {0: 2, 1: 3, 2: 7, 3: 15, 4: 16, 5: 17, 6: 18, 7: 31, 8: 33, 9: 64, 10: 300, 11: 5000}
    for row, group in sizes.items():
        logits[row] = _grouped_row(rng, group)
    logits[12] = np.round(logits[12] * 2) / 2                     # a few dozen values, thousands of times each
    logits[13, 1000:40000] = np.float32(1.25)                     # a padded stretch of equal logits among spread ones
    logits[14] = _grouped_row(rng, 40)
    logits[14] = -np.sort(-logits[14])                            # long groups, in order already (descending logits)
    # logits that were rounded to bf16 on their way (an LM head in bf16, its output widened): every key ends in the same bytes
    logits[15] = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(logits[15]))
    for trial in range(2):
        uniforms = rng.random(ROWS, dtype=np.float32)
        _, disordered = _sample_with_three_passes_and_four(sampler, logits, params, uniforms, "groups in the lowest byte, draw %d" % trial)
        expected = np.zeros(ROWS, dtype=bool)
        expected[[row for row, group in sizes.items() if group > 16]] = True
        assert (disordered.astype(bool) == expected).all(), (np.nonzero(disordered)[0], np.nonzero(expected)[0])


def test_parts_of_several_tiles():
    """Rows longer than sixteen tiles: a part of the spread sort holds several tiles (three here), and the row's
    cut, its three passes and the touch-up of the lowest byte work across them."""
    rows, vocab = 6, 300007
    rng = np.random.default_rng(4800)
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["temperature"] = np.array([0.3, 0.6, 0.9, 1.1, 1.3, 1.5], dtype=np.float32)
    params["top_p"] = np.array([0.9, 0.95, 0.99, 1.0, 0.8, 0.999], dtype=np.float32)
    with hip_sampler.HipSampler(rows, vocab, testing=True) as handle:
        for trial in range(2):
            uniforms = rng.random(rows, dtype=np.float32)
            _announce("parts of three tiles, %d x %d, draw %d" % (rows, vocab, trial))
            handle.upload_logits(logits)
            gpu = handle.sample(params, uniforms, None)
            assert not handle.disordered_rows(rows).any()
            cpu = parity_util.run_oracle(logits, params, uniforms)
            parity_util.assert_results_match(gpu, cpu, "f32", "parts of three tiles, draw %d" % trial)
            assert (gpu["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()


@pytest.mark.parametrize("vocab", [24577, 32768, 32769, 65543, 131072, 131073, 200003])
def test_row_lengths_around_the_tiles_and_parts_of_the_sort(vocab):
    """Rows that end at, just behind and just in front of a tile of the spread sort (8,192 keys) and of the terms
    kernel (2,048), and rows of one tile and of two tiles per part: the cut, the three passes and the touch-up of
    the lowest byte at the row's end, against the oracle and the four-pass sort."""
    rows = 5
    rng = np.random.default_rng(4900 + vocab)
    logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    logits[3] = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(logits[3]))
    logits[4, -3000:] = logits[4, -1]  # a run of equal logits at the row's end (in index order)
    params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
    params["temperature"] = np.array([0.2, 0.7, 1.2, 1.0, 1.5], dtype=np.float32)
    params["top_p"] = np.array([0.9, 0.97, 1.0, 0.95, 0.999], dtype=np.float32)
    with hip_sampler.HipSampler(rows, vocab, testing=True) as handle:
        handle.upload_logits(logits)
        for trial in range(2):
            uniforms = rng.random(rows, dtype=np.float32)
            _announce("rows of %d logits, draw %d" % (vocab, trial))
            three = handle.sample(params, uniforms, None)
            # (row 4 may go to the second launch: a spread logit that shares its upper 24 bits with the run's value and
            # has a larger lowest byte would have to cross the whole run)
            assert not handle.disordered_rows(rows)[:4].any()
            handle.skip_low_digit(False)
            try:
                four = handle.sample(params, uniforms, None)
            finally:
                handle.skip_low_digit(True)
            cpu = parity_util.run_oracle(logits, params, uniforms)
            parity_util.assert_results_match(three, cpu, "f32", "rows of %d logits, draw %d" % (vocab, trial))
            assert three.tobytes() == four.tobytes()
            assert (three["flags"] & hip_sampler.FLAG_GENERAL_PATH != 0).all()


def test_random_rows_three_passes_and_four():
    """Thirty random batches (row length, spread, offset, quantisation, infinities, options drawn at random): the
    three-pass sort against the oracle and, byte for byte, against the four-pass sort."""
    rng = np.random.default_rng(5000)
    for case in range(30):
        rows = int(rng.integers(1, 9))
        vocab = int(rng.integers(24577, 150000))
        spread = float(rng.choice([0.05, 0.5, 2.0, 6.0]))
        logits = (rng.standard_normal((rows, vocab)) * spread + float(rng.choice([0.0, -30.0, 100.0]))).astype(np.float32)
        kind = case % 5
        if kind == 1:
            logits = np.round(logits * 8) / 8                              # few distinct values
        elif kind == 2:
            logits = workloads.bf16_bits_to_float32(workloads.float32_to_bf16_bits(logits))
        elif kind == 3:
            logits[:, rng.integers(0, vocab, vocab // 3)] = -np.inf
            logits[0, rng.integers(0, vocab, 3)] = np.nan
        elif kind == 4:
            logits[:, vocab // 2:] = logits[:, :1]                         # half of every row one value
        params = hip_sampler.make_params(rows, 1.0, 0, 1.0, 0.0)
        params["temperature"] = rng.choice(np.array([0.1, 0.5, 0.9, 1.3, 2.0], dtype=np.float32), size=rows)
        params["top_p"] = rng.choice(np.array([0.3, 0.9, 0.99, 1.0], dtype=np.float32), size=rows)
        params["min_p"] = rng.choice(np.array([0.0, 0.0, 0.01], dtype=np.float32), size=rows)
        params["top_k"] = rng.choice(np.array([0, 0, 2000, 70000], dtype=np.uint32), size=rows)
        uniforms = rng.random(rows, dtype=np.float32)
        context = "random case %d: %d x %d, spread %.2f, kind %d" % (case, rows, vocab, spread, kind)
        _announce(context)
        with hip_sampler.HipSampler(rows, vocab, testing=True) as handle:
            handle.upload_logits(logits)
            three = handle.sample(params, uniforms, None)
            handle.skip_low_digit(False)
            four = handle.sample(params, uniforms, None)
        cpu = parity_util.run_oracle(logits, params, uniforms)
        parity_util.assert_results_match(three, cpu, "f32", context)
        assert three.tobytes() == four.tobytes(), context


def test_rows_that_a_select_hands_on_beside_listed_rows():
    """The rows of the partial sort are listed, cut and counted by their options while the first select is still
    running.  A row with a Top-K window whose select kernel cannot finish it (hundreds or thousands of equal logits at
    the window's edge, more than its list holds) is pending afterwards and in no list: the walk leaves it to the
    second launch, which sorts it whole.  Rows of every kind in one call, 300 rows (whole-row select) and 40 (split)."""
    rng = np.random.default_rng(8128)
    vocab = 129280
    for rows in (300, 40):
        logits = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
        kind = np.arange(rows) % 5   # 0, 1: no window (listed) | 2: window 20 | 3: window 1000 | 4: window 50 with ties
        logits[kind == 4] = np.round(logits[kind == 4] / 2.0) * 2.0  # hundreds of equal logits at the window's edge
        logits[3::10] = np.round(logits[3::10] * 2.0) / 2.0        # ... also for half of the wide windows
        params = hip_sampler.make_params(rows, 1.0, 0, 0.95, 0.0)
        params["temperature"] = rng.uniform(0.3, 1.4, size=rows).astype(np.float32)
        params["top_k"] = np.array([0, 0, 20, 1000, 50], dtype=np.uint32)[kind]
        uniforms = rng.random(rows, dtype=np.float32)
        context = "rows handed on beside listed rows, %d rows" % rows
        _announce(context)
        with hip_sampler.HipSampler(rows, vocab, testing=True) as handle:
            handle.upload_logits(logits)
            early = handle.sample(params, uniforms, None)
            flagged = handle.disordered_rows(rows)
            again = handle.sample(params, uniforms, None)
        cpu = parity_util.run_oracle(logits, params, uniforms)
        parity_util.assert_results_match(early, cpu, "f32", context)
        assert early.tobytes() == again.tobytes(), context
        general = (early["flags"] & hip_sampler.FLAG_GENERAL_PATH) != 0
        assert general[kind <= 1].all() and general[kind == 4].all(), context      # listed rows and rows handed on
        assert not general[kind == 2].any(), context
        assert not flagged[kind >= 2].any(), context                               # (the hook names disordered rows only)
