"""Seeded synthetic workloads: the five benchmark configurations of the generation sampler.

Every array is produced on the host from numpy's PCG64 streams with fixed seeds, so the CPU oracle
and the GPU sampler see identical logits, per-row parameters, uniforms and stop ids.  bf16 logits
are returned as uint16 bit patterns, rounded to nearest even from fp32.
"""
import numpy as np

PARAMS_DTYPE = np.dtype([("temperature", "<f4"), ("top_k", "<u4"), ("top_p", "<f4"),
                         ("min_p", "<f4"), ("stop_begin", "<u4"), ("stop_count", "<u4")])

CONFIGS = {
    # name: (rows, vocab, dtype)
    "cfg1_plumbing": (1, 32000, "f32"),
    "cfg2_topk_topp": (64, 151936, "f32"),
    "cfg3_full_nucleus": (256, 201088, "bf16"),
    "cfg4_service_mix": (512, 129280, "f32"),
    "cfg5_tie_stress": (1024, 262144, "bf16"),
}


def float32_to_bf16_bits(values):
    """Round to nearest even, as float_to_bfloat16 does: (bits + 0x7fff + lsb) >> 16."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounding = np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    return ((bits + rounding) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_float32(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def _uniforms(rows, seed):
    # 24 random bits per draw -> float32 in [0, 1)
    rng = np.random.Generator(np.random.PCG64(seed + 7919))
    return (rng.integers(0, 1 << 24, size=rows, dtype=np.uint32).astype(np.float32) * np.float32(2.0 ** -24))


def _params(rows, temperature, top_k, top_p, min_p):
    params = np.zeros(rows, dtype=PARAMS_DTYPE)
    params["temperature"] = temperature
    params["top_k"] = top_k
    params["top_p"] = top_p
    params["min_p"] = min_p
    return params


def make_workload(name, rows=None, seed=2024, vocab=None):
    """Returns a dict: logits [rows, vocab] (float32, or uint16 bf16 bits), dtype ("f32"/"bf16"),
    params, uniforms, stop_ids (or None), rows, vocab, description."""
    base_rows, base_vocab, dtype = CONFIGS[name]
    rows = base_rows if rows is None else rows
    vocab = base_vocab if vocab is None else vocab
    rng = np.random.Generator(np.random.PCG64(seed))
    stop_ids = None
    if name == "cfg1_plumbing":
        logits = (rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(2.5))
        params = _params(rows, 0.8, 50, 0.9, 0.0)
        description = "B=%d V=%d fp32 N(0,2.5^2); T 0.8, Top-K 50, Top-P 0.9" % (rows, vocab)
    elif name == "cfg2_topk_topp":
        logits = (rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(3.0))
        for row in range(rows):
            spikes = rng.choice(vocab, size=8, replace=False)
            logits[row, spikes] += np.float32(12.0)
        params = _params(rows, 0.7, 20, 0.8, 0.0)
        description = "B=%d V=%d fp32 N(0,3^2)+8 spikes at +12; T 0.7, Top-K 20, Top-P 0.8" % (rows, vocab)
    elif name == "cfg3_full_nucleus":
        logits = np.empty((rows, vocab), dtype=np.uint16)
        for row in range(rows):
            mix = rng.gumbel(0.0, 1.0, size=vocab).astype(np.float32) + rng.standard_normal(vocab, dtype=np.float32)
            logits[row] = float32_to_bf16_bits(mix)
        params = _params(rows, 1.0, 0, 0.95, 0.0)
        description = "B=%d V=%d bf16 Gumbel(0,1)+N(0,1); T 1.0, no Top-K, Top-P 0.95" % (rows, vocab)
    elif name == "cfg4_service_mix":
        logits = (rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(2.0))
        temperature = rng.uniform(0.0, 1.5, size=rows).astype(np.float32)
        temperature[rng.random(rows) < 0.10] = 0.0
        top_k = rng.choice(np.array([0, 1, 20, 50, 1000], dtype=np.uint32), size=rows)
        top_p = rng.uniform(0.5, 1.0, size=rows).astype(np.float32)
        min_p = rng.uniform(0.0, 0.1, size=rows).astype(np.float32)
        params = _params(rows, temperature, top_k, top_p, min_p)
        # four stop ids per row: three random ids plus, on every other row, the row's best token
        stop_ids = rng.integers(0, vocab, size=(rows, 4), dtype=np.int64).astype(np.int32)
        best = np.argmax(logits, axis=1).astype(np.int32)
        stop_ids[::2, 3] = best[::2]
        params["stop_begin"] = np.arange(rows, dtype=np.uint32) * 4
        params["stop_count"] = 4
        stop_ids = stop_ids.reshape(-1)
        description = ("B=%d V=%d fp32 N(0,2^2); per-row T U[0,1.5] (10%% greedy), Top-K {0,1,20,50,1000}, "
                       "Top-P U[0.5,1], Min-P U[0,0.1], 4 stop ids per row" % (rows, vocab))
    elif name == "cfg5_tie_stress":
        logits = np.empty((rows, vocab), dtype=np.uint16)
        for row in range(rows):
            logits[row] = float32_to_bf16_bits(rng.standard_normal(vocab, dtype=np.float32) * np.float32(1.5))
        params = _params(rows, 0.6, 64, 0.9, 0.02)
        description = "B=%d V=%d N(0,1.5^2) quantised to bf16; T 0.6, Top-K 64, Top-P 0.9, Min-P 0.02" % (rows, vocab)
    else:
        raise KeyError(name)
    return {
        "name": name, "rows": rows, "vocab": vocab, "dtype": dtype, "logits": logits, "params": params,
        "uniforms": _uniforms(rows, seed), "stop_ids": stop_ids, "description": description,
    }


def synthetic_model_logits(vocab, session, position, fed_token):
    """Logits of the stand-in model that the generation-loop test program uses (synthetic_logits in
    tests/cpp/test_session_sampler.cpp): an integer hash of (session, position, token fed), every value
    a multiple of 2^-20 in [-8, 14), so that C++ and numpy produce the same fp32 rows."""
    mask = 0xFFFFFFFF
    seed = ((session * 0x9E3779B1) ^ (position * 0x85EBCA77) ^ ((fed_token & mask) * 0xC2B2AE3D) ^ 0x27D4EB2F) & mask
    h = (np.arange(vocab, dtype=np.uint64) * 2654435761 + seed) & mask
    h ^= h >> np.uint64(15)
    h = (h * 2246822519) & mask
    h ^= h >> np.uint64(13)
    h = (h * 3266489917) & mask
    h ^= h >> np.uint64(16)
    values = (h >> np.uint64(8)).astype(np.float32) * np.float32(1.0 / 1048576.0) - np.float32(8.0)
    values[(h & np.uint64(1023)) == 0] += np.float32(6.0)
    return values.astype(np.float32)
