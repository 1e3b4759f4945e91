#!/usr/bin/env python3
"""Writes tests/golden/router_golden.npz from the REFERENCE library (oracle/_ref/libref_sampler.so).

Run in the build container only, where the reference checkout exists:

    make -C oracle && python tests/golden/make_golden_router.py

The file holds inputs and expected outputs only (data, no reference code): router logits, options,
selection bias and explicit expert ids of seeded cases, and what the reference's own
ExpertDispatcher::dispatch (src/graph/expert_dispatcher.cpp:76-157) returned for them: the return
code, the per-expert offsets and the routes (token, rank, weight) in plan order.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402

CASES = 96
MAX_TOKENS = 8
MAX_EXPERTS = 256
MAX_TOP_K = 16


def main():
    if not ol.reference_available():
        sys.exit("the reference library is not built: run `make -C oracle` where /root/reference exists")
    rng = np.random.default_rng(626262)
    logits = np.zeros((CASES, MAX_TOKENS, MAX_EXPERTS), dtype=np.float32)
    bias = np.zeros((CASES, MAX_EXPERTS), dtype=np.float32)
    explicit = np.zeros((CASES, MAX_TOKENS * MAX_TOP_K), dtype=np.uint32)
    # tokens, experts, top_k, score function, normalization, flags, has bias, has explicit ids
    shape = np.zeros((CASES, 8), dtype=np.uint32)
    scaling = np.zeros(CASES, dtype=np.float32)
    rc = np.zeros(CASES, dtype=np.int32)
    offsets = np.zeros((CASES, MAX_EXPERTS + 1), dtype=np.uint32)
    route_tokens = np.zeros((CASES, MAX_TOKENS * MAX_TOP_K), dtype=np.uint32)
    route_ranks = np.zeros_like(route_tokens)
    route_weights = np.zeros((CASES, MAX_TOKENS * MAX_TOP_K), dtype=np.float32)
    for case in range(CASES):
        tokens = int(rng.integers(1, MAX_TOKENS + 1))
        experts = int(rng.choice([1, 4, 8, 60, 64, 128, 160, 256]))
        top_k = int(min(experts, rng.choice([1, 2, 4, 6, 8, 16])))
        score = int(rng.integers(0, 3))
        normalization = int(rng.integers(0, 2))  # ExpertWeightNormalization: None, SelectedExperts
        flags = int(rng.integers(0, 2))          # bit 0: ExpertDispatchNormalizeTopKWeights
        values = (rng.standard_normal((tokens, experts)) * rng.choice([0.5, 2.0, 10.0, 40.0])).astype(np.float32)
        if case % 6 == 0:
            values = np.round(values)  # ties
        if case % 23 == 5:
            values[tokens - 1, experts // 2] = (np.nan, np.inf)[case % 2]
        if case % 29 == 11:
            score, normalization = 1, 1
            values[0, :] = -200.0  # sigmoid scores of exactly zero: a non-positive selected sum
        has_bias = case % 3 == 1
        has_explicit = case % 4 == 2
        if has_bias:
            bias[case, :experts] = (rng.standard_normal(experts) * 0.5).astype(np.float32)
        if has_explicit:
            ids = rng.integers(0, experts, size=tokens * top_k).astype(np.uint32)
            if case % 20 == 10:
                ids[-1] = experts  # out of range
            explicit[case, :ids.size] = ids
        scaling[case] = np.float32(rng.choice([1.0, 2.5, 0.125, 16.0]))
        if case % 31 == 7:
            scaling[case] = 0.0
        logits[case, :tokens, :experts] = values
        shape[case] = (tokens, experts, top_k, score, normalization, flags, has_bias, has_explicit)
        rc[case], case_offsets, routes, _ = ol.reference_router_dispatch(
            values, top_k, score, normalization, flags, float(scaling[case]),
            bias[case, :experts] if has_bias else None,
            explicit[case, :tokens * top_k] if has_explicit else None)
        if rc[case] == 0:
            offsets[case, :experts + 1] = case_offsets
            route_tokens[case, :routes.size] = routes["token_index"]
            route_ranks[case, :routes.size] = routes["rank"]
            route_weights[case, :routes.size] = routes["weight"]
    path = os.path.join(HERE, "router_golden.npz")
    np.savez_compressed(path, logits=logits, bias=bias, explicit=explicit, shape=shape, scaling=scaling, rc=rc,
                        offsets=offsets, route_tokens=route_tokens, route_ranks=route_ranks, route_weights=route_weights)
    print("wrote %s: %d cases, %d dispatched, %d bytes" % (path, CASES, int((rc == 0).sum()), os.path.getsize(path)))
    print("return codes:", dict(zip(*np.unique(rc, return_counts=True))))


if __name__ == "__main__":
    main()
