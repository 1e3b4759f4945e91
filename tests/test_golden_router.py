"""The router oracle against vectors recorded from the reference's own ExpertDispatcher::dispatch
(tests/golden/router_golden.npz, written by tests/golden/make_golden_router.py where the reference
builds).  Runs wherever the repository is."""
import os

import numpy as np
import pytest

import oracle_lib as ol

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "router_golden.npz")
# 1 + ErrorCode (include/ncnn/moe/result.h:12-19): InvalidArgument = 0, InvalidModel = 2
REF_CODE_OF_STATUS = {0: 0, 1: 1, 2: 1, 3: 1, 4: 1, 5: 1, 6: 3}


def golden_cases():
    golden = np.load(GOLDEN)
    for case in range(golden["rc"].size):
        tokens, experts, top_k, score, normalization, flags, has_bias, has_explicit = (int(v) for v in golden["shape"][case])
        yield dict(
            case=case, logits=golden["logits"][case, :tokens, :experts].copy(), top_k=top_k, score_function=score,
            renormalize=bool(normalization == 1 or (flags & 1)), routed_scaling_factor=float(golden["scaling"][case]),
            selection_bias=golden["bias"][case, :experts].copy() if has_bias else None,
            explicit_expert_ids=golden["explicit"][case, :tokens * top_k].copy() if has_explicit else None,
            rc=int(golden["rc"][case]), offsets=golden["offsets"][case, :experts + 1],
            route_tokens=golden["route_tokens"][case, :tokens * top_k], route_ranks=golden["route_ranks"][case, :tokens * top_k],
            route_weights=golden["route_weights"][case, :tokens * top_k])


def check_against_golden(dispatch, minimum_dispatched=80):
    dispatched = 0
    codes = set()
    for g in golden_cases():
        status, offsets, routes = dispatch(
            g["logits"], g["top_k"], score_function=g["score_function"], renormalize=g["renormalize"],
            routed_scaling_factor=g["routed_scaling_factor"], selection_bias=g["selection_bias"],
            explicit_expert_ids=g["explicit_expert_ids"])
        assert REF_CODE_OF_STATUS[status] == g["rc"], (g["case"], status, g["rc"])
        codes.add(status)
        if status != 0:
            continue
        dispatched += 1
        assert np.array_equal(offsets, g["offsets"]), g["case"]
        assert np.array_equal(routes["token_index"], g["route_tokens"]), g["case"]
        assert np.array_equal(routes["rank"], g["route_ranks"]), g["case"]
        assert np.array_equal(routes["weight"].view(np.uint32), g["route_weights"].view(np.uint32)), g["case"]
    assert dispatched >= minimum_dispatched
    return codes


def test_oracle_reproduces_the_recorded_plans():
    codes = check_against_golden(ol.oracle_router_dispatch)
    assert {0, 3, 4, 5, 6} <= codes  # scaling, non-finite logit, id out of range and zero sum are all recorded


@pytest.mark.gpu
def test_gpu_router_reproduces_the_recorded_plans():
    from ncnn_moe_runtime_amd import hip_router
    print("[case] router golden vectors", flush=True)
    router = hip_router.HipRouter(16)
    try:
        check_against_golden(router.dispatch)
    finally:
        router.close()
