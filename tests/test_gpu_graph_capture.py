"""The device entries enqueue kernels only (no allocation, no copy, no memset), so a caller can record them
into a HIP graph: ncnn_moe_hip_sampler_sample_device and ncnn_moe_hip_router_dispatch_device are captured
through the C ABI on a torch stream and replayed several times, with new inputs copied into the same
buffers and eager work between the replays; every replay is checked against the CPU oracle."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import oracle_lib
import parity_util
from ncnn_moe_runtime_amd import hip_router, hip_sampler

pytestmark = pytest.mark.gpu


def _bytes(array):
    return torch.from_numpy(np.ascontiguousarray(array).view(np.uint8).reshape(-1))


@pytest.mark.parametrize("passes", [hip_sampler.PASSES_FULL_ORDER, hip_sampler.PASSES_FULL_ORDER | hip_sampler.PASSES_SIDE_BY_SIDE])
def test_sampler_step_in_a_graph(passes):
    """Every pass in one captured call; with the side-by-side flag the handle's second stream forks from
    and joins the captured stream, so the graph holds two branches."""
    print("[case] sample_device captured in a HIP graph (passes %d), 4 replays" % passes, flush=True)
    rng = np.random.default_rng(31)
    rows, vocab = 48, 40013
    params = hip_sampler.make_params(rows, 0.8, 0, 0.9, 0.0)
    params["top_k"] = np.array([(1, 20, 64, 300, 0, 1000)[i % 6] for i in range(rows)], dtype=np.uint32)
    params["temperature"][::7] = 0.0
    device = torch.device("cuda:0")
    d_logits = torch.zeros(rows * vocab, dtype=torch.float32, device=device)
    d_params = _bytes(params).to(device)
    d_uniforms = torch.zeros(rows, dtype=torch.float32, device=device)
    d_results = torch.zeros(rows * 16, dtype=torch.uint8, device=device)
    stream = torch.cuda.Stream(device=device)
    with hip_sampler.HipSampler(rows, vocab) as sampler:
        def enqueue():
            sampler.sample_device(d_logits.data_ptr(), hip_sampler.LOGITS_F32, rows, vocab, vocab, d_params.data_ptr(),
                                  d_uniforms.data_ptr(), None, d_results.data_ptr(), passes, stream.cuda_stream)

        with torch.cuda.stream(stream):
            enqueue()  # eager once: everything the entry sets up lazily exists before the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            enqueue()
        for replay in range(4):
            logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
            if replay == 2:
                logits[5, :] = 1.0  # every logit tied: this row takes the full-order kernels inside the graph
            uniforms = rng.random(rows).astype(np.float32)
            d_logits.copy_(torch.from_numpy(logits).reshape(-1))   # eager work between the replays
            d_uniforms.copy_(torch.from_numpy(uniforms))
            d_results.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            gpu = d_results.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows)
            cpu = parity_util.run_oracle(logits, params, uniforms)
            parity_util.assert_results_match(gpu, cpu, "f32", "graph replay %d" % replay)


def test_router_dispatch_in_a_graph():
    print("[case] router dispatch_device captured in a HIP graph, 4 replays", flush=True)
    rng = np.random.default_rng(32)
    device = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=device)
    for tokens, experts, top_k in [(200, 128, 8), (1000, 256, 6)]:   # one launch (fused), and two
        options = hip_router.make_options(experts, top_k, hip_router.SOFTMAX, True, 1.5)
        d_logits = torch.zeros(tokens * experts, dtype=torch.float32, device=device)
        d_offsets = torch.zeros(experts + 1, dtype=torch.int32, device=device)
        d_routes = torch.zeros(tokens * top_k * 3, dtype=torch.int32, device=device)
        d_status = torch.zeros(1, dtype=torch.int32, device=device)
        router = hip_router.HipRouter(tokens, experts, top_k)
        try:
            def enqueue():
                host_status = router.dispatch_device(d_logits.data_ptr(), tokens, options, d_offsets.data_ptr(),
                                                     d_routes.data_ptr(), d_status.data_ptr(), stream=stream.cuda_stream)
                assert host_status == 0

            with torch.cuda.stream(stream):
                enqueue()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                enqueue()
            for replay in range(4):
                logits = (rng.standard_normal((tokens, experts)) * 2).astype(np.float32)
                if replay == 1:
                    logits[tokens // 2, 3] = np.nan   # a failing call inside the graph, then good ones again
                d_logits.copy_(torch.from_numpy(logits).reshape(-1))
                d_routes.zero_()
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                cpu_status, cpu_offsets, cpu_routes = oracle_lib.oracle_router_dispatch(
                    logits, top_k, score_function=hip_router.SOFTMAX, routed_scaling_factor=1.5)
                assert int(d_status.item()) == cpu_status, (tokens, replay)
                if cpu_status != 0:
                    continue
                assert np.array_equal(d_offsets.cpu().numpy().view(np.uint32), cpu_offsets)
                got = d_routes.cpu().numpy().view(np.uint32).reshape(-1, 3)
                assert np.array_equal(got[:, 0], cpu_routes["token_index"]) and np.array_equal(got[:, 1], cpu_routes["rank"])
                assert np.array_equal(got[:, 2], cpu_routes["weight"].view(np.uint32))
        finally:
            router.close()
