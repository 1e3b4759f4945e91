#!/usr/bin/env python3
"""Benchmark of the MI355X generation sampler: sampled rows/s and HBM GB/s on the logits read.

A step is one pass of the sampler (ncnn_moe_hip_sampler_sample_device, every kernel of the path) over
one batch of synthetic logits that is already resident in HBM.  The workload is the headline
configuration: B=64, V=151,936 fp32 logits N(0, 3^2) with 8 spikes at +12 per row, temperature 0.7,
Top-K 20, Top-P 0.8.  Steps rotate over several distinct logits buffers whose total size exceeds the
256 MB Infinity Cache, so the logits come from HBM and not from a cache warmed by the previous step.

Prints ONE JSON line.  `roofline` prices the dominant kernel (the one HBM pass over the logits)
against the 8 TB/s HBM peak using the algorithmic bytes of a launch and the average step time
measured with HIP events on the launch stream.  `cpu_baseline` times the reference's own
Session::sample loop (oracle/_ref, kind "reference") or, where that library is absent, the CPU
oracle (kind "port") on the host cores, on the same rows.

--workload speculative_verify and --workload router_dispatch time the two other entry points (one
verification step of speculative generation; one expert dispatch of a MoE layer) in the same JSON
shape; they are not the headline metric.
"""
import argparse
import ctypes
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
PACKAGE_DIR = os.path.join(ROOT, "ncnn-moe-runtime_amd")
HBM_PEAK_BYTES_PER_S = 8.0e12


def load_package():
    if "ncnn_moe_runtime_amd" in sys.modules:
        return sys.modules["ncnn_moe_runtime_amd"]
    spec = importlib.util.spec_from_file_location(
        "ncnn_moe_runtime_amd", os.path.join(PACKAGE_DIR, "__init__.py"),
        submodule_search_locations=[PACKAGE_DIR])
    module = importlib.util.module_from_spec(spec)
    sys.modules["ncnn_moe_runtime_amd"] = module
    spec.loader.exec_module(module)
    return module


def algorithmic_bytes(rows, vocab, element_bytes):
    """Logits read once, parameters (24 B) and uniform (4 B) in, result (16 B) out, per row."""
    return rows * vocab * element_bytes + rows * (24 + 4) + rows * 16


def measured_traffic(workload_name):
    """HBM bytes per launch of the dominant kernel (per step of all the step's kernels, for a workload whose step is
    several) as measured with rocprofv3 --pmc FETCH_SIZE and
    WRITE_SIZE (each scaled by the reading of a 256 MiB copy), recorded beside the profile summaries:
    a stored figure from those counter runs, not something this run measures.  Returns (bytes, file)."""
    for name in ("%s_hbm_traffic.json" % workload_name, "split_select_%s_traffic.json" % workload_name):
        path = os.path.join(ROOT, "profiles", name)
        if os.path.exists(path):
            with open(path) as handle:
                return json.load(handle).get("hbm_bytes_per_launch"), "profiles/" + name
    return None, None


def host_description():
    """CPU model, physical cores and hardware threads of this host (from /proc/cpuinfo)."""
    model, cores, threads = "unknown", set(), 0
    try:
        physical = core = None
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                key, _, value = line.partition(":")
                key, value = key.strip(), value.strip()
                if key == "model name":
                    model = value
                elif key == "processor":
                    threads += 1
                elif key == "physical id":
                    physical = value
                elif key == "core id":
                    core = value
                elif not key and physical is not None and core is not None:
                    cores.add((physical, core))
                    physical = core = None
    except OSError:
        pass
    return {"cpu_model": model, "physical_cores": len(cores) if cores else None, "hardware_threads": threads or os.cpu_count()}


METRICS = {
    "cfg1_plumbing": "sampled rows/sec + HBM GB/s (% peak), B=1 V=32000 fp32 temp+topk+topp",
    "cfg2_topk_topp": "sampled rows/sec + HBM GB/s (% peak), B=64 V=151936 fp32 temp+topk+topp",
    "cfg3_full_nucleus": "sampled rows/sec + HBM GB/s (% peak), B=256 V=201088 bf16 full-vocabulary nucleus top_p 0.95",
    "cfg4_service_mix": "sampled rows/sec + HBM GB/s (% peak), B=512 V=129280 fp32 per-row mixed options + stop ids",
    "cfg5_tie_stress": "sampled rows/sec + HBM GB/s (% peak), B=1024 V=262144 bf16 temp+topk+topp+minp, tie-heavy",
}


def cpu_baseline(workload, host_threads, sample_rows):
    """Times the CPU sampler on the first sample_rows rows of the workload."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib

    rows = min(sample_rows, workload["rows"])
    logits = workload["logits"][:rows]
    params = workload["params"][:rows]
    uniforms = workload["uniforms"][:rows]
    fp32 = logits if workload["dtype"] == "f32" else oracle_lib.widen_bf16(logits)
    fp32 = np.ascontiguousarray(fp32, dtype=np.float32)

    if oracle_lib.reference_available():
        kind = "reference"
        sessions = [oracle_lib.ReferenceSession(seed) for seed in range(rows)]
        handles = (ctypes.c_void_p * rows)(*[s.handle for s in sessions])
        temperature = np.ascontiguousarray(params["temperature"])
        top_k = np.ascontiguousarray(params["top_k"])
        top_p = np.ascontiguousarray(params["top_p"])
        min_p = np.ascontiguousarray(params["min_p"])
        stop_begin = np.ascontiguousarray(params["stop_begin"])
        stop_count = np.ascontiguousarray(params["stop_count"])
        stops = workload["stop_ids"]
        tokens = np.zeros(rows, dtype=np.int32)
        probabilities = np.zeros(rows, dtype=np.float32)
        is_stop = np.zeros(rows, dtype=np.uint8)
        status = np.zeros(rows, dtype=np.int32)

        def run(threads):
            oracle_lib.reference().ref_sample_rows(
                handles, fp32.ctypes.data, rows, fp32.shape[1], fp32.shape[1],
                temperature.ctypes.data, top_k.ctypes.data, top_p.ctypes.data, min_p.ctypes.data,
                None if stops is None else stops.ctypes.data, stop_begin.ctypes.data, stop_count.ctypes.data,
                tokens.ctypes.data, probabilities.ctypes.data, is_stop.ctypes.data, status.ctypes.data, threads)
    else:
        kind = "port"

        def run(threads):
            oracle_lib.oracle_sample_batch(fp32, params, uniforms, workload["stop_ids"], threads=threads)

    def best_of(threads, repetitions):
        best = float("inf")
        for _ in range(repetitions):
            start = time.perf_counter()
            run(threads)
            best = min(best, time.perf_counter() - start)
        return best

    single = best_of(1, 2)
    multi = best_of(host_threads, 3) if host_threads > 1 else single
    host = host_description()
    return {
        "value": rows / multi,
        "unit": "rows/s",
        "cores": host_threads,
        "cpu_model": host["cpu_model"],
        "host_physical_cores": host["physical_cores"],
        "host_hardware_threads": host["hardware_threads"],
        "kind": kind,
        "sample": "%d rows of the benchmark batch, best of 3 passes on %d threads (one Session per row); "
                  "1 thread: %.1f rows/s" % (rows, host_threads, rows / single),
        "single_thread_value": rows / single,
    }


def bench_speculative_verify(args, hip_sampler):
    """One verification step of speculative generation per step: 2 D + 1 rows of V = 151,936 fp32 logits
    resident in the handle's buffer, the small operands and the result crossing PCIe as the host entry
    does.  Not the headline metric; printed in the same JSON shape."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib

    if hip_sampler.device_count() < 1:
        sys.exit("bench.py needs a GPU: no HIP device is visible")
    drafts, vocab = args.drafts, 151936
    options = dict(temperature=0.7, top_k=20, top_p=0.8, min_p=0.0)
    if args.dense_verify:
        # no Top-K window: the filtered distributions are longer than the verification's lists, and the step takes the
        # dense path (full-order kernels that export every row's distribution, the accept loop over dense rows)
        options = dict(temperature=1.0, top_k=0, top_p=0.95, min_p=0.0)
    options_text = "T %.1f, Top-K %d, Top-P %.2f" % (options["temperature"], options["top_k"], options["top_p"])
    rng = np.random.Generator(np.random.PCG64(77))
    target = (rng.standard_normal((drafts + 1, vocab), dtype=np.float32) * np.float32(3.0))
    draft = target[:drafts] + rng.standard_normal((drafts, vocab), dtype=np.float32) * np.float32(0.5)
    proposed = [int(oracle_lib.oracle_sample(row, 0.37, **options)["token_id"]) for row in draft]
    uniform_sets = [rng.random(drafts + 1, dtype=np.float32) for _ in range(64)]
    sampler = hip_sampler.HipSampler(2 * drafts + 1, vocab)
    sampler.upload_logits(np.concatenate([target, draft], axis=0))
    mismatches = 0
    accepted_total = 0
    for uniforms in uniform_sets[:16]:
        gpu, gpu_accepted = sampler.speculative_verify(proposed, uniforms, **options)
        cpu, cpu_accepted = oracle_lib.oracle_speculative_verify(target, draft, proposed, uniforms, **options)
        same = all(gpu[f] == cpu[f] for f in ("status", "accepted", "next_token_id", "accept_draws", "final_draw_consumed"))
        same = same and np.float32(gpu["next_probability"]).view(np.uint32) == np.float32(cpu["next_probability"]).view(np.uint32)
        same = same and np.array_equal(gpu_accepted[:cpu["accepted"]].view(np.uint32), cpu_accepted[:cpu["accepted"]].view(np.uint32))
        mismatches += 0 if same else 1
        accepted_total += int(cpu["accepted"])
    for index in range(args.warmup):
        sampler.speculative_verify(proposed, uniform_sets[index % 64], **options)
    start = time.perf_counter()
    for index in range(args.steps):
        sampler.speculative_verify(proposed, uniform_sets[index % 64], **options)
    seconds_per_step = (time.perf_counter() - start) / args.steps
    cpu_start = time.perf_counter()
    cpu_steps = 3
    for index in range(cpu_steps):
        oracle_lib.oracle_speculative_verify(target, draft, proposed, uniform_sets[index], **options)
    cpu_seconds = (time.perf_counter() - cpu_start) / cpu_steps
    bytes_per_step = (2 * drafts + 1) * vocab * 4
    line = {
        "metric": "speculative verification steps/sec, D=%d V=151936 fp32 %s" % (drafts, "full-vocabulary nucleus (dense path)" if args.dense_verify else "temp+topk+topp"),
        "value": 1.0 / seconds_per_step, "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": seconds_per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "speculative verification, %d drafted tokens, %d x %d fp32 logits resident in HBM; "
                               "%s" % (drafts, 2 * drafts + 1, vocab, options_text),
                   "entry_point": "ncnn_moe_hip_sampler_speculative_verify (host operands, synchronous)"},
        "roofline": {"bound": "hbm", "achieved": bytes_per_step / seconds_per_step / 1e9, "peak": HBM_PEAK_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": bytes_per_step / seconds_per_step / HBM_PEAK_BYTES_PER_S, "traffic": None,
                     "kernel": ("full-order kernels with exported distributions + speculative_verify_dense_kernel" if args.dense_verify
                                else "scan_select_kernel + speculative_verify_kernel") + ", wall clock of the synchronous call",
                     "algorithmic_bytes_per_launch": bytes_per_step},
        "parity": {"steps_checked": 16, "step_mismatches": mismatches, "mean_accepted": accepted_total / 16.0},
        "cpu_baseline": {"value": 1.0 / cpu_seconds, "unit": "steps/s", "cores": 1, "kind": "port",
                         "sample": "%d steps of the CPU oracle's verification (two full sorts per tested position)" % cpu_steps},
    }
    sampler.close()
    print(json.dumps(line))


def bench_router_dispatch(args):
    """One expert dispatch of a MoE layer per step (ExpertDispatcher::dispatch): --rows tokens (4096 by
    default, a prefill chunk) x 256 experts, Top-8, sqrt-softplus scores with a selection bias, scaling
    1.5, every array resident in HBM (ncnn_moe_hip_router_dispatch_device).  Not the headline metric;
    printed in the same JSON shape."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    from ncnn_moe_runtime_amd import hip_router

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: no HIP device is visible")
    tokens = args.rows if args.rows > 0 else 4096
    score_name = args.router_score
    experts, top_k, scaling = 256, 8, 1.5
    score = {"softmax": hip_router.SOFTMAX, "sigmoid": hip_router.SIGMOID, "sqrt_softplus": hip_router.SQRT_SOFTPLUS}[score_name]
    rng = np.random.Generator(np.random.PCG64(88))
    buffers = 16
    host_logits = [(rng.standard_normal((tokens, experts), dtype=np.float32) * np.float32(2.0)) for _ in range(buffers)]
    bias = (rng.standard_normal(experts, dtype=np.float32) * np.float32(0.1))
    device = torch.device("cuda:0")
    logits = [torch.from_numpy(values).to(device) for values in host_logits]
    device_bias = torch.from_numpy(bias).to(device)
    offsets = torch.zeros(experts + 1, dtype=torch.int32, device=device)
    routes = torch.zeros(tokens * top_k * 3, dtype=torch.int32, device=device)
    status = torch.zeros(1, dtype=torch.int32, device=device)
    options = hip_router.make_options(experts, top_k, score, True, scaling)
    router = hip_router.HipRouter(tokens, experts, top_k)
    stream = torch.cuda.current_stream()

    def step(index):
        host_status = router.dispatch_device(
            logits[index % buffers].data_ptr(), tokens, options, offsets.data_ptr(), routes.data_ptr(), status.data_ptr(),
            bias_pointer=device_bias.data_ptr(), stream=stream.cuda_stream)
        if host_status != 0:
            sys.exit("router dispatch rejected its arguments: status %d" % host_status)

    # parity of what is timed: every buffer against the oracle, bit for bit
    mismatches = 0
    cpu_seconds = []
    for index in range(buffers):
        step(index)
        torch.cuda.synchronize()
        start = time.perf_counter()
        cpu_status, cpu_offsets, cpu_routes = oracle_lib.oracle_router_dispatch(
            host_logits[index], top_k, score_function=score, routed_scaling_factor=scaling, selection_bias=bias)
        cpu_seconds.append(time.perf_counter() - start)
        got = routes.cpu().numpy().view(np.uint32).reshape(-1, 3)
        same = int(status.item()) == cpu_status == 0 and np.array_equal(offsets.cpu().numpy().view(np.uint32), cpu_offsets)
        same = same and np.array_equal(got[:, 0], cpu_routes["token_index"]) and np.array_equal(got[:, 1], cpu_routes["rank"])
        same = same and np.array_equal(got[:, 2], cpu_routes["weight"].view(np.uint32))
        mismatches += 0 if same else 1
    for index in range(args.warmup):
        step(index)
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start = time.perf_counter()
    begin.record(stream)
    for index in range(args.steps):
        step(index)
    end.record(stream)
    torch.cuda.synchronize()
    seconds_per_step = (time.perf_counter() - start) / args.steps
    device_seconds_per_step = begin.elapsed_time(end) * 1e-3 / args.steps
    bytes_per_step = tokens * experts * 4 + experts * 4 + tokens * top_k * 12 + (experts + 1) * 4 + 4
    cpu_best = min(cpu_seconds)
    line = {
        "metric": "expert dispatch tokens/sec, %d experts Top-%d %s + bias, fp32 router logits" % (experts, top_k, score_name),
        "value": tokens / seconds_per_step, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": seconds_per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "expert dispatch of one MoE layer: %d tokens x %d experts, Top-%d, %s scores, "
                               "selection bias, scaling %.1f; logits resident in HBM" % (tokens, experts, top_k, score_name, scaling),
                   "entry_point": "ncnn_moe_hip_router_dispatch_device (no host synchronisation inside the timed region)"},
        "roofline": {"bound": "hbm", "achieved": bytes_per_step / device_seconds_per_step / 1e9, "peak": HBM_PEAK_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": bytes_per_step / device_seconds_per_step / HBM_PEAK_BYTES_PER_S, "traffic": None,
                     "kernel": "router_clear_kernel + router_select_kernel + router_group_kernel, device time per dispatch "
                               "between two events on the launch stream",
                     "algorithmic_bytes_per_launch": bytes_per_step, "device_us_per_step": device_seconds_per_step * 1e6},
        "parity": {"dispatches_checked": buffers, "dispatch_mismatches": mismatches},
        "cpu_baseline": {"value": tokens / cpu_best, "unit": "tokens/s", "cores": 1, "kind": "port",
                         "sample": "best of %d dispatches of the same %d tokens by the CPU oracle" % (buffers, tokens)},
    }
    router.close()
    print(json.dumps(line))


def bench_generation_loop(args):
    """The batched generation loop of the C++ host mirror (BatchGenerationLoop::generate): --rows Sessions
    (64 by default) generate --steps tokens each from device-resident V = 151,936 fp32 logits, one device
    call per token index; the model's decode step is outside this path and costs nothing here (the rows
    stay resident).  Runs the C++ program and wraps its figures in the JSON shape of the other modes."""
    import subprocess
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    from ncnn_moe_runtime_amd.workloads import synthetic_model_logits as synthetic_logits

    program = os.path.join(PACKAGE_DIR, "test_session_sampler")
    if not os.path.exists(program):
        sys.exit("%s is missing: build it with make -C %s" % (program, PACKAGE_DIR))
    sessions = args.rows if args.rows > 0 else 64
    vocab, steps = 151936, args.steps
    done = subprocess.run([program, "--generation-bench", str(sessions), str(vocab), str(steps)],
                          capture_output=True, text=True, timeout=1200)
    if done.returncode != 0:
        sys.exit("generation bench failed: " + done.stdout[-1000:] + done.stderr[-1000:])
    fields = done.stdout.split()
    figures = {fields[i]: fields[i + 1] for i in range(1, len(fields) - 1, 2)}
    seconds = float(figures["seconds"]) - float(figures["prefill_seconds"])
    tokens = int(figures["tokens"])
    sample_seconds = int(figures["sample_time_microseconds"]) * 1e-6
    # parity of the run that was timed: Session 0's first token, recomputed with the CPU oracle
    first = oracle_lib.oracle_sample(synthetic_logits(vocab, 0, 0, -1), oracle_lib.OracleRng(1000).uniform(), 0.7, 20, 0.8, 0.0)
    same = int(first["token_id"]) == int(figures["first_token"]) and \
        int(np.float32(first["probability"]).view(np.uint32)) == int(figures["first_probability_bits"])
    # CPU baseline: the oracle over the same rows, one thread
    rows = np.stack([synthetic_logits(vocab, i, 0, -1) for i in range(min(sessions, 32))])
    params = np.zeros(rows.shape[0], dtype=oracle_lib.ROW_PARAMS_DTYPE)
    params["temperature"], params["top_k"], params["top_p"] = 0.7, 20, 0.8
    uniforms = np.full(rows.shape[0], 0.5, dtype=np.float32)
    start = time.perf_counter()
    oracle_lib.oracle_sample_batch(rows, params, uniforms, threads=1)
    cpu_seconds = time.perf_counter() - start
    bytes_per_step = sessions * vocab * 4
    line = {
        "metric": "generated tokens/sec, %d Sessions, V=151936 fp32 temp+topk+topp, device-resident logits" % sessions,
        "value": tokens / seconds, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 20,
        "ms_per_step": seconds / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "batched generation loop: %d Sessions x %d tokens, one device call per token index over "
                               "%d x %d fp32 logits resident in HBM; T 0.7, Top-K 20, Top-P 0.8; decode step not included" % (
                                   sessions, steps, sessions, vocab),
                   "entry_point": "BatchGenerationLoop::generate (C++ host mirror) over ncnn_moe_hip_sampler_logits_buffer + _sample"},
        "roofline": {"bound": "hbm", "achieved": bytes_per_step * steps / sample_seconds / 1e9, "peak": HBM_PEAK_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": bytes_per_step * steps / sample_seconds / HBM_PEAK_BYTES_PER_S, "traffic": None,
                     "kernel": "scan_select_kernel, wall clock of the synchronous sampling calls (SamplingStatistics::sample_time_microseconds)",
                     "algorithmic_bytes_per_launch": bytes_per_step, "sample_us_per_step": sample_seconds / steps * 1e6},
        "parity": {"first_token_matches_oracle": bool(same)},
        "cpu_baseline": {"value": rows.shape[0] / cpu_seconds, "unit": "tokens/s", "cores": 1, "kind": "port",
                         "sample": "%d rows of the same logits through the CPU oracle" % rows.shape[0]},
    }
    print(json.dumps(line))


def bench_scheduler(args):
    """Micro-batches through the scheduler seam of the C++ host mirror: BatchSampleScheduler over --samplers
    samplers (2 by default), a worker each, --rows device-resident rows (64 by default) of V = 151,936 fp32 per
    batch, as many batches in flight as there are samplers, every batch one synchronous device call of the
    worker that runs it (ncnn_moe_hip_sampler_sample: enqueue, wait, read the results).  Runs the C++ program
    and wraps its figures in the JSON shape of the other modes; the tokens of the first batch are checked
    against the CPU oracle."""
    import subprocess
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    from ncnn_moe_runtime_amd.workloads import synthetic_model_logits as synthetic_logits

    program = os.path.join(PACKAGE_DIR, "test_session_sampler")
    if not os.path.exists(program):
        sys.exit("%s is missing: build it with make -C %s" % (program, PACKAGE_DIR))
    rows = args.rows if args.rows > 0 else 64
    vocab, steps, samplers = 151936, args.steps, args.samplers
    done = subprocess.run([program, "--scheduler-bench", str(rows), str(vocab), str(samplers), str(steps)],
                          capture_output=True, text=True, timeout=1200)
    if done.returncode != 0:
        sys.exit("scheduler bench failed: " + done.stdout[-1000:] + done.stderr[-1000:])
    fields = done.stdout.split()
    at = fields.index("first_batch")
    figures = {fields[i]: fields[i + 1] for i in range(1, at, 2)}
    first_batch = [tuple(int(v) for v in entry.split(":")) for entry in fields[at + 1:]]
    seconds = float(figures["seconds"])
    mismatches = 0
    checked = min(rows, 16)
    for i in range(checked):
        expected = oracle_lib.oracle_sample(synthetic_logits(vocab, i, 0, -1), oracle_lib.OracleRng(5000 + i).uniform(), 0.7, 20, 0.8, 0.0)
        same = int(expected["token_id"]) == first_batch[i][0] and int(np.float32(expected["probability"]).view(np.uint32)) == first_batch[i][1]
        mismatches += 0 if same else 1
    sample = np.stack([synthetic_logits(vocab, i, 0, -1) for i in range(min(rows, 32))])
    params = np.zeros(sample.shape[0], dtype=oracle_lib.ROW_PARAMS_DTYPE)
    params["temperature"], params["top_k"], params["top_p"] = 0.7, 20, 0.8
    start = time.perf_counter()
    oracle_lib.oracle_sample_batch(sample, params, np.full(sample.shape[0], 0.5, dtype=np.float32), threads=1)
    cpu_seconds = time.perf_counter() - start
    bytes_per_step = rows * vocab * 4 + rows * 44
    line = {
        "metric": "sampled rows/sec through BatchSampleScheduler, %d samplers, B=%d V=151936 fp32 temp+topk+topp, device-resident logits" % (samplers, rows),
        "value": rows * steps / seconds, "unit": "rows/s", "n_gpus": 1, "steps": steps, "warmup": 4 * samplers,
        "ms_per_step": seconds / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "scheduler seam: batches of %d x %d fp32 rows resident in HBM, %d samplers and workers, %d batches in flight; "
                               "T 0.7, Top-K 20, Top-P 0.8" % (rows, vocab, samplers, samplers),
                   "entry_point": "BatchSampleScheduler::submit_sample (C++ host mirror) over ncnn_moe_hip_sampler_sample"},
        "roofline": {"bound": "hbm", "achieved": bytes_per_step * steps / seconds / 1e9, "peak": HBM_PEAK_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": bytes_per_step * steps / seconds / HBM_PEAK_BYTES_PER_S, "traffic": None,
                     "kernel": "split_select_kernel, wall clock of the whole loop (host threads, synchronous device calls)",
                     "algorithmic_bytes_per_launch": bytes_per_step},
        "parity": {"rows_checked": checked, "token_or_probability_mismatches": mismatches},
        "detail": {"device_calls": int(figures["device_calls"]), "device_calls_begun_while_another_ran": int(figures["overlapped_device_calls"])},
        "cpu_baseline": {"value": sample.shape[0] / cpu_seconds, "unit": "rows/s", "cores": 1, "kind": "port",
                         "sample": "%d rows of the same logits through the CPU oracle" % sample.shape[0]},
    }
    print(json.dumps(line))


def bench_geometry_sweep(args):
    """The select path over batch sizes, row lengths and both logits types at configuration 2's options (T 0.7,
    Top-K 20, Top-P 0.8): one run of this script per shape (--rows, --vocab, --logits-dtype; one rotated buffer
    checked against the CPU oracle), one table line each: microseconds per step, share of the 8 TB/s roofline,
    the kernel variant that served the shape, token mismatches."""
    import subprocess
    print("%5s %8s %5s  %-58s %9s %8s %11s" % ("rows", "vocab", "type", "kernel, grid", "us/step", "% peak", "mismatches"), flush=True)
    for dtype in ((args.logits_dtype,) if args.logits_dtype else ("f32", "bf16")):
        for vocab in (32000, 129280, 151936, 201088, 262144):
            for rows in (1, 8, 32, 64, 128, 192, 256, 384, 512):
                steps = max(60, min(600, int(3e9 / (rows * vocab * (4 if dtype == "f32" else 2)))))
                done = subprocess.run([sys.executable, os.path.abspath(__file__), "--workload", "cfg2_topk_topp", "--rows", str(rows),
                                       "--vocab", str(vocab), "--logits-dtype", dtype, "--steps", str(steps), "--warmup", "10",
                                       "--no-cpu-baseline", "--parity-buffers", "1"], capture_output=True, text=True, timeout=600)
                if done.returncode != 0:
                    sys.exit("shape %d x %d %s failed: %s" % (rows, vocab, dtype, done.stderr[-600:]))
                line = json.loads(done.stdout.strip().splitlines()[-1])
                parity = line["parity"]
                print("%5d %8d %5s  %-58s %9.2f %8.1f %11d" % (
                    rows, vocab, dtype, line["roofline"]["kernel"][:58], line["ms_per_step"] * 1e3, 100.0 * line["roofline"]["frac"],
                    parity["token_mismatches"] + parity["probability_bit_mismatches"] + parity["status_mismatches"]), flush=True)


def bench_timeline(args):
    """Where the time of a split-row launch goes: the library built with wall-clock stamps in the split
    kernel (make -C ncnn-moe-runtime_amd timeline) runs bursts of 12 launches over rotated logits buffers;
    the stamps of every burst's last launch are read back.  Prints a table (text, not the JSON line): times
    are microseconds after the launch's first workgroup entered the kernel."""
    import torch
    from ncnn_moe_runtime_amd import hip_sampler, workloads

    library = os.path.join(PACKAGE_DIR, "libncnn_moe_hip_sampler_timeline.so")
    if not os.path.exists(library):
        sys.exit("%s is missing: build it with make -C %s timeline" % (library, PACKAGE_DIR))
    hip_sampler.LIBRARY_PATH = library
    lib = hip_sampler.load_library()
    lib.ncnn_moe_hip_sampler_debug_timeline.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.ncnn_moe_hip_sampler_debug_timeline_rows.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    names = ["entered", "logits arrived", "bound", "collected", "counted itself"]
    merge_names = ["counted itself", "records read, checked, candidates placed in their bins", "bins scanned, window ordered", "result written"]
    device = torch.device("cuda:0")
    for rows in sorted({1, args.rows if args.rows > 0 else 64}):
        workload = workloads.make_workload(args.workload, rows=rows)
        vocab = workload["vocab"]
        dtype_code = hip_sampler.LOGITS_F32 if workload["dtype"] == "f32" else hip_sampler.LOGITS_BF16
        segments, chunks, variant = hip_sampler.select_geometry(dtype_code, rows, vocab)
        if variant != hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK or rows > 64:
            sys.exit("--timeline covers the split kernel (one-chunk workgroups) at up to 64 rows")
        host = torch.from_numpy(workload["logits"].view(np.int16) if workload["dtype"] != "f32" else workload["logits"])
        buffers = [host.to(device)]
        for _ in range(8):
            buffers.append(buffers[0][:, torch.randperm(vocab, device=device)].contiguous())
        params = torch.from_numpy(workload["params"].view(np.uint8).reshape(rows, -1)).to(device)
        uniforms = torch.from_numpy(workload["uniforms"]).to(device)
        results = torch.zeros(rows * 16, dtype=torch.uint8, device=device)
        stream = torch.cuda.current_stream()
        segment_times, merge_times, fine_times, retries = [], [], [], []
        with hip_sampler.HipSampler(rows, vocab) as sampler:
            for burst in range(40):
                for launch in range(12):
                    sampler.sample_device(buffers[(burst * 12 + launch) % 9].data_ptr(), dtype_code, rows, vocab, vocab,
                                          params.data_ptr(), uniforms.data_ptr(), None, results.data_ptr(), 0, stream.cuda_stream)
                torch.cuda.synchronize()
                if burst < 10:
                    continue
                stamps = np.zeros(64 * 16 * 16, dtype=np.uint64)
                fine = np.zeros(64 * 16, dtype=np.uint64)
                assert lib.ncnn_moe_hip_sampler_debug_timeline(stamps.ctypes.data, stamps.size) == 0
                assert lib.ncnn_moe_hip_sampler_debug_timeline_rows(fine.ctypes.data, fine.size) == 0
                t = stamps.reshape(64, 16, 16)[:rows, :segments].astype(np.int64)
                start = t[:, :, 0].min()
                relative = (t[:, :, :8] - start) / 100.0  # the clock ticks at 100 MHz
                merger = relative[:, :, 7].argmax(axis=1)  # the stamps of an earlier launch's merge are older
                merge = relative[np.arange(rows), merger]
                segment_times.append(relative[:, :, :5])
                merge_times.append(merge[:, 4:8])
                epilogue = (fine.reshape(64, 16)[:rows, :7].astype(np.int64) - start) / 100.0
                fine_times.append(np.concatenate([merge[:, 6:7], epilogue, merge[:, 7:8]], axis=1))
                retries.append(t[np.arange(rows), merger, 8] - 1)
        seg, mer, fin = np.stack(segment_times), np.stack(merge_times), np.stack(fine_times)
        print("%s, %d rows x %d (%d workgroups per row), %d launches sampled: microseconds after the first workgroup entered" % (
            args.workload, rows, vocab, segments, len(segment_times)))
        for slot, name in enumerate(names):
            v = seg[..., slot]
            print("  every workgroup: %-26s min %6.2f  median %6.2f  p90 %6.2f  max %6.2f" % (name, v.min(), np.median(v), np.percentile(v, 90), v.max()))
        for slot, name in enumerate(merge_names):
            v = mer[..., slot]
            print("  row's last workgroup: %-21s min %6.2f  median %6.2f  p90 %6.2f  max %6.2f" % (name, v.min(), np.median(v), np.percentile(v, 90), v.max()))
        d, dm, df = np.diff(seg, axis=-1), np.diff(mer, axis=-1), np.diff(fin, axis=-1)
        print("  phases of a workgroup (medians): wait for the logits %.2f | maxima + bound %.2f | collect %.2f | entries out + counter atomic %.2f" % tuple(
            np.median(d[..., k]) for k in range(4)))
        print("  phases of the merge (medians): records read, checked, placed %.2f | bins scanned, window ordered %.2f | epilogue %.2f" % tuple(
            np.median(dm[..., k]) for k in range(3)))
        print("  inside the epilogue (medians): last ordering %.2f | divide + expf %.2f | normaliser %.2f | divide + Min-P + Top-P %.2f | export %.2f | draw %.2f | "
              "result store %.2f | exit %.2f" % tuple(np.median(df[..., k]) for k in range(8)))
        print("  last result of a launch (median over launches) %.2f us; last logits of a launch %.2f us; re-reads of records per merge: mean %.2f" % (
            np.median(mer[..., 3].max(axis=1)), np.median(seg[..., 1].reshape(len(segment_times), -1).max(axis=1)), np.concatenate(retries).mean()))


def bench_full_order_timeline(args):
    """Where the time of the later passes goes (rows without a Top-K window, or with one wider than 64): the
    stamped library runs the workload's batch a few times; the stamps that the first 64 rows' workgroups left
    in the last launch are read back.  Prints a table (text, not the JSON line), microseconds."""
    import torch
    from ncnn_moe_runtime_amd import hip_sampler, workloads

    library = os.path.join(PACKAGE_DIR, "libncnn_moe_hip_sampler_timeline.so")
    if not os.path.exists(library):
        sys.exit("%s is missing: build it with make -C %s timeline" % (library, PACKAGE_DIR))
    hip_sampler.LIBRARY_PATH = library
    lib = hip_sampler.load_library()
    lib.ncnn_moe_hip_sampler_debug_timeline.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    workload = workloads.make_workload(args.workload)
    rows, vocab = workload["rows"], workload["vocab"]
    device = torch.device("cuda:0")
    dtype_code = hip_sampler.LOGITS_F32 if workload["dtype"] == "f32" else hip_sampler.LOGITS_BF16
    logits = torch.from_numpy(workload["logits"].view(np.int16) if workload["dtype"] != "f32" else workload["logits"]).to(device)
    params = torch.from_numpy(workload["params"].view(np.uint8).reshape(rows, -1)).to(device)
    uniforms = torch.from_numpy(workload["uniforms"]).to(device)
    stop_ids = None if workload["stop_ids"] is None else torch.from_numpy(workload["stop_ids"]).to(device)
    results = torch.zeros(rows * 16, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream()

    def read_stamps():
        stamps = np.zeros(64 * 16 * 16, dtype=np.uint64)
        assert lib.ncnn_moe_hip_sampler_debug_timeline(stamps.ctypes.data, stamps.size) == 0
        return stamps.reshape(64, 16, 16).astype(np.int64)

    with hip_sampler.HipSampler(rows, vocab) as sampler:
        for _ in range(6):
            before = read_stamps()
            sampler.sample_device(logits.data_ptr(), dtype_code, rows, vocab, vocab, params.data_ptr(), uniforms.data_ptr(),
                                  None if stop_ids is None else stop_ids.data_ptr(), results.data_ptr(),
                                  hip_sampler.PASSES_FULL_ORDER, stream.cuda_stream)
            torch.cuda.synchronize()
            after = read_stamps()
    out = results.cpu().numpy().view(hip_sampler.RESULT_DTYPE)
    top_k = workload["params"]["top_k"][:64]
    sampled = workload["params"]["temperature"][:64] != 0
    full_order = np.nonzero((out["flags"][:64] & hip_sampler.FLAG_GENERAL_PATH) != 0)[0]
    wide = np.nonzero(sampled & (top_k > 64) & (top_k <= 1024) & ((out["flags"][:64] & hip_sampler.FLAG_GENERAL_PATH) == 0))[0]
    print("%s, %d rows x %d %s; of the first 64 rows %d took the full-order kernels and %d the wide select" % (
        args.workload, rows, vocab, workload["dtype"], full_order.size, wide.size))

    def table(title, stamps, names):
        relative = (stamps - stamps[:, :1]) / 100.0  # the clock ticks at 100 MHz
        phases = np.diff(stamps, axis=1) / 100.0
        print("  " + title)
        for slot, name in enumerate(names[1:]):
            print("    %-46s at %7.1f (median)   phase: median %6.1f  max %6.1f" % (
                name, np.median(relative[:, slot + 1]), np.median(phases[:, slot]), phases[:, slot].max()))

    if full_order.size:
        if workload["dtype"] != "f32":
            table("bf16_counting_replay_kernel, one workgroup per row: the count, after the kernel's entry:", after[full_order, 14, :3],
                  ["entered", "row counted (one pass, 16-bit counters)", "runs written (into the counters' LDS)"])
        table("general_replay_kernel, one workgroup per row, after its entry:" if workload["dtype"] == "f32" else
              "bf16_counting_replay_kernel: the walk, after the count:", after[full_order, 15, :8],
              ["entered", "exp terms of the row ready", "finite prefix found", "normaliser (exact running sum)", "Min-P cut",
               "Top-P walk (exact running sum)", "draw (exact running sum)", "token index recovered from the logits"])
        rounds = (after - before)[full_order, 15, 12:14].sum(axis=1)
        print("    rounds of the exact running sums per row: median %d, max %d" % (np.median(rounds), rounds.max()))
    if wide.size:
        table("scan_select_kernel<wide>, one workgroup per row, after its entry:", after[wide, 12, :5],
              ["entered", "row streamed, candidates listed", "list cut to the window", "window sorted (bitonic, LDS)", "window walked, result written"])


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=2000)
    parser.add_argument("--warmup", type=int, default=200)
    parser.add_argument("--workload", default="cfg2_topk_topp")
    parser.add_argument("--rows", type=int, default=0, help="batch rows (0: the configuration's own)")
    parser.add_argument("--vocab", type=int, default=0, help="row length (0: the configuration's own)")
    parser.add_argument("--logits-dtype", default="", choices=["", "f32", "bf16"],
                        help="store the configuration's logits as fp32 or bf16 instead of its own type")
    parser.add_argument("--parity-buffers", type=int, default=0,
                        help="rotated buffers checked against the CPU oracle (0: every one; a sweep over large shapes checks one)")
    parser.add_argument("--geometry-sweep", action="store_true",
                        help="the select path at B x V x {fp32, bf16}, K = 20 (configuration 2's options): one table line per shape")
    parser.add_argument("--batches-in-flight", action="store_true",
                        help="also time 2 and 4 independent batches in flight (detail only; their launches overlap, "
                             "so leave it off under a kernel trace)")
    parser.add_argument("--router-score", default="sqrt_softplus", choices=["softmax", "sigmoid", "sqrt_softplus"],
                        help="score function of --workload router_dispatch")
    parser.add_argument("--samplers", type=int, default=2, help="samplers (and workers) of --workload scheduler")
    parser.add_argument("--drafts", type=int, default=5, help="drafted tokens per step of --workload speculative_verify")
    parser.add_argument("--dense-verify", action="store_true",
                        help="--workload speculative_verify without a Top-K window (T 1.0, Top-P 0.95): the dense path")
    parser.add_argument("--buffers", type=int, default=0, help="distinct logits buffers (0: enough to exceed 320 MB)")
    parser.add_argument("--cpu-rows", type=int, default=64)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--host-entry", action="store_true",
                        help="also time the host-buffer entry (upload_logits + sample(): the logits cross PCIe); detail only")
    parser.add_argument("--timeline", action="store_true",
                        help="print where the time of a launch goes: the split kernel's phases (cfg2 and the like), or the later "
                             "passes' (cfg3, cfg4); needs the stamped library (make timeline); a table, not the JSON line")
    parser.add_argument("--copy-calibration", type=int, default=0,
                        help="after the timed steps, copy a 256 MiB buffer this many times (a kernel of known "
                             "traffic for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every box of this build has one MI355X; run with --gpus 1")

    load_package()
    from ncnn_moe_runtime_amd import hip_sampler, workloads
    if args.geometry_sweep:
        bench_geometry_sweep(args)
        return
    if args.timeline:
        if args.workload in ("cfg3_full_nucleus", "cfg4_service_mix"):
            bench_full_order_timeline(args)
        else:
            bench_timeline(args)
        return
    if args.workload == "router_dispatch":
        bench_router_dispatch(args)
        return
    if args.workload == "generation_loop":
        bench_generation_loop(args)
        return
    if args.workload == "scheduler":
        bench_scheduler(args)
        return
    if args.workload == "speculative_verify":
        return bench_speculative_verify(args, hip_sampler)
    import torch

    if not torch.cuda.is_available() or hip_sampler.device_count() < 1:
        sys.exit("bench.py needs a GPU: no HIP device is visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    workload = workloads.make_workload(args.workload, rows=args.rows if args.rows > 0 else None, vocab=args.vocab if args.vocab > 0 else None)
    if args.logits_dtype and args.logits_dtype != workload["dtype"]:
        if args.logits_dtype == "bf16":
            workload["logits"] = workloads.float32_to_bf16_bits(workload["logits"])
        else:
            workload["logits"] = workloads.bf16_bits_to_float32(workload["logits"])
        workload["dtype"] = args.logits_dtype
        workload["description"] += " [logits stored as %s]" % args.logits_dtype
    rows, vocab = workload["rows"], workload["vocab"]
    element_bytes = 4 if workload["dtype"] == "f32" else 2
    dtype_code = hip_sampler.LOGITS_F32 if workload["dtype"] == "f32" else hip_sampler.LOGITS_BF16
    batch_bytes = rows * vocab * element_bytes
    buffers = args.buffers if args.buffers > 0 else max(2, -(-320 * 1024 * 1024 // batch_bytes))

    # buffer 0 holds the seeded host workload (checked against the oracle); the others hold rows of the
    # same distribution generated on the device, so that consecutive steps read different HBM lines
    host_logits = torch.from_numpy(workload["logits"].view(np.int16) if element_bytes == 2 else workload["logits"])
    logits = [host_logits.to(device)]
    generator = torch.Generator(device=device)
    generator.manual_seed(1234)
    for _ in range(buffers - 1):
        permutation = torch.randperm(vocab, device=device, generator=generator)
        logits.append(logits[0][:, permutation].contiguous())
    params = torch.from_numpy(workload["params"].view(np.uint8).reshape(rows, -1)).to(device)
    uniforms = torch.from_numpy(workload["uniforms"]).to(device)
    stop_ids = None if workload["stop_ids"] is None else torch.from_numpy(workload["stop_ids"]).to(device)
    results = torch.zeros((rows, 16), dtype=torch.uint8, device=device)

    sampler = hip_sampler.HipSampler(rows, vocab)
    stream = torch.cuda.Stream(device=device)
    stream_pointer = stream.cuda_stream

    # the scheduler holds every Session's SamplingOptions on the host, so it knows whether a batch can
    # need the full-order kernels (no Top-K window, or one wider than 64)
    effective_k = np.where((workload["params"]["top_k"] == 0) | (workload["params"]["top_k"] >= vocab),
                           vocab, workload["params"]["top_k"])
    sampled = workload["params"]["temperature"] != 0
    may_need_full_order = int(np.any(sampled & (effective_k > 64)))
    if np.count_nonzero(sampled & (effective_k > 64) & (effective_k <= 1024)) >= 32 and np.count_nonzero(sampled & (effective_k > 1024)) >= 32:
        may_need_full_order |= hip_sampler.PASSES_SIDE_BY_SIDE  # as a scheduler that knows its Sessions' options would
    if may_need_full_order and not np.any(sampled & (effective_k > 64) & (effective_k <= 1024)):
        may_need_full_order |= hip_sampler.PASSES_NO_WIDE_WINDOWS

    def step(index):
        sampler.sample_device(
            logits[index % buffers].data_ptr(), dtype_code, rows, vocab, vocab,
            params.data_ptr(), uniforms.data_ptr(), None if stop_ids is None else stop_ids.data_ptr(),
            results.data_ptr(), may_need_full_order, stream_pointer)

    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        # parity of the measured path against the CPU oracle on EVERY buffer that the timed steps rotate
        # over (the oracle runs after the timed region, on host copies of the buffers)
        gpu_per_buffer = []
        for index in range(buffers):
            step(index)
            stream.synchronize()
            gpu_per_buffer.append(results.cpu().numpy().view(hip_sampler.RESULT_DTYPE).reshape(rows).copy())
        gpu = gpu_per_buffer[0]
        for index in range(args.warmup):
            step(index)
        stream.synchronize()
        torch.cuda.synchronize()
        start_event = torch.cuda.Event(enable_timing=True)
        stop_event = torch.cuda.Event(enable_timing=True)
        wall_start = time.perf_counter()
        start_event.record(stream)
        for index in range(args.steps):
            step(index)
        stop_event.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wall_seconds = time.perf_counter() - wall_start
    event_seconds = start_event.elapsed_time(stop_event) * 1e-3
    seconds_per_step = event_seconds / args.steps

    # Beside the headline: the spread of single launches (one event pair per launch, which adds the
    # event's own cost to each) and the same loop on ONE buffer, which the 256 MB Infinity Cache holds.
    detail_steps = 200
    with torch.cuda.stream(stream):
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(detail_steps)]
        for index, (first, last) in enumerate(pairs):
            first.record(stream)
            step(index)
            last.record(stream)
        stream.synchronize()
        single_launch_us = np.array([first.elapsed_time(last) * 1e3 for first, last in pairs])
        resident_start = torch.cuda.Event(enable_timing=True)
        resident_stop = torch.cuda.Event(enable_timing=True)
        for _ in range(10):
            step(0)
        resident_start.record(stream)
        for _ in range(detail_steps):
            step(0)
        resident_stop.record(stream)
        stream.synchronize()
    torch.cuda.synchronize()
    detail = {
        "single_launch_us_p10_median_p90": [float(np.percentile(single_launch_us, q)) for q in (10, 50, 90)],
        "single_launches": detail_steps,
        "single_launch_note": "one HIP event pair per launch, %d launches; includes the events' own cost" % detail_steps,
        "cache_resident_ms_per_step": resident_start.elapsed_time(resident_stop) / detail_steps,
        "cache_resident_note": "same loop on one logits buffer (%.1f MB), held by the Infinity Cache where it fits; "
                               "not the reported value" % (batch_bytes / 1e6),
    }
    if os.path.exists(hip_sampler.TESTING_LIBRARY_PATH) and \
            hip_sampler.select_geometry(dtype_code, rows, vocab)[2] == hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK:
        # what a launch of this grid costs for streaming the logits alone: the split kernel's loads with
        # nothing behind them, over the same rotated buffers (a probe kernel of the library's testing build)
        probe = hip_sampler.HipSampler(rows, vocab, testing=True)
        with torch.cuda.stream(stream):
            for index in range(20):
                probe.stream_only(logits[index % buffers].data_ptr(), dtype_code, rows, vocab, vocab, stream_pointer)
            stream_start = torch.cuda.Event(enable_timing=True)
            stream_stop = torch.cuda.Event(enable_timing=True)
            stream_start.record(stream)
            for index in range(detail_steps * 4):
                probe.stream_only(logits[index % buffers].data_ptr(), dtype_code, rows, vocab, vocab, stream_pointer)
            stream_stop.record(stream)
            stream.synchronize()
        probe.close()
        detail["stream_only_ms_per_launch"] = stream_start.elapsed_time(stream_stop) / (detail_steps * 4)
        detail["stream_only_note"] = ("the split kernel's grid and loads with nothing behind them (%d launches over the rotated "
                                      "buffers): the cost of streaming the logits alone; not the reported value" % (detail_steps * 4))
    # Several independent batches in flight (one handle and one stream each, steps dealt round robin): what
    # a server that keeps several micro-batches going sees.  A decode loop of ONE batch cannot do this (step
    # n + 1 needs step n's tokens), so these are reported beside the value, never as it.
    if args.batches_in_flight and rows <= 256:
        lanes = [(sampler, stream, results)]
        in_flight = {}
        for lane_count in (2, 4):
            while len(lanes) < lane_count:
                lanes.append((hip_sampler.HipSampler(rows, vocab), torch.cuda.Stream(device=device), torch.zeros_like(results)))

            def overlapped_step(index):
                handle, lane_stream, lane_results = lanes[index % lane_count]
                handle.sample_device(
                    logits[index % buffers].data_ptr(), dtype_code, rows, vocab, vocab,
                    params.data_ptr(), uniforms.data_ptr(), None if stop_ids is None else stop_ids.data_ptr(),
                    lane_results.data_ptr(), may_need_full_order, lane_stream.cuda_stream)

            for index in range(20):
                overlapped_step(index)
            torch.cuda.synchronize()
            overlapped_start = time.perf_counter()
            for index in range(detail_steps * 4):
                overlapped_step(index)
            enqueue_seconds = time.perf_counter() - overlapped_start
            torch.cuda.synchronize()
            in_flight[str(lane_count)] = (time.perf_counter() - overlapped_start) / (detail_steps * 4) * 1e3
            detail["host_enqueue_ms_per_call"] = enqueue_seconds / (detail_steps * 4) * 1e3
        detail["batches_in_flight_ms_per_step"] = in_flight
        detail["batches_in_flight_note"] = ("2 and 4 independent batches, one handle and one stream each, steps dealt round "
                                            "robin, wall clock over %d steps; not the reported value" % (detail_steps * 4))
        for handle, _, _ in lanes[1:]:
            handle.close()
    if args.host_entry:
        # the boundary's host-buffer entry: logits cross PCIe from pageable host memory, then the synchronous call
        upload_seconds, sample_seconds = [], []
        for _ in range(12):
            begin = time.perf_counter()
            sampler.upload_logits(workload["logits"])
            middle = time.perf_counter()
            sampler.sample(workload["params"], workload["uniforms"], workload["stop_ids"])
            upload_seconds.append(middle - begin)
            sample_seconds.append(time.perf_counter() - middle)
        upload, call = float(np.median(upload_seconds[2:])), float(np.median(sample_seconds[2:]))
        detail["host_entry"] = {
            "upload_logits_ms": upload * 1e3, "upload_GB_per_s": rows * vocab * element_bytes / upload / 1e9,
            "sample_call_ms": call * 1e3, "rows_per_s_including_pcie": rows / (upload + call),
            "note": "upload_logits from pageable host memory + the synchronous sample() through the Python binding, "
                    "medians of 10 calls; never the reported value"}
    if args.copy_calibration > 0:
        source = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        for _ in range(args.copy_calibration):
            target.copy_(source)
        torch.cuda.synchronize()

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    import parity_util
    host_threads = min(16, os.cpu_count() or 1)
    parity = None
    checked_buffers = buffers if args.parity_buffers <= 0 else min(buffers, args.parity_buffers)
    for index in range(checked_buffers):
        host_buffer = workload["logits"] if index == 0 else logits[index].cpu().numpy().view(workload["logits"].dtype)
        cpu = oracle_lib.oracle_sample_batch(host_buffer, workload["params"], workload["uniforms"],
                                             workload["stop_ids"], threads=host_threads)
        counters = parity_util.parity_counters(gpu_per_buffer[index], cpu)
        counters["status_mismatches"] = int(np.count_nonzero(gpu_per_buffer[index]["status"] != cpu["status"]))
        counters["kept_count_mismatches"] = int(np.count_nonzero(gpu_per_buffer[index]["kept_count"] != cpu["kept_count"]))
        if parity is None:
            parity = counters
        else:
            for key, value in counters.items():
                parity[key] += value
    parity["buffers_checked"] = checked_buffers

    bytes_per_launch = algorithmic_bytes(rows, vocab, element_bytes)
    achieved = bytes_per_launch / seconds_per_step
    own_shape = args.rows == 0 and args.vocab == 0 and not args.logits_dtype
    traffic, traffic_file = measured_traffic(workload["name"]) if own_shape else (None, None)
    segments, chunks, variant = hip_sampler.select_geometry(dtype_code, rows, vocab)
    kernel = {hip_sampler.GEOMETRY_WHOLE_ROW: "scan_select_kernel (one workgroup per row)",
              hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK: "split_select_kernel (%d one-chunk workgroups per row)" % segments,
              hip_sampler.GEOMETRY_SPLIT_LOOPED: "scan_select_kernel (%d workgroups per row, %d chunks each)" % (segments, chunks)}[variant]
    if may_need_full_order:
        kernel += " + the later passes for rows without a Top-K window of at most 64 (wide select, sort, replay)"
    metric = METRICS.get(workload["name"], "sampled rows/sec + HBM GB/s (% peak), " + workload["name"])
    if not own_shape:
        metric += " [shape overridden: %d x %d %s]" % (rows, vocab, workload["dtype"])
    line = {
        "metric": metric,
        "value": rows / seconds_per_step,
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": seconds_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if element_bytes == 4 else "bf16",
        "data": "synthetic",
        "config": {
            "workload": workload["description"],
            "name": workload["name"],
            "rows": rows,
            "vocab": vocab,
            "logits_buffers_rotated": buffers,
            "logits_bytes_per_step": batch_bytes,
            "entry_point": "ncnn_moe_hip_sampler_sample_device",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved / 1e9,
            "peak": HBM_PEAK_BYTES_PER_S / 1e9,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_BYTES_PER_S,
            "traffic": traffic,
            "traffic_source": None if traffic is None else "stored from %s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                                                           "command, scaled by a copy kernel); not measured in this run" % traffic_file,
            "kernel": kernel,
            "algorithmic_bytes_per_launch": bytes_per_launch,
        },
        "parity": parity,
        "wall_ms_per_step": wall_seconds / args.steps * 1e3,
        "detail": detail,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(workload, host_threads, args.cpu_rows)
    sampler.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
