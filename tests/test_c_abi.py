"""The C-ABI library loads without a GPU and exports every function include/*.h declares;
the C++ host mirror's host-only tests pass."""
import ctypes
import os
import re
import subprocess

import pytest

from ncnn_moe_runtime_amd import hip_router, hip_sampler

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PACKAGE_DIR = os.path.join(ROOT, "ncnn-moe-runtime_amd")
TEST_PROGRAM = os.path.join(PACKAGE_DIR, "test_session_sampler")


def declared_functions(header="ncnn_moe_hip_sampler.h", prefix="ncnn_moe_hip_sampler_"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def router_functions():
    return declared_functions("ncnn_moe_hip_router.h", "ncnn_moe_hip_router_")


def test_header_and_binding_agree():
    assert declared_functions() == sorted(hip_sampler.EXPORTED_SYMBOLS)
    assert declared_functions("ncnn_moe_hip_sampler_testing.h") == sorted(hip_sampler.TESTING_SYMBOLS)
    assert not [name for name in declared_functions() if "_debug_" in name], "test hooks belong in the testing header"


def test_library_exports_every_declared_function():
    """The shipped library exports the boundary and none of the test hooks; the testing build exports both."""
    library = hip_sampler.load_library()
    for name in declared_functions():
        assert getattr(library, name) is not None
    for name in declared_functions("ncnn_moe_hip_sampler_testing.h"):
        assert not hasattr(library, name), "%s is a test hook: it belongs in the testing build only" % name
    exported = subprocess.run(["nm", "-D", "--defined-only", hip_sampler.LIBRARY_PATH], capture_output=True, text=True, check=True).stdout
    assert "_debug_" not in exported and "stream_only" not in exported
    testing = hip_sampler.load_testing_library()
    for name in declared_functions() + declared_functions("ncnn_moe_hip_sampler_testing.h"):
        assert getattr(testing, name) is not None


def test_select_geometry_of_the_benchmark_shapes():
    """The kernel variant behind each benchmark configuration, and the shapes that the GPU tests name."""
    f32, bf16 = hip_sampler.LOGITS_F32, hip_sampler.LOGITS_BF16
    assert hip_sampler.select_geometry(f32, 64, 151936) == (15, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
    assert hip_sampler.select_geometry(f32, 1, 32000) == (4, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
    assert hip_sampler.select_geometry(f32, 512, 129280)[2] == hip_sampler.GEOMETRY_WHOLE_ROW
    assert hip_sampler.select_geometry(bf16, 1024, 262144)[2] == hip_sampler.GEOMETRY_WHOLE_ROW
    for rows in (1, 8, 64, 130, 200, 255):
        # rows of 17 to 32 chunks: one-chunk workgroups (fp32 always, bf16 up to 2,304 of them); longer rows: looped
        assert hip_sampler.select_geometry(f32, rows, 163841) == (17, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
        assert hip_sampler.select_geometry(f32, rows, 262144) == (26, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
        segments, chunks, variant = hip_sampler.select_geometry(bf16, rows, 262144)
        if rows * 22 <= 2304:
            assert (segments, chunks, variant) == (22, 1, hip_sampler.GEOMETRY_SPLIT_ONE_CHUNK)
        else:
            assert variant == hip_sampler.GEOMETRY_SPLIT_LOOPED and chunks > 1 and 1 < segments <= 16
        segments, chunks, variant = hip_sampler.select_geometry(f32, rows, 340000)
        assert variant == hip_sampler.GEOMETRY_SPLIT_LOOPED and chunks > 1 and 1 < segments <= 16


def test_router_header_and_binding_agree():
    assert router_functions() == sorted(hip_router.EXPORTED_SYMBOLS)
    library = hip_router.load_library()
    for name in router_functions():
        assert getattr(library, name) is not None


def test_router_status_messages_are_the_dispatcher_messages():
    """src/graph/expert_dispatcher.cpp:80-103, :122, :133"""
    expected = {
        1: "expert dispatch requires at least one token",
        2: "expert dispatch requires 0 < top_k <= expert_count",
        3: "routed scaling factor must be finite and positive",
        4: "router logits must be finite",
        5: "explicit expert id is out of range",
        6: "selected router weights have a non-positive sum",
    }
    for status, message in expected.items():
        assert hip_router.status_message(status) == message
    assert hip_router.status_message(0) == ""
    assert hip_router.OPTIONS_DTYPE.itemsize == 20 and hip_router.ROUTE_DTYPE.itemsize == 12


def test_router_create_without_gpu_fails_loudly():
    if hip_sampler.device_count() > 0:
        pytest.skip("a GPU is visible")
    with pytest.raises(hip_router.RouterError):
        hip_router.HipRouter(16)


def test_status_messages_are_the_cpu_sampler_messages():
    expected = {
        1: "cannot sample empty logits",
        2: "temperature must be finite and non-negative",
        3: "top_p must be in the range (0, 1]",
        4: "min_p must be in the range [0, 1]",
        5: "sampling requires at least one finite logit",
        6: "sampling distribution is invalid",
    }
    for status, message in expected.items():
        assert hip_sampler.status_message(status) == message
    assert hip_sampler.status_message(0) == ""


def test_struct_layouts():
    assert hip_sampler.PARAMS_DTYPE.itemsize == 24
    assert hip_sampler.RESULT_DTYPE.itemsize == 16


def test_exp2_table_is_correctly_rounded():
    """2^(i/32) as double bits minus i << 47, recomputed with 80-digit decimal arithmetic."""
    from decimal import Decimal, getcontext
    import struct
    getcontext().prec = 80
    table = hip_sampler.exp2_table()
    for i in range(32):
        value = float(Decimal(2) ** (Decimal(i) / Decimal(32)))
        bits = struct.unpack("<Q", struct.pack("<d", value))[0] - (i << 47)
        assert int(table[i]) == bits


def test_create_without_gpu_fails_loudly():
    if hip_sampler.device_count() > 0:
        pytest.skip("a GPU is visible")
    with pytest.raises(hip_sampler.SamplerError):
        hip_sampler.HipSampler(4, 1000)


def test_host_mirror_host_only_tests():
    assert os.path.exists(TEST_PROGRAM), "build it with make -C ncnn-moe-runtime_amd"
    done = subprocess.run([TEST_PROGRAM, "--host"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "all host-side session sampler tests passed" in done.stdout


@pytest.mark.gpu
def test_host_mirror_on_gpu():
    print("[case] C++ host mirror test program", flush=True)
    done = subprocess.run([TEST_PROGRAM], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "all session sampler tests passed" in done.stdout


DISPATCHER_TEST_PROGRAM = os.path.join(PACKAGE_DIR, "test_expert_dispatcher")


def test_dispatcher_mirror_host_only_tests():
    assert os.path.exists(DISPATCHER_TEST_PROGRAM), "build it with make -C ncnn-moe-runtime_amd"
    done = subprocess.run([DISPATCHER_TEST_PROGRAM, "--host"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "all host-side expert dispatcher tests passed" in done.stdout


@pytest.mark.gpu
def test_dispatcher_mirror_on_gpu():
    print("[case] C++ expert dispatcher mirror test program", flush=True)
    done = subprocess.run([DISPATCHER_TEST_PROGRAM], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "all expert dispatcher tests passed" in done.stdout


REFERENCE_INCLUDE = "/root/reference/include"


@pytest.mark.reference
@pytest.mark.parametrize("source, forced_includes", [
    ("hip_session_sampler.cpp", ["ncnn/moe/session.h"]),
    ("worker_wire.cpp", ["ncnn/moe/session.h"]),
    ("hip_expert_dispatcher.cpp", ["ncnn/moe/session.h", "ncnn/moe/expert_dispatcher.h"]),
])
def test_host_mirrors_compile_inside_the_runtime(source, forced_includes):
    """The host mirrors are meant to be compiled inside the runtime, where its own headers come first and
    the mirrors must use the runtime's types instead of their stand-alone equivalents: syntax-check each
    source with the runtime's public headers force-included (nothing is linked or run)."""
    if not os.path.exists(os.path.join(REFERENCE_INCLUDE, "ncnn", "moe", "session.h")):
        pytest.skip("the runtime's headers are not present on this machine")
    command = ["g++", "-std=c++20", "-fsyntax-only", "-I" + REFERENCE_INCLUDE, "-I" + os.path.join(ROOT, "include"),
               "-I" + os.path.join(PACKAGE_DIR, "csrc")]
    for header in forced_includes:
        command += ["-include", header]
    command.append(os.path.join(PACKAGE_DIR, "csrc", source))
    done = subprocess.run(command, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]
