"""The inspection commands and the benchmark summary of the ROCm arm (CPU only).

`yvex-rocm inspect backend rocm` and `yvex-rocm inspect rocm [bandwidth]` are run as the
reference's fail-closed test runs `yvex inspect backend cuda` (tests/test_cuda_failclosed.sh:
46-80): exit code 5 with the "unsupported" lines where the device runtime cannot be opened,
exit code 0 with the capability lines where it can (here: the stand-in HIP runtime of
tests/fake_hip, whose launches do nothing).  The sample summary is checked on values worked out
by hand from the nearest-rank rule of src/runtime/benchmark.c:421-447.
"""
import os
import subprocess

import pytest

from clori_amd import backend as K
from clori_amd import binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "clori_amd", "yvex-rocm")
FAKE_DIR = os.path.join(ROOT, "tests", "fake_hip")
FAKE_SO = os.path.join(FAKE_DIR, "libfakehip.so")

pytestmark = pytest.mark.skipif(not os.path.exists(PROGRAM), reason="yvex-rocm is not built")


def run(*arguments, driver=None, extra=None):
    env = {k: v for k, v in os.environ.items() if not k.startswith("YVEX_TEST_ROCM_")}
    if driver:
        env["YVEX_TEST_ROCM_DRIVER_LIBRARY"] = driver
    env.update(extra or {})
    done = subprocess.run([PROGRAM, *arguments], env=env, capture_output=True, text=True, timeout=60)
    return done.returncode, done.stdout, done.stderr


@pytest.fixture(scope="module")
def fake_runtime():
    subprocess.check_call(["gcc", "-std=c11", "-O1", "-fPIC", "-shared", "-I/opt/rocm/include",
                           "-o", FAKE_SO, os.path.join(FAKE_DIR, "fake_hip.c")])
    return FAKE_SO


def test_backend_unsupported_exits_5_with_the_reference_lines():
    rc, out, _ = run("inspect", "backend", "rocm", driver="/nonexistent/libamdhip64.so")
    assert rc == 5
    assert "backend: rocm\n" in out and "status: unsupported\n" in out
    assert "reason: " in out and out.endswith("status: backend-unsupported\n")


def test_rocm_info_unsupported_exits_5():
    for arguments in (("inspect", "rocm"), ("inspect", "rocm", "bandwidth")):
        rc, out, _ = run(*arguments, driver="/nonexistent/libamdhip64.so")
        assert rc == 5
        assert out.startswith("rocm: unavailable\nreason: ")
        assert out.endswith("status: rocm-unavailable\n")


def test_other_backend_kinds_are_unsupported_not_errors():
    rc, out, _ = run("inspect", "backend", "cuda")
    assert rc == 5 and "backend: cuda\n" in out and "status: backend-unsupported\n" in out


def test_grammar_errors_exit_2():
    for arguments in (("inspect", "rocm", "nope"), ("inspect", "backend"),
                      ("inspect", "backend", "vulkan"), ("inspect",), ("bench", "x", "y")):
        rc, out, err = run(*arguments)
        assert rc == 2 and out == "" and err
    rc, out, _ = run("inspect", "rocm", "--help")
    assert rc == 0 and out.startswith("usage: yvex inspect rocm [bandwidth]")


def test_backend_capabilities_on_the_stand_in_runtime(fake_runtime):
    rc, out, _ = run("inspect", "backend", "rocm", driver=fake_runtime)
    assert rc == 0
    for line in ("backend: rocm", "status: ready", "name: fake-gfx950", "  tensor_alloc: yes",
                 "  tensor_read_write: yes", "  op_embed: no", "  op_rms_norm: no", "  op_rope: no",
                 "  op_matmul: no", "  op_mlp: no", "  op_attention: yes", "context_available: yes",
                 "kernel_bundle: admitted", "kernel_bundle_reason: none", "kernel_bundle_native: yes",
                 "kernel_bundle_architecture: gfx950", "  embed-f32-to-f32: unsupported (variant-unsupported)",
                 "  attention-causal-f32: supported (none)",
                 "  encoded-attention: unsupported (variant-unsupported)",
                 "  rocm-attention-paged-q8-0: supported (none)",
                 "  rocm-attention-mla-bf16: supported (none)"):
        assert line + "\n" in out, line
    assert out.endswith("status: backend-capabilities\n")


def test_rejected_bundle_is_reported_not_hidden(fake_runtime):
    rc, out, _ = run("inspect", "backend", "rocm", driver=fake_runtime,
                     extra={"YVEX_TEST_ROCM_BUNDLE_FAILURE": "module"})
    assert rc == 0
    assert "kernel_bundle: rejected\n" in out and "kernel_bundle_native: no\n" in out
    assert "  op_attention: no\n" in out
    assert "  rocm-attention-gqa-bf16: failed (" in out


def test_rocm_info_and_bandwidth_on_the_stand_in_runtime(fake_runtime):
    rc, out, _ = run("inspect", "rocm", driver=fake_runtime)
    assert rc == 0 and out.startswith("rocm: available\ndevice_count: >=1\n\ndevice 0:\n")
    assert "  name: fake-gfx950\n" in out and "kernel_bundle: admitted\n" in out
    assert out.endswith("\nstatus: rocm-info\n")
    rc, out, _ = run("inspect", "rocm", "bandwidth", driver=fake_runtime,
                     extra={"YVEX_TEST_ROCM_BANDWIDTH_BYTES": "1048576"})
    assert rc == 0
    assert out.startswith("rocm_bandwidth_schema: 1\nworking_set_bytes: 1048576\n")
    assert "sample_count: 5\n" in out and "  5: stream_ns=" in out
    assert out.endswith("status: rocm-bandwidth\n")


def test_benchmark_summary_nearest_rank_by_hand():
    # ten samples 1..10 ms, shuffled: rank (10*p+99)//100 -> p50 5th, p90 9th, p95/p99 10th;
    # mean 5.5 ms; population variance 8.25 ms^2 -> 2.872281 ms
    seconds = [0.007, 0.001, 0.010, 0.003, 0.005, 0.002, 0.009, 0.004, 0.008, 0.006]
    got = K.benchmark_summarize(seconds)
    assert got == {"minimum_ns": 1_000_000, "p50_ns": 5_000_000, "p90_ns": 9_000_000,
                   "p95_ns": 10_000_000, "p99_ns": 10_000_000, "maximum_ns": 10_000_000,
                   "mean_ns": 5_500_000, "standard_deviation_ns": 2_872_281}
    # one sample: every percentile is that sample, no spread
    one = K.benchmark_summarize([12.5e-6], prefix="device_")
    assert one == {"device_minimum_ns": 12_500, "device_p50_ns": 12_500, "device_p90_ns": 12_500,
                   "device_p95_ns": 12_500, "device_p99_ns": 12_500, "device_maximum_ns": 12_500,
                   "device_mean_ns": 12_500, "device_standard_deviation_ns": 0}
    # 101 samples 1..101 us: ranks 51, 91, 96, 100
    many = K.benchmark_summarize([i * 1e-6 for i in range(101, 0, -1)])
    assert (many["p50_ns"], many["p90_ns"], many["p95_ns"], many["p99_ns"]) == (51_000, 91_000, 96_000, 100_000)


def test_benchmark_summary_refuses_bad_samples():
    for bad in ([], [0.0, 1.0], [1.0, -1.0], [float("nan")], [float("inf")], [1e-12]):
        with pytest.raises(K.YvexError) as e:
            K.benchmark_summarize(bad)
        assert e.value.code == B.YVEX_ERR_BOUNDS and e.value.where == "runtime.benchmark"


def test_library_loads_and_refuses_without_any_hip_runtime():
    """The library reaches the HIP runtime through dlopen only (no DT_NEEDED entry for it), so on
    a machine without the runtime the program still starts, the backend answers "unsupported"
    and the commands exit with 5 (tests/test_cuda_failclosed.sh:46-79 of the reference asks the
    same of the CUDA arm).  Here: no library search path at all and a runtime name that does
    not exist."""
    library = os.path.join(ROOT, "clori_amd", "libyvex_rocm.so")
    needed = subprocess.run(["readelf", "-d", library], capture_output=True, text=True, check=True).stdout
    needed = [line for line in needed.splitlines() if "(NEEDED)" in line]
    assert needed and not any("hip" in line.lower() or "hsa" in line.lower() for line in needed), needed
    bare = {"LD_LIBRARY_PATH": "", "PATH": os.environ.get("PATH", "")}
    for arguments in (("inspect", "backend", "rocm"), ("inspect", "rocm")):
        env = dict(bare, YVEX_TEST_ROCM_DRIVER_LIBRARY="/nonexistent/libamdhip64.so")
        done = subprocess.run([PROGRAM, *arguments], env=env, capture_output=True, text=True, timeout=60)
        assert done.returncode == 5, (arguments, done.stdout, done.stderr)
        assert "unsupported" in done.stdout or "unavailable" in done.stdout


def test_scratch_companion_is_the_only_object_linked_against_the_runtime():
    """The fixed device array of the entry point that allocates nothing sits in its own shared
    object beside the library; that object, and nothing else, names the HIP runtime."""
    companion = os.path.join(ROOT, "clori_amd", "libyvex_rocm_scratch.so")
    if not os.path.exists(companion):
        pytest.skip("the companion object is not built")
    needed = subprocess.run(["readelf", "-d", companion], capture_output=True, text=True, check=True).stdout
    assert "libamdhip64" in needed
    symbols = subprocess.run(["nm", "-D", "--defined-only", companion], capture_output=True, text=True,
                             check=True).stdout
    assert "yvex_rocm_static_scratch_resolve" in symbols
