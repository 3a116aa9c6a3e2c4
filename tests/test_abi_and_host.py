"""No-GPU checks of the boundary: the shared library loads and exports every symbol the header
declares, the Python signature table covers them all, and the C++ host layer's device-free tests pass."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_TESTS = os.path.join(ROOT, "deep8_amd", "host", "deep8_host_tests")


def _declared():
    text = open(os.path.join(ROOT, "include", "deep8_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(d8_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import ctypes
    from deep8_amd import capi
    names = _declared()
    assert len(names) >= 40
    lib = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.SIGNATURES) == names
    capi.load()


def test_missing_library_fails_loudly(monkeypatch):
    from deep8_amd import capi
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", os.path.join(ROOT, "deep8_amd", "no_such_library.so"))
    with pytest.raises(capi.Deep8HipError):
        capi.load()


def test_product_never_imports_the_oracle():
    """Nothing under deep8_amd/ or include/ may refer to the CPU checkers."""
    for base, _, files in os.walk(os.path.join(ROOT, "deep8_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")) or f == "Makefile":
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(base, f)


def test_host_layer_device_free_tests():
    assert os.path.exists(HOST_TESTS), "build the host layer first (__graft_entry__.build())"
    out = subprocess.run([HOST_TESTS, "--cpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "PASS half_conversion" in out.stdout and "PASS node_shape_inference" in out.stdout
    listed = subprocess.run([HOST_TESTS, "--list"], capture_output=True, text=True, timeout=60).stdout
    assert "gpu matrix_multiply_float_collapsed_batch" in listed and "gpu eager_executor_matmul_chain" in listed


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "ONE GPU" in out.stderr


def test_cpu_pieces_run_clean_under_the_sanitizers():
    """The oracle's C restatement and the host layer's device-free tests under AddressSanitizer +
    UndefinedBehaviorSanitizer (`make asan` in oracle/ and deep8_amd/host/): any report aborts the run."""
    import shutil
    import subprocess
    if not shutil.which("make") or not shutil.which("gcc") or not shutil.which("g++"):
        pytest.skip("no host toolchain")
    for where in ("oracle", os.path.join("deep8_amd", "host")):
        r = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, where), "asan"], capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, (where, r.stdout[-2000:], r.stderr[-2000:])
        assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, (where, r.stderr[-2000:])


def test_bench_reads_its_traffic_figures_from_the_committed_profiles():
    """bench.py must import without a GPU, and every workload that reports `traffic` must find its rows in the
    rocprofv3 summary under profiles/ (a renamed kernel or a regenerated summary would otherwise turn it into null)."""
    import bench
    for key, (fname, rows) in bench.TRAFFIC_ROWS.items():
        assert os.path.exists(os.path.join(ROOT, "profiles", fname)), fname
        parts = list(rows) if isinstance(rows, dict) else [None]
        for part in parts:
            t = bench.profile_traffic(key, part)
            assert t is not None and t["bytes"] > 0, (key, part)
    # the algorithmic bytes of the im2col launch at configuration 4's size are what the counters saw
    assert abs(bench.profile_traffic("i4", "im2col")["bytes"] - 256.9e6) < 2e6


def test_planner_keeps_the_plans_of_the_benchmark_configs():
    """The split planner's choices for the benchmark configurations (bench.py workloads c2a, c2b, c3, c4, c5), read off the scratch queries (host code only; with
    no device the planner assumes the MI355X's 256 CUs): a change of its rules or constants that moves one of them
    shows up here before it shows up in a benchmark."""
    import ctypes
    from deep8_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name, (res, args) in capi.SIGNATURES.items():
        if name.endswith("scratch_bytes") or name == "d8_gemm_workspace_bytes":
            getattr(lib, name).restype, getattr(lib, name).argtypes = res, args
    F16, F32 = capi.FLOAT16, capi.FLOAT32
    # C2b's dY: 512 x 512 over 16 384 in 16 pieces
    assert lib.d8_matmul_scratch_bytes(F32, 2, 32, 512, 512, 1, 512, 512) == 16 * 512 * 512 * 4
    # C2a and C3: whole
    assert lib.d8_matmul_scratch_bytes(F32, 2, 32, 512, 512, 32, 512, 512) == 0
    assert lib.d8_matmul_scratch_bytes(F16, 2, 1, 4096, 4096, 1, 4096, 4096) == 0
    # C4: the remainder band of 2048 rows in nine pieces (forward, dX), dW on 64 x 64 tiles in 85 pieces
    c4 = (32, 56, 56, 64, 64, 3, 3, 1, 1, 1, 1, 1)
    assert lib.d8_conv2d_scratch_bytes(F32, 0, *c4) == 9 * 2048 * 64 * 4
    assert lib.d8_conv2d_scratch_bytes(F32, 1, *c4) == 9 * 2048 * 64 * 4
    assert lib.d8_conv2d_scratch_bytes(F32, 2, *c4) == 85 * 64 * 576 * 4
    # C5: forward by classes and dX on half tiles stage nothing, dW in 22 pieces
    c5 = (16, 28, 28, 128, 64, 4, 4, 0, 2, 2)
    assert lib.d8_deconv2d_scratch_bytes(F16, 0, *c5) == 0
    assert lib.d8_deconv2d_scratch_bytes(F16, 1, *c5) == 0
    assert lib.d8_deconv2d_scratch_bytes(F16, 2, *c5) == 22 * 1024 * 128 * 4
