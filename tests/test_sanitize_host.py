"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer: the engine (host-only mode), the
C-ABI and the wire front end's message handlers are compiled with the sanitizers on the host pass
and fed well-formed, mutated and random messages (tests/native/fuzz_wire.cpp).  CPU only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = "/opt/rocm/bin/hipcc"
# the engine's host translation units (the Makefile's .cpp sources)
HOST_SOURCES = ("engine.cpp", "engine_swap.cpp", "engine_request.cpp", "engine_exec.cpp", "capi.cpp")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_wire_handlers_and_engine_under_sanitizers(tmp_path):
    csrc = os.path.join(ROOT, "torpor_amd", "csrc")
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined"]
    flags = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops"] + san
    objs = []
    # the kernels come from the regular build (device code is not instrumented); host files are rebuilt
    for src in HOST_SOURCES:
        o = str(tmp_path / (src + ".o"))
        subprocess.check_call([HIPCC] + flags + ["-x", "hip", "-c", os.path.join(csrc, src), "-o", o],
                              stderr=subprocess.DEVNULL)
        objs.append(o)
    for k in ("gemm", "conv", "winograd", "ops", "attention"):
        o = os.path.join(ROOT, "build", "obj", "kernels", k + ".hip.o")
        if not os.path.exists(o):
            pytest.skip("kernel objects not built (run make -C torpor_amd/csrc)")
        objs.append(o)
    drv = str(tmp_path / "fuzz_wire.o")
    subprocess.check_call([HIPCC] + flags + ["-x", "hip", "-c", os.path.join(ROOT, "tests", "native", "fuzz_wire.cpp"),
                                             "-o", drv], stderr=subprocess.DEVNULL)
    exe = str(tmp_path / "fuzz_wire")
    # link step: the sanitizer runtimes for the host objects only (device code is never instrumented)
    subprocess.check_call([HIPCC, "--offload-arch=gfx950"] + san + ["-o", exe, drv] + objs + ["-lpthread"],
                          stderr=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TORPOR_IPC_DIR=str(tmp_path))
    r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "fuzz ok" in r.stdout, (r.stdout[-2000:], r.stderr[-4000:])
    shutil.rmtree(tmp_path, ignore_errors=True)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_c_abi_from_three_threads_under_thread_sanitizer(tmp_path):
    """A controller, an executor and an observer thread on one host-only engine (tests/native/race_abi.cpp),
    host code built with ThreadSanitizer: no report, and the run must have reached swap-ins and evictions."""
    csrc = os.path.join(ROOT, "torpor_amd", "csrc")
    san = ["-Xarch_host", "-fsanitize=thread"]
    flags = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops"] + san
    objs = []
    for k in ("gemm", "conv", "winograd", "ops", "attention"):
        o = os.path.join(ROOT, "build", "obj", "kernels", k + ".hip.o")
        if not os.path.exists(o):
            pytest.skip("kernel objects not built (run make -C torpor_amd/csrc)")
        objs.append(o)
    for src in [os.path.join(csrc, f) for f in HOST_SOURCES] + [os.path.join(ROOT, "tests", "native", "race_abi.cpp")]:
        o = str(tmp_path / (os.path.basename(src) + ".o"))
        subprocess.check_call([HIPCC] + flags + ["-x", "hip", "-c", src, "-o", o], stderr=subprocess.DEVNULL)
        objs.append(o)
    exe = str(tmp_path / "race_abi")
    subprocess.check_call([HIPCC, "--offload-arch=gfx950"] + san + ["-o", exe] + objs + ["-lpthread"],
                          stderr=subprocess.DEVNULL)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:exitcode=66")
    env.pop("EXECUTOR_LOG_LEVEL", None)
    r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "race ok" in r.stdout and "ThreadSanitizer" not in r.stderr, \
        (r.returncode, r.stdout[-2000:], r.stderr[-4000:])
    shutil.rmtree(tmp_path, ignore_errors=True)
