"""The dispatch layer of libphysattn (shape checks, workspace plans, argument errors) under ASan + UBSan.

hipcc compiles the library's own sources with the sanitizers on the host pass only (the device code is untouched and
never runs: there is no GPU here) and links them with tests/host_sanitize_main.cpp into one executable, which walks
the query / workspace functions over a wide grid of shapes (extreme ones included) and the argument-error paths of the
compute entry points.  Any sanitizer report aborts the run.
"""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from physicsnemo_amd import build as pa_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SAN = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
       "-Xarch_host", "-fno-sanitize-recover=undefined"]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not found")
def test_dispatch_layer_is_clean_under_host_sanitizers(tmp_path):
    flags = [f for f in pa_build.HIPCC_FLAGS if not f.startswith("-O")] + ["-O1", "-g"]
    srcs = [os.path.join(pa_build.CSRC, s) for s in pa_build.SOURCES] + [os.path.join(ROOT, "tests", "host_sanitize_main.cpp")]
    objs = [str(tmp_path / (os.path.basename(s) + ".o")) for s in srcs]

    def compile_one(pair):
        src, obj = pair
        lang = ["-x", "hip"] if src.endswith(".cpp") else []
        proc = subprocess.run([HIPCC, *flags, *SAN, *lang, "-c", src, "-o", obj], capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr[-4000:]

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    exe = str(tmp_path / "host_sanitize")
    link = subprocess.run([HIPCC, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize",
                           *objs, "-o", exe], capture_output=True, text=True)
    assert link.returncode == 0, link.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-6000:])
    assert "0 failures" in run.stdout
    shutil.rmtree(tmp_path, ignore_errors=True)
