"""The host-side rules (ratchet_amd/csrc/spec.cpp) and the GGUF parser (gguf.cpp) built with
g++ -fsanitize=address,undefined and driven over hostile inputs (tests/host_sanitize_driver.cpp):
truncated and corrupted images, wrapping tensor offsets, descriptors with out-of-range ranks, dtypes
and extents.  No HIP is involved: the parser is compiled with -DRT_HOST_ONLY."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ratchet_amd", "csrc")
G = os.path.join(ROOT, "tests", "golden")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_parser_and_shape_rules_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_sanitize")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-DRT_HOST_ONLY", os.path.join(ROOT, "tests", "host_sanitize_driver.cpp"),
           os.path.join(CSRC, "spec.cpp"), os.path.join(CSRC, "gguf.cpp"), "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)   # the sanitizer runtime must come first in the process
    images = [os.path.join(G, f"gguf_v{v}.gguf") for v in (1, 2, 3)]
    res = subprocess.run([exe, *images], capture_output=True, text=True, env=env, timeout=600)
    assert res.returncode == 0, res.stderr[-4000:]
    assert res.stdout.startswith("ok "), res.stdout
    fields = dict(kv.split("=") for kv in res.stdout.split()[1:])
    # the run really exercised both outcomes
    assert int(fields["parsed"]) > 100 and int(fields["rejected"]) > 1000
    assert int(fields["ranges_rejected"]) > 0 and int(fields["descriptors"]) == 200000
