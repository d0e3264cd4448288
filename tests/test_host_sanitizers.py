"""The library's host-only C++ (bundle reader with its own JSON parser, the threaded quantisers)
under AddressSanitizer and UndefinedBehaviorSanitizer: thousands of damaged meta.json files
(truncated, bytes flipped, holes, stray tokens, offsets and sizes past the file) must be refused or
opened without a single sanitizer report, and the quantisers must take zero rows, NaN / inf bit
patterns and the Q4 block-size refusal without one.  CPU only; the device half is stubbed out."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_bundle_reader_and_quantisers_under_sanitizers(tmp_path):
    exe = str(tmp_path / "drv")
    cmd = ["g++", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-fno-omit-frame-pointer", "-std=c++17", "-I", os.path.join(ROOT, "include"), "-o", exe,
           os.path.join(ROOT, "tests", "host_sanitizer_driver.cpp"),
           os.path.join(ROOT, "adreno-llms_amd", "csrc", "quantize.cpp"),
           os.path.join(ROOT, "adreno-llms_amd", "csrc", "bundle.cpp"), "-lpthread"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    if build.returncode != 0 and "sanitize" in build.stderr and "cannot find" in build.stderr:
        pytest.skip("this g++ has no sanitizer runtime")
    assert build.returncode == 0, build.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0")
    run = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, run.stderr[-3000:]
    assert "AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr, run.stderr[-3000:]
    assert "good bundle" in run.stdout and "3 tensors" in run.stdout
    last = run.stdout.strip().splitlines()[-1]           # "mutated metas: A opened, B refused"
    opened, refused = int(last.split()[2]), int(last.split()[4])
    assert opened + refused == 6000 and refused > 3000
