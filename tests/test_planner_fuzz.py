"""The launch planners (hpt_amd/csrc/layout.cpp) under AddressSanitizer and
UndefinedBehaviorSanitizer on the host: tests/cpp/planner_fuzz.cpp feeds them random views
(permuted, sliced with steps of either sign, broadcast, off the 16-byte grid, dims up to
2^32 + 5) and checks that every plan keeps the view's element counts and a launch shape the
kernels accept. Pure host code: no GPU, no HIP runtime."""
import pathlib
import shutil
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parents[1]


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_planners_clean_under_sanitizers(tmp_path):
    exe = tmp_path / "planner_fuzz"
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           f"-I{ROOT / 'include'}", f"-I{ROOT / 'hpt_amd' / 'csrc'}", "-I/opt/rocm/include",
           "-D__HIP_PLATFORM_AMD__", "-x", "c++", str(ROOT / "hpt_amd" / "csrc" / "layout.cpp"),
           str(ROOT / "tests" / "cpp" / "planner_fuzz.cpp"), "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-4000:]
    for seed in (1, 2, 3):
        r = subprocess.run([str(exe), "100000", str(seed)], capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, f"seed {seed}:\n{r.stdout[-2000:]}\n{r.stderr[-6000:]}"
