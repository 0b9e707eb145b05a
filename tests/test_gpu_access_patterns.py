"""The measurement program behind the transposed plans (tests/cpp/transposed_access_patterns.hip) runs, and
the two hardware facts the planner relies on hold on this device: whole 128-byte lines load faster than
half lines shared between workgroups, and whole-row stores beat 128-byte pieces of eight rows."""
import re
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

BIN = Path(__file__).resolve().parent.parent / "hpt_amd" / "lib" / "transposed_access_patterns"


def test_access_pattern_ceilings(dev):
    assert BIN.exists(), f"{BIN} is missing: build it with `python -m hpt_amd.build`"
    r = subprocess.run([str(BIN)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    print(r.stdout)
    us = {m.group(1).strip(): float(m.group(2)) for m in re.finditer(r"^(.*?)\s+([0-9.]+) us", r.stdout, re.M)}
    assert len(us) == 10, r.stdout
    launch = us["launch only"]
    assert 0.5 < launch < 20
    half, whole = us["load 1: 64 B segments, line partners on one XCD"], us["load 2: whole 128 B lines, 64 rows x 2048 cols"]
    assert whole < half, f"whole lines {whole} us, half lines {half} us"
    pieces, rows = us["store 2: 8 rows x 128 B per instruction"], us["store 3: 1 row x 1 KiB per instruction, non-temporal"]
    assert rows < pieces, f"whole rows {rows} us, 128-byte pieces {pieces} us"
