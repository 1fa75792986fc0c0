"""bench/membench runs and reports sane ceilings (needs the GPU): what bench.py puts beside its roofline."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

EXE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench", "membench")


def test_membench_reports_chunk_read_rates():
    assert os.path.exists(EXE), "membench is not built: make -C bench"
    out = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    rates = {int(m.group(1)): float(m.group(2)) for m in re.finditer(r"random reads,\s+(\d+) B chunks, .*:\s+(\d+) GB/s", out.stdout)}
    assert set(rates) == {256, 512, 768, 1024, 2048, 5120}
    # longer chunks are never slower per byte, nothing beats the 8 TB/s streaming peak, and 1 KiB chunks get a fair share of it
    assert rates[256] < rates[512] < rates[1024] <= rates[5120] * 1.05 < 8000 * 1.05
    assert rates[1024] > 3000
    with_atomics = [float(m.group(1)) for m in re.finditer(r"returning atomics per chunk:\s+(\d+) GB/s", out.stdout)]
    assert len(with_atomics) == 3 and max(with_atomics) < rates[1024]
