"""The C program of allan-poe_amd/examples drives build and search through include/apoe.h alone (no Python, no C++):
it must compile as C99, link against the library, find the brute-force closest document of its queries and report
distances that equal the metric computed on the host."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_example_builds_searches_and_checks_itself(tmp_path):
    import apoe
    libdir = os.path.dirname(apoe.LIB_PATH)
    exe = tmp_path / "c_abi_example"
    subprocess.run(["gcc", "-std=c99", "-O2", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "allan-poe_amd", "examples", "c_abi_example.c"), "-o", str(exe), "-L", libdir, "-lapoe",
                    "-Wl,-rpath," + libdir, "-lm"], check=True, capture_output=True)
    run = subprocess.run([str(exe), "3000", "64", "64"], check=True, capture_output=True, text=True, timeout=120)
    lines = run.stdout.strip().splitlines()
    assert len(lines) == 65 and all(re.match(r"q \d+:( \d+){5} \| -?\d+\.\d+$", ln) for ln in lines[:64]), run.stdout[-500:]
    m = re.match(r"brute-force best document in the pool for (\d+) of 64 queries; reported distance equals the metric for (\d+) of 64", lines[-1])
    assert m, lines[-1]
    assert int(m.group(2)) == 64
    assert int(m.group(1)) >= 60
    assert "ms of GPU time" in run.stderr
