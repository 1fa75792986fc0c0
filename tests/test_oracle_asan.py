"""The oracle's C++ under AddressSanitizer + UndefinedBehaviorSanitizer (CPU): `make -C oracle asan-test` on the
distance, merge/search and knowledge-graph tests. The whole oracle suite runs the same way by hand (`make -C oracle
asan-test`, about three minutes); this keeps a slice of it in the CPU suite."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_is_clean_under_sanitizers():
    env = dict(os.environ)
    env.pop("APOE_ORACLE_LIB", None)
    out = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "asan-test",
                          "ASAN_TESTS=../tests/test_oracle_distance.py ../tests/test_oracle_merge_search.py ../tests/test_oracle_kg.py"],
                         capture_output=True, text=True, env=env, timeout=900)
    text = out.stdout + out.stderr
    assert out.returncode == 0, text[-4000:]
    assert "ERROR: AddressSanitizer" not in text and "runtime error" not in text, text[-4000:]
    assert " passed" in text
