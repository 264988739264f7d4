"""The arithmetic short cut of the int8 append for binary16 rows, checked on the CPU over its whole
domain: tests/cpp/i8h_f16_codes_exhaustive.c walks every (block amax, value) pair of binary16
numbers and compares the code the kernel's fused multiply-add produces (with reciprocals one ulp
off either way) against the rule round-half-away(clamp(x / scale)).  Host code only."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "cpp", "i8h_f16_codes_exhaustive.c")
BIN = os.path.join(HERE, "cpp", "i8h_f16_codes_exhaustive")


def test_biased_reciprocal_codes_equal_the_rule_for_every_binary16_pair():
    if not os.path.exists(BIN) or os.path.getmtime(BIN) < os.path.getmtime(SRC):
        subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", SRC, "-o", BIN, "-lm"], check=True)
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    pairs = int(r.stdout.split()[0])
    # 22527 amax codes above 2^-6, every code up to the amax, both signs
    assert pairs > 900_000_000, r.stdout
    assert "all codes equal the rule's" in r.stdout
