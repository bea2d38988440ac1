"""The bag kernel's launch plan on the CPU: tests/cpp/bag_plan_test.cpp walks every workgroup
number of ~900 plans (the 26-table configuration, tables of mixed bag lengths, 1 .. 70 tables of
ragged sizes, per-table run sizes on / off, devices of 1 .. 16 dies) through the decode the kernel
itself uses and checks that every bag is reduced exactly once and nothing reaches past the bags,
the per-die segments or the LDS carve-up.  Built here with g++ and the address / undefined-
behaviour sanitizers from the same sources the library compiles (no GPU, no HIP)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bag_plan_test")
SOURCES = ["forward_amd/csrc/status.cpp", "forward_amd/csrc/kernels/bag_plan.cpp", "tests/cpp/bag_plan_test.cpp"]


def test_every_bag_of_every_plan_is_reduced_exactly_once():
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Wextra", "-Werror", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-I" + os.path.join(ROOT, "include")]
    cmd += [os.path.join(ROOT, s) for s in SOURCES] + ["-o", BIN]
    b = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert b.returncode == 0, b.stderr
    # a library preloaded into every process of this machine would otherwise trip the sanitizer's
    # "runtime does not come first" start-up check
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    p = subprocess.run([BIN], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0 and "0 failures" in p.stdout, p.stdout[-2000:] + p.stderr[-4000:]
