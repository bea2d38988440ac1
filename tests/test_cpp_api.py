"""Runs the C++ host program that drives the plugin classes through include/fwdmi_plugin.h the
way the reference's layer creator and TensorRT do (tests/cpp/plugin_cpp_test.cpp, built by
`make -C forward_amd/csrc cpptest` / `__graft_entry__.build()`)."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "plugin_cpp_test")


def run(mode):
    assert os.path.exists(BIN), "build it first: make -C forward_amd/csrc cpptest"
    p = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and "PASS" in p.stdout, p.stdout + p.stderr


def test_cpp_plugin_interface_host_side():
    run("host")


@pytest.mark.gpu
def test_cpp_plugin_interface_on_device():
    run("gpu")
