"""The C-ABI library loads without a GPU and exports exactly what include/fwdmi.h declares."""
import os
import re
import subprocess

import numpy as np
import pytest

from forward_amd import lib


def declared_symbols():
    text = open(lib.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(fwdmi_[a-z0-9_]+)\s*\(", text))


def test_header_matches_binding_table():
    assert declared_symbols() == set(lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    out = subprocess.check_output(["nm", "-D", "--defined-only", lib.LIB_PATH], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    missing = declared_symbols() - exported
    assert not missing, missing
    extra = {s for s in exported if s.startswith("fwdmi_")} - declared_symbols()
    assert not extra, extra


def test_basic_calls_without_gpu():
    assert lib.dll.fwdmi_version().startswith(b"fwdmi")
    assert lib.dll.fwdmi_device_count() >= 0
    assert lib.dll.fwdmi_registry_size() == 6


def test_launchers_validate_before_touching_the_gpu():
    import ctypes as C
    x = lib.BagExt()
    x.table_dtype, x.index_dtype, x.out_dtype = lib.I8, lib.I32, lib.F32
    rc = lib.dll.fwdmi_embedding_bag(None, None, None, 0, 4, None, 10, 8, 0, 0, C.byref(x), None)
    assert rc == lib.ERR_UNSUPPORTED and "dtype" in lib.last_error()
    rc = lib.dll.fwdmi_embedding_bag(None, None, None, 0, 4, None, 10, 8, 0, 7, None, None)
    assert rc == lib.ERR_UNSUPPORTED
    rc = lib.dll.fwdmi_embedding_bag(None, None, None, 0, 4, None, 10, 8, 0, 0, None, None)
    assert rc == lib.ERR_BAD_ARG                       # null output
    rc = lib.dll.fwdmi_embedding_bag(None, None, None, 0, 0, None, 10, 8, 0, 0, None, None)
    assert rc == lib.OK                                # zero bags: nothing to do
    rc = lib.dll.fwdmi_embedding_bag(None, None, None, 0, 4, None, 10, (1 << 24) + 1, 0, 0, None, None)
    assert rc == lib.ERR_BAD_ARG and "dim" in lib.last_error()
    rc = lib.dll.fwdmi_embedding_bag_fixed(None, None, 1 << 40, 1 << 40, None, 10, 8, 0, 0, None, None)
    assert rc == lib.ERR_BAD_ARG                       # batch x length leaves 64 bits
    rc = lib.dll.fwdmi_gather(None, None, 1 << 62, 4, None, 10, 8, 0, None, None)
    assert rc == lib.ERR_BAD_ARG
    rc = lib.dll.fwdmi_layer_norm(None, 10, 25, None, None, None, None, None, lib.F32, 0.0)
    assert rc == lib.ERR_BAD_ARG and "multiple" in lib.last_error()
    rc = lib.dll.fwdmi_layer_norm(None, 10, 20, None, None, None, None, None, lib.I8, 0.0)
    assert rc == lib.ERR_UNSUPPORTED
    rc = lib.dll.fwdmi_emb_layer_norm(None, 4, 2, 8, None, None, None, None, None, None, None, None, 1, 1, 1, None,
                                      None, lib.F16, 0.0, None)
    assert rc == lib.ERR_BAD_ARG


def test_table_cost_estimate():
    import ctypes as C
    nbytes = np.array([1 << 10, 2 << 20, 32 << 20, 512 << 20, 8 << 30], np.int64)
    cost = np.zeros(5, np.float32)
    assert lib.dll.fwdmi_bag_table_cost(nbytes.ctypes.data, 5, cost.ctypes.data) == 0
    assert cost[0] == 1.0 and cost[1] == 1.0 and cost[3] == cost[4] and 1.0 < cost[2] < cost[3] < 2.0
    np.testing.assert_allclose(cost[2], 1.0 + 0.45 * 0.5, rtol=1e-6)    # 32 MiB is half way in log size
    assert lib.dll.fwdmi_bag_table_cost(None, 5, cost.ctypes.data) == lib.ERR_BAD_ARG


def test_c_header_is_plain_c(tmp_path):
    """include/fwdmi.h is what a C host (cgo, JNI glue, plain C) includes: it must compile as C99."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "fwdmi.h"\n'
                   'int main(void) { fwdmi_bag_ext e = {0}; fwdmi_bag_table t = {0}; (void)e; (void)t;\n'
                   '  return FWDMI_BAG_INLINE_TABLES > 0 && FWDMI_OP_SUM == 0 ? 0 : 1; }\n')
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    p = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, "-fsyntax-only", str(src)],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
