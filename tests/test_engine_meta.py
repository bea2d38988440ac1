"""The engine sidecar ("<engine>.meta"), typed: reader and writer of the library against (a) fixtures
written by the reference's own JSON library (tests/golden/meta/, made by make_meta_fixtures.py),
byte for byte and member for member, (b) what trt_meta_data.cpp:49-79 accepts and rejects, and
(c) where oracle/_ref/meta_ref is built (the reference tree is present), that program live: files
written by one side read by the other, and the same verdict on a battery of malformed documents."""
import importlib.util
import json
import os
import subprocess

import numpy as np
import pytest

from forward_amd import lib, plugin
from forward_amd.plugin import EngineMetaData

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "meta")
REF = os.path.join(ROOT, "oracle", "_ref", "meta_ref")

_spec = importlib.util.spec_from_file_location("make_meta_fixtures", os.path.join(ROOT, "tests", "golden",
                                                                                  "make_meta_fixtures.py"))
_fx = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_fx)
CASES = _fx.CASES

GOOD = {"infer_mode": 1, "opt_batch_size": 8, "max_batch_size": 16, "unused_input_indices": [2], "output_indices": [1, 0],
        "torch_module_path": "m.pth"}


def meta_of(case):
    mode, opt, mx, unused, outs, path = case
    return EngineMetaData(mode, opt, mx, unused, outs, path)


@pytest.mark.parametrize("name", sorted(CASES))
def test_writer_and_reader_against_files_of_the_reference_json_library(name, tmp_path):
    want = open(os.path.join(GOLDEN, name + ".meta"), "rb").read()
    m = meta_of(CASES[name])
    assert m.to_json().encode() == want
    out = str(tmp_path / "x.meta")
    m.SaveMetaData(out)
    assert open(out, "rb").read() == want
    back = EngineMetaData.LoadMetaData(os.path.join(GOLDEN, name + ".meta"))
    assert back == m
    assert back.unused_input_indices == sorted(set(CASES[name][3]))      # a set in the reference: ascending
    assert back.output_indices == CASES[name][4]                         # a vector: the order is kept


def test_defaults_are_the_reference_defaults():
    m = EngineMetaData()
    assert (m.infer_mode, m.opt_batch_size, m.max_batch_size) == (0, -1, -1)      # trt_meta_data.h:75-79
    assert m.unused_input_indices == [] and m.output_indices == [] and m.torch_module_path == ""
    assert EngineMetaData("float16").infer_mode == 1 and EngineMetaData("int8_calib").infer_mode == 3


# (document, loads?) -- what value.get<int>() / get<std::string>() / iteration accept, trt_meta_data.cpp:59-70
BATTERY = [
    (GOOD, True),
    ({k: v for k, v in GOOD.items() if k != "infer_mode"}, False),
    ({k: v for k, v in GOOD.items() if k != "opt_batch_size"}, False),
    ({k: v for k, v in GOOD.items() if k != "max_batch_size"}, False),
    ({k: v for k, v in GOOD.items() if k != "torch_module_path"}, False),
    ({k: v for k, v in GOOD.items() if k != "unused_input_indices"}, True),      # iterating null: empty
    ({k: v for k, v in GOOD.items() if k != "output_indices"}, True),
    (dict(GOOD, infer_mode="float16"), False),                                   # a string is no int
    (dict(GOOD, infer_mode=None), False),
    (dict(GOOD, infer_mode=[1]), False),
    (dict(GOOD, infer_mode=1.75), True),                                         # a fraction is cut off
    (dict(GOOD, opt_batch_size=True), True),                                     # booleans convert
    (dict(GOOD, max_batch_size="16"), False),
    (dict(GOOD, torch_module_path=7), False),
    (dict(GOOD, torch_module_path=None), False),
    (dict(GOOD, output_indices=[0, "1"]), False),
    (dict(GOOD, output_indices=[0, 2.5]), True),
    (dict(GOOD, unused_input_indices=[5, 5, 1]), True),                          # repeats collapse
    (dict(GOOD, extra_key={"nested": [1, 2, {"a": None}]}), True),               # unknown keys are ignored
]


@pytest.mark.parametrize("case", range(len(BATTERY)))
def test_reader_accepts_and_rejects_what_the_reference_reader_does(case, tmp_path):
    doc, loads = BATTERY[case]
    path = str(tmp_path / "m.meta")
    open(path, "w").write(json.dumps(doc))
    if loads:
        m = EngineMetaData.LoadMetaData(path)
        assert m.infer_mode == int(doc["infer_mode"]) and m.opt_batch_size == int(doc["opt_batch_size"])
        assert m.output_indices == [int(v) for v in doc.get("output_indices", [])]
        assert m.unused_input_indices == sorted(set(int(v) for v in doc.get("unused_input_indices", [])))
    else:
        with pytest.raises(lib.FwdmiError, match="engine meta data"):
            EngineMetaData.LoadMetaData(path)
    if os.path.exists(REF):                       # the reference's JSON library gives the same verdict
        got = subprocess.run([REF, "read", path], capture_output=True, text=True, timeout=30).stdout.split()
        assert (got[0] == "ok") == loads, got
        if loads:
            assert [int(v) for v in got[1:4]] == [m.infer_mode, m.opt_batch_size, m.max_batch_size]


@pytest.mark.parametrize("text", ["", "{", "[1, 2]", '{"infer_mode": 1,}', '{"infer_mode": 01}', "not json",
                                  '{"infer_mode": 1} trailing', '{"a": "\\x"}', '{"a": "\\ud800"}'])
def test_text_that_is_not_a_json_object_fails(text, tmp_path):
    path = str(tmp_path / "bad.meta")
    open(path, "w").write(text)
    with pytest.raises(lib.FwdmiError, match="engine meta data"):
        EngineMetaData.LoadMetaData(path)
    with pytest.raises(lib.FwdmiError):
        EngineMetaData.LoadMetaData(str(tmp_path / "absent.meta"))


def test_string_escapes_and_number_forms(tmp_path):
    path = str(tmp_path / "e.meta")
    open(path, "w").write('{"infer_mode": 1e0, "opt_batch_size": -0, "max_batch_size": 2.0E1, '
                          '"torch_module_path": "a\\"b\\\\c\\/d\\n\\u00e9\\ud83d\\ude00\\t", "output_indices": [ ]}')
    m = EngineMetaData.LoadMetaData(path)
    assert (m.infer_mode, m.opt_batch_size, m.max_batch_size) == (1, 0, 20)
    assert m.torch_module_path == 'a"b\\c/d\né\U0001F600\t'
    again = EngineMetaData.from_dict(json.loads(m.to_json()))           # what is written reads back the same
    assert again == m
    for bad in (2 ** 31, -2 ** 31 - 1, 1e30):                               # no int holds it: refused, not wrapped
        with pytest.raises(lib.FwdmiError, match="not an integer"):
            EngineMetaData.from_dict(dict(GOOD, max_batch_size=bad))


@pytest.mark.skipif(not os.path.exists(REF), reason="oracle/_ref/meta_ref is built only where the reference tree is present")
def test_files_cross_between_the_library_and_the_reference_json_library(tmp_path):
    rng = np.random.Generator(np.random.PCG64(5))
    for i in range(40):
        unused = sorted(set(int(v) for v in rng.integers(0, 12, rng.integers(0, 5))))
        outs = [int(v) for v in rng.integers(0, 9, rng.integers(0, 6))]
        path_text = "".join(rng.choice(list("abc/_. -\"\\"), rng.integers(0, 12)))
        m = EngineMetaData(int(rng.integers(0, 4)), int(rng.integers(-1, 70000)), int(rng.integers(-1, 70000)), unused,
                           outs, path_text)
        ours, theirs = str(tmp_path / ("o%d.meta" % i)), str(tmp_path / ("t%d.meta" % i))
        m.SaveMetaData(ours)
        subprocess.check_call([REF, "write", theirs, str(m.infer_mode), str(m.opt_batch_size), str(m.max_batch_size),
                               ",".join(map(str, unused)), ",".join(map(str, outs)), path_text])
        assert open(ours, "rb").read() == open(theirs, "rb").read()
        assert EngineMetaData.LoadMetaData(theirs) == m
        got = subprocess.run([REF, "read", ours], capture_output=True, text=True, timeout=30).stdout
        assert got.startswith("ok %d %d %d " % (m.infer_mode, m.opt_batch_size, m.max_batch_size)), got


def test_reader_survives_mutated_sidecars_under_the_sanitizers():
    """tests/cpp/engine_meta_mutation_test.cpp: 300 000 seeded mutations of valid sidecars and nesting
    200 000 levels deep through the reader, built with the address / undefined-behaviour sanitizers from
    the sources the library compiles; what the reader accepts must survive its own writer unchanged."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "engine_meta_mutation_test")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Wextra", "-Werror", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-I" + os.path.join(root, "include")]
    cmd += [os.path.join(root, s) for s in ("forward_amd/csrc/status.cpp", "forward_amd/csrc/plugins/engine_meta.cpp",
                                            "tests/cpp/engine_meta_mutation_test.cpp")] + ["-o", exe]
    b = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert b.returncode == 0, b.stderr
    # a library preloaded into every process of this machine would otherwise trip the sanitizer's
    # "runtime does not come first" start-up check
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    p = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0 and " 0 failures" in p.stdout, p.stdout[-2000:] + p.stderr[-4000:]
