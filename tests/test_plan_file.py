"""Plan files (plugins of an engine in one file + JSON sidecar) and tables kept by file
reference.  The host half runs anywhere; the run-after-load half needs the GPU."""
import json
import os
import struct

import numpy as np
import pytest

from forward_amd import lib, plugin
from forward_amd.plugin import PluginFieldData as F

REG = plugin.getPluginRegistry()
# infer_mode is the number of the reference's InferMode (1 = half), as trt_meta_data.cpp:60,83 reads and writes it
META = {"infer_mode": 1, "max_batch_size": 65536, "opt_batch_size": 65536, "output_indices": [0],
        "unused_input_indices": [], "torch_module_path": "dlrm.pth"}


def bag_fields(table, op=0):
    return [F("dim", table.shape[1]), F("count", table.shape[0]), F("offset", 0), F("op", op), F("data", table)]


def make_layers(rng):
    t = rng.standard_normal((30, 8)).astype(np.float32)
    bag = REG.getPluginCreator("EmbeddingBag_TRT", "001").createPlugin("emb_0", bag_fields(t))
    ln = REG.getPluginCreator("CustomSkipLayerNormPluginDynamic", "1").createPlugin("skip_ln", [
        F("beta", rng.standard_normal(16).astype(np.float32)), F("gamma", rng.standard_normal(16).astype(np.float32)),
        F("ld", 16), F("type_id", lib.F16)])
    ln.setPluginNamespace("bert")
    g16 = [rng.standard_normal((r, 8)).astype(np.float16) for r in (4, 9)]
    group = REG.getPluginCreator("EmbeddingBagGroup_TRT", "001").createPlugin("sparse_stage", [
        F("dim", 8), F("op", 0), F("count", np.array([4, 9], np.int32)),
        F("data", np.concatenate([x.reshape(-1) for x in g16])), F("output_fp16", 1)])
    return [("emb_0", bag), ("encoder_layer_0_skip_layer_norm", ln), ("sparse_stage", group)], t


def test_plan_roundtrip_and_sidecar(tmp_path):
    layers, _ = make_layers(np.random.default_rng(0))
    path = str(tmp_path / "engine.plan")
    plugin.save_plan(path, layers, META)
    raw = open(path, "rb").read()
    assert raw[:8] == b"FWDMIPL1" and struct.unpack("<I", raw[8:12]) == (3,)
    assert json.load(open(path + ".meta")) == META           # keys of trt_meta_data.cpp:42-97
    # the very bytes the reference's JSON library writes for these members (tests/golden/meta/)
    assert open(path + ".meta", "rb").read() == open(os.path.join(os.path.dirname(__file__), "golden", "meta",
                                                                  "dlrm_half.meta"), "rb").read()
    loaded, meta = plugin.load_plan(path)
    assert meta.to_dict() == META and [n for n, _ in loaded] == [n for n, _ in layers]
    # a sidecar the reference's reader rejects is refused before anything is written, and fails a load
    with pytest.raises(lib.FwdmiError, match="infer_mode"):
        plugin.save_plan(str(tmp_path / "bad.plan"), layers, dict(META, infer_mode="float16"))
    assert not os.path.exists(str(tmp_path / "bad.plan"))
    good_meta = open(path + ".meta").read()
    open(path + ".meta", "w").write(good_meta.replace('"max_batch_size": 65536', '"max_batch_size": "many"'))
    with pytest.raises(lib.FwdmiError, match="max_batch_size"):
        plugin.load_plan(path)
    os.remove(path + ".meta")
    assert plugin.load_plan(path)[1] is None                 # no sidecar: a plan without engine settings
    open(path + ".meta", "w").write(good_meta)
    for (_, a), (_, b) in zip(layers, loaded):
        assert (a.getPluginType(), a.getPluginVersion(), a.getPluginNamespace()) == \
               (b.getPluginType(), b.getPluginVersion(), b.getPluginNamespace())
        assert a.serialize() == b.serialize()
    # failure modes: truncated file, foreign file, unknown creator version
    for cut in (0, 7, 11, 40, len(raw) - 1):
        open(path, "wb").write(raw[:cut])
        with pytest.raises(lib.FwdmiError):
            plugin.load_plan(path)
    open(path, "wb").write(b"NOTAPLAN" + raw[8:])
    with pytest.raises(lib.FwdmiError, match="not a plan file"):
        plugin.load_plan(path)
    open(path, "wb").write(raw.replace(b"\x03\x00\x00\x00001", b"\x03\x00\x00\x00009", 1))
    with pytest.raises(lib.FwdmiError, match="no creator"):
        plugin.load_plan(path)
    with pytest.raises(lib.FwdmiError):
        plugin.load_plan(str(tmp_path / "missing.plan"))


def test_table_by_file_reference_host_side(tmp_path):
    rng = np.random.default_rng(1)
    table = rng.standard_normal((100, 16)).astype(np.float16)
    tf = str(tmp_path / "tables.bin")
    with open(tf, "wb") as f:
        f.write(b"\0" * (10 * 16 * 2))                       # ten rows of another table first
        f.write(table.tobytes())
    c = REG.getPluginCreator("EmbeddingBag_TRT", "002")
    path_field = F("data_file", np.frombuffer(tf.encode(), np.int8), lib.FIELD_CHAR)
    fields = [F("dim", 16), F("count", 100), F("offset", 0), F("op", 0), path_field, F("table_type", lib.F16),
              F("data_file_row_offset", 10), F("output_fp16", 1)]
    p = c.createPlugin("emb", fields)
    blob = p.serialize()
    assert len(blob) < 200                                   # a reference, not 3200 bytes of table
    head = struct.unpack("<10iQQ", blob[:56])
    assert head[:10] == (16, 100, 0, 0, lib.F16, lib.I32, lib.F16, 0, 0, 0) and head[10] == 2**64 - 1 and head[11] == len(tf)
    assert blob[56:56 + len(tf)] == tf.encode() and struct.unpack("<Q", blob[-8:]) == (10 * 16 * 2,)
    q = c.deserializePlugin("emb", blob)
    assert q.serialize() == blob and q.clone().serialize() == blob
    # the same table given by value serializes by value
    byval = c.createPlugin("emb", bag_fields(table) + [F("output_fp16", 1)])
    assert byval.serialize()[48:] == table.tobytes()
    # a file that is too short, a missing file, both 'data' and 'data_file'
    with pytest.raises(lib.FwdmiError, match="shorter"):
        c.createPlugin("emb", fields[:6] + [F("data_file_row_offset", 50)])
    # a corrupt file offset in the blob (offset + size would wrap 64 bits) is "too short", not a mapping
    for off in (2**64 - 8, 2**64 - 1, 2**63):
        with pytest.raises(lib.FwdmiError, match="shorter"):
            c.deserializePlugin("emb", blob[:-8] + struct.pack("<Q", off))
    os.remove(tf)
    with pytest.raises(lib.FwdmiError, match="cannot open"):
        c.deserializePlugin("emb", blob)
    with pytest.raises(lib.FwdmiError, match="excludes"):
        c.createPlugin("emb", fields + [F("data", table)])


@pytest.mark.gpu
def test_plan_load_then_run(tmp_path, oracle):
    import torch
    from gpu_util import assert_bits_equal, dev, host
    rng = np.random.default_rng(2)
    table = rng.standard_normal((500, 64)).astype(np.float16)
    tf = str(tmp_path / "t.bin")
    table.tofile(tf)
    c2 = REG.getPluginCreator("EmbeddingBag_TRT", "002")
    ref_plugin = c2.createPlugin("emb_ref", [F("dim", 64), F("count", 500), F("offset", 0), F("op", 0),
                                             F("data_file", np.frombuffer(tf.encode(), np.int8), lib.FIELD_CHAR),
                                             F("table_type", lib.F16), F("output_fp16", 1)])
    layers, t32 = make_layers(rng)
    path = str(tmp_path / "engine.plan")
    plugin.save_plan(path, layers + [("emb_ref", ref_plugin)], META)
    assert os.path.getsize(path) < 4000                      # the 64 KB fp16 table is not inside
    loaded, _ = plugin.load_plan(path)
    lengths = rng.integers(0, 9, 40)
    idx = rng.integers(0, 30, int(lengths.sum())).astype(np.int32)
    off = (np.cumsum(lengths) - lengths).astype(np.int32)
    want, _, _ = oracle.embedding_bag(t32, idx, off, 0)
    assert_bits_equal(host(loaded[0][1](dev(idx), dev(off))), want, "by-value table after load")
    idx2 = rng.integers(0, 500, int(lengths.sum())).astype(np.int32)
    want, _, _ = oracle.embedding_bag(table, idx2, off, 0)
    assert loaded[3][0] == "emb_ref"
    assert_bits_equal(host(loaded[3][1](dev(idx2), dev(off))), want, "file-mapped table after load")
    x = torch.randn(3, 5, 16, device="cuda", dtype=torch.float16)
    a = layers[1][1](x, x)
    b = loaded[1][1](x, x)
    assert torch.equal(a, b)
