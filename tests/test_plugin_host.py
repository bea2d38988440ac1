"""Host-side plugin contract: registry, creator fields, shape / format rules, serialized bytes,
clone, error statuses.  Everything here runs without a GPU (no configure / enqueue)."""
import struct

import numpy as np
import pytest

from forward_amd import lib, plugin
from forward_amd.plugin import PluginFieldData as F

REG = plugin.getPluginRegistry()


def bag_fields(table, op=0, offset=0):
    count, dim = table.shape
    # order and types of trt_embedding_bag_creator.h:56-65
    return [F("dim", dim), F("count", count), F("offset", offset), F("op", op), F("data", table)]


def test_registry_lookup():
    names = {(c.getPluginName(), c.getPluginVersion()) for c in REG.getPluginCreatorList()}
    assert names == {("EmbeddingBag_TRT", "001"), ("EmbeddingBag_TRT", "002"), ("EmbeddingBagGroup_TRT", "001"),
                     ("ForwardLayerNormPluginDynamic", "1"), ("CustomSkipLayerNormPluginDynamic", "1"),
                     ("CustomEmbLayerNormPluginDynamic", "1")}
    assert REG.getPluginCreator("EmbeddingBag_TRT", "003") is None
    assert REG.getPluginCreator("Nope", "1") is None


def test_embedding_bag_creator_fields():
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    assert c.getFieldNames() == [("dim", lib.FIELD_I32), ("count", lib.FIELD_I32), ("offset", lib.FIELD_I32),
                                 ("op", lib.FIELD_I32), ("data", lib.FIELD_F32)]
    table = np.arange(20, dtype=np.float32).reshape(5, 4)
    p = c.createPlugin("embedding_bag", bag_fields(table))
    assert p.getPluginType() == "EmbeddingBag_TRT" and p.getPluginVersion() == "001"
    assert p.getNbOutputs() == 1 and p.getPluginNamespace() == ""
    assert p.getWorkspaceSize([((5,), lib.I32), ((5,), lib.I32)], [((5, 4), lib.F32)]) == 0
    # contract violations: wrong field count, unknown name, wrong type (the reference aborts)
    with pytest.raises(lib.FwdmiError, match="expected 5 fields"):
        c.createPlugin("x", bag_fields(table)[:4])
    with pytest.raises(lib.FwdmiError, match="unknown field"):
        c.createPlugin("x", bag_fields(table)[:4] + [F("weights", table)])
    with pytest.raises(lib.FwdmiError, match="INT32"):
        c.createPlugin("x", [F("dim", np.array([4.0], np.float32))] + bag_fields(table)[1:])
    with pytest.raises(lib.FwdmiError, match="FLOAT32"):
        c.createPlugin("x", bag_fields(table)[:4] + [F("data", table.astype(np.float16))])
    with pytest.raises(lib.FwdmiError, match="dim\\*count"):
        c.createPlugin("x", bag_fields(table)[:4] + [F("data", table[:3])])
    with pytest.raises(lib.FwdmiError, match="dim\\*count"):           # a 1-element placeholder is not a table
        c.createPlugin("x", bag_fields(table)[:4] + [F("data", table[:1, :1])])


def test_embedding_bag_output_dimensions_and_formats():
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    table = np.zeros((50, 16), np.float32)
    p = c.createPlugin("embedding_bag", bag_fields(table, op=0))
    assert p.getOutputDimensions(0, [(10, 5)]) == [10, 16]                  # fixed-length bags
    assert p.getOutputDimensions(0, [(1056,), (64,)]) == [64, 16]           # ids + offsets
    assert p.getOutputDimensions(0, [(1056,), (1, 64)]) == [64, 16]         # offsets selected from a [1,B] slice
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(0, [(1056,)])                                 # single input must be 2-D
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(0, [(1056,), (2, 64)])
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(1, [(10, 5)])
    g = c.createPlugin("gather", bag_fields(table, op=999))
    assert g.getOutputDimensions(0, [(1, 10)]) == [1, 10, 16]
    with pytest.raises(lib.FwdmiError, match="GATHER"):
        g.getOutputDimensions(0, [(10,), (2,)])
    g1 = c.createPlugin("gather", bag_fields(np.zeros((50, 1), np.float32), op=999))
    assert g1.getOutputDimensions(0, [(1, 3)]) == [1, 3]                    # dim == 1 keeps the input shape

    io = [((100,), lib.I32), ((8,), lib.I32), ((8, 16), lib.F32)]
    assert all(p.supportsFormatCombination(i, io, 2, 1) for i in range(3))
    assert not p.supportsFormatCombination(0, [((100,), lib.I64)] + io[1:], 2, 1)
    assert not p.supportsFormatCombination(2, io[:2] + [((8, 16), lib.F16)], 2, 1)
    assert not p.supportsFormatCombination(0, [((100,), lib.I32, 1)] + io[1:], 2, 1)   # non-linear format
    assert not p.supportsFormatCombination(0, io + io, 3, 1)                          # at most two inputs
    assert p.getOutputDataType(0, [lib.I32, lib.I32]) == lib.F32


def test_embedding_bag_serialization_layout_and_roundtrip():
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    table = np.random.default_rng(0).standard_normal((7, 3)).astype(np.float32)
    p = c.createPlugin("embedding_bag", bag_fields(table, op=3, offset=11))
    blob = p.serialize()
    # int dim | int count | int data_offset | int op | size_t n | float[n]   (embedding_bag_plugin.cpp:191-202)
    assert len(blob) == p.getSerializationSize() == 24 + 4 * 21
    assert struct.unpack("<iiiiQ", blob[:24]) == (3, 7, 11, 3, 21)
    assert blob[24:] == table.tobytes()
    q = c.deserializePlugin("embedding_bag", blob)
    assert q.serialize() == blob
    assert q.clone().serialize() == blob
    for cut in (0, 3, 23, 24, len(blob) - 1):
        with pytest.raises(lib.FwdmiError):
            c.deserializePlugin("embedding_bag", blob[:cut])
    bad = bytearray(blob)
    bad[0:4] = struct.pack("<i", 4)                                          # dim no longer matches n
    with pytest.raises(lib.FwdmiError, match="inconsistent"):
        c.deserializePlugin("embedding_bag", bytes(bad))


def test_embedding_bag_extended_version():
    c = REG.getPluginCreator("EmbeddingBag_TRT", "002")
    table = np.random.default_rng(1).standard_normal((9, 8)).astype(np.float16)
    p = c.createPlugin("embedding_bag", bag_fields(table) + [F("index_type", lib.I64), F("output_fp16", 1),
                                                            F("include_last_offset", 1), F("per_sample_weights", 1)])
    assert p.getPluginVersion() == "002"
    assert p.getOutputDimensions(0, [(40,), (5,), (40,)]) == [4, 8]          # include_last_offset: B+1 offsets
    io = [((40,), lib.I64), ((5,), lib.I64), ((40,), lib.F16), ((4, 8), lib.F16)]
    assert all(p.supportsFormatCombination(i, io, 3, 1) for i in range(4))
    assert not p.supportsFormatCombination(0, [((40,), lib.I32)] + io[1:], 3, 1)
    assert p.getOutputDataType(0, [lib.I64, lib.I64, lib.F16]) == lib.F16
    blob = p.serialize()
    assert struct.unpack("<10iQ", blob[:48]) == (8, 9, 0, 0, lib.F16, lib.I64, lib.F16, 1, 1, 0, 72)
    assert blob[48:] == table.tobytes()
    assert c.deserializePlugin("e", blob).serialize() == blob
    with pytest.raises(lib.FwdmiError, match="SUM"):
        c.createPlugin("e", bag_fields(table, op=2) + [F("per_sample_weights", 1)])
    # the five reference fields alone are accepted by the extended creator too
    assert c.createPlugin("e", bag_fields(table.astype(np.float32))).getOutputDataType(0, [lib.I32]) == lib.F32


def group_fields(tables, op=0, extra=()):
    dim = tables[0].shape[1]
    return [F("dim", dim), F("op", op), F("count", np.array([t.shape[0] for t in tables], np.int32)),
            F("data", np.concatenate([t.reshape(-1) for t in tables]))] + list(extra)


def test_embedding_bag_group_host_contract(tmp_path):
    rng = np.random.default_rng(5)
    c = REG.getPluginCreator("EmbeddingBagGroup_TRT", "001")
    assert [n for n, _ in c.getFieldNames()][:5] == ["dim", "op", "count", "offset", "data"]
    tables = [rng.standard_normal((r, 8)).astype(np.float16) for r in (3, 7, 2)]
    p = c.createPlugin("sparse", group_fields(tables, extra=[F("output_fp16", 1), F("index_type", lib.I64),
                                                             F("offset", np.array([0, 5, 0], np.int32))]))
    assert p.getPluginType() == "EmbeddingBagGroup_TRT" and p.getPluginVersion() == "001" and p.getNbOutputs() == 1
    shapes = [(11,), (4,), (0,), (1, 4), (9,), (4,)]
    assert p.getOutputDimensions(0, shapes) == [4, 24]
    with pytest.raises(lib.FwdmiError, match="3 tables need 6"):
        p.getOutputDimensions(0, shapes[:4])
    with pytest.raises(lib.FwdmiError, match="offsets"):
        p.getOutputDimensions(0, shapes[:5] + [(5,)])                      # tables disagree on the bag count
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(0, [(11, 2)] + shapes[1:])                   # ids must be 1-D
    io = [(s, lib.I64) for s in shapes] + [((4, 24), lib.F16)]
    assert all(p.supportsFormatCombination(i, io, 6, 1) for i in range(7))
    assert not p.supportsFormatCombination(6, io[:6] + [((4, 24), lib.F32)], 6, 1)
    assert not p.supportsFormatCombination(1, [io[0], ((4,), lib.I32)] + io[2:], 6, 1)
    assert p.getOutputDataType(0, [lib.I64] * 6) == lib.F16
    assert p.getWorkspaceSize(io[:6], io[6:]) == 256                       # 3 descriptors of 64 bytes, rounded up
    blob = p.serialize()
    head = struct.unpack("<9i", blob[:36])
    assert head == (8, 0, 3, lib.F16, lib.I64, lib.F16, 0, 1, 0)
    assert struct.unpack("<3i3i", blob[36:60]) == (3, 7, 2, 0, 5, 0)
    assert all(x == 1.0 for x in struct.unpack("<3f", blob[60:72]))        # tiny tables: equal cost
    assert struct.unpack("<Q", blob[72:80]) == (12 * 8,)
    assert blob[80:] == b"".join(t.tobytes() for t in tables)
    assert c.deserializePlugin("x", blob).serialize() == blob and p.clone().serialize() == blob
    for cut in (0, 35, 44, 79, len(blob) - 1):
        with pytest.raises(lib.FwdmiError):
            c.deserializePlugin("x", blob[:cut])
    rc = p.enqueue_raw(io[:6], io[6:], [0] * 6, [0], stream_handle=0)
    assert rc == lib.ERR_NOT_CONFIGURED

    # contract violations
    with pytest.raises(lib.FwdmiError, match="required"):
        c.createPlugin("x", group_fields(tables)[:3])
    with pytest.raises(lib.FwdmiError, match="dim \\* sum"):
        c.createPlugin("x", group_fields(tables)[:3] + [F("data", np.zeros(5, np.float16))])
    with pytest.raises(lib.FwdmiError, match="op must"):
        c.createPlugin("x", group_fields(tables, op=999))
    with pytest.raises(lib.FwdmiError, match="one entry per table"):
        c.createPlugin("x", group_fields(tables, extra=[F("table_cost", np.ones(2, np.float32))]))
    with pytest.raises(lib.FwdmiError, match="positive"):
        c.createPlugin("x", group_fields(tables, extra=[F("table_cost", np.array([1, 0, 1], np.float32))]))
    with pytest.raises(lib.FwdmiError, match="unknown field"):
        c.createPlugin("x", group_fields(tables, extra=[F("max_norm", 1)]))
    with pytest.raises(lib.FwdmiError, match="requires op 0"):
        c.createPlugin("x", group_fields(tables, op=2, extra=[F("per_sample_weights", 1)]))
    # a blob whose table sizes would wrap 64 bits when multiplied out is refused, not trusted
    T = 127
    crafted = struct.pack("<9i", 1 << 24, 0, T, lib.F32, lib.I32, lib.F32, 0, 1, 0) + \
        struct.pack("<%di" % T, *([2 ** 31 - 1] * T)) + struct.pack("<%di" % T, *([0] * T)) + \
        struct.pack("<%df" % T, *([1.0] * T)) + struct.pack("<Q", 0)
    with pytest.raises(lib.FwdmiError, match="too large"):
        c.deserializePlugin("x", crafted)
    # per-sample weights: a third input per table, in the table's type
    w = c.createPlugin("x", group_fields(tables, extra=[F("per_sample_weights", 1)]))
    wshapes = [(11,), (4,), (11,), (0,), (4,), (0,), (9,), (4,), (9,)]
    assert w.getOutputDimensions(0, wshapes) == [4, 24]
    with pytest.raises(lib.FwdmiError, match="one weight per id"):
        w.getOutputDimensions(0, wshapes[:2] + [(10,)] + wshapes[3:])
    wio = [(s_, lib.F16 if i % 3 == 2 else lib.I32) for i, s_ in enumerate(wshapes)] + [((4, 24), lib.F32)]
    assert all(w.supportsFormatCombination(i, wio, 9, 1) for i in range(10))
    assert not w.supportsFormatCombination(2, wio[:2] + [((11,), lib.F32)] + wio[3:], 9, 1)
    assert struct.unpack("<9i", w.serialize()[:36])[8] == 1

    # tables kept by file reference: the blob names the file instead of carrying the rows
    path = tmp_path / "tables.bin"
    path.write_bytes(b"".join(t.tobytes() for t in tables))
    by_ref = c.createPlugin("x", group_fields(tables)[:3] + [
        F("data_file", np.frombuffer(str(path).encode(), np.int8), lib.FIELD_CHAR),
        F("table_type", lib.F16)])
    ref_blob = by_ref.serialize()
    assert len(ref_blob) == 36 + 36 + 8 + 8 + len(str(path)) + 8 and str(path).encode() in ref_blob
    assert c.deserializePlugin("x", ref_blob).serialize() == ref_blob


def test_enqueue_before_configure_and_wrong_dtype():
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    p = c.createPlugin("embedding_bag", bag_fields(np.zeros((5, 4), np.float32)))
    rc = p.enqueue_raw([((5,), lib.I32), ((5,), lib.I32)], [((5, 4), lib.F32)], [0, 0], [0], stream_handle=0)
    assert rc == lib.ERR_NOT_CONFIGURED
    p.terminate()            # harmless before configure
    p.setPluginNamespace("ns")
    assert p.getPluginNamespace() == "ns" and p.clone().getPluginNamespace() == "ns"


def ln_fields(ld, type_id, rng, bias=False, extra=()):
    # order of trt_normalization_creator.h:147-157 (ld, beta, gamma, type_id, has_skip, batch_size)
    f = [F("ld", ld), F("beta", rng.standard_normal(ld).astype(np.float32)),
         F("gamma", rng.standard_normal(ld).astype(np.float32)), F("type_id", type_id)]
    if bias:
        f.append(F("bias", rng.standard_normal(ld).astype(np.float32)))
    return f + list(extra)


@pytest.mark.parametrize("name,n_in", [("ForwardLayerNormPluginDynamic", 1), ("CustomSkipLayerNormPluginDynamic", 2)])
def test_layer_norm_plugins_host_contract(name, n_in):
    rng = np.random.default_rng(2)
    c = REG.getPluginCreator(name, "1")
    assert [n for n, _ in c.getFieldNames()][:5] == ["ld", "type_id", "beta", "gamma", "bias"]
    fields = ln_fields(10, lib.F32, rng, extra=[F("has_skip", 0), F("batch_size", 16)])   # unknown fields ignored
    p = c.createPlugin("skip_layer_norm", fields)
    assert p.getPluginType() == name and p.getPluginVersion() == "1" and p.getNbOutputs() == 1
    shapes = [(20, 5, 10)] * n_in
    assert p.getOutputDimensions(0, shapes) == [20, 5, 10]
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(0, shapes + [(20, 5, 10)])
    io = [((20, 5, 10), lib.F32)] * (n_in + 1)
    assert all(p.supportsFormatCombination(i, io, n_in, 1) for i in range(n_in + 1))
    assert not p.supportsFormatCombination(0, [((20, 5, 10), lib.F16)] * (n_in + 1), n_in, 1)
    assert not p.supportsFormatCombination(n_in, io[:-1] + [((20, 5, 10), lib.F16)], n_in, 1)
    assert p.getOutputDataType(0, [lib.F32] * n_in) == lib.F32
    # DataType mType | DataType mCfgType | size_t mLd | bool mHasBias | beta | gamma   (layer_norm_plugin.cpp:257-277)
    blob = p.serialize()
    assert len(blob) == p.getSerializationSize() == 4 + 4 + 8 + 1 + 2 * 10 * 4
    assert struct.unpack("<iiQ?", blob[:17]) == (lib.F32, lib.F32, 10, False)
    assert blob[17:57] == fields[1].array.tobytes() and blob[57:97] == fields[2].array.tobytes()
    assert c.deserializePlugin("x", blob).serialize() == blob
    assert p.clone().serialize() == blob
    for cut in (0, 16, 17, 96):
        with pytest.raises(lib.FwdmiError):
            c.deserializePlugin("x", blob[:cut])

    # half precision: parameters are stored (and serialized) as fp16; bias and eps extend the blob
    f16 = ln_fields(8, lib.F16, rng, bias=True, extra=[F("eps", np.array([1e-12], np.float32))])
    h = c.createPlugin("ln", f16)
    blob = h.serialize()
    assert len(blob) == 17 + 3 * 8 * 2 + 4
    assert struct.unpack("<iiQ?", blob[:17]) == (lib.F16, lib.F16, 8, True)
    assert blob[17:33] == f16[1].array.astype(np.float16).tobytes()
    assert struct.unpack("<f", blob[-4:])[0] == np.float32(1e-12)
    assert c.deserializePlugin("ln", blob).serialize() == blob

    with pytest.raises(lib.FwdmiError, match="int8"):
        c.createPlugin("ln", ln_fields(8, lib.I8, rng))
    with pytest.raises(lib.FwdmiError, match="Invalid type ID"):
        c.createPlugin("ln", ln_fields(8, 7, rng))
    with pytest.raises(lib.FwdmiError, match="ld=9"):
        c.createPlugin("ln", [F("ld", 9)] + ln_fields(8, lib.F32, rng)[1:])


def emb_fields(rng, ld=16, vocab=40, pos=12, fp16=0):
    # names and order of trt_bert_creator.h:130-141
    r = lambda *s: rng.standard_normal(s).astype(np.float32)
    return [F("bert_embeddings_layernorm_beta", r(ld)), F("bert_embeddings_layernorm_gamma", r(ld)),
            F("bert_embeddings_word_embeddings", r(vocab, ld)), F("bert_embeddings_token_type_embeddings", r(2, ld)),
            F("bert_embeddings_position_embeddings", r(pos, ld)), F("output_fp16", fp16), F("mha_type_id", fp16)]


def test_emb_layer_norm_plugin_that_also_stands_for_the_skip_layer_norm_host_contract():
    """Optional fields skip_beta / skip_gamma (/ skip_bias, skip_eps): the plugin takes the SkipLayerNorm's
    second input (the residual) as its fourth and stands for both layers (trt_bert_creator.h:113-155,199-239)."""
    rng = np.random.default_rng(5)
    c = REG.getPluginCreator("CustomEmbLayerNormPluginDynamic", "1")
    r = lambda n: rng.standard_normal(n).astype(np.float32)
    base = emb_fields(rng, fp16=1)
    for with_bias in (False, True):
        extra = [F("skip_beta", r(16)), F("skip_gamma", r(16)), F("skip_eps", np.array([1e-6], np.float32))]
        if with_bias:
            extra.append(F("skip_bias", r(16)))
        p = c.createPlugin("embeddings", base + extra)
        ins = [(12, 4)] * 3 + [(12, 4, 16, 1, 1)]
        assert p.getNbOutputs() == 2
        assert p.getOutputDimensions(0, ins) == [12, 4, 16, 1, 1] and p.getOutputDimensions(1, ins) == [4, 1]
        assert p.getOutputDimensions(0, ins[:3] + [(12, 4, 16)]) == [12, 4, 16, 1, 1]
        with pytest.raises(lib.FwdmiError, match="takes 4"):
            p.getOutputDimensions(0, ins[:3])
        with pytest.raises(lib.FwdmiError, match="residual"):
            p.getOutputDimensions(0, ins[:3] + [(12, 4, 17, 1, 1)])
        io = [((12, 4), lib.I32)] * 3 + [((12, 4, 16, 1, 1), lib.F16), ((12, 4, 16, 1, 1), lib.F16), ((4, 1), lib.I32)]
        assert all(p.supportsFormatCombination(i, io, 4, 2) for i in range(6))
        assert not p.supportsFormatCombination(3, io[:3] + [((12, 4, 16, 1, 1), lib.F32)] + io[4:], 4, 2)
        assert not p.supportsFormatCombination(0, io[:3] + io[4:], 3, 2)               # the plain plugin's shape
        blob = p.serialize()
        plain = c.createPlugin("embeddings", base).serialize()
        n2 = (3 if with_bias else 2) * 16 * 4
        assert len(blob) == p.getSerializationSize() == len(plain) + 4 + 12 + n2
        assert blob[:len(plain)] == plain                                                # the plain plugin's bytes first
        assert struct.unpack("<iifi", blob[len(plain):len(plain) + 16]) == (0, 1, np.float32(1e-6), int(with_bias))
        assert blob[len(plain) + 16:len(plain) + 16 + 64] == extra[0].array.tobytes()
        q = c.deserializePlugin("e", blob)
        assert q.serialize() == blob and p.clone().serialize() == blob
        assert q.getOutputDimensions(0, ins) == [12, 4, 16, 1, 1]
        for cut in (1, 5, 64, n2 + 3):
            with pytest.raises(lib.FwdmiError):
                c.deserializePlugin("e", blob[:-cut])
    with pytest.raises(lib.FwdmiError, match="skip_beta"):
        c.createPlugin("x", base + [F("skip_beta", r(16))])                              # gamma missing
    with pytest.raises(lib.FwdmiError, match="skip_beta"):
        c.createPlugin("x", base + [F("skip_beta", r(16)), F("skip_gamma", r(15))])


def test_emb_layer_norm_plugin_host_contract():
    rng = np.random.default_rng(3)
    c = REG.getPluginCreator("CustomEmbLayerNormPluginDynamic", "1")
    fields = emb_fields(rng, fp16=1)
    p = c.createPlugin("embeddings", fields)
    assert p.getNbOutputs() == 2
    ins = [(12, 4)] * 3                                                       # [S, B]
    assert p.getOutputDimensions(0, ins) == [12, 4, 16, 1, 1]                 # consumed as [S,B,H,1,1]
    assert p.getOutputDimensions(1, ins) == [4, 1]                            # one mask index per batch row
    with pytest.raises(lib.FwdmiError):
        p.getOutputDimensions(0, [(12, 4), (12, 4), (12, 5)])
    io = [((12, 4), lib.I32)] * 3 + [((12, 4, 16, 1, 1), lib.F16), ((4, 1), lib.I32)]
    assert all(p.supportsFormatCombination(i, io, 3, 2) for i in range(5))
    assert not p.supportsFormatCombination(3, io[:3] + [((12, 4, 16, 1, 1), lib.F32), io[4]], 3, 2)
    assert p.getOutputDataType(0, [lib.I32] * 3) == lib.F16 and p.getOutputDataType(1, [lib.I32] * 3) == lib.I32
    blob = p.serialize()
    assert struct.unpack("<6if", blob[:28]) == (lib.F16, lib.F16, 16, 40, 12, 2, 0.0)
    assert blob[28:28 + 64] == fields[0].array.tobytes()
    assert blob[28 + 128:28 + 128 + 40 * 16 * 2] == fields[2].array.astype(np.float16).tobytes()
    assert len(blob) == p.getSerializationSize() == 28 + 128 + (40 + 12 + 2) * 16 * 2
    assert c.deserializePlugin("e", blob).serialize() == blob and p.clone().serialize() == blob
    with pytest.raises(lib.FwdmiError):
        c.deserializePlugin("e", blob[:-1])
    # crafted headers: sizes whose product would wrap 64 bits, or that the blob cannot hold, are
    # refused with a status (never an allocation failure inside a noexcept call)
    for ld, word, pos, tok in ((2**31 - 1, 2**31 - 1, 2**31 - 1, 2**31 - 1), (2**24 + 1, 40, 12, 2),
                               (16, 2**31 - 1, 12, 2), (2**24, 2**31 - 1, 2**31 - 1, 2**31 - 1), (0, 40, 12, 2),
                               (16, -1, 12, 2)):
        bad = struct.pack("<6if", lib.F16, lib.F16, ld, word, pos, tok, 0.0) + blob[28:]
        with pytest.raises(lib.FwdmiError):
            c.deserializePlugin("e", bad)
    # batch-major variant: [B,S] ids, [B,S,H,1,1] output, one trailing int in the blob
    bm = c.createPlugin("embeddings", fields + [F("batch_major", 1)])
    assert bm.getOutputDimensions(0, [(4, 12)] * 3) == [4, 12, 16, 1, 1] and bm.getOutputDimensions(1, [(4, 12)] * 3) == [4, 1]
    bblob = bm.serialize()
    assert bblob[:-4] == blob and struct.unpack("<i", bblob[-4:]) == (1,)
    assert c.deserializePlugin("e", bblob).getOutputDimensions(1, [(4, 12)] * 3) == [4, 1]
    with pytest.raises(lib.FwdmiError, match="inconsistent sizes"):
        c.createPlugin("e", fields[:2] + [F("bert_embeddings_word_embeddings", np.zeros(17, np.float32))] + fields[3:])


def test_creators_and_plugins_are_thread_safe():
    """Build-time calls from several host threads at once (ctypes releases the GIL): creators are
    shared registry objects, plugins and their clones share table storage."""
    import threading
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    shared = c.createPlugin("shared", bag_fields(np.arange(200, dtype=np.float32).reshape(50, 4)))
    want = shared.serialize()
    errors = []

    def work(seed):
        try:
            rng = np.random.default_rng(seed)
            for _ in range(30):
                t = rng.standard_normal((int(rng.integers(1, 40)), 8)).astype(np.float32)
                p = c.createPlugin("t%d" % seed, bag_fields(t))
                blob = p.serialize()
                assert blob[24:] == t.tobytes()
                q = c.deserializePlugin("t", blob)
                assert q.getOutputDimensions(0, [(9,), (3,)]) == [3, 8]
                k = shared.clone()
                assert k.serialize() == want
                with pytest.raises(lib.FwdmiError, match="expected 5 fields"):
                    c.createPlugin("bad", bag_fields(t)[:3])       # error text is per thread
                for o in (p, q, k):
                    o.destroy()
        except Exception as e:       # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=work, args=(s,)) for s in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert shared.serialize() == want


def test_damaged_engine_bytes_under_the_sanitizers():
    """`make santest` compiles the library's host code (plugin classes, C handles, plan files, sidecar,
    launch plan) with the address / undefined-behaviour sanitizers and runs two programs against it:
    tests/cpp/plugin_mutation_test.cpp (every truncation and 30 000 seeded mutations of every plugin's
    serialized form, 6 000 damaged plan files with good, damaged and missing sidecars: each must come
    back as NULL with a reason or as an object that serializes, clones and destroys) and the C++
    interface test in its host mode.  No GPU: nothing is configured or enqueued."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    b = subprocess.run(["make", "-C", os.path.join(root, "forward_amd", "csrc"), "-j8", "santest"], capture_output=True,
                       text=True, timeout=1500)
    assert b.returncode == 0, b.stdout[-2000:] + b.stderr[-4000:]
    # a library preloaded into every process of this machine would otherwise trip the sanitizer's
    # "runtime does not come first" start-up check
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    p = subprocess.run([os.path.join(root, "tests", "cpp", "plugin_mutation_test")], capture_output=True, text=True,
                       timeout=600, env=env)
    assert p.returncode == 0 and " 0 failures" in p.stdout, p.stdout[-2000:] + p.stderr[-4000:]
    q = subprocess.run([os.path.join(root, "tests", "cpp", "plugin_cpp_test_san"), "host"], capture_output=True, text=True,
                       timeout=600, env=env)
    assert q.returncode == 0 and "PASS" in q.stdout, q.stdout[-2000:] + q.stderr[-4000:]
