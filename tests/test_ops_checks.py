"""Argument checks of forward_amd.ops that guard the launchers' device-memory accesses.  They
run before any launch, so they are exercised here on CPU tensors with the "is in device memory"
test switched off; every case must raise ValueError (and would otherwise index device memory out
of bounds)."""
import pytest
import torch

from forward_amd import ops


@pytest.fixture(autouse=True)
def host_tensors_pass_as_device(monkeypatch):
    def dev(t, name):
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(name)
        if not t.is_contiguous():
            raise ValueError(name)
        return t
    monkeypatch.setattr(ops, "_dev", dev)


def f32(*shape):
    return torch.zeros(shape, dtype=torch.float32)


def i32(*shape):
    return torch.zeros(shape, dtype=torch.int32)


def test_tables_without_rows_are_refused():
    empty, ok = f32(0, 8), f32(5, 8)
    ids, off = i32(3), i32(2)
    with pytest.raises(ValueError, match="rows > 0"):
        ops.MultiTableBatch([ok, empty], [ids, ids], [off, off])
    with pytest.raises(ValueError, match="rows > 0"):
        ops.embedding_bag_group([empty, ok], [ids, ids], [off, off])


def test_embedding_bag_column_block_must_fit():
    table, ids, off = f32(5, 8), i32(3), i32(2)
    for out, col in ((f32(2, 20), -1), (f32(2, 20), 13), (f32(2, 7), 0), (f32(3, 20), 0), (f32(40), 0)):
        with pytest.raises(ValueError):
            ops.embedding_bag(table, ids, off, out=out, out_col=col)


def test_layer_norm_parameter_lengths():
    x = f32(4, 16)
    with pytest.raises(ValueError, match="ld"):
        ops.layer_norm(x, f32(15), f32(16))
    with pytest.raises(ValueError, match="ld"):
        ops.layer_norm(x, f32(16), f32(8))
    with pytest.raises(ValueError, match="bias"):
        ops.layer_norm(x, f32(16), f32(16), bias=f32(4))
    with pytest.raises(ValueError, match="bias"):
        ops.skip_layer_norm(x, f32(16), f32(16), skip=f32(4, 16), bias=f32(17))
    with pytest.raises(ValueError, match="element count"):
        ops.layer_norm(x, f32(16), f32(16), out=f32(3, 16))
    with pytest.raises(ValueError, match="element count"):
        ops.skip_layer_norm(x, f32(16), f32(16), out=torch.zeros((4, 16), dtype=torch.float16))


def test_emb_layer_norm_shapes():
    S, B, H = 6, 2, 16
    ids, seg, msk = i32(S, B), i32(S, B), i32(S, B)
    word, pos, tok, g, b = f32(30, H), f32(8, H), f32(2, H), f32(H), f32(H)
    bad = [
        dict(pos=f32(8, H + 1)), dict(tok=f32(2, H - 1)), dict(gamma=f32(H - 1)), dict(beta=f32(H + 3)),
        dict(input_mask=i32(S, B + 1)), dict(input_mask=torch.zeros((S, B), dtype=torch.int64)),
        dict(out=f32(S, B, H - 1)), dict(out=torch.zeros((S, B, H), dtype=torch.float16)),
        dict(mask_idx=i32(B + 1)), dict(mask_idx=torch.zeros(B, dtype=torch.int64)),
        dict(skip=f32(S, B, H), gamma2=f32(H), beta2=f32(H - 1)),
        dict(skip=f32(S, B, H), gamma2=f32(H), beta2=f32(H), bias2=f32(1)),
    ]
    for change in bad:
        kw = dict(input_ids=ids, segment_ids=seg, input_mask=msk, word=word, pos=pos, tok=tok, gamma=g, beta=b)
        kw.update(change)
        with pytest.raises(ValueError):
            ops.emb_layer_norm(**kw)
