"""The PyTorch adapter (torch.ops.fwdmi.* and the drop-in modules) against PyTorch's own
embedding_bag / embedding on the same device, and a DLRM-style model with its modules swapped."""
import numpy as np
import pytest
import torch

from forward_amd import torch_ops, workloads

pytestmark = pytest.mark.gpu


def test_custom_ops_match_torch_on_device():
    wl = workloads.config2(variant=8, rows=20000, n_bags=500)
    w, idx, off = (torch.from_numpy(a).cuda() for a in (wl.table, wl.indices.astype(np.int64), wl.offsets.astype(np.int64)))
    for mode, code in (("sum", 0), ("mean", 1), ("max", 2)):
        ref = torch.nn.functional.embedding_bag(idx, w, off, mode=mode)
        got = torch.ops.fwdmi.embedding_bag(w, idx, off, code, None, False)
        torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-6)
    psw = torch.rand(idx.numel(), device="cuda")
    ref = torch.nn.functional.embedding_bag(idx, w, off, mode="sum", per_sample_weights=psw)
    torch.testing.assert_close(torch.ops.fwdmi.embedding_bag(w, idx, off, 0, psw, False), ref, rtol=1e-5, atol=1e-6)
    ids = torch.randint(0, 20000, (7, 3, 5), device="cuda")
    assert torch.equal(torch.ops.fwdmi.embedding(w, ids), torch.nn.functional.embedding(ids, w))
    x = torch.randn(9, 4, 768, device="cuda", dtype=torch.float16)
    sk = torch.randn_like(x)
    g, b = torch.randn(768, device="cuda"), torch.randn(768, device="cuda")
    ref = torch.nn.functional.layer_norm((x.float() + sk.float()), (768,), g, b, 1e-5)
    torch.testing.assert_close(torch.ops.fwdmi.skip_layer_norm(x, sk, g, b, None, 1e-5).float(), ref, rtol=5e-3, atol=1e-2)


class TinyDlrm(torch.nn.Module):
    """Sparse stage of the reference's DLRM test model (test_torch_dlrm.h:34-57): three sum-mode bags, concatenated."""

    def __init__(self, tables):
        super().__init__()
        self.emb_l = torch.nn.ModuleList([torch.nn.EmbeddingBag(t.shape[0], t.shape[1], mode="sum") for t in tables])
        for m, t in zip(self.emb_l, tables):
            m.weight.data = torch.tensor(t)
        self.word = torch.nn.Embedding(11, 4)

    def forward(self, offsets, indices, tokens):
        bags = [m(i, o) for m, i, o in zip(self.emb_l, indices, offsets)]
        return torch.cat(bags, dim=1), self.word(tokens)


def test_swapped_modules_reproduce_the_reference_dlrm_case(kats):
    d = kats["dlrm"]
    model = TinyDlrm([np.array(t, np.float32) for t in d["tables"]]).cuda().eval()
    idx = [torch.tensor(i, device="cuda") for i in d["indices"]]
    off = [torch.tensor(o, device="cuda") for o in d["offsets"]]
    tok = torch.tensor([[1, 2, 10], [0, 0, 3]], device="cuda")
    with torch.no_grad():
        want_bags, want_tok = model(off, idx, tok)
        swapped = torch_ops.replace_embedding_modules(model)
        assert all(isinstance(m, torch_ops.EmbeddingBag) for m in swapped.emb_l) and isinstance(swapped.word, torch_ops.Embedding)
        got_bags, got_tok = swapped(off, idx, tok)
    torch.testing.assert_close(got_bags, want_bags, rtol=1e-6, atol=1e-7)
    assert torch.equal(got_tok, want_tok)
    expect = np.concatenate([[[0.48071694, 0.18480009], [0.41585842, -0.29087239]],
                             [[-0.18103497, 0.26449448], [-0.25194445, -0.24395032]],
                             [[-0.44896644, -0.45899662], [-0.44896644, -0.45899662]]], axis=1)
    np.testing.assert_allclose(got_bags.cpu().numpy(), expect, atol=1e-4)      # test_torch_dlrm.h:56


def test_collection_is_the_concatenation_of_its_bags(kats):
    # the reference's DLRM case: the three bags as one module, one launch
    d = kats["dlrm"]
    model = TinyDlrm([np.array(t, np.float32) for t in d["tables"]]).cuda().eval()
    idx = [torch.tensor(i, device="cuda") for i in d["indices"]]
    off = [torch.tensor(o, device="cuda") for o in d["offsets"]]
    coll = torch_ops.EmbeddingBagCollection.from_torch(model.emb_l)
    with torch.no_grad():
        want = torch.cat([m(i, o) for m, i, o in zip(model.emb_l, idx, off)], dim=1)
        got = coll(idx, off)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-7)
    expect = np.concatenate([[[0.48071694, 0.18480009], [0.41585842, -0.29087239]],
                             [[-0.18103497, 0.26449448], [-0.25194445, -0.24395032]],
                             [[-0.44896644, -0.45899662], [-0.44896644, -0.45899662]]], axis=1)
    np.testing.assert_allclose(got.cpu().numpy(), expect, atol=1e-4)           # test_torch_dlrm.h:56

    # a larger stage: every mode and table type, trailing end offsets, against the single-table op bit for bit
    wl = workloads.config4(variant=6, n_tables=7, n_bags=1500, max_rows=50000)
    for tdt in (torch.float16, torch.float32):
        ws = [torch.from_numpy(wl.host_table(t)).cuda().to(tdt) for t in range(7)]
        ids = [torch.from_numpy(i.astype(np.int64)).cuda() for i in wl.indices]
        offs = [torch.from_numpy(np.append(o, i.size).astype(np.int64)).cuda() for o, i in zip(wl.offsets, wl.indices)]
        for mode, code in (("sum", 0), ("mean", 1), ("max", 2)):
            got = torch.ops.fwdmi.embedding_bag_group(ws, ids, offs, code, True, [None] * 7)
            one = torch.cat([torch.ops.fwdmi.embedding_bag(w, i, o, code, None, True) for w, i, o in zip(ws, ids, offs)], dim=1)
            assert got.shape == (1500, 7 * 128) and torch.equal(got, one), (tdt, mode)
            ref = torch.cat([torch.nn.functional.embedding_bag(i, w.float(), o, mode=mode, include_last_offset=True)
                             for w, i, o in zip(ws, ids, offs)], dim=1)
            tol = dict(rtol=5e-3, atol=1e-2) if tdt == torch.float16 else dict(rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(got.float(), ref, **tol)
        # per-sample weights on some of the tables only
        psw = [torch.rand(i.numel(), device="cuda").to(tdt) if t % 2 == 0 else None for t, i in enumerate(ids)]
        got = torch.ops.fwdmi.embedding_bag_group(ws, ids, offs, 0, True, psw)
        one = torch.cat([torch.ops.fwdmi.embedding_bag(w, i, o, 0, p, True) for w, i, o, p in zip(ws, ids, offs, psw)], dim=1)
        assert torch.equal(got, one), (tdt, "weighted")
    mixed = [torch.nn.EmbeddingBag(5, 4, mode="sum"), torch.nn.EmbeddingBag(5, 4, mode="mean")]
    with pytest.raises(ValueError):
        torch_ops.EmbeddingBagCollection.from_torch(mixed)


def _bert_inputs(wl):
    """[B, S] tensors as a PyTorch model holds them (int64 ids), plus the plugin-layout originals."""
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    bs = lambda a: dev(a.T).long()
    return (bs(wl.input_ids), bs(wl.segment_ids), bs(wl.input_mask), dev(wl.word), dev(wl.pos), dev(wl.tok),
            dev(wl.gamma.astype(np.float32)), dev(wl.beta.astype(np.float32)))


@pytest.mark.parametrize("cfg", ["config3", "config5"])
def test_bert_ops_against_the_oracle(oracle, cfg):
    """torch.ops.fwdmi.emb_layer_norm / emb_skip_layer_norm on [B, S] int64 tensors (scaled configs 3 and 5)
    against the oracle: fp16 abs 1e-2 / rel 5e-3, mask index exact; the fused op equal to the two ops in a row."""
    wl = workloads.config3(variant=4, batch=5, seq=48) if cfg == "config3" else workloads.config5(variant=4, batch=3, seq=96)
    ids, seg, msk, word, pos, tok, g, b = _bert_inputs(wl)
    out, midx = torch.ops.fwdmi.emb_layer_norm(ids, seg, msk, word, pos, tok, g, b, wl.eps, True)
    want, want_midx, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                               wl.gamma, wl.beta, eps=wl.eps)
    assert out.shape == (ids.shape[0], ids.shape[1], wl.word.shape[1]) and out.dtype == torch.float16
    np.testing.assert_allclose(out.float().cpu().numpy().transpose(1, 0, 2), want.astype(np.float32), atol=1e-2, rtol=5e-3)
    assert np.array_equal(midx.cpu().numpy(), want_midx) and np.array_equal(want_midx, wl.valid_len)
    # the plugin's own [S, B] layout through the same op
    out_sb, midx_sb = torch.ops.fwdmi.emb_layer_norm(ids.T.contiguous(), seg.T.contiguous(), msk.T.contiguous(), word, pos,
                                                     tok, g, b, wl.eps, False)
    assert torch.equal(out_sb.transpose(0, 1), out) and torch.equal(midx_sb, midx)
    # without a mask: no mask index
    _, none = torch.ops.fwdmi.emb_layer_norm(ids, seg, None, word, pos, tok, g, b, wl.eps, True)
    assert none.numel() == 0
    # into the caller's tensors
    out2, midx2 = torch.full_like(out, 7.0), torch.full_like(midx, -1)
    torch.ops.fwdmi.emb_layer_norm_out(out2, midx2, ids, seg, msk, word, pos, tok, g, b, wl.eps, None, None, None, None,
                                       0.0, True)
    assert torch.equal(out2, out) and torch.equal(midx2, midx)
    mod = torch_ops.BertEmbeddings(word, pos, tok, g, b, wl.eps)
    m_out, m_len = mod(ids, seg, msk)
    assert torch.equal(m_out, out) and torch.equal(m_len, midx)
    if wl.skip is None:
        return
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    skip = dev(wl.skip.transpose(1, 0, 2))
    g2, b2, bi2 = (dev(a.astype(np.float32)) for a in (wl.skip_gamma, wl.skip_beta, wl.skip_bias))
    fused, fmidx = torch.ops.fwdmi.emb_skip_layer_norm(ids, seg, msk, word, pos, tok, g, b, wl.eps, skip, g2, b2, bi2,
                                                       wl.eps, True)
    chained = torch.ops.fwdmi.skip_layer_norm(out, skip, g2, b2, bi2, wl.eps)
    assert torch.equal(fused, chained) and torch.equal(fmidx, midx)
    want2 = oracle.skip_layer_norm(want, wl.skip_gamma, wl.skip_beta, skip=wl.skip, bias=wl.skip_bias, eps=wl.eps)
    np.testing.assert_allclose(fused.float().cpu().numpy().transpose(1, 0, 2), want2.astype(np.float32), atol=1e-2, rtol=5e-3)
    buf = torch.zeros_like(fused)
    torch.ops.fwdmi.emb_layer_norm_out(buf, None, ids, seg, msk, word, pos, tok, g, b, wl.eps, skip, g2, b2, bi2, wl.eps, True)
    assert torch.equal(buf, fused)
    buf.zero_()
    torch.ops.fwdmi.skip_layer_norm_out(buf, out, skip, g2, b2, bi2, wl.eps)
    assert torch.equal(buf, chained)


def test_out_forms_write_into_the_callers_tensors(kats, oracle):
    """*_out ops: declared to PyTorch as mutating `out`, results equal to the returning forms; on the reference's
    DLRM case (test_torch_dlrm.h:34-57) and on a larger stage, against the oracle."""
    d = kats["dlrm"]
    ws = [torch.tensor(np.array(t, np.float32), device="cuda") for t in d["tables"]]
    idx = [torch.tensor(i, device="cuda") for i in d["indices"]]
    off = [torch.tensor(o, device="cuda") for o in d["offsets"]]
    out = torch.full((2, 6), 9.0, device="cuda")
    for t in range(3):
        torch.ops.fwdmi.embedding_bag_out(out, ws[t], idx[t], off[t], 0, None, False, 2 * t)
    expect = np.concatenate([[[0.48071694, 0.18480009], [0.41585842, -0.29087239]],
                             [[-0.18103497, 0.26449448], [-0.25194445, -0.24395032]],
                             [[-0.44896644, -0.45899662], [-0.44896644, -0.45899662]]], axis=1)
    np.testing.assert_allclose(out.cpu().numpy(), expect, atol=1e-6)           # test_torch_dlrm.h:56
    out2 = torch.full((2, 6), 9.0, device="cuda")
    torch.ops.fwdmi.embedding_bag_group_out(out2, ws, idx, off, 0, False, [None] * 3)
    assert torch.equal(out2, out)
    assert "Tensor(a0!) out" in str(torch.ops.fwdmi.embedding_bag_out.default._schema)
    assert "Tensor(a0!) out" in str(torch.ops.fwdmi.embedding_bag_group_out.default._schema)

    wl = workloads.config4(variant=3, n_tables=5, n_bags=2000, max_rows=30000)
    tabs = [wl.host_table(t) for t in range(5)]
    ws = [torch.from_numpy(t).cuda() for t in tabs]
    ids = [torch.from_numpy(i.astype(np.int64)).cuda() for i in wl.indices]
    offs = [torch.from_numpy(o.astype(np.int64)).cuda() for o in wl.offsets]
    want = np.zeros((2000, 5 * 128), np.float16)
    for t in range(5):
        oracle.embedding_bag(tabs[t], wl.indices[t], wl.offsets[t], oracle.OP_SUM, out=want, out_col=128 * t)
    buf = torch.zeros((2000, 5 * 128), dtype=torch.float16, device="cuda")
    torch.ops.fwdmi.embedding_bag_group_out(buf, ws, ids, offs, 0, False, [None] * 5)
    assert np.array_equal(buf.cpu().numpy().view(np.uint16), want.view(np.uint16))
    buf.zero_()
    for t in range(5):
        torch.ops.fwdmi.embedding_bag_out(buf, ws[t], ids[t], offs[t], 0, None, False, 128 * t)
    assert np.array_equal(buf.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # PyTorch's own checks of a custom op: schema (which arguments are written) and shape inference
    torch.library.opcheck(torch.ops.fwdmi.embedding_bag_out.default, (buf, ws[0], ids[0], offs[0], 0, None, False, 0),
                          test_utils=("test_schema",))
    ids3, seg3 = torch.zeros((2, 4), dtype=torch.int64, device="cuda"), torch.zeros((2, 4), dtype=torch.int64, device="cuda")
    word = torch.randn(10, 64, device="cuda", dtype=torch.float16)
    args = (ids3, seg3, torch.ones_like(ids3), word, word[:4].clone(), word[:2].clone(), torch.ones(64, device="cuda"),
            torch.zeros(64, device="cuda"), 1e-12, True)
    torch.library.opcheck(torch.ops.fwdmi.emb_layer_norm.default, args, test_utils=("test_schema", "test_faketensor"))
