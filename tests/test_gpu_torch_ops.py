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
