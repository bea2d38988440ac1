"""Pins the CPU oracle's LayerNorm family: float64 closed form, libtorch CPU vectors,
standardisation invariants, and the BERT embedding composition.  CPU only."""
import numpy as np
import torch

from forward_amd import workloads


def ln64(x, gamma, beta, eps):
    x = x.astype(np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * gamma.astype(np.float64) + beta.astype(np.float64)


def test_layer_norm_torch_vectors(oracle, torch_vectors):
    v = torch_vectors
    for eps, key in ((1e-5, "ln_out_eps1e-5"), (1e-12, "ln_out_eps1e-12")):
        out = oracle.layer_norm(v["ln_x"], v["ln_gamma"], v["ln_beta"], eps=eps)
        np.testing.assert_allclose(out, v[key], rtol=1e-5, atol=1e-6)


def test_layer_norm_reference_held_weights(oracle, kats):
    """LayerNorm(10) with the weights stored in layer_norm_with_weights.pth (gamma=1, beta=0)."""
    k = kats["layer_norm_with_weights"]
    a, b = np.array(k["data0"], np.float32), np.array(k["data1"], np.float32)
    gamma, beta = (a, b) if a.sum() > b.sum() else (b, a)
    np.testing.assert_array_equal(gamma, 1.0)
    np.testing.assert_array_equal(beta, 0.0)
    rng = np.random.Generator(np.random.PCG64(5))
    x = rng.standard_normal(k["input_shape"]).astype(np.float32)
    out = oracle.layer_norm(x, gamma, beta, eps=0.0)
    # gamma=1, beta=0 reduces to plain standardisation of each row
    np.testing.assert_allclose(out.mean(-1), 0.0, atol=1e-6)
    np.testing.assert_allclose(out.std(-1), 1.0, rtol=1e-5)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (10,), eps=k["eps"]).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-3)      # the reference's own tolerance (eps ignored by the plugin)


def test_skip_layer_norm_closed_form(oracle):
    rng = np.random.Generator(np.random.PCG64(6))
    for dt, tol in ((np.float32, 2e-6), (np.float16, 2e-3)):
        x = rng.standard_normal((7, 3, 96)).astype(dt)
        sk = rng.standard_normal((7, 3, 96)).astype(dt)
        g = (1 + 0.1 * rng.standard_normal(96)).astype(np.float32)
        b = (0.1 * rng.standard_normal(96)).astype(np.float32)
        bi = (0.1 * rng.standard_normal(96)).astype(np.float32)
        out = oracle.skip_layer_norm(x, g, b, skip=sk, bias=bi, eps=1e-12)
        want = ln64(x.astype(np.float64) + sk.astype(np.float64) + bi, g, b, 1e-12)
        np.testing.assert_allclose(out.astype(np.float64), want, atol=tol * 4, rtol=tol)
        # a dropped operand must be visible
        assert np.abs(oracle.skip_layer_norm(x, g, b, skip=None, bias=bi).astype(np.float64) - want).max() > 0.1
        assert np.abs(oracle.skip_layer_norm(x, g, b, skip=sk, bias=None).astype(np.float64) - want).max() > 0.01


def test_emb_layer_norm_composition(oracle):
    wl = workloads.config3(variant=2, dtype=np.float32, batch=4, seq=24)
    out, midx, oob = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                           wl.gamma, wl.beta, eps=wl.eps)
    assert oob == 0 and out.shape == (24, 4, 768)
    S, B = wl.input_ids.shape
    x = (wl.word[wl.input_ids].astype(np.float64) + wl.pos[:S, None, :].astype(np.float64)
         + wl.tok[wl.segment_ids].astype(np.float64))
    np.testing.assert_allclose(out, ln64(x, wl.gamma, wl.beta, wl.eps), rtol=1e-5, atol=1e-6)
    # libtorch CPU composition: embedding x3 + add + layer_norm
    tw, tp, tt = (torch.from_numpy(a) for a in (wl.word, wl.pos, wl.tok))
    e = (torch.nn.functional.embedding(torch.from_numpy(wl.input_ids).long(), tw)
         + tp[:S].unsqueeze(1) + torch.nn.functional.embedding(torch.from_numpy(wl.segment_ids).long(), tt))
    ref = torch.nn.functional.layer_norm(e, (768,), torch.from_numpy(wl.gamma), torch.from_numpy(wl.beta), wl.eps)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-5, atol=2e-6)
    # mask index = valid length for prefix masks; first zero in general
    np.testing.assert_array_equal(midx, wl.valid_len)
    m = wl.input_mask.copy()
    m[5, 2] = 0
    _, midx2, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, m, wl.word, wl.pos, wl.tok, wl.gamma, wl.beta)
    assert midx2[2] == min(5, wl.valid_len[2])
    full = np.ones_like(m)
    _, midx3, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, full, wl.word, wl.pos, wl.tok, wl.gamma, wl.beta)
    np.testing.assert_array_equal(midx3, S)


def test_workload_generators_are_deterministic():
    a, b = workloads.config1(), workloads.config1()
    np.testing.assert_array_equal(a.indices, b.indices)
    np.testing.assert_array_equal(a.table, b.table)
    assert a.offsets[0] == 0 and a.n_bags == 64 and a.table.shape == (10000, 64)
    w = workloads.config4(n_tables=4, n_bags=2048, max_rows=1e5)
    assert len(w.rows) == 4 and all(1000 <= r <= 100000 for r in w.rows)
    lens = np.diff(np.append(w.offsets[0], w.indices[0].size))
    assert lens.min() >= 1 and lens.max() <= 100 and 12 < lens.mean() < 21
    assert w.indices[0].max() < w.rows[0] and w.indices[0].min() >= 0
    c5 = workloads.config5(batch=2, seq=32)
    assert c5.skip.shape == (32, 2, 1024) and c5.input_ids[0, 0] == 101
    assert (c5.input_ids[c5.valid_len[0]:, 0] == 0).all()
