"""GPU parity of the LayerNorm-family kernels against the CPU oracle (float64 closed form),
through the C ABI launchers and the plugin objects.  Tolerances: fp32 rel 1e-5 (abs 1e-5 floor,
outputs are O(1)); fp16 abs 1e-2 / rel 5e-3; the mask index is bit-exact."""
import numpy as np
import pytest
import torch

from forward_amd import lib, ops, plugin, workloads
from forward_amd.plugin import PluginFieldData as F
from gpu_util import assert_close, dev, host

pytestmark = pytest.mark.gpu
REG = plugin.getPluginRegistry()


def f32(a):
    return dev(np.asarray(a, np.float32))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_config3_emb_layer_norm(oracle, dtype):
    wl = workloads.config3(dtype=dtype)
    assert wl.input_ids.shape == (128, 32) and wl.word.shape == (30522, 768)
    out, midx = ops.emb_layer_norm(dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask), dev(wl.word),
                                   dev(wl.pos), dev(wl.tok), f32(wl.gamma), f32(wl.beta), eps=wl.eps)
    want, wmidx, oob = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                             wl.gamma, wl.beta, eps=wl.eps)
    assert oob == 0
    assert_close(host(out), want, dtype)
    np.testing.assert_array_equal(host(midx), wmidx)
    np.testing.assert_array_equal(host(midx), wl.valid_len)
    if dtype == np.float16:
        # next to the oracle: libtorch CPU's own fp16 path (embedding x3, add, layer_norm, rounding per op)
        S = wl.input_ids.shape[0]
        tw, tp, tt = (torch.from_numpy(a) for a in (wl.word, wl.pos, wl.tok))
        e = (torch.nn.functional.embedding(torch.from_numpy(wl.input_ids).long(), tw) + tp[:S].unsqueeze(1)
             + torch.nn.functional.embedding(torch.from_numpy(wl.segment_ids).long(), tt))
        ref = torch.nn.functional.layer_norm(e.float(), (768,), torch.from_numpy(wl.gamma).float(),
                                             torch.from_numpy(wl.beta).float(), wl.eps)
        assert_close(host(out), ref.numpy(), np.float16)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_config5_emb_then_skip_layer_norm(oracle, dtype):
    wl = workloads.config5(dtype=dtype)
    assert wl.input_ids.shape == (512, 16) and wl.skip.shape == (512, 16, 1024)
    emb, midx = ops.emb_layer_norm(dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask), dev(wl.word),
                                   dev(wl.pos), dev(wl.tok), f32(wl.gamma), f32(wl.beta), eps=wl.eps)
    out = ops.skip_layer_norm(emb, f32(wl.skip_gamma), f32(wl.skip_beta), skip=dev(wl.skip), bias=f32(wl.skip_bias),
                              eps=wl.eps)
    wemb, wmidx, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                           wl.gamma, wl.beta, eps=wl.eps)
    assert_close(host(emb), wemb, dtype)
    np.testing.assert_array_equal(host(midx), wmidx)
    # second stage checked on the GPU's own first-stage output, so errors do not compound
    want = oracle.skip_layer_norm(host(emb), wl.skip_gamma, wl.skip_beta, skip=wl.skip, bias=wl.skip_bias, eps=wl.eps)
    assert_close(host(out), want, dtype)
    # next to the oracle: libtorch CPU itself on the same parameters (embedding x3 + add + layer_norm, then
    # the residual / bias add + layer_norm), evaluated in fp32
    Fn = torch.nn.functional
    S, H = wl.input_ids.shape[0], wl.word.shape[1]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).float()
    e = Fn.layer_norm(Fn.embedding(torch.from_numpy(wl.input_ids).long(), t(wl.word)) + t(wl.pos)[:S].unsqueeze(1)
                      + Fn.embedding(torch.from_numpy(wl.segment_ids).long(), t(wl.tok)), (H,), t(wl.gamma), t(wl.beta),
                      wl.eps)
    assert_close(host(emb), e.numpy(), dtype)
    ref = Fn.layer_norm(e + t(wl.skip) + t(wl.skip_bias), (H,), t(wl.skip_gamma), t(wl.skip_beta), wl.eps)
    assert_close(host(out), ref.numpy(), dtype, scale=4.0)


@pytest.mark.parametrize("ld,dtype", [(1, np.float32), (7, np.float32), (10, np.float32), (32, np.float16),
                                      (48, np.float32), (100, np.float16), (256, np.float32), (768, np.float32),
                                      (1000, np.float16), (1024, np.float16), (4096, np.float16),
                                      (2048, np.float32), (5000, np.float32), (8192, np.float16),
                                      # several rows per wavefront (rows of at most 512 bytes)
                                      (8, np.float16), (16, np.float16), (64, np.float16), (128, np.float16),
                                      (248, np.float16), (256, np.float16), (4, np.float32), (128, np.float32),
                                      (3, np.float16), (31, np.float16), (25, np.float32), (33, np.float32),
                                      # no 16-byte slices: one element per lane, a workgroup per row
                                      (513, np.float32), (1001, np.float16), (2050, np.float16), (8191, np.float32),
                                      (8193, np.float32),
                                      # a workgroup per row, and beyond it the strided kernel
                                      (4104, np.float16), (12000, np.float16), (16384, np.float16),
                                      (16392, np.float16), (4096, np.float32), (8192, np.float32),
                                      (8196, np.float32),
                                      # beyond a workgroup's registers: streamed twice
                                      (40000, np.float16), (20001, np.float32), (65536, np.float32)])
def test_layer_norm_row_lengths(oracle, ld, dtype):
    rng = np.random.Generator(np.random.PCG64(ld))
    x = (rng.standard_normal((37, ld)) * 2 + 0.5).astype(dtype)
    sk = rng.standard_normal((37, ld)).astype(dtype)
    g = (1 + 0.1 * rng.standard_normal(ld)).astype(np.float32)
    b = (0.1 * rng.standard_normal(ld)).astype(np.float32)
    bi = (0.1 * rng.standard_normal(ld)).astype(np.float32)
    eps = 1e-5
    got = host(ops.layer_norm(dev(x), dev(g), dev(b), eps=eps))
    assert_close(got, oracle.layer_norm(x, g, b, eps=eps), dtype)
    got = host(ops.layer_norm(dev(x), dev(g), dev(b), bias=dev(bi), eps=eps))
    assert_close(got, oracle.layer_norm(x, g, b, bias=bi, eps=eps), dtype)
    got = host(ops.skip_layer_norm(dev(x), dev(g), dev(b), skip=dev(sk), bias=dev(bi), eps=eps))
    assert_close(got, oracle.skip_layer_norm(x, g, b, skip=sk, bias=bi, eps=eps), dtype)


@pytest.mark.parametrize("ld", [1024, 24, 6000, 20000])
def test_layer_norm_large_mean_is_stable(oracle, ld):
    """|mean| >> std: the E[x^2]-mean^2 form of the reference loses all digits here; Welford (and, for
    streamed rows, sums shifted by the row's first element) does not.  One length per kernel variant."""
    rng = np.random.Generator(np.random.PCG64(9))
    x = (1000.0 + 0.1 * rng.standard_normal((64, ld))).astype(np.float32)
    g, b = np.ones(ld, np.float32), np.zeros(ld, np.float32)
    got = host(ops.layer_norm(dev(x), dev(g), dev(b), eps=0.0))
    want = oracle.layer_norm(x, g, b, eps=0.0)
    np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-3)
    assert np.isfinite(got).all()


def test_many_rows_loop_path(oracle):
    rng = np.random.Generator(np.random.PCG64(10))
    x = rng.standard_normal((20000, 64)).astype(np.float16)     # more rows than wavefronts in the grid
    g, b = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32), (0.1 * rng.standard_normal(64)).astype(np.float32)
    got = host(ops.layer_norm(dev(x), dev(g), dev(b), eps=1e-5))
    assert_close(got, oracle.layer_norm(x, g, b, eps=1e-5), np.float16)


def test_unaligned_operands(oracle):
    """Operands that start one element into a buffer: no 128-bit access, same results."""
    rng = np.random.Generator(np.random.PCG64(13))
    for dtype, ld in ((np.float16, 1024), (np.float32, 768), (np.float16, 16)):
        x = rng.standard_normal((50, ld)).astype(dtype)
        sk = rng.standard_normal((50, ld)).astype(dtype)
        g, b = (1 + 0.1 * rng.standard_normal(ld)).astype(np.float32), (0.1 * rng.standard_normal(ld)).astype(np.float32)
        shifted = lambda a: dev(np.concatenate([[0], a.reshape(-1)]).astype(a.dtype))[1:].reshape(a.shape)
        dx, dsk = shifted(x), shifted(sk)
        assert dx.data_ptr() % 16 != 0 and dx.is_contiguous()
        got = host(ops.skip_layer_norm(dx, dev(g), dev(b), skip=dsk, eps=1e-5))
        assert_close(got, oracle.skip_layer_norm(x, g, b, skip=sk, eps=1e-5), dtype)


def test_many_wide_rows_loop_path(oracle):
    rng = np.random.Generator(np.random.PCG64(12))
    x = rng.standard_normal((2500, 8192)).astype(np.float16)    # more rows than workgroups in the grid
    sk = rng.standard_normal((2500, 8192)).astype(np.float16)
    g, b = (1 + 0.1 * rng.standard_normal(8192)).astype(np.float32), (0.1 * rng.standard_normal(8192)).astype(np.float32)
    got = host(ops.skip_layer_norm(dev(x), dev(g), dev(b), skip=dev(sk), eps=1e-5))
    assert_close(got, oracle.skip_layer_norm(x, g, b, skip=sk, eps=1e-5), np.float16)


def test_emb_layer_norm_mask_and_out_of_table_ids(oracle):
    wl = workloads.config3(variant=7, dtype=np.float32, batch=5, seq=70)
    ids, seg, msk = wl.input_ids.copy(), wl.segment_ids.copy(), wl.input_mask.copy()
    msk[3, 1] = 0                      # a hole: mask index is the first zero, not the count of ones
    msk[:, 4] = 1                      # no zero at all -> S
    ids[2, 0] = 40000                  # outside the word table: contributes a zero row, raises the flag
    seg[6, 3] = 9
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    out, midx = ops.emb_layer_norm(dev(ids), dev(seg), dev(msk), dev(wl.word), dev(wl.pos), dev(wl.tok),
                                   f32(wl.gamma), f32(wl.beta), eps=wl.eps, oob_flag=flag)
    want, wmidx, oob = oracle.emb_layer_norm(ids, seg, msk, wl.word, wl.pos, wl.tok, wl.gamma, wl.beta, eps=wl.eps)
    assert oob == 2 and int(flag.item()) == 1
    assert_close(host(out), want, np.float32)
    np.testing.assert_array_equal(host(midx), wmidx)
    assert wmidx[1] == 3 and wmidx[4] == 70


# ---- through the plugin objects ------------------------------------------------------------------
def test_plugin_layer_norm_with_weights_reference_shape(oracle, kats):
    """test_torch_nodes.h:293-299: input [20,5,10], LayerNorm(10) with the stored weights, threshold 1e-3."""
    k = kats["layer_norm_with_weights"]
    a, b = np.array(k["data0"], np.float32), np.array(k["data1"], np.float32)
    gamma, beta = (a, b) if a.sum() > b.sum() else (b, a)
    c = REG.getPluginCreator("ForwardLayerNormPluginDynamic", "1")
    # fields as trt_normalization_creator.h:147-157 sends them (no eps reaches the plugin)
    p = c.createPlugin("skip_layer_norm", [F("ld", 10), F("beta", beta), F("gamma", gamma), F("type_id", lib.F32),
                                           F("has_skip", 0), F("batch_size", 20)])
    x = np.random.Generator(np.random.PCG64(12)).standard_normal(k["input_shape"]).astype(np.float32)
    out = host(p(dev(x)))
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (10,), torch.from_numpy(gamma), torch.from_numpy(beta),
                                         k["eps"]).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-3)
    assert_close(out, oracle.layer_norm(x, gamma, beta, eps=0.0), np.float32)
    again = host(c.deserializePlugin("ln", p.serialize())(dev(x)))
    np.testing.assert_array_equal(out, again)


def test_plugin_layer_norm_without_weights_reference_shape(oracle):
    """test_torch_nodes.h:285-291 (layer_norm.pth: torch.layer_norm(x, x.shape[1:], None, None, 1e-5) on
    [3,3,14,32]): the normalised axes are flattened to one row of 1344 elements, gamma 1 and beta 0."""
    x = np.random.Generator(np.random.PCG64(14)).standard_normal((3, 3, 14, 32)).astype(np.float32)
    ld = 3 * 14 * 32
    c = REG.getPluginCreator("ForwardLayerNormPluginDynamic", "1")
    p = c.createPlugin("layer_norm", [F("ld", ld), F("beta", np.zeros(ld, np.float32)),
                                      F("gamma", np.ones(ld, np.float32)), F("type_id", lib.F32),
                                      F("eps", np.array([1e-5], np.float32))])
    out = host(p(dev(x.reshape(3, ld)))).reshape(x.shape)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (3, 14, 32), None, None, 1e-5).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-3)                      # the reference test's threshold
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5)
    assert_close(out.reshape(3, ld), oracle.layer_norm(x.reshape(3, ld), np.ones(ld, np.float32),
                                                       np.zeros(ld, np.float32), eps=1e-5), np.float32)


def test_plugins_config5_chain(oracle):
    wl = workloads.config5(variant=1, batch=4, seq=64)
    up = lambda a: a.astype(np.float32)
    ce = REG.getPluginCreator("CustomEmbLayerNormPluginDynamic", "1")
    emb = ce.createPlugin("embeddings", [
        F("bert_embeddings_layernorm_beta", up(wl.beta)), F("bert_embeddings_layernorm_gamma", up(wl.gamma)),
        F("bert_embeddings_word_embeddings", up(wl.word)), F("bert_embeddings_token_type_embeddings", up(wl.tok)),
        F("bert_embeddings_position_embeddings", up(wl.pos)), F("output_fp16", 1), F("mha_type_id", lib.F16),
        F("eps", np.array([wl.eps], np.float32))])
    e, midx = emb(dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask))
    assert tuple(e.shape) == (64, 4, 1024, 1, 1) and tuple(midx.shape) == (4, 1) and e.dtype == torch.float16
    wemb, wmidx, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                           wl.gamma, wl.beta, eps=wl.eps)
    assert_close(host(e).reshape(64, 4, 1024), wemb, np.float16)
    np.testing.assert_array_equal(host(midx).reshape(-1), wmidx)

    cs = REG.getPluginCreator("CustomSkipLayerNormPluginDynamic", "1")
    skip = cs.createPlugin("skip_ln", [F("beta", up(wl.skip_beta)), F("gamma", up(wl.skip_gamma)), F("ld", 1024),
                                       F("type_id", lib.F16), F("bias", up(wl.skip_bias)),
                                       F("eps", np.array([wl.eps], np.float32))])
    res = dev(wl.skip.reshape(64, 4, 1024, 1, 1))
    out = skip(e, res)
    want = oracle.skip_layer_norm(host(e).reshape(64, 4, 1024), wl.skip_gamma, wl.skip_beta, skip=wl.skip,
                                  bias=wl.skip_bias, eps=wl.eps)
    assert_close(host(out).reshape(64, 4, 1024), want, np.float16)
    # save / load keeps the result
    out2 = cs.deserializePlugin("skip_ln", skip.serialize())(e, res)
    np.testing.assert_array_equal(host(out), host(out2))
    e2, _ = ce.deserializePlugin("embeddings", emb.serialize())(dev(wl.input_ids), dev(wl.segment_ids),
                                                                dev(wl.input_mask))
    np.testing.assert_array_equal(host(e), host(e2))
    # a half-precision plugin refuses float input at configure time
    with pytest.raises(lib.FwdmiError):
        skip.configurePlugin([((64, 4, 1024), lib.F32)] * 2, [((64, 4, 1024), lib.F32)])


@pytest.mark.parametrize("batch_major", [False, True])
def test_one_plugin_for_embedding_and_skip_layer_norm_equals_the_two_plugins(oracle, batch_major):
    """CustomEmbLayerNormPluginDynamic with the skip_* fields stands for the embedding plugin and the
    SkipLayerNorm plugin behind it: one enqueue, bit-identical to the chain of the two, in both id layouts,
    also after serialize -> deserialize; against the oracle within the fp16 bar."""
    wl = workloads.config5(variant=2, batch=3, seq=80)
    up = lambda a: a.astype(np.float32)
    S, B, H = 80, 3, 1024
    lay = (lambda a: np.ascontiguousarray(np.swapaxes(a, 0, 1))) if batch_major else (lambda a: a)
    ids, seg, msk = (dev(lay(a)) for a in (wl.input_ids, wl.segment_ids, wl.input_mask))
    res = dev(lay(wl.skip).reshape(tuple(lay(wl.input_ids).shape) + (H, 1, 1)))
    emb_f = [F("bert_embeddings_layernorm_beta", up(wl.beta)), F("bert_embeddings_layernorm_gamma", up(wl.gamma)),
             F("bert_embeddings_word_embeddings", up(wl.word)), F("bert_embeddings_token_type_embeddings", up(wl.tok)),
             F("bert_embeddings_position_embeddings", up(wl.pos)), F("output_fp16", 1), F("mha_type_id", lib.F16),
             F("eps", np.array([wl.eps], np.float32)), F("batch_major", int(batch_major))]
    ce = REG.getPluginCreator("CustomEmbLayerNormPluginDynamic", "1")
    cs = REG.getPluginCreator("CustomSkipLayerNormPluginDynamic", "1")
    e, midx = ce.createPlugin("embeddings", emb_f)(ids, seg, msk)
    want = cs.createPlugin("skip_ln", [F("beta", up(wl.skip_beta)), F("gamma", up(wl.skip_gamma)), F("ld", H),
                                       F("type_id", lib.F16), F("bias", up(wl.skip_bias)),
                                       F("eps", np.array([wl.eps], np.float32))])(e, res)
    both = ce.createPlugin("embeddings+skip", emb_f + [
        F("skip_beta", up(wl.skip_beta)), F("skip_gamma", up(wl.skip_gamma)), F("skip_bias", up(wl.skip_bias)),
        F("skip_eps", np.array([wl.eps], np.float32))])
    got, gmidx = both(ids, seg, msk, res)
    assert tuple(got.shape) == tuple(e.shape)
    np.testing.assert_array_equal(host(got).view(np.uint16), host(want).view(np.uint16))
    np.testing.assert_array_equal(host(gmidx), host(midx))
    got2, _ = ce.deserializePlugin("embeddings+skip", both.serialize())(ids, seg, msk, res)
    np.testing.assert_array_equal(host(got2).view(np.uint16), host(want).view(np.uint16))
    wemb, wmidx, _ = oracle.emb_layer_norm(wl.input_ids, wl.segment_ids, wl.input_mask, wl.word, wl.pos, wl.tok,
                                           wl.gamma, wl.beta, eps=wl.eps)
    wout = oracle.skip_layer_norm(wemb, wl.skip_gamma, wl.skip_beta, skip=wl.skip, bias=wl.skip_bias, eps=wl.eps)
    g = host(got).reshape(tuple(lay(wl.input_ids).shape) + (H,))
    assert_close(np.swapaxes(g, 0, 1) if batch_major else g, wout, np.float16)
    np.testing.assert_array_equal(host(gmidx).reshape(-1), wmidx)
    # without a bias, and a residual of the wrong type is refused
    nob = ce.createPlugin("embeddings+skip", emb_f + [F("skip_beta", up(wl.skip_beta)), F("skip_gamma", up(wl.skip_gamma)),
                                                      F("skip_eps", np.array([wl.eps], np.float32))])
    got3, _ = nob(ids, seg, msk, res)
    want3 = cs.createPlugin("skip_ln", [F("beta", up(wl.skip_beta)), F("gamma", up(wl.skip_gamma)), F("ld", H),
                                        F("type_id", lib.F16), F("eps", np.array([wl.eps], np.float32))])(e, res)
    np.testing.assert_array_equal(host(got3).view(np.uint16), host(want3).view(np.uint16))
    with pytest.raises(lib.FwdmiError):
        nob(ids, seg, msk, res.float())


def test_launches_can_be_captured_in_a_hip_graph(oracle):
    """enqueue allocates nothing and never synchronises, so a chain of launches can be captured
    once and replayed; every replay (with eager work in between) must equal the eager result."""
    wl = workloads.config5(variant=2, batch=4, seq=64)
    a = [dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask), dev(wl.word), dev(wl.pos), dev(wl.tok),
         f32(wl.gamma), f32(wl.beta)]
    sk, g, b, bi = dev(wl.skip), f32(wl.skip_gamma), f32(wl.skip_beta), f32(wl.skip_bias)
    emb = torch.empty((64, 4, 1024), dtype=torch.float16, device="cuda")
    midx = torch.empty((4,), dtype=torch.int32, device="cuda")
    out = torch.empty_like(emb)
    bw = workloads.config2(variant=6, table_dtype=np.float16, rows=5000, n_bags=300)
    tb, ix, of = dev(bw.table), dev(bw.indices), dev(bw.offsets)
    bag_out = torch.empty((300, 128), dtype=torch.float16, device="cuda")

    def chain():
        ops.emb_layer_norm(*a, eps=wl.eps, out=emb, mask_idx=midx)
        ops.skip_layer_norm(emb, g, b, skip=sk, bias=bi, eps=wl.eps, out=out)
        ops.embedding_bag(tb, ix, of, "sum", out=bag_out)

    chain()
    torch.cuda.synchronize()
    want = [t.clone() for t in (emb, midx, out, bag_out)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    for i in range(4):
        for t in (emb, midx, out, bag_out):
            t.fill_(0)                                   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip((emb, midx, out, bag_out), want):
            assert torch.equal(got, w), "replay %d differs from the eager result" % i


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_batch_major_layout_equals_transposed_sequence_major(oracle, dtype):
    """[B,S] ids in, [B,S,H] out: the transposes the reference wraps around the plugin
    (trt_bert_creator.h:64-71,106-109) folded into the kernel's indexing."""
    wl = workloads.config3(variant=11, dtype=dtype, batch=6, seq=40)
    a = [dev(wl.word), dev(wl.pos), dev(wl.tok), f32(wl.gamma), f32(wl.beta)]
    ref, rmidx = ops.emb_layer_norm(dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask), *a, eps=wl.eps)
    t = lambda x: np.ascontiguousarray(x.T)
    got, midx = ops.emb_layer_norm(dev(t(wl.input_ids)), dev(t(wl.segment_ids)), dev(t(wl.input_mask)), *a,
                                   eps=wl.eps, batch_major=True)
    assert tuple(got.shape) == (6, 40, 768)
    np.testing.assert_array_equal(host(got), host(ref).transpose(1, 0, 2))
    np.testing.assert_array_equal(host(midx), host(rmidx))
    np.testing.assert_array_equal(host(midx), wl.valid_len)
    # through the plugin: optional creator field "batch_major"
    up = lambda x: x.astype(np.float32)
    c = REG.getPluginCreator("CustomEmbLayerNormPluginDynamic", "1")
    p = c.createPlugin("embeddings", [
        F("bert_embeddings_layernorm_beta", up(wl.beta)), F("bert_embeddings_layernorm_gamma", up(wl.gamma)),
        F("bert_embeddings_word_embeddings", up(wl.word)), F("bert_embeddings_token_type_embeddings", up(wl.tok)),
        F("bert_embeddings_position_embeddings", up(wl.pos)), F("output_fp16", int(dtype == np.float16)),
        F("mha_type_id", 0), F("eps", np.array([wl.eps], np.float32)), F("batch_major", 1)])
    assert p.getOutputDimensions(0, [(6, 40)] * 3) == [6, 40, 768, 1, 1] and p.getOutputDimensions(1, [(6, 40)] * 3) == [6, 1]
    e, m = p(dev(t(wl.input_ids)), dev(t(wl.segment_ids)), dev(t(wl.input_mask)))
    np.testing.assert_array_equal(host(e).reshape(6, 40, 768), host(got))
    np.testing.assert_array_equal(host(m).reshape(-1), wl.valid_len)
    q = c.deserializePlugin("embeddings", p.serialize())
    e2, _ = q(dev(t(wl.input_ids)), dev(t(wl.segment_ids)), dev(t(wl.input_mask)))
    np.testing.assert_array_equal(host(e2), host(e))


@pytest.mark.parametrize("dtype,hidden", [(np.float16, 128), (np.float16, 256), (np.float32, 64), (np.float32, 128),
                                          (np.float16, 8)])
def test_small_hidden_sizes_share_a_wavefront(oracle, dtype, hidden):
    """BERT-tiny / -mini sized embeddings: several tokens per wavefront.  Values against the oracle,
    mask index and out-of-table ids exactly, batch-major equal to the transposed sequence-major run."""
    rng = np.random.Generator(np.random.PCG64(100 + hidden))
    S, B, V, P = 37, 9, 500, 40
    mk = lambda *s, mu=0.0, sd=0.02: (mu + sd * rng.standard_normal(s)).astype(np.float32).astype(dtype)
    word, pos, tok = mk(V, hidden), mk(P, hidden), mk(2, hidden)
    g, b = mk(hidden, mu=1.0).astype(np.float32), mk(hidden).astype(np.float32)
    ids = rng.integers(0, V, (S, B)).astype(np.int32)
    seg = rng.integers(0, 2, (S, B)).astype(np.int32)
    lens = rng.integers(1, S + 1, B)
    msk = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    tabs = [dev(word), dev(pos), dev(tok), dev(g), dev(b)]
    got, midx = ops.emb_layer_norm(dev(ids), dev(seg), dev(msk), *tabs, eps=1e-12, oob_flag=flag)
    want, wmidx, n_oob = oracle.emb_layer_norm(ids, seg, msk, word, pos, tok, g, b, eps=1e-12)
    assert n_oob == 0 and not flag.item()
    assert_close(host(got), want, dtype)
    np.testing.assert_array_equal(host(midx), wmidx)
    t = lambda x: np.ascontiguousarray(x.T)
    bm, bmidx = ops.emb_layer_norm(dev(t(ids)), dev(t(seg)), dev(t(msk)), *tabs, eps=1e-12, batch_major=True)
    np.testing.assert_array_equal(host(bm), host(got).transpose(1, 0, 2))
    np.testing.assert_array_equal(host(bmidx), wmidx)
    # ids outside their tables contribute zero rows and raise the flag
    bad_ids, bad_seg = ids.copy(), seg.copy()
    bad_ids[3, 2], bad_ids[10, 0], bad_seg[5, 5] = V + 7, -1, 2
    got, _ = ops.emb_layer_norm(dev(bad_ids), dev(bad_seg), dev(msk), *tabs, eps=1e-12, oob_flag=flag)
    want, _, n_oob = oracle.emb_layer_norm(bad_ids, bad_seg, msk, word, pos, tok, g, b, eps=1e-12)
    assert n_oob == 3 and flag.item() == 1
    assert_close(host(got), want, dtype)


@pytest.mark.parametrize("dtype,hidden", [(np.float16, 1024), (np.float32, 1024), (np.float16, 768), (np.float16, 100),
                                          (np.float16, 128), (np.float32, 64)])
def test_fused_emb_skip_equals_two_launches(oracle, dtype, hidden):
    """One pass computing LN2(LN(word+pos+tok) + residual + bias) is bit-identical to the
    EmbLayerNorm launch followed by the SkipLayerNorm launch (hidden=100 takes the fallback)."""
    rng = np.random.Generator(np.random.PCG64(hidden))
    S, B, V = 48, 5, 300
    mk = lambda *s, mu=0.0, sd=0.02: (mu + sd * rng.standard_normal(s)).astype(np.float32).astype(dtype)
    word, pos, tok = mk(V, hidden), mk(64, hidden), mk(2, hidden)
    g1, b1, g2, b2, bias2 = mk(hidden, mu=1.0), mk(hidden), mk(hidden, mu=1.0), mk(hidden), mk(hidden)
    ids = rng.integers(0, V, (S, B)).astype(np.int32)
    seg = rng.integers(0, 2, (S, B)).astype(np.int32)
    msk = (rng.random((S, B)) < 0.9).astype(np.int32)
    skip = rng.standard_normal((S, B, hidden)).astype(dtype)
    common = [dev(ids), dev(seg), dev(msk), dev(word), dev(pos), dev(tok), f32(g1), f32(b1)]
    emb, midx = ops.emb_layer_norm(*common, eps=1e-12)
    two = ops.skip_layer_norm(emb, f32(g2), f32(b2), skip=dev(skip), bias=f32(bias2), eps=1e-6)
    keep = torch.zeros_like(emb)
    one, midx1 = ops.emb_layer_norm(*common, eps=1e-12, skip=dev(skip), gamma2=f32(g2), beta2=f32(b2),
                                    bias2=f32(bias2), eps2=1e-6, emb_out=keep)
    np.testing.assert_array_equal(host(one), host(two))
    np.testing.assert_array_equal(host(keep), host(emb))
    np.testing.assert_array_equal(host(midx1), host(midx))
    # without the optional copy and without bias2
    two_nb = ops.skip_layer_norm(emb, f32(g2), f32(b2), skip=dev(skip), eps=0.0)
    one_nb, _ = ops.emb_layer_norm(*common, eps=1e-12, skip=dev(skip), gamma2=f32(g2), beta2=f32(b2))
    np.testing.assert_array_equal(host(one_nb), host(two_nb))
    # and against the oracle, stage by stage
    want = oracle.skip_layer_norm(host(emb), g2, b2, skip=skip, bias=bias2, eps=1e-6)
    assert_close(host(one), want, dtype)
