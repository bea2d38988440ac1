"""Writes ``torch_cpu_vectors.npz``: small input/output vectors produced by the libtorch CPU
operators the reference's unit tests use as ground truth
(source/unit_test/unit_test_torch_helper.h:82-87): ``aten::_embedding_bag`` in sum / mean / max
mode (ties, NaN, empty bags, argmax = row id, int32 and int64 ids, fp16 tables, per-sample
weights) and ``aten::layer_norm``.  torch is an installed library, not reference code.

  python tests/golden/make_torch_vectors.py        (torch 2.10.0 wrote the committed file)
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def bag(w, idx, off, mode, psw=None):
    out, _, _, maxi = torch.ops.aten._embedding_bag(w, idx, off, False, mode, False, psw, False, -1)
    return out.numpy(), maxi.numpy()


def main():
    v = {}
    nan = float("nan")
    # hand-made table exercising ties (first wins), NaN in first / later position, negatives
    w = torch.tensor([[1., 5., nan, -1.], [2., 5., 0., -3.], [nan, 4., 1., -1.], [0., 0., 0., 0.],
                      [-7., 9., -0., 2.]])
    idx = torch.tensor([0, 1, 2, 2, 0, 1, 1, 4, 3, 4], dtype=torch.int64)
    off = torch.tensor([0, 3, 3, 5, 7, 10, 10], dtype=torch.int64)  # bags: 3, 0, 2, 2, 3, 0 ids
    v["tie_table"], v["tie_idx"], v["tie_off"] = w.numpy(), idx.numpy(), off.numpy()
    v["tie_max_out"], v["tie_max_arg"] = bag(w, idx, off, 2)
    v["tie_mean_out"], _ = bag(w, idx, off, 1)
    v["tie_sum_out"], _ = bag(w, idx, off, 0)

    g = torch.Generator().manual_seed(1234)
    w = torch.randn(200, 24, generator=g)
    # quantise so that ties are common in max mode
    wq = (w * 2).round() / 2
    lengths = torch.randint(0, 9, (40,), generator=g)
    off = torch.cumsum(lengths, 0) - lengths
    idx = torch.randint(0, 200, (int(lengths.sum()),), generator=g)
    psw = torch.rand(idx.numel(), generator=g)
    v["rnd_table"], v["rnd_tableq"], v["rnd_idx"], v["rnd_off"], v["rnd_psw"] = (
        w.numpy(), wq.numpy(), idx.numpy(), off.numpy(), psw.numpy())
    v["rnd_sum"], _ = bag(w, idx, off, 0)
    v["rnd_mean"], _ = bag(w, idx, off, 1)
    v["rnd_max"], v["rnd_max_arg"] = bag(wq, idx, off, 2)
    v["rnd_wsum"], _ = bag(w, idx, off, 0, psw)
    o32, a32 = bag(wq, idx.int(), off.int(), 2)
    v["rnd_max_i32"], v["rnd_max_arg_i32"] = o32, a32
    wh = w.half()
    v["rnd_sum_f16"] = torch.nn.functional.embedding_bag(idx, wh, off, mode="sum").numpy()
    v["rnd_mean_f16"] = torch.nn.functional.embedding_bag(idx, wh, off, mode="mean").numpy()
    v["rnd_max_f16"] = torch.nn.functional.embedding_bag(idx, wq.half(), off, mode="max").numpy()

    x = torch.randn(6, 5, 48, generator=g)
    gam, bet = 1 + 0.1 * torch.randn(48, generator=g), 0.1 * torch.randn(48, generator=g)
    v["ln_x"], v["ln_gamma"], v["ln_beta"] = x.numpy(), gam.numpy(), bet.numpy()
    v["ln_out_eps1e-5"] = torch.nn.functional.layer_norm(x, (48,), gam, bet, 1e-5).numpy()
    v["ln_out_eps1e-12"] = torch.nn.functional.layer_norm(x, (48,), gam, bet, 1e-12).numpy()
    np.savez_compressed(os.path.join(HERE, "torch_cpu_vectors.npz"), **v)
    print({k: a.shape for k, a in v.items()})


if __name__ == "__main__":
    main()
