"""PyTorch adapter: the kernels as ``torch.ops.fwdmi.*`` custom ops plus drop-in modules.

Counterpart of the reference's torch-side glue (``TorchEngine::ParseInput`` / ``CopyFromBuffers``,
source/fwd_torch/torch_engine/torch_engine.cpp:134-174): there, int64 ids are copied to int32 and
outputs are copied out of engine buffers; here the ops consume int32 or int64 ids as they are and
write straight into the tensors they return.  ``nn.EmbeddingBag`` / ``nn.Embedding`` modules of an
inference model can be swapped for the HIP path with ``replace_embedding_modules``.
"""
from typing import List, Optional

import torch

from . import ops

_MODE = {"sum": 0, "mean": 1, "max": 2}


@torch.library.custom_op("fwdmi::embedding_bag", mutates_args=())
def embedding_bag(weight: torch.Tensor, indices: torch.Tensor, offsets: torch.Tensor, mode: int,
                  per_sample_weights: Optional[torch.Tensor], include_last_offset: bool) -> torch.Tensor:
    return ops.embedding_bag(weight, indices.contiguous(), offsets.contiguous().to(indices.dtype), mode,
                             per_sample_weights=per_sample_weights, include_last_offset=include_last_offset)


@embedding_bag.register_fake
def _(weight, indices, offsets, mode, per_sample_weights, include_last_offset):
    n = offsets.numel() - (1 if include_last_offset else 0)
    return weight.new_empty((n, weight.shape[1]))


@torch.library.custom_op("fwdmi::embedding_bag_group", mutates_args=())
def embedding_bag_group(weights: List[torch.Tensor], indices: List[torch.Tensor], offsets: List[torch.Tensor],
                        mode: int, include_last_offset: bool,
                        per_sample_weights: List[Optional[torch.Tensor]]) -> torch.Tensor:
    """The embedding bags of a sparse stage and their concatenation: ``[B, T*dim]`` from one launch.
    ``per_sample_weights``: one entry per table, ``None`` for a table without weights (sum only)."""
    idt = indices[0].dtype
    psw = [None if w is None else w.to(weights[0].dtype).contiguous() for w in per_sample_weights]
    if all(w is None for w in psw):
        psw = None
    return ops.embedding_bag_group(weights, [i.contiguous() for i in indices],
                                   [o.contiguous().to(idt) for o in offsets], mode,
                                   include_last_offset=include_last_offset, per_sample_weights=psw)


@embedding_bag_group.register_fake
def _(weights, indices, offsets, mode, include_last_offset, per_sample_weights):
    n = offsets[0].numel() - (1 if include_last_offset else 0)
    return weights[0].new_empty((n, len(weights) * weights[0].shape[1]))


@torch.library.custom_op("fwdmi::embedding_bag_fixed", mutates_args=())
def embedding_bag_fixed(weight: torch.Tensor, indices: torch.Tensor, mode: int) -> torch.Tensor:
    return ops.embedding_bag_fixed(weight, indices.contiguous(), mode)


@embedding_bag_fixed.register_fake
def _(weight, indices, mode):
    return weight.new_empty((indices.shape[0], weight.shape[1]))


@torch.library.custom_op("fwdmi::embedding", mutates_args=())
def embedding(weight: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``aten::embedding`` as the plain row gather (op 999); out-of-range ids give zero rows."""
    flat = indices.contiguous().reshape(1, -1)
    return ops.gather(weight, flat).reshape(tuple(indices.shape) + (weight.shape[1],))


@embedding.register_fake
def _(weight, indices):
    return weight.new_empty(tuple(indices.shape) + (weight.shape[1],))


@torch.library.custom_op("fwdmi::skip_layer_norm", mutates_args=())
def skip_layer_norm(x: torch.Tensor, skip: Optional[torch.Tensor], gamma: torch.Tensor, beta: torch.Tensor,
                    bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    f = lambda t: None if t is None else t.float().contiguous()
    return ops.skip_layer_norm(x.contiguous(), f(gamma), f(beta), skip=None if skip is None else skip.contiguous(),
                               bias=f(bias), eps=eps)


@skip_layer_norm.register_fake
def _(x, skip, gamma, beta, bias, eps):
    return torch.empty_like(x)


class EmbeddingBag(torch.nn.Module):
    """Inference replacement of ``torch.nn.EmbeddingBag`` (1-D ids + offsets, or 2-D ids)."""

    def __init__(self, weight, mode="sum", include_last_offset=False):
        super().__init__()
        self.weight = torch.nn.Parameter(weight.detach().contiguous(), requires_grad=False)
        self.mode, self.include_last_offset = mode, include_last_offset

    @classmethod
    def from_torch(cls, m):
        if m.padding_idx is not None or m.max_norm is not None:
            raise NotImplementedError("padding_idx / max_norm are not part of the plugin path")
        return cls(m.weight, m.mode, m.include_last_offset)

    def forward(self, input, offsets=None, per_sample_weights=None):
        if input.dim() == 2:
            if per_sample_weights is not None:
                raise NotImplementedError("per_sample_weights with 2-D ids")
            return torch.ops.fwdmi.embedding_bag_fixed(self.weight, input, _MODE[self.mode])
        psw = None if per_sample_weights is None else per_sample_weights.to(self.weight.dtype).contiguous()
        return torch.ops.fwdmi.embedding_bag(self.weight, input, offsets, _MODE[self.mode], psw,
                                             self.include_last_offset)


class EmbeddingBagCollection(torch.nn.Module):
    """The ``nn.EmbeddingBag`` list of a DLRM-style model (equal dim, mode and dtype) as one module:
    ``forward(indices_list, offsets_list)`` returns what ``torch.cat([bag_t(ids_t, offsets_t)], dim=1)``
    returns, from one launch."""

    def __init__(self, weights, mode="sum", include_last_offset=False):
        super().__init__()
        self.weights = torch.nn.ParameterList(
            [torch.nn.Parameter(w.detach().contiguous(), requires_grad=False) for w in weights])
        self.mode, self.include_last_offset = mode, include_last_offset

    @classmethod
    def from_torch(cls, bags):
        bags = list(bags)
        first = bags[0]
        for m in bags:
            if m.padding_idx is not None or m.max_norm is not None:
                raise NotImplementedError("padding_idx / max_norm are not part of the plugin path")
            if (m.mode, m.include_last_offset, m.embedding_dim, m.weight.dtype) != \
                    (first.mode, first.include_last_offset, first.embedding_dim, first.weight.dtype):
                raise ValueError("the bags of a collection share mode, include_last_offset, dim and dtype")
        return cls([m.weight for m in bags], first.mode, first.include_last_offset)

    def forward(self, indices, offsets, per_sample_weights=None):
        psw = [None] * len(self.weights) if per_sample_weights is None else list(per_sample_weights)
        return torch.ops.fwdmi.embedding_bag_group(list(self.weights), list(indices), list(offsets),
                                                   _MODE[self.mode], self.include_last_offset, psw)


class Embedding(torch.nn.Module):
    """Inference replacement of ``torch.nn.Embedding`` (plain gather)."""

    def __init__(self, weight):
        super().__init__()
        self.weight = torch.nn.Parameter(weight.detach().contiguous(), requires_grad=False)

    def forward(self, input):
        return torch.ops.fwdmi.embedding(self.weight, input)


def replace_embedding_modules(model):
    """Swaps every ``nn.EmbeddingBag`` / ``nn.Embedding`` (without padding_idx / max_norm) in place."""
    for name, child in list(model.named_children()):
        if isinstance(child, torch.nn.EmbeddingBag) and child.padding_idx is None and child.max_norm is None:
            setattr(model, name, EmbeddingBag.from_torch(child))
        elif isinstance(child, torch.nn.Embedding) and child.padding_idx is None and child.max_norm is None:
            setattr(model, name, Embedding(child.weight))
        else:
            replace_embedding_modules(child)
    return model
