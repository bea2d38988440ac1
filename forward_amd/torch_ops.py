"""PyTorch adapter: the kernels as ``torch.ops.fwdmi.*`` custom ops plus drop-in modules.

Counterpart of the reference's torch-side glue (``TorchEngine::ParseInput`` / ``CopyFromBuffers``,
source/fwd_torch/torch_engine/torch_engine.cpp:134-174): there, int64 ids are copied to int32 and
outputs are copied out of engine buffers; here the bag ops consume int32 or int64 ids as they are and
write straight into the tensors they return, or, in their ``*_out`` forms, into tensors the caller
supplies (declared to PyTorch as mutated arguments), so that a serving loop reuses its buffers.
The BERT ops (``emb_layer_norm``, ``emb_skip_layer_norm``) take the ``[B, S]`` tensors a PyTorch model
holds (``batch_major``) or the plugin's ``[S, B]``.  ``nn.EmbeddingBag`` / ``nn.Embedding`` modules of an
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


def _i32(t):
    """ids of the BERT ops: the launchers read int32 (int64 ids are narrowed, as the reference's
    ParseInput does for every integer input, torch_engine.cpp:134-140)."""
    return None if t is None else t.to(torch.int32).contiguous()


def _f32(t):
    return None if t is None else t.float().contiguous()


@torch.library.custom_op("fwdmi::emb_layer_norm", mutates_args=())
def emb_layer_norm(input_ids: torch.Tensor, segment_ids: torch.Tensor, input_mask: Optional[torch.Tensor],
                   word: torch.Tensor, pos: torch.Tensor, tok: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                   eps: float, batch_major: bool) -> List[torch.Tensor]:
    """BERT embedding + LayerNorm: ``[out, mask_idx]``.  ids / mask are ``[B, S]`` with ``batch_major``
    (out ``[B, S, H]``), else the plugin's ``[S, B]`` (out ``[S, B, H]``); ``mask_idx`` is int32 ``[B]``
    (empty without a mask)."""
    out, midx = ops.emb_layer_norm(_i32(input_ids), _i32(segment_ids), _i32(input_mask), word, pos, tok, _f32(gamma),
                                   _f32(beta), eps=eps, batch_major=batch_major)
    return [out, midx if midx is not None else torch.empty((0,), dtype=torch.int32, device=out.device)]


@emb_layer_norm.register_fake
def _(input_ids, segment_ids, input_mask, word, pos, tok, gamma, beta, eps, batch_major):
    b = input_ids.shape[0] if batch_major else input_ids.shape[1]
    return [word.new_empty(tuple(input_ids.shape) + (word.shape[1],)),
            input_ids.new_empty((b if input_mask is not None else 0,), dtype=torch.int32)]


@torch.library.custom_op("fwdmi::emb_skip_layer_norm", mutates_args=())
def emb_skip_layer_norm(input_ids: torch.Tensor, segment_ids: torch.Tensor, input_mask: Optional[torch.Tensor],
                        word: torch.Tensor, pos: torch.Tensor, tok: torch.Tensor, gamma: torch.Tensor,
                        beta: torch.Tensor, eps: float, skip: torch.Tensor, gamma2: torch.Tensor, beta2: torch.Tensor,
                        bias2: Optional[torch.Tensor], eps2: float, batch_major: bool) -> List[torch.Tensor]:
    """The embedding stage and the SkipLayerNorm that consumes it in one launch:
    ``out = LN2(LN(word + pos + tok) + skip (+ bias2))``, equal bit for bit to the two ops in a row."""
    out, midx = ops.emb_layer_norm(_i32(input_ids), _i32(segment_ids), _i32(input_mask), word, pos, tok, _f32(gamma),
                                   _f32(beta), eps=eps, batch_major=batch_major, skip=skip.contiguous(),
                                   gamma2=_f32(gamma2), beta2=_f32(beta2), bias2=_f32(bias2), eps2=eps2)
    return [out, midx if midx is not None else torch.empty((0,), dtype=torch.int32, device=out.device)]


@emb_skip_layer_norm.register_fake
def _(input_ids, segment_ids, input_mask, word, pos, tok, gamma, beta, eps, skip, gamma2, beta2, bias2, eps2, batch_major):
    b = input_ids.shape[0] if batch_major else input_ids.shape[1]
    return [word.new_empty(tuple(input_ids.shape) + (word.shape[1],)),
            input_ids.new_empty((b if input_mask is not None else 0,), dtype=torch.int32)]


# ---- forms that write into the caller's tensors ------------------------------------------------
# Where the reference copies every output out of an engine buffer into a fresh tensor
# (TorchEngine::CopyFromBuffers, torch_engine.cpp:150-174), these write the result where the caller
# wants it; PyTorch is told which argument is written (mutates_args), nothing is returned.

@torch.library.custom_op("fwdmi::embedding_bag_out", mutates_args=("out",))
def embedding_bag_out(out: torch.Tensor, weight: torch.Tensor, indices: torch.Tensor, offsets: torch.Tensor, mode: int,
                      per_sample_weights: Optional[torch.Tensor], include_last_offset: bool, out_col: int) -> None:
    """``out[:, out_col : out_col + dim]`` = the bags; ``out`` is ``[n_bags, W]`` of the table's dtype."""
    ops.embedding_bag(weight, indices.contiguous(), offsets.contiguous().to(indices.dtype), mode,
                      per_sample_weights=per_sample_weights, include_last_offset=include_last_offset, out=out,
                      out_col=out_col, out_dtype=out.dtype)


@torch.library.custom_op("fwdmi::embedding_bag_group_out", mutates_args=("out",))
def embedding_bag_group_out(out: torch.Tensor, weights: List[torch.Tensor], indices: List[torch.Tensor],
                            offsets: List[torch.Tensor], mode: int, include_last_offset: bool,
                            per_sample_weights: List[Optional[torch.Tensor]]) -> None:
    idt = indices[0].dtype
    psw = [None if w is None else w.to(weights[0].dtype).contiguous() for w in per_sample_weights]
    if all(w is None for w in psw):
        psw = None
    ops.embedding_bag_group(weights, [i.contiguous() for i in indices], [o.contiguous().to(idt) for o in offsets], mode,
                            include_last_offset=include_last_offset, per_sample_weights=psw, out=out, out_dtype=out.dtype)


@torch.library.custom_op("fwdmi::skip_layer_norm_out", mutates_args=("out",))
def skip_layer_norm_out(out: torch.Tensor, x: torch.Tensor, skip: Optional[torch.Tensor], gamma: torch.Tensor,
                        beta: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> None:
    """``out``: a tensor of ``x``'s shape and dtype (not ``x`` or ``skip`` themselves)."""
    ops.skip_layer_norm(x.contiguous(), _f32(gamma), _f32(beta), skip=None if skip is None else skip.contiguous(),
                        bias=_f32(bias), eps=eps, out=out)


@torch.library.custom_op("fwdmi::emb_layer_norm_out", mutates_args=("out", "mask_idx"))
def emb_layer_norm_out(out: torch.Tensor, mask_idx: Optional[torch.Tensor], input_ids: torch.Tensor,
                       segment_ids: torch.Tensor, input_mask: Optional[torch.Tensor], word: torch.Tensor,
                       pos: torch.Tensor, tok: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, eps: float,
                       skip: Optional[torch.Tensor], gamma2: Optional[torch.Tensor], beta2: Optional[torch.Tensor],
                       bias2: Optional[torch.Tensor], eps2: float, batch_major: bool) -> None:
    """Both BERT forms (``skip`` given: the fused embedding + SkipLayerNorm) into ``out`` / ``mask_idx``."""
    ops.emb_layer_norm(_i32(input_ids), _i32(segment_ids), _i32(input_mask), word, pos, tok, _f32(gamma), _f32(beta),
                       eps=eps, batch_major=batch_major, out=out, mask_idx=mask_idx,
                       skip=None if skip is None else skip.contiguous(), gamma2=_f32(gamma2), beta2=_f32(beta2),
                       bias2=_f32(bias2), eps2=eps2)


class BertEmbeddings(torch.nn.Module):
    """Inference replacement of a BERT embedding block (word + position + token-type lookup, then
    LayerNorm) on ``[B, S]`` tensors: ``forward(input_ids, token_type_ids, attention_mask)`` returns
    ``(embeddings [B, S, H], valid_length int32 [B])``, the two outputs of the embedding plugin the
    reference wires in (trt_bert_creator.h:113-155), without its transposes to and from ``[S, B]``."""

    def __init__(self, word, pos, tok, gamma, beta, eps=1e-12):
        super().__init__()
        p = lambda t: torch.nn.Parameter(t.detach().contiguous(), requires_grad=False)
        self.word, self.pos, self.tok = p(word), p(pos), p(tok)
        self.gamma, self.beta, self.eps = p(gamma.float()), p(beta.float()), float(eps)

    def forward(self, input_ids, token_type_ids=None, attention_mask=None):
        if token_type_ids is None:
            token_type_ids = torch.zeros_like(input_ids)
        out, midx = torch.ops.fwdmi.emb_layer_norm(input_ids, token_type_ids, attention_mask, self.word, self.pos,
                                                   self.tok, self.gamma, self.beta, self.eps, True)
        return out, midx


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
