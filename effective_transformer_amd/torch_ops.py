"""The three ops as torch.library custom ops (namespace `effective_transformer`), so that they can sit inside
PyTorch-ROCm graphs (torch.compile / export trace them through the registered fake kernels) the way the reference's
ops sit inside a TensorFlow graph (tf_op/bert_transformer_op.cc:31-77, 249-262, 359-372).

    to_tensor, valid_word_num, batch_idx, word_idx = torch.ops.effective_transformer.input(from_tensor, mask, heads, d)
    out = torch.ops.effective_transformer.layer(x, x, attr_mask, valid_word_num, batch_idx, word_idx, weights, heads, d)
    y = torch.ops.effective_transformer.output(out, valid_word_num, batch_idx, word_idx, heads, d)

`weights` is the list of the 16 tensors of one layer in the order of the reference's `weights_value`
(python/effective_transformer/__init__.py:55-74), already on the device in the dtype of the activations.
The valid-token count stays on the device (no host read-back), so the ops never synchronise.
"""
from __future__ import annotations

from typing import List, Tuple

import torch
from torch import Tensor

from . import ops

_NS = "effective_transformer"


@torch.library.custom_op(_NS + "::input", mutates_args=(), device_types="cuda")
def et_input(from_tensor: Tensor, mask: Tensor, head_num: int, size_per_head: int) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    B, S = mask.shape
    return ops.effective_transformer_input(from_tensor, mask, B, S, S, head_num, size_per_head)


@et_input.register_fake
def _(from_tensor, mask, head_num, size_per_head):
    return (torch.empty_like(from_tensor), mask.new_empty((1,)), torch.empty_like(mask), torch.empty_like(mask))


@torch.library.custom_op(_NS + "::layer", mutates_args=(), device_types="cuda")
def et_layer(from_tensor: Tensor, to_tensor: Tensor, attr_mask: Tensor, valid_word_num: Tensor, batch_idx: Tensor,
             word_idx: Tensor, weights: List[Tensor], head_num: int, size_per_head: int) -> Tensor:
    B, S = batch_idx.shape
    for w in weights:
        if w.device != from_tensor.device or w.dtype != from_tensor.dtype or not w.is_contiguous():
            raise ValueError("layer weights must be contiguous device tensors in the dtype of the activations")
    lw = ops.LayerWeights.from_slots(from_tensor.device, from_tensor.dtype, weights)   # no copies: pointers only
    return ops.effective_transformer(from_tensor, to_tensor, attr_mask, valid_word_num, batch_idx, word_idx, lw, B, S, S,
                                     head_num, size_per_head)


@et_layer.register_fake
def _(from_tensor, to_tensor, attr_mask, valid_word_num, batch_idx, word_idx, weights, head_num, size_per_head):
    if len(weights) != 16:
        raise ValueError("a layer has 16 weight tensors")
    return torch.empty_like(from_tensor)


@torch.library.custom_op(_NS + "::output", mutates_args=(), device_types="cuda")
def et_output(from_tensor: Tensor, valid_word_num: Tensor, batch_idx: Tensor, word_idx: Tensor, head_num: int,
              size_per_head: int) -> Tensor:
    B, S = batch_idx.shape
    return ops.effective_transformer_output(from_tensor, valid_word_num, batch_idx, word_idx, B, S, S, head_num,
                                            size_per_head)


@et_output.register_fake
def _(from_tensor, valid_word_num, batch_idx, word_idx, head_num, size_per_head):
    return torch.empty_like(from_tensor)


def encoder(from_tensor: Tensor, input_mask: Tensor, attention_mask: Tensor, layer_weights: List[List[Tensor]],
            head_num: int, size_per_head: int) -> Tensor:
    """Input -> L x Layer -> Output through the registered ops (traceable)."""
    op = getattr(torch.ops, _NS)
    x, vwn, bidx, widx = op.input(from_tensor, input_mask, head_num, size_per_head)
    for w in layer_weights:
        x = op.layer(x, x, attention_mask, vwn, bidx, widx, w, head_num, size_per_head)
    return op.output(x, vwn, bidx, widx, head_num, size_per_head)
