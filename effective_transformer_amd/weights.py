"""Encoder weights from local checkpoint files into the 16-slot layout of the reference's `weights_value`
(python/effective_transformer/__init__.py:55-74: per layer q_k, q_b, k_k, k_b, v_k, v_b, ao_k, ao_b, ao_ln_beta,
ao_ln_gamma, i_k, i_b, o_k, o_b, o_ln_beta, o_ln_gamma, which is the creation order of the variables in
sample/tensorflow/modeling.py:828-882).

Two naming schemes are understood, in `.npz` or `.safetensors` files (both are loaded without executing anything
from the file):

* TF-BERT variable names: `<prefix>layer_<l>/attention/self/query/kernel` ...; kernels are `[in, out]` already.
* Hugging Face BertModel names: `<prefix>layer.<l>.attention.self.query.weight` ...; Linear weights are `[out, in]`
  and are transposed on import.
"""
from __future__ import annotations

import os
import re
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

# slot -> (TF suffix, HF suffix, is_kernel)
SLOTS: Tuple[Tuple[str, str, bool], ...] = (
    ("attention/self/query/kernel", "attention.self.query.weight", True),
    ("attention/self/query/bias", "attention.self.query.bias", False),
    ("attention/self/key/kernel", "attention.self.key.weight", True),
    ("attention/self/key/bias", "attention.self.key.bias", False),
    ("attention/self/value/kernel", "attention.self.value.weight", True),
    ("attention/self/value/bias", "attention.self.value.bias", False),
    ("attention/output/dense/kernel", "attention.output.dense.weight", True),
    ("attention/output/dense/bias", "attention.output.dense.bias", False),
    ("attention/output/LayerNorm/beta", "attention.output.LayerNorm.bias", False),
    ("attention/output/LayerNorm/gamma", "attention.output.LayerNorm.weight", False),
    ("intermediate/dense/kernel", "intermediate.dense.weight", True),
    ("intermediate/dense/bias", "intermediate.dense.bias", False),
    ("output/dense/kernel", "output.dense.weight", True),
    ("output/dense/bias", "output.dense.bias", False),
    ("output/LayerNorm/beta", "output.LayerNorm.bias", False),
    ("output/LayerNorm/gamma", "output.LayerNorm.weight", False),
)


def read_tensors(path: str) -> Dict[str, np.ndarray]:
    """name -> array from a `.npz` or `.safetensors` file."""
    ext = os.path.splitext(path)[1].lower()
    if ext == ".npz":
        with np.load(path, allow_pickle=False) as z:
            return {k: z[k] for k in z.files}
    if ext == ".safetensors":
        from safetensors.numpy import load_file
        return dict(load_file(path))
    raise ValueError("unsupported checkpoint format %r (want .npz or .safetensors)" % ext)


def _clean(name: str) -> str:
    return name[:-2] if name.endswith(":0") else name


def _find(tensors: Dict[str, np.ndarray], tail: str, prefix: Optional[str]) -> Optional[str]:
    hits = [k for k in tensors if _clean(k).endswith(tail) and (prefix is None or _clean(k).startswith(prefix))]
    # "layer_1/..." must not match "layer_11/...": the character in front of the tail has to be a separator
    hits = [k for k in hits if len(_clean(k)) == len(tail) or _clean(k)[-len(tail) - 1] in "/._"]
    if len(hits) > 1:
        raise ValueError("ambiguous tensor name for %r: %s (pass prefix=...)" % (tail, sorted(hits)))
    return hits[0] if hits else None


def count_layers(tensors: Dict[str, np.ndarray]) -> int:
    ids = set()
    for k in tensors:
        m = re.search(r"layer[_.](\d+)[/.]", _clean(k))
        if m:
            ids.add(int(m.group(1)))
    return max(ids) + 1 if ids else 0


def weights_from_tensors(tensors: Dict[str, np.ndarray], num_layers: Optional[int] = None,
                         prefix: Optional[str] = None) -> List[np.ndarray]:
    """The 16 * num_layers arrays in slot order.  Kernels come out `[in, out]` (row-major)."""
    if num_layers is None:
        num_layers = count_layers(tensors)
    if num_layers < 1:
        raise ValueError("no encoder layers found")
    out: List[np.ndarray] = []
    for l in range(num_layers):
        for tf_tail, hf_tail, is_kernel in SLOTS:
            key = _find(tensors, "layer_%d/%s" % (l, tf_tail), prefix)
            transpose = False
            if key is None:
                key = _find(tensors, "layer.%d.%s" % (l, hf_tail), prefix)
                transpose = is_kernel
            if key is None:
                raise KeyError("layer %d: neither layer_%d/%s nor layer.%d.%s in the checkpoint" % (l, l, tf_tail, l, hf_tail))
            a = np.asarray(tensors[key])
            if transpose:
                a = a.T
            out.append(np.ascontiguousarray(a))
        q, ao, i, o_ = out[-16], out[-10], out[-6], out[-4]
        H = q.shape[0]
        if q.shape != (H, H) or ao.shape != (H, H) or i.shape[0] != H or o_.shape != (i.shape[1], H):
            raise ValueError("layer %d: kernel shapes %s %s %s %s are not an encoder layer" % (l, q.shape, ao.shape, i.shape, o_.shape))
    return out


def load_weights(path: str, num_layers: Optional[int] = None, prefix: Optional[str] = None) -> List[np.ndarray]:
    return weights_from_tensors(read_tensors(path), num_layers, prefix)


def save_weights(path: str, weights_value: Sequence[np.ndarray], prefix: str = "bert/encoder/") -> None:
    """Writes `weights_value` under TF-BERT names (`.npz` or `.safetensors`)."""
    if len(weights_value) % 16:
        raise ValueError("expected a multiple of 16 tensors")
    named = {}
    for n, a in enumerate(weights_value):
        named["%slayer_%d/%s" % (prefix, n // 16, SLOTS[n % 16][0])] = np.ascontiguousarray(a)
    ext = os.path.splitext(path)[1].lower()
    if ext == ".npz":
        np.savez(path, **named)
    elif ext == ".safetensors":
        from safetensors.numpy import save_file
        save_file(named, path)
    else:
        raise ValueError("unsupported checkpoint format %r" % ext)


def fuse_qkv(weights_value: Sequence[np.ndarray], layer: int) -> Tuple[np.ndarray, np.ndarray]:
    """Kernel `[H, 3H]` and bias `[3H]` of one layer's fused Q/K/V projection (for callers that want one GEMM operand;
    the layer op itself takes the three kernels as they are and runs them as one grouped launch)."""
    s = weights_value[16 * layer:16 * layer + 6]
    return np.concatenate([s[0], s[2], s[4]], axis=1), np.concatenate([s[1], s[3], s[5]])
