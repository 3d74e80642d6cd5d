"""torch-tensor wrappers of the kernel-level entry points of the C ABI (one per launcher of
the reference's cuda/cuda_kernels.h and cuda/attention.h, plus the fused attention and the
GEMM).  Used by the unit tests, the per-kernel benchmark and profiling runs."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from .ops import _dtype_code, _p, _stream, _workspace, handle


def _call(name, dev, *args):
    lib = _lib.load()
    h = handle(dev)
    _lib.check(getattr(lib, name)(h, *args), h)


def exclusive_scan(d_in: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    n = d_in.numel()
    out = torch.empty_like(d_in)
    ws = _workspace(d_in.device, "scan", lib.et_input_workspace_bytes(1, n))
    _call("et_exclusive_scan", d_in.device, _p(out), _p(d_in), n, _p(ws), ws.numel(), _stream())
    return out


def compress(from_tensor, mask, prefix_sum):
    B, S, H = from_tensor.shape
    to = torch.zeros_like(from_tensor)
    bidx = torch.full_like(mask, -1)
    widx = torch.full_like(mask, -1)
    _call("et_compress", from_tensor.device, _dtype_code(from_tensor.dtype), _p(from_tensor), _p(mask),
          _p(prefix_sum), _p(to), _p(bidx), _p(widx), B, S, H, _stream())
    return to, bidx, widx


def restore(from_tensor, batch_idx, word_idx, valid_word_num, B, S):
    H = from_tensor.shape[-1]
    to = torch.empty(B, S, H, dtype=from_tensor.dtype, device=from_tensor.device)
    _call("et_restore", from_tensor.device, _dtype_code(from_tensor.dtype), _p(to), _p(from_tensor), _p(batch_idx),
          _p(word_idx), _p(valid_word_num), B, S, H, _stream())
    return to


def add_bias_act(out, bias, m: Optional[int] = None, m_dev: Optional[torch.Tensor] = None):
    rows, n = out.shape
    _call("et_add_bias_act", out.device, _dtype_code(out.dtype), _p(out), _p(bias), rows if m is None else m, n,
          _p(m_dev), _stream())
    return out


def add_bias_input_layernorm(out, inp, bias, gamma, beta, m: Optional[int] = None,
                             m_dev: Optional[torch.Tensor] = None):
    rows, n = out.shape
    _call("et_add_bias_input_layernorm", out.device, _dtype_code(out.dtype), _p(out), _p(inp), _p(bias), _p(gamma),
          _p(beta), rows if m is None else m, n, _p(m_dev), _stream())
    return out


def add_qkv_bias_padding(q, bq, k, bk, v, bv, valid_word_num, B, S, heads, d, batch_idx, word_idx):
    lib = _lib.load()
    dev = q.device
    bufs = [torch.full((B, heads, S, d), float("nan"), dtype=q.dtype, device=dev) for _ in range(3)]
    ws = _workspace(dev, "seq", lib.et_seq_workspace_bytes(B))
    _call("et_add_qkv_bias_padding", dev, _dtype_code(q.dtype), _p(q), _p(bq), _p(k), _p(bk), _p(v), _p(bv),
          _p(bufs[0]), _p(bufs[1]), _p(bufs[2]), _p(valid_word_num), B, S, heads, d, _p(batch_idx), _p(word_idx),
          _p(ws), ws.numel(), _stream())
    return bufs


def softmax(qk, attr_mask, scaler: float):
    B, heads, S, _ = qk.shape
    _call("et_softmax", qk.device, _dtype_code(qk.dtype), _p(qk), _p(attr_mask), B, heads, S, C.c_float(scaler),
          _stream())
    return qk


def transpose_rm_padding(src, valid_word_num, batch_idx, word_idx):
    B, heads, S, d = src.shape
    dst = torch.zeros(B * S, heads * d, dtype=src.dtype, device=src.device)
    _call("et_transpose_rm_padding", src.device, _dtype_code(src.dtype), _p(src), _p(dst), _p(valid_word_num), B, S,
          heads, d, _p(batch_idx), _p(word_idx), _stream())
    return dst


def attention(q, k, v, layout: int, packed_ld: int, attr_mask, valid_word_num, B, S, heads, d, batch_idx, word_idx,
              dst: Optional[torch.Tensor] = None, seq_start: Optional[torch.Tensor] = None):
    """seq_start: the table of ops.sequence_starts for this batch; the call is then the attention kernel alone."""
    lib = _lib.load()
    dev = attr_mask.device
    if dst is None:
        dst = torch.zeros(B * S, heads * d, dtype=attr_mask.dtype, device=dev)
    if seq_start is not None:
        _call("et_attention_with_starts", dev, _dtype_code(attr_mask.dtype), _p(q), _p(k), _p(v), layout, packed_ld,
              _p(attr_mask), _p(dst), _p(valid_word_num), B, S, heads, d, _p(batch_idx), _p(word_idx), _p(seq_start), None,
              seq_start.numel() * seq_start.element_size(), _stream())
        return dst
    ws = _workspace(dev, "seq", lib.et_seq_workspace_bytes(B))
    _call("et_attention", dev, _dtype_code(attr_mask.dtype), _p(q), _p(k), _p(v), layout, packed_ld, _p(attr_mask),
          _p(dst), _p(valid_word_num), B, S, heads, d, _p(batch_idx), _p(word_idx), _p(ws), ws.numel(), _stream())
    return dst


def gemm(a, b, bias=None, m: Optional[int] = None, m_dev: Optional[torch.Tensor] = None,
         out: Optional[torch.Tensor] = None, gelu: bool = False):
    """a [m, k] . b [k, n] (+ bias); gelu=True applies bias + GELU to the product on its way out."""
    rows, k = a.shape
    n = b.shape[1]
    if out is None:
        out = torch.zeros(rows, n, dtype=a.dtype, device=a.device)
    _call("et_gemm_bias_gelu" if gelu else "et_gemm", a.device, _dtype_code(a.dtype), _p(a), _p(b), _p(out), _p(bias),
          rows if m is None else m, n, k, _p(m_dev), _stream())
    return out


def transpose_weight(w, out: Optional[torch.Tensor] = None):
    """[k, n] -> [n, k] (fp16), the layout gemm_bt takes."""
    k, n = w.shape
    if out is None:
        out = torch.empty(n, k, dtype=w.dtype, device=w.device)
    _call("et_transpose_weight", w.device, _dtype_code(w.dtype), _p(w), _p(out), k, n, _stream())
    return out


def gemm_bt(a, bt, bias=None, m: Optional[int] = None, m_dev: Optional[torch.Tensor] = None,
            out: Optional[torch.Tensor] = None, gelu: bool = False):
    """a [m, k] . bt [n, k]^T (+ bias): the large-M kernel of the encoder layer.  gelu=True applies bias + GELU to the
    product on its way out (what add_bias_act would do in a second pass)."""
    rows, k = a.shape
    n = bt.shape[0]
    if out is None:
        out = torch.zeros(rows, n, dtype=a.dtype, device=a.device)
    _call("et_gemm_bt_bias_gelu" if gelu else "et_gemm_bt", a.device, _dtype_code(a.dtype), _p(a), _p(bt), _p(out),
          _p(bias), rows if m is None else m, n, k, _p(m_dev), _stream())
    return out
