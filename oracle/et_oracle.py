"""CPU oracle for the padding-free BERT encoder path (TEST INFRASTRUCTURE ONLY).

This module restates, in numpy, the arithmetic of the reference's GPU kernels and
host orchestration so that the HIP implementation can be checked against it.  It is
imported only by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline
leg; the shipped library never calls it.

Each function cites the reference lines it follows (paths relative to the
reference tree).  Two numeric modes exist:

* "fp32": every value is held in float32; contractions are evaluated in float64
  and rounded once to float32 (the reference accumulates in float32 inside cuBLAS
  in an unspecified order, so the ideal value is the tightest neutral statement).
* "fp16": values are rounded to IEEE binary16 (round-to-nearest-even) at exactly
  the points where the reference stores or computes in half; contractions are
  evaluated in float64 and rounded once to half.

Pinning status (what independent check covers each function is listed in
tests/test_oracle_pins.py):
  exclusive_scan / input_op / restore ... pinned by the worked examples in the
      reference's Readme.md:14-21 and images/1.png and by brute force.
  add_bias_act ... pinned against torch gelu(approximate="tanh").
  add_bias_input_layernorm ... pinned against torch layer_norm(eps=1e-6).
  softmax ... pinned against torch.softmax with the additive -10000 mask.
  add_qkv_bias_padding / transpose_rm_padding ... pinned by round trip + brute force.
  embedding_postprocess / embedding_input ... pinned against transformers' BertEmbeddings with the
      same tables, torch layer_norm(eps=1e-12) and a position-by-position loop.
  layer / encoder ... pinned against a HuggingFace BertLayer built from a local
      config and against tf_graph_encoder (the reference benchmark's own check).
  cuBLAS half-accumulate ordering and device-intrinsic ULP behaviour (__expf,
      rsqrtf, tanhf): parity unpinned (only a run of the reference on NVIDIA
      hardware could pin them); the tolerances absorb them.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

# --------------------------------------------------------------------------- #
# rounding helpers
# --------------------------------------------------------------------------- #

def _np_dtype(dtype: str):
    if dtype == "fp32":
        return np.float32
    if dtype == "fp16":
        return np.float16
    raise ValueError("dtype must be 'fp32' or 'fp16'")


def rnd(x, dtype: str):
    """Round an array (any float type) to the storage type, round-to-nearest-even."""
    return np.asarray(x).astype(_np_dtype(dtype))


def hadd(a, b):
    """IEEE half add with a single rounding (the sum of two halves is exact in float64)."""
    return (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)


def hmul(a, b):
    """IEEE half multiply with a single rounding (the product is exact in float32)."""
    return (a.astype(np.float32) * b.astype(np.float32)).astype(np.float16)


def gemm(a, b, dtype: str):
    """C = A.B with alpha=1, beta=0 (tf_op/bert_transformer_op.cu.cc:110-119 and the
    other cublasGemmEx call sites); weights are [in,out] row-major and used untransposed."""
    c = a.astype(np.float64) @ b.astype(np.float64)
    return rnd(c, dtype)


# --------------------------------------------------------------------------- #
# Input op: scan, valid-token count, index build, compress
# --------------------------------------------------------------------------- #

def exclusive_scan(mask_flat) -> np.ndarray:
    """prefix[i] = sum_{j<i} mask[j] over the flattened int32 mask
    (cuda/cuda_kernels.cu:709-718)."""
    m = np.asarray(mask_flat, dtype=np.int32).reshape(-1)
    out = np.zeros_like(m)
    if m.size > 1:
        np.cumsum(m[:-1], out=out[1:])
    return out


def input_op(from_tensor, mask):
    """EffectiveTransformerInput (tf_op/bert_transformer_op.cu.cc:266-331 and
    cuda/cuda_kernels.cu:278-340).

    Returns (to_tensor[T,H], T, batch_idx[T], word_idx[T], prefix[B*S]).  Entries of
    the reference's index outputs beyond T are uninitialised, so only T are returned."""
    mask = np.asarray(mask, dtype=np.int32)
    B, S = mask.shape
    prefix = exclusive_scan(mask)
    flat = mask.reshape(-1)
    # T = prefix[last] + (mask[last] == 1)   (bert_transformer_op.cu.cc:306-315)
    T = int(prefix[-1]) + (1 if flat[-1] == 1 else 0)
    H = from_tensor.shape[-1]
    to_tensor = np.zeros((T, H), dtype=from_tensor.dtype)
    batch_idx = np.zeros(T, dtype=np.int32)
    word_idx = np.zeros(T, dtype=np.int32)
    src = np.asarray(from_tensor).reshape(B * S, H)
    for p in range(B * S):                       # cuda_kernels.cu:285-306
        if flat[p] > 0.5:
            t = prefix[p]
            batch_idx[t] = p // S
            word_idx[t] = p % S
            to_tensor[t] = src[p]
    return to_tensor, T, batch_idx, word_idx, prefix


def input_op_fast(from_tensor, mask):
    """Vectorised form of input_op for large inputs (same results; checked against
    the loop form in the tests)."""
    mask = np.asarray(mask, dtype=np.int32)
    B, S = mask.shape
    prefix = exclusive_scan(mask)
    flat = mask.reshape(-1)
    T = int(prefix[-1]) + (1 if flat[-1] == 1 else 0)
    pos = np.nonzero(flat > 0.5)[0]
    batch_idx = (pos // S).astype(np.int32)
    word_idx = (pos % S).astype(np.int32)
    H = from_tensor.shape[-1]
    to_tensor = np.ascontiguousarray(np.asarray(from_tensor).reshape(B * S, H)[pos])
    return to_tensor, T, batch_idx, word_idx, prefix


def embedding_postprocess(input_ids, token_type_ids, word_table, type_table, pos_table, gamma, beta, dtype: str):
    """Padded embedding block of the reference's sample model, [B,S] ids -> [B,S,H]
    (sample/tensorflow/modeling.py:380-521 with dropout off): output = word_table[ids];
    output += type_table[type_ids]; output += pos_table[:S]; layer_norm (tf.contrib.layers.layer_norm: biased
    variance + 1e-12).  Sums in the element type in that order, statistics in float.  Ids outside a table give a zero
    row (tf.gather on a GPU).  type_table / pos_table may be None."""
    ids = np.asarray(input_ids, dtype=np.int64)
    B, S = ids.shape
    H = word_table.shape[1]
    npdt = _np_dtype(dtype)

    def gather(table, idx):
        ok = (idx >= 0) & (idx < table.shape[0])
        rows = np.asarray(table).astype(npdt)[np.where(ok, idx, 0)]
        return np.where(ok[..., None], rows, npdt(0)).astype(npdt)

    x = gather(word_table, ids)
    if type_table is not None:
        t = gather(type_table, np.asarray(token_type_ids, dtype=np.int64))
        x = hadd(x, t) if dtype == "fp16" else (x + t).astype(np.float32)
    if pos_table is not None:
        p = np.broadcast_to(np.asarray(pos_table).astype(npdt)[:S][None], (B, S, H))
        x = hadd(x, p) if dtype == "fp16" else (x + p).astype(np.float32)
    x = x.astype(np.float64)
    mean = x.sum(axis=-1, keepdims=True) / H
    var = ((x - mean) ** 2).sum(axis=-1, keepdims=True) / H + 1e-12
    y = (x - mean) / np.sqrt(var) * np.asarray(gamma).astype(np.float64) + np.asarray(beta).astype(np.float64)
    return rnd(y, dtype)


def embedding_input(input_ids, token_type_ids, mask, word_table, type_table, pos_table, gamma, beta, dtype: str):
    """embedding_postprocess followed by input_op (the order in which the reference runs them,
    python/effective_transformer/__init__.py:40-45 on the output of modeling.py:171-194)."""
    padded = embedding_postprocess(input_ids, token_type_ids, word_table, type_table, pos_table, gamma, beta, dtype)
    return input_op_fast(padded, mask)


def restore(from_tensor, T: int, batch_idx, word_idx, B: int, S: int):
    """EffectiveTransformerOutput: zero [B,S,H] then scatter T rows
    (tf_op/bert_transformer_op.cu.cc:351-360, cuda/cuda_kernels.cu:396-406)."""
    H = from_tensor.shape[-1]
    out = np.zeros((B * S, H), dtype=from_tensor.dtype)
    dst = batch_idx[:T].astype(np.int64) * S + word_idx[:T]
    out[dst] = from_tensor[:T]
    return out.reshape(B, S, H)


# --------------------------------------------------------------------------- #
# Row kernels
# --------------------------------------------------------------------------- #

_GELU_C = np.float32(0.7978845608028654)
_GELU_A = np.float32(0.044715)


def add_bias_act(out, bias, dtype: str):
    """gelu_tanh(out + bias) (cuda/cuda_kernels.cu:29-51, 88-130)."""
    if dtype == "fp32":
        x = (out.astype(np.float32) + bias.astype(np.float32)).astype(np.float32)
        x64 = x.astype(np.float64)
        # float expression 0.7978845608028654f * (x + 0.044715f * x * x * x)
        u = np.float64(_GELU_C) * (x64 + np.float64(_GELU_A) * x64 * x64 * x64)
        cdf = 0.5 * (1.0 + np.tanh(u))
        return (x64 * cdf).astype(np.float32)
    v = hadd(out.astype(np.float16), bias.astype(np.float16))          # __hadd2
    v3 = hmul(v, hmul(v, v))                                             # two half roundings
    vf = v.astype(np.float64)
    u = np.float64(_GELU_C) * (vf + np.float64(_GELU_A) * v3.astype(np.float64))
    cdf = (0.5 * (1.0 + np.tanh(u))).astype(np.float32).astype(np.float16)  # __float22half2_rn
    return hmul(v, cdf)


def add_bias_input_layernorm(out, inp, bias, gamma, beta, dtype: str):
    """LN(out + input + bias) * gamma + beta, eps 1e-6 added to the biased variance,
    two-pass statistics in float (cuda/cuda_kernels.cu:157-237)."""
    n = out.shape[-1]
    if dtype == "fp32":
        x = ((out.astype(np.float32) + inp.astype(np.float32)).astype(np.float32)
             + bias.astype(np.float32)).astype(np.float32)
    else:
        x = hadd(hadd(out.astype(np.float16), inp.astype(np.float16)), bias.astype(np.float16))
    x = x.astype(np.float64)
    mean = x.sum(axis=-1, keepdims=True) / n
    var = ((x - mean) ** 2).sum(axis=-1, keepdims=True) / n + 1e-6
    y = (x - mean) / np.sqrt(var) * gamma.astype(np.float64) + beta.astype(np.float64)
    return rnd(y, dtype)


# --------------------------------------------------------------------------- #
# Attention side
# --------------------------------------------------------------------------- #

def add_qkv_bias_padding(q, bq, k, bk, v, bv, T, B, S, heads, d, batch_idx, word_idx, dtype: str):
    """[T,H] + bias -> zero-initialised [B,heads,S,d] for Q, K and V
    (cuda/attention.cu:105-176; zero fill at tf_op/bert_transformer_op.cu.cc:146)."""
    outs = []
    for src, b in ((q, bq), (k, bk), (v, bv)):
        if dtype == "fp32":
            val = (src[:T].astype(np.float32) + b.astype(np.float32)).astype(np.float32)
        else:
            val = hadd(src[:T].astype(np.float16), b.astype(np.float16))
        dst = np.zeros((B, heads, S, d), dtype=_np_dtype(dtype))
        dst[batch_idx[:T], :, word_idx[:T], :] = val.reshape(T, heads, d)
        outs.append(dst)
    return outs


def softmax(qk, attr_mask, scaler: float, dtype: str):
    """Masked, scaled softmax over the last axis of qk[B,heads,S,S] with
    attr_mask[B,S,S] (cuda/attention.cu:249-334):
      t = qk*scale + (1-mask)*(-10000); m = max(max_k t, 0); e = exp(t-m);
      p = e / (sum e + 1e-6).
    The clamp of the maximum at 0 comes from the second stage of blockReduceMax
    (cuda/attention.cu:91-92), which feeds 0 for idle lanes whenever the block has
    fewer than 32 warps, i.e. for every S <= 512.  For 512 < S < 1024 the block has 1024
    threads (:345-356) and the threads beyond S feed -1e-20 into the reduction
    (:267-270), which in float acts exactly like the clamp at 0 (t - (-1e-20) == t);
    only S = 1024 has neither and uses the true maximum."""
    S = qk.shape[-1]
    t = (qk.astype(np.float32) * np.float32(scaler)).astype(np.float32)
    mv = ((np.float32(1.0) - attr_mask.astype(np.float32)) * np.float32(-10000.0)).astype(np.float32)
    t = (t + mv[:, None, :, :]).astype(np.float32)
    m = np.maximum(t.max(axis=-1, keepdims=True), np.float32(0.0)) if S < 1024 else t.max(axis=-1, keepdims=True)
    e = np.exp((t - m).astype(np.float64))
    e = np.where((t - m) < -103.0, 0.0, e)        # float32 exp underflows to 0 below ~-103.97
    p = e / (e.sum(axis=-1, keepdims=True) + 1e-6)
    return rnd(p, dtype)


def transpose_rm_padding(src, T, batch_idx, word_idx):
    """[B,heads,S,d] -> packed [T,heads*d] (cuda/attention.cu:387-440)."""
    B, heads, S, d = src.shape
    return np.ascontiguousarray(src[batch_idx[:T], :, word_idx[:T], :]).reshape(T, heads * d)


def attention(qp, kp, vp, attr_mask, T, batch_idx, word_idx, dtype: str):
    """batched QK^T (unscaled, stored in T) -> softmax -> batched PV -> un-pad
    (tf_op/bert_transformer_op.cu.cc:159-192)."""
    d = qp.shape[-1]
    qk = rnd(np.einsum("bhqd,bhkd->bhqk", qp.astype(np.float64), kp.astype(np.float64)), dtype)
    scaler = 1.0 / math.sqrt(float(d))
    if dtype == "fp16":
        scaler = float(np.float16(scaler))        # DataType_ scaler (half) at :172
    p = softmax(qk, attr_mask, scaler, dtype)
    ctx = rnd(np.einsum("bhqk,bhkd->bhqd", p.astype(np.float64), vp.astype(np.float64)), dtype)
    return transpose_rm_padding(ctx, T, batch_idx, word_idx)


# --------------------------------------------------------------------------- #
# Layer op and whole encoder
# --------------------------------------------------------------------------- #

WEIGHT_SLOTS = (
    # order of python/effective_transformer/__init__.py:55-74 (beta before gamma)
    "attr_kernel_q", "attr_bias_q", "attr_kernel_k", "attr_bias_k",
    "attr_kernel_v", "attr_bias_v", "attr_output_kernel", "attr_output_bias",
    "attr_output_layernorm_beta", "attr_output_layernorm_gamma",
    "inter_kernel", "inter_bias", "output_kernel", "output_bias",
    "output_layernorm_beta", "output_layernorm_gamma",
)


def layer(from_tensor, to_tensor, attr_mask, T, batch_idx, word_idx, w: Sequence[np.ndarray],
          B, S, heads, d, dtype: str, return_intermediates: bool = False):
    """EffectiveTransformer layer op on packed tokens
    (tf_op/bert_transformer_op.cu.cc:104-247).  `w` is the 16-slot list in
    WEIGHT_SLOTS order."""
    (wq, bq, wk, bk, wv, bv, wo, bo, ln1_b, ln1_g, wi, bi, wo2, bo2, ln2_b, ln2_g) = w
    x = from_tensor[:T]
    xt = to_tensor[:T]
    q = gemm(x, wq, dtype)
    k = gemm(xt, wk, dtype)
    v = gemm(xt, wv, dtype)
    qp, kp, vp = add_qkv_bias_padding(q, bq, k, bk, v, bv, T, B, S, heads, d, batch_idx, word_idx, dtype)
    ctx = attention(qp, kp, vp, attr_mask, T, batch_idx, word_idx, dtype)
    a = gemm(ctx, wo, dtype)
    y1 = add_bias_input_layernorm(a, x, bo, ln1_g, ln1_b, dtype)
    inter = add_bias_act(gemm(y1, wi, dtype), bi, dtype)
    o = gemm(inter, wo2, dtype)
    y2 = add_bias_input_layernorm(o, y1, bo2, ln2_g, ln2_b, dtype)
    if return_intermediates:
        return y2, dict(q=q, k=k, v=v, qp=qp, kp=kp, vp=vp, ctx=ctx, a=a, y1=y1, inter=inter, o=o)
    return y2


def encoder(from_tensor, mask, attr_mask, weights: Sequence[np.ndarray], heads: int, d: int, dtype: str):
    """Input -> L x Layer (from == to) -> Output
    (python/effective_transformer/__init__.py:41-82).  Returns [B,S,H] with zeros at padding."""
    B, S = mask.shape
    x, T, bidx, widx, _ = input_op_fast(rnd(from_tensor, dtype), mask)
    L = len(weights) // 16
    for l in range(L):
        x = layer(x, x, attr_mask, T, bidx, widx, weights[16 * l:16 * l + 16], B, S, heads, d, dtype)
    return restore(x, T, bidx, widx, B, S)


# --------------------------------------------------------------------------- #
# The reference's CPU path: the TF BERT encoder graph, restated
# --------------------------------------------------------------------------- #

def tf_graph_encoder(from_tensor, attr_mask, weights: Sequence[np.ndarray], heads: int, d: int):
    """modeling.transformer_model (sample/tensorflow/modeling.py:755-893) on the padded
    [B*S,H] matrix in float32: dense Q/K/V, scores * 1/sqrt(d), + (1-mask)*-10000, exact
    softmax (:702-721), dense + residual + LayerNorm (:858-864), dense + tanh-GELU
    (:264-277, :867-872), dense + residual + LayerNorm (:875-882); no dropout
    (sample/tensorflow/benchmark.py:29-30).  LayerNorm epsilon is 1e-12
    (tf.contrib.layers.layer_norm's variance_epsilon).  Runs on torch CPU kernels so
    that all host cores are used; this is also the timed CPU baseline."""
    import torch

    B, S, H = from_tensor.shape
    x = torch.from_numpy(np.ascontiguousarray(from_tensor, dtype=np.float32)).reshape(B * S, H)
    adder = (1.0 - torch.from_numpy(np.ascontiguousarray(attr_mask, dtype=np.float32))) * -10000.0
    adder = adder[:, None, :, :]
    tw = [torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)) for a in weights]
    L = len(tw) // 16
    scale = 1.0 / math.sqrt(float(d))
    with torch.no_grad():
        for l in range(L):
            (wq, bq, wk, bk, wv, bv, wo, bo, ln1_b, ln1_g, wi, bi, wo2, bo2, ln2_b, ln2_g) = tw[16 * l:16 * l + 16]
            q = (x @ wq + bq).reshape(B, S, heads, d).permute(0, 2, 1, 3)
            k = (x @ wk + bk).reshape(B, S, heads, d).permute(0, 2, 1, 3)
            v = (x @ wv + bv).reshape(B, S, heads, d).permute(0, 2, 1, 3)
            sc = torch.matmul(q, k.transpose(-1, -2)) * scale + adder
            p = torch.softmax(sc, dim=-1)
            ctx = torch.matmul(p, v).permute(0, 2, 1, 3).reshape(B * S, H)
            a = ctx @ wo + bo
            y1 = torch.nn.functional.layer_norm(a + x, (H,), ln1_g, ln1_b, eps=1e-12)
            u = y1 @ wi + bi
            inter = u * 0.5 * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * torch.pow(u, 3))))
            o = inter @ wo2 + bo2
            x = torch.nn.functional.layer_norm(o + y1, (H,), ln2_g, ln2_b, eps=1e-12)
    return x.reshape(B, S, H).numpy()


# --------------------------------------------------------------------------- #
# Seeded synthetic workloads (mirrors sample/tensorflow/benchmark.py:38-61)
# --------------------------------------------------------------------------- #


# the benchmark's workload generator lives with the benchmark sample; the tests reach it through this module
from effective_transformer_amd.sample.workloads import (  # noqa: E402,F401
    WORKLOADS, Workload, draw_lens, make_layer_weights, make_masks, make_workload)
