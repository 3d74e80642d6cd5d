"""Host-side mirror of the reference's three custom ops and of its Python glue
(python/effective_transformer/__init__.py:32-84), on torch-ROCm tensors.

torch is used for device memory and the current stream only; all computation happens in
libet_hip.so through the C ABI.
"""
from __future__ import annotations

import ctypes as C
import threading
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib

_handles: Dict[int, C.c_void_p] = {}
_workspaces: Dict[tuple, torch.Tensor] = {}
_lock = threading.Lock()


def _dtype_code(t: torch.dtype) -> int:
    if t == torch.float32:
        return _lib.ET_FP32
    if t == torch.float16:
        return _lib.ET_FP16
    raise TypeError("only float32 and float16 tensors are supported, got %s" % t)


def handle(device: torch.device) -> C.c_void_p:
    """One library handle per GPU."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    with _lock:
        h = _handles.get(idx)
        if h is None:
            h = C.c_void_p()
            _lib.check(_lib.load().et_create(C.byref(h), idx), None)
            _handles[idx] = h
        return h


_scope = threading.local()      # .owner: set while a GraphedEncoder warms up and captures (its buffers are its own)


def _workspace(device: torch.device, kind: str, nbytes: int) -> torch.Tensor:
    """One scratch buffer per (GPU, stream, kind, owner, host thread), grown on demand: calls queued on one stream by
    one thread run in order and may share it; calls on different streams get their own, so does every captured graph
    (a graph keeps the addresses it was captured with, and replays of two graphs on different streams may overlap),
    and so does every host thread (the layer op keeps its intermediate tensors there between the calls of one encoder
    pass, and two threads' passes interleave on a shared stream call by call)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    key = (idx, torch.cuda.current_stream(idx).cuda_stream, kind, getattr(_scope, "owner", None), threading.get_ident())
    with _lock:
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
            _workspaces[key] = ws
        return ws


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("tensors must live on the GPU")
        if not t.is_contiguous():
            raise ValueError("tensors must be contiguous")


# --------------------------------------------------------------------------- the three ops

def effective_transformer_input(from_tensor: torch.Tensor, mask: torch.Tensor, batch_size: int, from_seq_len: int,
                                to_seq_len: int, head_num: int, size_per_head: int, return_host_count: bool = False):
    """EffectiveTransformerInput (tf_op/bert_transformer_op.cc:249-340): returns
    (to_tensor, valid_word_num, batch_idx, word_idx) with the shapes of the reference op; the
    batch is taken from from_tensor.shape[0] ("dynamic batch size").  With
    return_host_count=True the valid-token count is also returned as a Python int (one
    stream synchronisation, as in the reference)."""
    lib = _lib.load()
    _require_cuda(from_tensor, mask)
    if mask.dtype != torch.int32:
        raise TypeError("mask must be int32")
    B = from_tensor.shape[0]
    S = from_seq_len
    dev = from_tensor.device
    to_tensor = torch.empty_like(from_tensor)
    valid_word_num = torch.empty(1, dtype=torch.int32, device=dev)
    batch_idx = torch.empty_like(mask)
    word_idx = torch.empty_like(mask)
    nbytes = lib.et_input_workspace_bytes(B, S)
    ws = _workspace(dev, "input", nbytes)
    host = C.c_int32(-1)
    h = handle(dev)
    st = lib.et_input(h, _dtype_code(from_tensor.dtype), _p(from_tensor), _p(mask), _p(to_tensor), _p(valid_word_num),
                      _p(batch_idx), _p(word_idx), B, S, head_num, size_per_head, _p(ws), ws.numel(), _stream(),
                      C.byref(host) if return_host_count else None)
    _lib.check(st, h)
    if return_host_count:
        return to_tensor, valid_word_num, batch_idx, word_idx, int(host.value)
    return to_tensor, valid_word_num, batch_idx, word_idx


class EmbeddingWeights:
    """The tables of the BERT embedding block on the device (sample/tensorflow/modeling.py:171-194):
    word_embeddings [V,H], token_type_embeddings [Vt,H] or None, position_embeddings [P,H] or None, LayerNorm
    gamma / beta [H]."""

    def __init__(self, device, dtype: torch.dtype, word_embeddings, layernorm_gamma, layernorm_beta,
                 token_type_embeddings=None, position_embeddings=None):
        def up(v):
            if v is None:
                return None
            if isinstance(v, np.ndarray):
                v = torch.from_numpy(np.ascontiguousarray(v))
            return v.to(device=device, dtype=dtype).contiguous()
        self.word, self.type, self.pos = up(word_embeddings), up(token_type_embeddings), up(position_embeddings)
        self.gamma, self.beta = up(layernorm_gamma), up(layernorm_beta)
        s = _lib.EmbeddingWeights()
        s.word_embeddings = self.word.data_ptr()
        s.token_type_embeddings = self.type.data_ptr() if self.type is not None else None
        s.position_embeddings = self.pos.data_ptr() if self.pos is not None else None
        s.layernorm_gamma, s.layernorm_beta = self.gamma.data_ptr(), self.beta.data_ptr()
        s.vocab_size = self.word.shape[0]
        s.type_vocab_size = self.type.shape[0] if self.type is not None else 0
        s.max_position_embeddings = self.pos.shape[0] if self.pos is not None else 0
        self.struct = s
        self.hidden = self.word.shape[1]
        self.dtype = dtype


def effective_transformer_embedding_input(input_ids: torch.Tensor, token_type_ids: Optional[torch.Tensor],
                                          mask: torch.Tensor, embeddings: EmbeddingWeights, head_num: int,
                                          size_per_head: int, return_host_count: bool = False):
    """Embedding block (modeling.py:380-521) fused with EffectiveTransformerInput: packed rows straight from the ids,
    the padded [B,S,H] embedding output is never written.  Returns what effective_transformer_input returns."""
    lib = _lib.load()
    _require_cuda(input_ids, mask)
    if token_type_ids is not None:
        _require_cuda(token_type_ids)
    for t in (input_ids, mask) + ((token_type_ids,) if token_type_ids is not None else ()):
        if t.dtype != torch.int32:
            raise TypeError("ids and mask must be int32")
    B, S = mask.shape
    dev = mask.device
    to_tensor = torch.empty(B, S, embeddings.hidden, dtype=embeddings.dtype, device=dev)
    valid_word_num = torch.empty(1, dtype=torch.int32, device=dev)
    batch_idx = torch.empty_like(mask)
    word_idx = torch.empty_like(mask)
    ws = _workspace(dev, "input", lib.et_input_workspace_bytes(B, S))
    host = C.c_int32(-1)
    h = handle(dev)
    st = lib.et_embedding_input(h, _dtype_code(embeddings.dtype), C.byref(embeddings.struct), _p(input_ids),
                                _p(token_type_ids), _p(mask), _p(to_tensor), _p(valid_word_num), _p(batch_idx),
                                _p(word_idx), B, S, head_num, size_per_head, _p(ws), ws.numel(), _stream(),
                                C.byref(host) if return_host_count else None)
    _lib.check(st, h)
    if return_host_count:
        return to_tensor, valid_word_num, batch_idx, word_idx, int(host.value)
    return to_tensor, valid_word_num, batch_idx, word_idx


class LayerWeights:
    """The 16 tensors of one layer on the device, keyed by the attribute names of the
    reference op (tf_op/bert_transformer_op.cc:44-77)."""

    ATTRS = ("attr_kernel_q", "attr_kernel_k", "attr_kernel_v", "attr_bias_q", "attr_bias_k", "attr_bias_v",
             "attr_output_kernel", "attr_output_bias", "attr_output_layernorm_beta", "attr_output_layernorm_gamma",
             "inter_kernel", "inter_bias", "output_kernel", "output_bias", "output_layernorm_beta",
             "output_layernorm_gamma")

    def __init__(self, device, dtype: torch.dtype, **tensors):
        missing = [a for a in self.ATTRS if a not in tensors]
        if missing:
            raise ValueError("missing weights: %s" % missing)
        self.t = {}
        for a in self.ATTRS:
            v = tensors[a]
            if isinstance(v, np.ndarray):
                v = torch.from_numpy(np.ascontiguousarray(v))
            self.t[a] = v.to(device=device, dtype=dtype).contiguous()
        s = _lib.LayerWeights()
        s.attr_kernel_Q = self.t["attr_kernel_q"].data_ptr()
        s.attr_kernel_K = self.t["attr_kernel_k"].data_ptr()
        s.attr_kernel_V = self.t["attr_kernel_v"].data_ptr()
        s.attr_bias_Q = self.t["attr_bias_q"].data_ptr()
        s.attr_bias_K = self.t["attr_bias_k"].data_ptr()
        s.attr_bias_V = self.t["attr_bias_v"].data_ptr()
        for name in ("attr_output_kernel", "attr_output_bias", "attr_output_layernorm_gamma",
                     "attr_output_layernorm_beta", "inter_kernel", "inter_bias", "output_kernel", "output_bias",
                     "output_layernorm_gamma", "output_layernorm_beta"):
            setattr(s, name, self.t[name].data_ptr())
        self.struct = s
        self.prepared: Optional[_lib.LayerPrepared] = None
        self.warm_block: Optional[torch.Tensor] = None
        self._prepared_tensors: List[torch.Tensor] = []

    def prepare(self, every_kernel: bool = True) -> "LayerWeights":
        """For weights that stay as they are: k-contiguous ([out,in]) copies of the dense kernels, made once, which the
        layer op then uses for its large-M GEMMs instead of transposing on every call (fp16 only; a no-op for fp32).
        every_kernel=False: only the kernels of the wide projections (Q, K, V, FFN up), the ones the layer op would
        transpose by itself."""
        if self.t["attr_kernel_q"].dtype != torch.float16:
            return self
        # the k-contiguous kernels take k in multiples of 64 and n in multiples of 8; other hidden sizes run the [k][n] kernels
        hq = self.t["attr_kernel_q"].shape[0]
        if hq % 64 != 0:
            return self
        lib = _lib.load()
        dev = self.t["attr_kernel_q"].device
        h = handle(dev)
        prep = _lib.LayerPrepared()
        names = [("attr_kernel_q", "attr_kernel_Q_t"), ("attr_kernel_k", "attr_kernel_K_t"),
                 ("attr_kernel_v", "attr_kernel_V_t"), ("inter_kernel", "inter_kernel_t")]
        if every_kernel:
            names += [("attr_output_kernel", "attr_output_kernel_t"), ("output_kernel", "output_kernel_t")]
        self._prepared_tensors = []
        with torch.cuda.device(dev):
            # the copies of Q, K, V and the attention output kernel lie one behind the other: one region for the layer in
            # front of this one to request (et_layer_prepared.warm)
            hq = self.t["attr_kernel_q"].shape[0]
            together = [nm for nm, _ in names if nm.startswith("attr_") and tuple(self.t[nm].shape) == (hq, hq)]
            block = torch.empty(len(together), hq, hq, dtype=torch.float16, device=dev)
            self.warm_block = block if len(together) >= 3 else None
            for src_name, field in names:
                src = self.t[src_name]
                k, n = src.shape
                dst = block[together.index(src_name)] if src_name in together else \
                    torch.empty(n, k, dtype=src.dtype, device=dev)
                _lib.check(lib.et_transpose_weight(h, _lib.ET_FP16, _p(src), _p(dst), k, n, _stream()), h)
                self._prepared_tensors.append(dst)
                setattr(prep, field, dst.data_ptr())
        self.prepared = prep
        return self

    @classmethod
    def from_slots(cls, device, dtype, slots: Sequence):
        """slots: the 16 arrays of one layer in the order of the reference's `weights_value`
        (python/effective_transformer/__init__.py:55-74):
        q_k,q_b,k_k,k_b,v_k,v_b,ao_k,ao_b,ao_ln_beta,ao_ln_gamma,i_k,i_b,o_k,o_b,o_ln_beta,o_ln_gamma."""
        if len(slots) != 16:
            raise ValueError("a layer has 16 weight tensors")
        return cls(device, dtype,
                   attr_kernel_q=slots[0], attr_bias_q=slots[1], attr_kernel_k=slots[2], attr_bias_k=slots[3],
                   attr_kernel_v=slots[4], attr_bias_v=slots[5], attr_output_kernel=slots[6],
                   attr_output_bias=slots[7], attr_output_layernorm_beta=slots[8],
                   attr_output_layernorm_gamma=slots[9], inter_kernel=slots[10], inter_bias=slots[11],
                   output_kernel=slots[12], output_bias=slots[13], output_layernorm_beta=slots[14],
                   output_layernorm_gamma=slots[15])


def effective_transformer(from_tensor: torch.Tensor, to_tensor: torch.Tensor, attr_mask: torch.Tensor,
                          valid_word_num: torch.Tensor, batch_idx: torch.Tensor, word_idx: torch.Tensor,
                          weights: LayerWeights, batch_size: int, from_seq_len: int, to_seq_len: int, head_num: int,
                          size_per_head: int, valid_word_num_hint: int = -1,
                          out: Optional[torch.Tensor] = None, seq_start: Optional[torch.Tensor] = None) -> torch.Tensor:
    """EffectiveTransformer layer op (tf_op/bert_transformer_op.cc:44-77, 180-221).  Output has
    the shape of from_tensor; rows beyond the valid-token count are left as allocated.
    seq_start: the table of `sequence_starts` for this batch (saves building it in every layer); weights that were
    `prepare()`d bring their transposed kernels along."""
    lib = _lib.load()
    _require_cuda(from_tensor, to_tensor, attr_mask, valid_word_num, batch_idx, word_idx)
    B = from_tensor.shape[0]
    dev = from_tensor.device
    if attr_mask.dtype != from_tensor.dtype:
        raise TypeError("attr_mask must have the dtype of from_tensor")
    if out is None:
        out = torch.empty_like(from_tensor)
    code = _dtype_code(from_tensor.dtype)
    nbytes = lib.et_layer_workspace_bytes(code, B, from_seq_len, head_num, size_per_head)
    ws = _workspace(dev, "layer", nbytes)
    h = handle(dev)
    if weights.prepared is None and seq_start is None:
        st = lib.et_layer(h, code, C.byref(weights.struct), _p(from_tensor), _p(to_tensor), _p(attr_mask),
                          _p(valid_word_num), _p(batch_idx), _p(word_idx), _p(out), B, from_seq_len, to_seq_len,
                          head_num, size_per_head, valid_word_num_hint, _p(ws), ws.numel(), _stream())
    else:
        # a copy per call: the weights object (and its prepared struct) may be shared by threads and streams, the
        # sequence start table belongs to this batch
        prep = _lib.LayerPrepared()
        if weights.prepared is not None:
            C.pointer(prep)[0] = weights.prepared
        prep.seq_start = seq_start.data_ptr() if seq_start is not None else None
        prep.seq_start_bytes = seq_start.numel() * seq_start.element_size() if seq_start is not None else 0
        st = lib.et_layer_with_prepared(h, code, C.byref(weights.struct), C.byref(prep), _p(from_tensor), _p(to_tensor),
                                        _p(attr_mask), _p(valid_word_num), _p(batch_idx), _p(word_idx), _p(out), B,
                                        from_seq_len, to_seq_len, head_num, size_per_head, valid_word_num_hint, _p(ws),
                                        ws.numel(), _stream())
    _lib.check(st, h)
    return out


def sequence_starts(valid_word_num: torch.Tensor, batch_idx: torch.Tensor, batch_size: int, seq_len: int,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The sequence table of a batch, int32[2 * batch_size + 1]: first packed row of every sequence (entry batch_size
    = valid-token count), then the sequence numbers in the order the attention kernel serves them (longest first); one
    per batch serves all layers."""
    lib = _lib.load()
    _require_cuda(valid_word_num, batch_idx)
    words = lib.et_seq_workspace_bytes(batch_size) // 4
    if out is None:
        out = torch.empty(words, dtype=torch.int32, device=batch_idx.device)
    elif out.dtype != torch.int32:
        raise TypeError("the sequence table is int32")
    h = handle(batch_idx.device)
    _lib.check(lib.et_sequence_starts(h, _p(batch_idx), _p(valid_word_num), batch_size, seq_len, _p(out),
                                      out.numel() * 4, _stream()), h)
    return out


def effective_transformer_output(from_tensor: torch.Tensor, valid_word_num: torch.Tensor, batch_idx: torch.Tensor,
                                 word_idx: torch.Tensor, batch_size: int, from_seq_len: int, to_seq_len: int,
                                 head_num: int, size_per_head: int) -> torch.Tensor:
    """EffectiveTransformerOutput (tf_op/bert_transformer_op.cc:359-431): [B,S,H] with zeros at
    padding."""
    lib = _lib.load()
    _require_cuda(from_tensor, valid_word_num, batch_idx, word_idx)
    B = from_tensor.shape[0]
    to_tensor = torch.empty_like(from_tensor)
    h = handle(from_tensor.device)
    st = lib.et_output(h, _dtype_code(from_tensor.dtype), _p(from_tensor), _p(valid_word_num), _p(batch_idx),
                       _p(word_idx), _p(to_tensor), B, from_seq_len, head_num, size_per_head, _stream())
    _lib.check(st, h)
    return to_tensor


def effective_transformer_first_token(from_tensor: torch.Tensor, valid_word_num: torch.Tensor, batch_idx: torch.Tensor,
                                      word_idx: torch.Tensor) -> torch.Tensor:
    """[B,H]: the row at position 0 of every sequence, read from the packed matrix (what the pooler takes from
    `sequence_output[:, 0]`, sample/tensorflow/modeling.py:224-232); zeros where position 0 holds no token."""
    lib = _lib.load()
    _require_cuda(from_tensor, valid_word_num, batch_idx, word_idx)
    B, S = batch_idx.shape
    H = from_tensor.shape[-1]
    out = torch.empty(B, H, dtype=from_tensor.dtype, device=from_tensor.device)
    h = handle(from_tensor.device)
    st = lib.et_first_token(h, _dtype_code(from_tensor.dtype), _p(from_tensor), _p(valid_word_num), _p(batch_idx),
                            _p(word_idx), _p(out), B, S, H, _stream())
    _lib.check(st, h)
    return out


# --------------------------------------------------------------------------- the glue

class EffectiveTransformerEncoder:
    """Input -> L x Layer -> Output with the weights resident on the device (the reference bakes
    them into op attributes at graph build, python/effective_transformer/__init__.py:48-76)."""

    def __init__(self, num_layers: int, head_num: int, size_per_head: int, weights_value: Sequence, dtype: torch.dtype,
                 device="cuda", prepare: bool = True):
        """prepare: the weights are constants of this object, so the k-contiguous copies the large-M GEMMs want are
        made here once (fp16) instead of in every layer call."""
        if len(weights_value) != 16 * num_layers:
            raise ValueError("expected %d weight tensors, got %d" % (16 * num_layers, len(weights_value)))
        self.device = torch.device(device)
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self.dtype = dtype
        self.head_num, self.size_per_head, self.num_layers = head_num, size_per_head, num_layers
        self.layers: List[LayerWeights] = [
            LayerWeights.from_slots(self.device, dtype, weights_value[16 * l:16 * l + 16]) for l in range(num_layers)]
        if prepare:
            for w in self.layers:
                w.prepare()
            # a layer's last kernel requests the next layer's attention weights, which would otherwise be read cold
            self._warm_refs = []         # the regions named below stay allocated as long as this encoder lives
            for w, nxt in zip(self.layers[:-1], self.layers[1:]):
                if w.prepared is not None and getattr(nxt, "warm_block", None) is not None:
                    w.prepared.warm = nxt.warm_block.data_ptr()
                    w.prepared.warm_bytes = nxt.warm_block.numel() * 2
                    self._warm_refs.append(nxt.warm_block)
        # ping-pong activations, sequence table and the pinned count, per (activation shape, stream, host thread): two
        # threads or streams that run this encoder at the same time each have their own
        self._bufs: Dict[tuple, list] = {}
        self._bufs_lock = threading.Lock()

    @classmethod
    def from_checkpoint(cls, path: str, head_num: int, size_per_head: int, dtype: torch.dtype, device="cuda",
                        num_layers: Optional[int] = None, prefix: Optional[str] = None):
        """Encoder from a local `.npz` / `.safetensors` file with TF-BERT or Hugging Face tensor names
        (see weights.py for the name map)."""
        from . import weights as _weights
        ws = _weights.load_weights(path, num_layers, prefix)
        return cls(len(ws) // 16, head_num, size_per_head, ws, dtype, device)

    def __call__(self, from_tensor: torch.Tensor, input_mask: torch.Tensor, attention_mask: torch.Tensor,
                 sync_count: bool = True, rows_bound: Optional[int] = None) -> torch.Tensor:
        """rows_bound (with sync_count=False): an upper bound of the valid-token count that the caller vouches for;
        the launches are sized for that many rows instead of B*S (rows beyond it would not be computed)."""
        B, S = input_mask.shape
        hn, d = self.head_num, self.size_per_head
        x, vwn, bidx, widx = effective_transformer_input(from_tensor, input_mask, B, S, S, hn, d)
        return self._layers_and_output(x, vwn, bidx, widx, sync_count, attention_mask, B, S, rows_bound)

    def forward_ids(self, input_ids, token_type_ids, input_mask, attention_mask, embeddings: "EmbeddingWeights",
                    sync_count: bool = True) -> torch.Tensor:
        """Embedding block + encoder from token ids: the packed token matrix is produced directly."""
        B, S = input_mask.shape
        hn, d = self.head_num, self.size_per_head
        r = effective_transformer_embedding_input(input_ids, token_type_ids, input_mask, embeddings, hn, d)
        x, vwn, bidx, widx = r[:4]
        return self._layers_and_output(x, vwn, bidx, widx, sync_count, attention_mask, B, S)

    def _layers_and_output(self, x, vwn, bidx, widx, sync_count, attention_mask, B, S, rows_bound=None):
        """sync_count: read the valid-token count back once per batch, so that the launches of layers 2 .. L are sized
        exactly (the reference reads it back in every layer).  The copy is asynchronous and the host waits for it
        behind the launches of the first layer, which is sized for B*S rows and bounded on the device: the GPU never
        idles for the read-back (waiting right after the input op left it without work for 0.13-0.19 ms per batch)."""
        hn, d = self.head_num, self.size_per_head
        key = (tuple(x.shape), torch.cuda.current_stream(x.device).cuda_stream, threading.get_ident(),
               getattr(_scope, "owner", None))
        with self._bufs_lock:
            bufs = self._bufs.get(key)
        if bufs is None:
            # (the pinned word for the count is made on first use: a pass under graph capture never reads the count back)
            bufs = [torch.empty_like(x), torch.empty_like(x),
                    torch.empty(_lib.load().et_seq_workspace_bytes(B) // 4, dtype=torch.int32, device=x.device), None]
            with self._bufs_lock:
                self._bufs[key] = bufs
        T, copied = -1, None
        if not sync_count and rows_bound is not None:
            if not 0 < rows_bound <= B * S:
                raise ValueError("rows_bound must be in 1 .. batch * seq_len")
            T = int(rows_bound)
        if sync_count and len(self.layers) > 1:
            if bufs[3] is None:
                bufs[3] = torch.empty(1, dtype=torch.int32, pin_memory=True)
            bufs[3].copy_(vwn, non_blocking=True)
            copied = torch.cuda.Event()
            copied.record()
        starts = sequence_starts(vwn, bidx, B, S, out=bufs[2])       # one table for all layers of the batch
        for l, w in enumerate(self.layers):
            out = bufs[l & 1]
            if l == 1 and copied is not None:
                copied.synchronize()
                T = int(bufs[3].item())
            effective_transformer(x, x, attention_mask, vwn, bidx, widx, w, B, S, S, hn, d, valid_word_num_hint=T,
                                  out=out, seq_start=starts)
            x = out
        return effective_transformer_output(x, vwn, bidx, widx, B, S, S, hn, d)

    def make_graph(self, from_tensor, input_mask, attention_mask,
                   max_valid_tokens: Optional[int] = None) -> "GraphedEncoder":
        """Captures the whole stack into one HIP graph (no host work between the launches).  max_valid_tokens: see
        GraphedEncoder."""
        return GraphedEncoder(self, from_tensor, input_mask, attention_mask, max_valid_tokens)


class GraphedEncoder:
    """One HIP graph holding Input -> L x Layer -> Output for fixed shapes.  The valid-token count stays on the
    device inside the graph (no host read-back), so every replay adapts to the mask it is given.

    A graph's launches are sized when it is captured, for B*S rows unless max_valid_tokens says that no mask replayed
    through this graph has more valid tokens than that (12 layers, batch 100 x 32 with 2000 valid tokens: 1.00 ms per
    replay sized for 3200 rows, 0.84 ms sized for 2000).  Rows beyond the bound are not computed, so a replay checks a
    new mask against it (one read-back of the mask's sum) unless check_mask=False."""

    def __init__(self, enc: EffectiveTransformerEncoder, from_tensor, input_mask, attention_mask,
                 max_valid_tokens: Optional[int] = None):
        self.enc = enc
        self.max_valid_tokens = max_valid_tokens
        if max_valid_tokens is not None and int(input_mask.sum().item()) > max_valid_tokens:
            raise ValueError("the mask holds more valid tokens than max_valid_tokens")
        self.x = from_tensor.clone()
        self.mask = input_mask.clone()
        self.attn = attention_mask.clone()
        # warm-up outside the capture (kernel attributes, allocator pools), on a side stream; its buffers are dropped
        # again.  The workspaces and the encoder's ping-pong buffers made under this owner during the capture come from
        # the graph's own memory pool, belong to this graph alone and are kept alive with it.
        _scope.owner = id(self)

        def drop_owned():
            with enc._bufs_lock:
                for key in [k for k in enc._bufs if k[3] == id(self)]:
                    del enc._bufs[key]
            with _lock:
                for key in [k for k in _workspaces if k[3] == id(self)]:
                    del _workspaces[key]

        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    enc(self.x, self.mask, self.attn, sync_count=False, rows_bound=max_valid_tokens)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            drop_owned()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.out = enc(self.x, self.mask, self.attn, sync_count=False, rows_bound=max_valid_tokens)
            with _lock:
                self._held = [ws for key, ws in _workspaces.items() if key[3] == id(self)]
            with enc._bufs_lock:
                self._held += [t for key, bufs in enc._bufs.items() if key[3] == id(self) for t in bufs if t is not None]
        finally:
            _scope.owner = None
            drop_owned()

    def __call__(self, from_tensor=None, input_mask=None, attention_mask=None, check_mask: bool = True) -> torch.Tensor:
        """Copies the given tensors into the graph's inputs (None = keep the previous ones), replays, and returns the
        graph's output tensor (overwritten by the next replay)."""
        if from_tensor is not None:
            self.x.copy_(from_tensor)
        if input_mask is not None:
            if self.max_valid_tokens is not None and check_mask and \
                    int(input_mask.sum().item()) > self.max_valid_tokens:
                raise ValueError("the mask holds more valid tokens than the graph's max_valid_tokens")
            self.mask.copy_(input_mask)
        if attention_mask is not None:
            self.attn.copy_(attention_mask)
        self.graph.replay()
        return self.out


def get_sequence_output(config, max_batch_size, max_seq_length, attention_mask, input_mask, from_tensor,
                        weights_value):
    """Same argument list as the reference's get_sequence_output
    (python/effective_transformer/__init__.py:32-35).  `config` needs num_attention_heads,
    hidden_size and num_hidden_layers."""
    head_num = config.num_attention_heads
    size_per_head = int(config.hidden_size / config.num_attention_heads)
    enc = EffectiveTransformerEncoder(config.num_hidden_layers, head_num, size_per_head, weights_value,
                                      from_tensor.dtype, from_tensor.device)
    return enc(from_tensor, input_mask, attention_mask)
