"""One handle entered by two host threads at once (the reference's layer op may be entered concurrently and serialises
on cublas_mutex_, tf_op/bert_transformer_op.cc:213,228): every thread on its own stream, workspace and buffers, through
the C ABI.  The results must be the bits of the sequential run, a failing call in one thread must not touch the other's
status, and every thread must read its own error message."""
import ctypes as C
import threading

import numpy as np
import pytest
import torch

from oracle import et_oracle as o
from gpu_util import TDT, dev

pytestmark = pytest.mark.gpu

ROUNDS = 20


class _Job:
    """Everything one thread needs for et_layer calls on its own stream: inputs, workspace, output."""

    def __init__(self, lib, h, name, seed, nseq=None):
        from effective_transformer_amd import _lib, ops
        w = o.make_workload(name, layers=1, random_affine=True)
        wl = w["wl"]
        self.wl, self.lib, self.h = wl, lib, h
        dt = TDT[wl.dtype]
        self.code = _lib.ET_FP16 if wl.dtype == "fp16" else _lib.ET_FP32
        rng = np.random.RandomState(seed)
        x = o.rnd(rng.randn(*w["x"].shape), wl.dtype)
        self.x, self.vwn, self.bidx, self.widx, self.T = ops.effective_transformer_input(
            dev(x, dt), dev(w["mask"].astype(np.int32)), wl.B, wl.S, wl.S, wl.heads, wl.d, return_host_count=True)
        self.attr = dev(w["attr_mask"], dt)
        self.weights = ops.LayerWeights.from_slots(self.x.device, dt, w["weights"][:16])
        self.ws_bytes = lib.et_layer_workspace_bytes(self.code, wl.B, wl.S, wl.heads, wl.d)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device="cuda")
        self.out = torch.zeros_like(self.x)
        self.stream = torch.cuda.Stream()
        torch.cuda.synchronize()

    def layer(self, ws_bytes=None, heads=None):
        wl = self.wl
        P = lambda t: C.c_void_p(t.data_ptr())
        return self.lib.et_layer(self.h, self.code, C.byref(self.weights.struct), P(self.x), P(self.x), P(self.attr),
                                 P(self.vwn), P(self.bidx), P(self.widx), P(self.out), wl.B, wl.S, wl.S,
                                 wl.heads if heads is None else heads, wl.d, self.T, P(self.ws),
                                 self.ws_bytes if ws_bytes is None else ws_bytes, C.c_void_p(self.stream.cuda_stream))

    def result(self):
        self.stream.synchronize()
        return self.out.reshape(self.wl.B * self.wl.S, -1)[:self.T].clone()


def test_two_threads_on_one_handle_give_the_sequential_bits():
    from effective_transformer_amd import _lib, ops
    lib = _lib.load()
    h = ops.handle(torch.device("cuda", 0))
    # thread 0: fp16 on the small-tile GEMMs and the short attention kernel; thread 1: fp32
    jobs = [_Job(lib, h, "cfg2", 5), _Job(lib, h, "cfg1", 6)]
    want = []
    for j in jobs:                                   # sequential reference runs
        assert j.layer() == 0, lib.et_last_error(h)
        want.append(j.result())
        j.out.zero_()
    # what each thread breaks on purpose, and what its message must name
    bad = [dict(ws_bytes=256), dict(heads=0)]
    expect = [(2, b"et_layer_workspace_bytes"), (1, b"head_num")]
    start = threading.Barrier(2)
    log = [[], []]

    def work(i):
        j = jobs[i]
        start.wait()
        for r in range(ROUNDS):
            st = j.layer()
            log[i].append(("ok", st))
            if r % 4 == 1:
                st = j.layer(**bad[i])
                msg = lib.et_last_error(h)           # this thread's own last failure, whatever the other thread did
                log[i].append(("bad", st, msg))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive()
    for i, j in enumerate(jobs):
        oks = [e for e in log[i] if e[0] == "ok"]
        bads = [e for e in log[i] if e[0] == "bad"]
        assert len(oks) == ROUNDS and all(e[1] == 0 for e in oks), oks
        assert len(bads) == ROUNDS // 4
        for _, st, msg in bads:
            assert st == expect[i][0] and expect[i][1] in msg, (i, st, msg)
        assert torch.equal(j.result(), want[i]), "thread %d: result differs from the sequential run" % i
    # a thread that never failed on the handle reads the handle's last message, from whichever thread it came
    seen = []
    t = threading.Thread(target=lambda: seen.append(lib.et_last_error(h)))
    t.start()
    t.join()
    assert any(e[1] in seen[0] for e in expect), seen


def test_two_threads_on_one_encoder_object():
    """The Python mirror from two threads, each on its own stream: buffers are per (stream, thread), so both passes give
    the bits of a pass on its own."""
    from effective_transformer_amd import ops
    w = o.make_workload("cfg2", layers=3, random_affine=True)
    wl = w["wl"]
    dt = TDT[wl.dtype]
    enc = ops.EffectiveTransformerEncoder(3, wl.heads, wl.d, w["weights"][:48], dt, "cuda")
    mask = dev(w["mask"].astype(np.int32))
    attr = dev(w["attr_mask"], dt)
    rng = np.random.RandomState(3)
    xs = [dev(o.rnd(rng.randn(*w["x"].shape), wl.dtype), dt) for _ in range(2)]
    want = [enc(x, mask, attr).clone() for x in xs]
    torch.cuda.synchronize()
    got = [None, None]
    start = threading.Barrier(2)

    def work(i):
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            start.wait()
            for _ in range(10):
                out = enc(xs[i], mask, attr)
            s.synchronize()
            got[i] = out.clone()

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive()
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(got[i], want[i]), i
