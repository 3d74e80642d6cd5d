"""et_input_static, the entry point that allocates nothing (its scan scratch is a static array in the library's device
image), against et_input through the C ABI: two calls in a row, the second on a smaller batch, both large enough for
the scan to go through the scratch (more than 128 tiles of 1024 positions); bit-exact."""
import ctypes as C

import numpy as np
import pytest
import torch

from effective_transformer_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _both(lib, h, dt, x, mask, heads, d):
    B, S = mask.shape
    res = []
    for static in (False, True):
        to = torch.full_like(x, -7.0)
        vwn = torch.full((1,), -1, dtype=torch.int32, device="cuda")
        bidx = torch.full_like(mask, -1)
        widx = torch.full_like(mask, -1)
        code = _lib.ET_FP16 if dt == torch.float16 else _lib.ET_FP32
        if static:
            st = lib.et_input_static(h, code, x.data_ptr(), mask.data_ptr(), to.data_ptr(), vwn.data_ptr(),
                                     bidx.data_ptr(), widx.data_ptr(), B, S, heads, d, None)
        else:
            nbytes = lib.et_input_workspace_bytes(B, S)
            ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            st = lib.et_input(h, code, x.data_ptr(), mask.data_ptr(), to.data_ptr(), vwn.data_ptr(), bidx.data_ptr(),
                              widx.data_ptr(), B, S, heads, d, ws.data_ptr(), nbytes, None, None)
        _lib.check(st, h)
        torch.cuda.synchronize()
        res.append((to, vwn, bidx, widx))
    return res


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
def test_static_scratch_input_equals_et_input_twice(dt):
    lib = _lib.load()
    h = ops.handle(torch.device("cuda", 0))
    heads, d, S = 1, 64, 64
    rng = np.random.RandomState(11)
    for B in (2400, 2100):                     # 150 and 132 scan tiles: both calls read tile totals from the scratch
        print("et_input_static", dt, "B", B, flush=True)
        lens = rng.randint(0, S + 1, size=B)
        mask_np = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
        mask_np[rng.randint(0, B, 50), rng.randint(0, S, 50)] ^= 1          # holes
        mask = torch.from_numpy(mask_np).cuda()
        x = torch.from_numpy(rng.randn(B, S, heads * d).astype(np.float32)).cuda().to(dt)
        (to0, n0, b0, w0), (to1, n1, b1, w1) = _both(lib, h, dt, x, mask, heads, d)
        T = int(mask_np.sum())
        assert int(n0.item()) == T and int(n1.item()) == T
        assert torch.equal(b0.ravel()[:T], b1.ravel()[:T]) and torch.equal(w0.ravel()[:T], w1.ravel()[:T])
        assert torch.equal(to0.reshape(B * S, -1)[:T], to1.reshape(B * S, -1)[:T])
        # and against the closed form
        pos = np.flatnonzero(mask_np.ravel())
        assert np.array_equal(b1.ravel()[:T].cpu().numpy(), pos // S)
        assert np.array_equal(w1.ravel()[:T].cpu().numpy(), pos % S)
        assert torch.equal(to1.reshape(B * S, -1)[:T], x.reshape(B * S, -1)[torch.from_numpy(pos).cuda()])


def test_static_scratch_input_rejects_sizes_beyond_its_scratch():
    lib = _lib.load()
    h = ops.handle(torch.device("cuda", 0))
    t = torch.zeros(64, dtype=torch.int32, device="cuda")
    p = t.data_ptr()
    st = lib.et_input_static(h, _lib.ET_FP16, p, p, p, p, p, p, 16385, 64, 1, 64, None)
    assert st == 3 and b"1048576" in lib.et_last_error(h)
    st = lib.et_input_static(h, _lib.ET_FP16, p, p, p, p, p, None, 4, 4, 1, 64, None)
    assert st == 1


def _static_call(lib, h, x, mask, stream):
    """One et_input_static call on `stream` (a torch stream or None) into fresh outputs; returns (status, outputs)."""
    B, S = mask.shape
    to = torch.full_like(x, -7.0)
    vwn = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    bidx = torch.full_like(mask, -1)
    widx = torch.full_like(mask, -1)
    if stream is not None:
        stream.wait_stream(torch.cuda.current_stream())      # the fills above run on torch's current stream
    st = lib.et_input_static(h, _lib.ET_FP16, x.data_ptr(), mask.data_ptr(), to.data_ptr(), vwn.data_ptr(),
                             bidx.data_ptr(), widx.data_ptr(), B, S, 1, x.shape[-1],
                             None if stream is None else C.c_void_p(stream.cuda_stream))
    return st, (to, vwn, bidx, widx)


def _big_batch(seed, B=2300, S=64, H=64):
    rng = np.random.RandomState(seed)
    lens = rng.randint(0, S + 1, size=B)
    mask_np = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
    x = torch.from_numpy(rng.randn(B, S, H).astype(np.float32)).cuda().half()
    return x, torch.from_numpy(mask_np).cuda(), mask_np


def test_static_scratch_slots_belong_to_handles():
    """Every handle owns a slot of the static scratch, so two handles on two streams may overlap; a ninth live handle
    on the GPU has no slot; the calls of one handle are refused on a second stream while the first still has work."""
    lib = _lib.load()
    ops.handle(torch.device("cuda", 0))                  # the package's own handle holds one slot
    handles = []
    try:
        for _ in range(8):
            h = C.c_void_p()
            _lib.check(lib.et_create(C.byref(h), 0), None)
            handles.append(h)
        x, mask, mask_np = _big_batch(21)
        x2, mask2, mask2_np = _big_batch(22, B=2200)
        torch.cuda.synchronize()
        # the ninth live handle of the GPU got no slot
        st, _ = _static_call(lib, handles[7], x, mask, None)
        assert st == 3 and b"slot" in lib.et_last_error(handles[7])
        # two handles, two streams, queued back to back: each scans through its own slot (144 / 138 tile totals)
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        for _ in range(3):
            st1, r1 = _static_call(lib, handles[0], x, mask, s1)
            st2, r2 = _static_call(lib, handles[1], x2, mask2, s2)
            assert st1 == 0 and st2 == 0
        torch.cuda.synchronize()
        for (to, vwn, bidx, widx), m_np, xin in ((r1, mask_np, x), (r2, mask2_np, x2)):
            pos = np.flatnonzero(m_np.ravel())
            T = len(pos)
            S = m_np.shape[1]
            assert int(vwn.item()) == T
            assert np.array_equal(bidx.ravel()[:T].cpu().numpy(), pos // S)
            assert np.array_equal(widx.ravel()[:T].cpu().numpy(), pos % S)
            assert torch.equal(to.reshape(-1, to.shape[-1])[:T], xin.reshape(-1, to.shape[-1])[torch.from_numpy(pos).cuda()])
        # one handle, second stream while the first is still busy (a 50 ms sleep queued behind the call): refused
        st, _ = _static_call(lib, handles[0], x, mask, s1)
        assert st == 0
        with torch.cuda.stream(s1):
            torch.cuda._sleep(int(50e-3 * 2.0e9))
        st, _ = _static_call(lib, handles[0], x, mask, s2)
        assert st == 1 and b"in flight" in lib.et_last_error(handles[0])
        s1.synchronize()
        st, _ = _static_call(lib, handles[0], x, mask, s2)      # the first stream is idle now: accepted
        assert st == 0
        torch.cuda.synchronize()
        # a destroyed handle gives its slot back
        _lib.check(lib.et_destroy(handles.pop(0)), None)
        h = C.c_void_p()
        _lib.check(lib.et_create(C.byref(h), 0), None)
        handles.append(h)
        st, _ = _static_call(lib, h, x, mask, None)
        assert st == 0
        torch.cuda.synchronize()
    finally:
        for h in handles:
            lib.et_destroy(h)


def test_static_scratch_input_under_graph_capture():
    """What the entry point is for: a caller under HIP graph capture.  Captured once on a handle of its own, replayed
    with several masks (eager work and synchronisations between the replays), every replay against et_input."""
    lib = _lib.load()
    h = C.c_void_p()
    _lib.check(lib.et_create(C.byref(h), 0), None)
    try:
        B, S, H = 2200, 64, 64
        x, mask, _ = _big_batch(31, B=B)
        to = torch.full_like(x, -7.0)
        vwn = torch.full((1,), -1, dtype=torch.int32, device="cuda")
        bidx = torch.full_like(mask, -1)
        widx = torch.full_like(mask, -1)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            st = lib.et_input_static(h, _lib.ET_FP16, x.data_ptr(), mask.data_ptr(), to.data_ptr(), vwn.data_ptr(),
                                     bidx.data_ptr(), widx.data_ptr(), B, S, 1, H,
                                     C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0, lib.et_last_error(h)
        hh = ops.handle(torch.device("cuda", 0))
        for seed in (41, 42, 43):
            x2, mask2, mask2_np = _big_batch(seed, B=B)
            x.copy_(x2)
            mask.copy_(mask2)
            g.replay()
            torch.cuda.synchronize()
            # the same batch through et_input (eager work between the replays)
            to_ref, n_ref, b_ref, w_ref = ops.effective_transformer_input(x2, mask2, B, S, S, 1, H)
            torch.cuda.synchronize()
            T = int(mask2_np.sum())
            assert int(vwn.item()) == T == int(n_ref.item())
            assert torch.equal(bidx.ravel()[:T], b_ref.ravel()[:T]) and torch.equal(widx.ravel()[:T], w_ref.ravel()[:T])
            assert torch.equal(to.reshape(B * S, -1)[:T], to_ref.reshape(B * S, -1)[:T])
        del g, hh
    finally:
        lib.et_destroy(h)
