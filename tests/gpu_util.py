"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import et_oracle as o

TDT = {"fp32": torch.float32, "fp16": torch.float16}


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def half_ulp(x):
    """Spacing of binary16 at |x| (as float64 array)."""
    ax = np.maximum(np.abs(np.asarray(x, dtype=np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(ax)) - 10)


def assert_half_close(got, want, ulps=1.0, frac=0.02, what="", atol=0.0):
    """got/want float16 arrays: every element within `ulps` half-ulps of want, and at most
    `frac` of the elements different at all."""
    g = np.asarray(got, dtype=np.float64)
    w = np.asarray(want, dtype=np.float64)
    assert g.shape == w.shape
    err = np.abs(g - w)
    lim = ulps * half_ulp(w) * 1.001 + atol
    bad = err > lim
    assert not bad.any(), "%s: %d elements beyond %.1f ulp, worst %g vs %g" % (
        what, bad.sum(), ulps, g[bad][0], w[bad][0])
    if frac is not None:
        assert (err > 0).mean() <= frac, "%s: %.4f of elements differ" % (what, (err > 0).mean())


def run_encoder(w, layers=None, hint=True, dtype=None, prepare=True, every_kernel=True):
    """Runs Input -> L x Layer -> Output on the GPU for an oracle workload dict.  Returns the output [B,S,H] as numpy.
    prepare=False: plain et_layer calls; every_kernel=False: only the wide projections' kernels pre-transposed."""
    from effective_transformer_amd import ops
    wl = w["wl"]
    dt = TDT[dtype or wl.dtype]
    weights = w["weights"] if layers is None else w["weights"][:16 * layers]
    L = len(weights) // 16
    enc = ops.EffectiveTransformerEncoder(L, wl.heads, wl.d, weights, dt, "cuda", prepare=prepare)
    if prepare and not every_kernel:
        for lw in enc.layers:
            lw.prepare(every_kernel=False)
    x = dev(w["x"], dt)
    mask = dev(w["mask"].astype(np.int32))
    attr = dev(w["attr_mask"], dt)
    out = enc(x, mask, attr, sync_count=hint)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def subset_workload(w, idx):
    """The same workload restricted to the sequences `idx` (weights shared)."""
    idx = np.asarray(idx)
    return dict(wl=o.Workload(**{**w["wl"].__dict__, "B": len(idx)}), lens=w["lens"][idx], mask=w["mask"][idx],
                attr_mask=w["attr_mask"][idx], x=w["x"][idx], weights=w["weights"])
