"""Shapes the tuned kernels are not built for -- head rows and token rows that are no whole number of 16-byte pieces,
GEMM dimensions the MFMA tiles cannot take -- run element-wise kernels with the same arithmetic.  The reference's op
accepts any size_per_head (tf_op/bert_transformer_op.cc:53-57); here every such entry point is checked against the
oracle: the three ops end to end, and the kernel-level entry points one by one."""
import numpy as np
import pytest
import torch

from oracle import et_oracle as o
from gpu_util import TDT, assert_half_close, dev, half_ulp, run_encoder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def k():
    from effective_transformer_amd import kernel_ops
    return kernel_ops


# (heads, size_per_head): hidden 15 (30-byte fp16 rows), 240 (k % 32 != 0, 40-byte head rows), 12 (k % 16 != 0), 1,
# and 66 (a 132-byte fp16 row: 4-byte pieces)
@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("heads,d", [(3, 5), (12, 20), (2, 6), (1, 1), (2, 33)])
def test_encoder_with_odd_head_sizes(dtype, heads, d):
    print("odd shapes", dtype, heads, d, flush=True)
    wl = o.Workload("odd", 100 + heads * 7 + d, dtype, 2, 7, 24, heads, d, 4 * heads * d, 3, 25)
    rng = np.random.RandomState(wl.seed)
    lens, mask, attr = o.make_masks(wl, rng)
    mask[2, 5] = 0                                                   # a hole
    attr = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (wl.B, wl.S, wl.S))).astype(attr.dtype)
    x = o.rnd(rng.randn(wl.B, wl.S, wl.H), dtype)
    weights = []
    for _ in range(wl.layers):
        lw = o.make_layer_weights(wl, rng, True)
        # kernels of a tiny hidden size drawn at 0.02 would leave the layer output to the LayerNorm's beta alone
        weights.extend([o.rnd(a.astype(np.float32) * (8.0 if a.ndim == 2 else 1.0), dtype) for a in lw])
    w = dict(wl=wl, lens=lens, mask=mask, attr_mask=attr, x=x, weights=weights)
    got = run_encoder(w)
    want = o.encoder(x, mask, attr, weights, heads, d, dtype)
    valid = mask.astype(bool)
    assert np.all(got[~valid] == 0)
    err = np.abs(got[valid].astype(np.float64) - want[valid].astype(np.float64)).max()
    print("  max abs diff", err, flush=True)
    assert err < (1e-4 if dtype == "fp32" else 2e-2), err
    # the device-side token count gives the same bits
    assert np.array_equal(run_encoder(w, hint=False), got)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("m,n,k_", [(37, 15, 23), (5, 1, 7), (130, 33, 100), (20, 24, 24)])
def test_gemm_any_dimensions(k, dtype, m, n, k_):
    print("generic gemm", dtype, m, n, k_, flush=True)
    rng = np.random.RandomState(m + n + k_)
    a = o.rnd(rng.randn(m, k_), dtype)
    b = o.rnd(0.3 * rng.randn(k_, n), dtype)
    bias = o.rnd(0.5 * rng.randn(n), dtype)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    got = k.gemm(dev(a), dev(b)).cpu().numpy()
    scale = np.abs(exact).max()
    if dtype == "fp32":
        assert np.abs(got - exact).max() <= 1e-5 * scale
    else:
        # one rounding to half of a float sum: half an ulp plus the float accumulation's error on sums that cancel
        assert np.all(np.abs(got.astype(np.float64) - exact) <= 0.51 * half_ulp(exact) + 1e-5 * scale)
    # + bias: one add in the element type on the rounded product; + bias + gelu: the stand-alone kernel's arithmetic
    gb = k.gemm(dev(a), dev(b), bias=dev(bias)).cpu().numpy()
    want_b = (got + bias) if dtype == "fp32" else o.hadd(got, bias)
    assert np.array_equal(gb, want_b.astype(got.dtype))
    gg = k.gemm(dev(a), dev(b), bias=dev(bias), gelu=True).cpu().numpy()
    two = k.add_bias_act(dev(got), dev(bias)).cpu().numpy()
    assert np.array_equal(gg, two)
    want_g = o.add_bias_act(got, bias, dtype)
    if dtype == "fp32":
        np.testing.assert_allclose(gg, want_g, rtol=1e-4, atol=1e-6)
    else:
        assert_half_close(gg, want_g, ulps=2.0, frac=None, what="gelu")
    # a row bound that lives on the device
    keep = torch.tensor([max(m - 3, 0)], dtype=torch.int32, device="cuda")
    out = torch.full((m, n), 7.0, dtype=TDT[dtype], device="cuda")
    k.gemm(dev(a), dev(b), m_dev=keep, out=out)
    kept = int(keep.item())
    assert np.array_equal(out.cpu().numpy()[:kept], got[:kept]) and np.all(out.cpu().numpy()[kept:] == 7.0)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("m,n", [(9, 15), (4, 1), (3, 4099), (17, 66)])
def test_row_kernels_with_odd_rows(k, dtype, m, n):
    print("generic rows", dtype, m, n, flush=True)
    rng = np.random.RandomState(m * 3 + n)
    out = o.rnd(rng.randn(m, n), dtype)
    inp = o.rnd(rng.randn(m, n), dtype)
    bias, gamma, beta = (o.rnd(v, dtype) for v in (0.3 * rng.randn(n), 1 + 0.2 * rng.randn(n), 0.2 * rng.randn(n)))
    if n > 1:          # a one-element row has variance 0: the result is beta whatever the input
        want = o.add_bias_input_layernorm(out, inp, bias, gamma, beta, dtype)
        got = k.add_bias_input_layernorm(dev(out), dev(inp), dev(bias), dev(gamma), dev(beta)).cpu().numpy()
        if dtype == "fp32":
            np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-5)
        else:
            assert_half_close(got, want, ulps=1.0, frac=0.02, what="layernorm")
    else:
        got = k.add_bias_input_layernorm(dev(out), dev(inp), dev(bias), dev(gamma), dev(beta)).cpu().numpy()
        assert np.array_equal(got, np.broadcast_to(beta, (m, n)))
    x = o.rnd(2.0 * rng.randn(m, n), dtype)
    want = o.add_bias_act(x, bias, dtype)
    got = k.add_bias_act(dev(x), dev(bias)).cpu().numpy()
    if dtype == "fp32":
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-6)
    else:
        assert_half_close(got, want, ulps=2.0, frac=None, what="gelu")


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("heads,d,S", [(3, 5, 13), (2, 33, 40), (1, 1, 7), (4, 12, 70)])
def test_attention_side_with_odd_head_sizes(k, dtype, heads, d, S):
    """qkv bias + padding, un-padding and the fused attention (both layouts) on head rows that are no whole number of
    16-byte pieces, with holes and an unrelated mask."""
    print("generic attention", dtype, heads, d, S, flush=True)
    from test_gpu_kernels import _attn_problem, _idx_dev
    p = _attn_problem(31 + d, 5, S, heads, dtype, holes=True, weird_mask=True, d=d)
    B, T, H = p["B"], p["T"], heads * d
    bi, wi, vwn = _idx_dev(p)
    want_pad = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], T, B, S, heads, d, p["bi"],
                                      p["wi"], dtype)
    got_pad = k.add_qkv_bias_padding(dev(p["q"]), dev(p["bq"]), dev(p["k"]), dev(p["bk"]), dev(p["v"]), dev(p["bv"]),
                                     vwn, B, S, heads, d, bi, wi)
    for g, w_ in zip(got_pad, want_pad):
        assert np.array_equal(g.cpu().numpy(), w_)
    un = k.transpose_rm_padding(got_pad[0], vwn, bi, wi).cpu().numpy()
    assert np.array_equal(un[:T], o.transpose_rm_padding(want_pad[0], T, p["bi"], p["wi"]))
    want = o.attention(want_pad[0], want_pad[1], want_pad[2], p["attr"], T, p["bi"], p["wi"], dtype)
    got0 = k.attention(got_pad[0], got_pad[1], got_pad[2], 0, 0, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    add = (lambda a, b: (a.astype(np.float32) + b.astype(np.float32)).astype(np.float32)) if dtype == "fp32" else o.hadd
    packed = np.zeros((B * S, 3 * H), o._np_dtype(dtype))
    packed[:T, :H] = add(p["q"], p["bq"]); packed[:T, H:2 * H] = add(p["k"], p["bk"]); packed[:T, 2 * H:] = add(p["v"], p["bv"])
    pk = dev(packed)
    got1 = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    assert np.array_equal(got0, got1)
    if dtype == "fp32":
        np.testing.assert_allclose(got0[:T], want, rtol=1e-4, atol=2e-5)
    else:
        np.testing.assert_allclose(got0[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("H", [15, 1, 66, 7])
def test_input_and_output_ops_with_odd_rows(dtype, H):
    from effective_transformer_amd import ops
    print("generic movers", dtype, H, flush=True)
    rng = np.random.RandomState(H)
    B, S = 9, 21
    mask = (rng.random_sample((B, S)) < 0.6).astype(np.int32)
    mask[3] = 0
    x = o.rnd(rng.randn(B, S, H), dtype)
    to, vwn, bidx, widx, T = ops.effective_transformer_input(dev(x, TDT[dtype]), dev(mask), B, S, S, 1, H,
                                                             return_host_count=True)
    wto, wT, wb, ww, _ = o.input_op_fast(x, mask)
    assert T == wT
    assert np.array_equal(bidx.cpu().numpy().reshape(-1)[:T], wb) and np.array_equal(widx.cpu().numpy().reshape(-1)[:T], ww)
    assert np.array_equal(to.cpu().numpy().reshape(B * S, H)[:T].view(np.uint8), wto.view(np.uint8))
    back = ops.effective_transformer_output(to, vwn, bidx, widx, B, S, S, 1, H).cpu().numpy()
    want = np.where(mask[:, :, None].astype(bool), x, 0).astype(x.dtype)
    assert np.array_equal(back.view(np.uint8), want.view(np.uint8))
    # the first-token gather moves rows in the same pieces
    first = ops.effective_transformer_first_token(to, vwn, bidx, widx).cpu().numpy()
    assert np.array_equal(first.view(np.uint8), want[:, 0, :].view(np.uint8))
