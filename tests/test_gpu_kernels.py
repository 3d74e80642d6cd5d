"""Parity of every kernel-level entry point of the C ABI against the CPU oracle, on a real
MI355X.  Integer/byte work is bit-exact; floating point carries the tolerance written at each
assertion."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import et_oracle as o
from gpu_util import TDT, assert_half_close, dev, half_ulp

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def k():
    from effective_transformer_amd import kernel_ops
    return kernel_ops


@pytest.fixture(scope="module")
def ops():
    from effective_transformer_amd import ops
    return ops


# ---------------------------------------------------------------------------- scan ---

@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 2048 + 17, 64000, (1 << 20) + 3,
                               1100 * 1024 + 5])
def test_exclusive_scan(k, n):
    print("scan n=%d" % n, flush=True)
    rng = np.random.RandomState(n % 1000)
    for kind in ("mask", "ints"):
        a = (rng.random_sample(n) < 0.63).astype(np.int32) if kind == "mask" else rng.randint(0, 50, n).astype(np.int32)
        got = k.exclusive_scan(dev(a)).cpu().numpy()
        assert np.array_equal(got, o.exclusive_scan(a)), kind


def _input_case(ops, x, mask, dtype):
    B, S, H = x.shape
    heads = H // 64 if H % 64 == 0 else 1
    d = H // heads
    to, vwn, bidx, widx, T = ops.effective_transformer_input(dev(x, TDT[dtype]), dev(mask), B, S, S, heads, d,
                                                             return_host_count=True)
    wto, wT, wb, ww, _ = o.input_op_fast(o.rnd(x, dtype), mask)
    assert T == wT == int(vwn.item())
    assert np.array_equal(bidx.cpu().numpy().reshape(-1)[:T], wb)
    assert np.array_equal(widx.cpu().numpy().reshape(-1)[:T], ww)
    got = to.cpu().numpy().reshape(B * S, H)[:T]
    assert np.array_equal(got.view(np.uint8), wto.view(np.uint8))
    return to, vwn, bidx, widx, T


def test_input_known_answers(ops):
    ka = json.load(open(os.path.join(GOLD, "known_answers.json")))
    fig = np.array(ka["figure_4x8"]["mask"], dtype=np.int32)
    x = np.random.RandomState(0).randn(4, 8, 64).astype(np.float32)
    to, vwn, bidx, widx, T = _input_case(ops, x, fig, "fp32")
    assert T == ka["figure_4x8"]["valid_word_num"]
    padded = (bidx.cpu().numpy().reshape(-1)[:T].astype(np.int64) * 8 + widx.cpu().numpy().reshape(-1)[:T])
    assert padded[:8].tolist() == ka["figure_4x8"]["packed_to_padded_first8"]
    rd = np.array(ka["readme_3x5"]["mask"], dtype=np.int32)
    tok = np.zeros((3, 5, 8), np.float16)
    tok[..., 0] = np.array(ka["readme_3x5"]["tokens_padded"])
    to, vwn, bidx, widx, T = _input_case(ops, tok, rd, "fp16")
    assert T == 7 and to.cpu().numpy().reshape(15, 8)[:7, 0].tolist() == ka["readme_3x5"]["tokens_packed"]


@pytest.mark.parametrize("case", ["holes", "ones", "zeros", "last0", "last1", "single"])
@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_input_edge_masks(ops, k, case, dtype):
    print("input edge", case, dtype, flush=True)
    rng = np.random.RandomState(len(case))
    B, S, H = 37, 29, 128
    mask = (rng.random_sample((B, S)) < 0.55).astype(np.int32)
    if case == "ones":
        mask[:] = 1
    elif case == "zeros":
        mask[:] = 0
    elif case == "last0":
        mask[-1, -1] = 0
    elif case == "last1":
        mask[-1, -1] = 1
    elif case == "single":
        B, S = 1, 1
        mask = np.ones((1, 1), np.int32)
    x = rng.randn(B, S, H).astype(np.float32)
    to, vwn, bidx, widx, T = _input_case(ops, x, mask, dtype)
    # Output op: zero at padding, original rows elsewhere (round trip)
    back = ops.effective_transformer_output(to, vwn, bidx, widx, B, S, S, 2, H // 2).cpu().numpy()
    want = o.rnd(x, dtype) * mask[..., None].astype(o._np_dtype(dtype))
    assert np.array_equal(back, want)


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
def test_input_output_on_workload_masks(ops, name):
    print("input workload", name, flush=True)
    w = o.make_workload(name, with_inputs=False)
    wl = w["wl"]
    rng = np.random.RandomState(7)
    x = rng.randn(wl.B, wl.S, wl.H).astype(np.float32)
    to, vwn, bidx, widx, T = _input_case(ops, x, w["mask"], wl.dtype)
    dig = json.load(open(os.path.join(GOLD, "workload_digests.json")))
    assert T == dig[name]["T"]
    back = ops.effective_transformer_output(to, vwn, bidx, widx, wl.B, wl.S, wl.S, wl.heads, wl.d).cpu().numpy()
    want = o.rnd(x, wl.dtype) * w["mask"][..., None].astype(o._np_dtype(wl.dtype))
    assert np.array_equal(back, want)
    # checksum of the packed rows equals the checksum of the valid rows
    assert np.array_equal(back.astype(np.float64).sum(axis=(0, 1)), want.astype(np.float64).sum(axis=(0, 1)))


def test_compress_and_restore_entry_points(k):
    rng = np.random.RandomState(3)
    B, S, H = 9, 17, 96
    mask = (rng.random_sample((B, S)) < 0.5).astype(np.int32)
    x = rng.randn(B, S, H).astype(np.float16)
    wto, T, wb, ww, prefix = o.input_op(x, mask)
    to, bidx, widx = k.compress(dev(x), dev(mask), dev(prefix))
    assert np.array_equal(to.cpu().numpy().reshape(B * S, H)[:T], wto)
    assert np.array_equal(bidx.cpu().numpy().reshape(-1)[:T], wb)
    assert np.array_equal(widx.cpu().numpy().reshape(-1)[:T], ww)
    vwn = torch.tensor([T], dtype=torch.int32, device="cuda")
    back = k.restore(to.reshape(B * S, H), bidx, widx, vwn, B, S).cpu().numpy()
    assert np.array_equal(back, o.restore(wto, T, wb, ww, B, S))


# -------------------------------------------------------------------- row kernels ---

@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("m,n", [(1, 64), (5, 3072), (134, 3072), (33, 4096), (7, 200)])
def test_add_bias_act(k, dtype, m, n):
    print("gelu", dtype, m, n, flush=True)
    rng = np.random.RandomState(m + n)
    x = o.rnd(2.5 * rng.randn(m, n), dtype)
    b = o.rnd(rng.randn(n), dtype)
    want = o.add_bias_act(x, b, dtype)
    got = k.add_bias_act(dev(x), dev(b)).cpu().numpy()
    if dtype == "fp32":
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    else:
        # the CDF is rounded to half before the last multiply: a CDF one half-ulp off (exp2/rcp vs exact
        # tanh) moves the product by up to 2 ulps, or by |x| * 2^-24 where the CDF is a half denormal
        assert_half_close(got, want, ulps=2.0, frac=0.01, what="gelu", atol=1e-6)
    # rows bounded on the device: rows >= *m_dev stay untouched
    if m > 3:
        keep = torch.tensor([m - 2], dtype=torch.int32, device="cuda")
        got2 = k.add_bias_act(dev(x), dev(b), m_dev=keep).cpu().numpy()
        assert np.array_equal(got2[:m - 2], got[:m - 2]) and np.array_equal(got2[m - 2:], x[m - 2:])


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("m,n", [(1, 768), (134, 768), (50, 1024), (9, 64), (6, 200), (3, 2048)])
def test_add_bias_input_layernorm(k, dtype, m, n):
    print("layernorm", dtype, m, n, flush=True)
    rng = np.random.RandomState(m * 7 + n)
    out = o.rnd(rng.randn(m, n), dtype)
    inp = o.rnd(rng.randn(m, n), dtype)
    bias, gamma, beta = (o.rnd(v, dtype) for v in (0.3 * rng.randn(n), 1 + 0.2 * rng.randn(n), 0.2 * rng.randn(n)))
    want = o.add_bias_input_layernorm(out, inp, bias, gamma, beta, dtype)
    got = k.add_bias_input_layernorm(dev(out), dev(inp), dev(bias), dev(gamma), dev(beta)).cpu().numpy()
    if dtype == "fp32":
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)    # fp32 bar: 1e-4 relative
    else:
        assert_half_close(got, want, ulps=1.0, frac=0.01, what="layernorm")
    if m > 3:
        keep = torch.tensor([2], dtype=torch.int32, device="cuda")
        got2 = k.add_bias_input_layernorm(dev(out), dev(inp), dev(bias), dev(gamma), dev(beta), m_dev=keep).cpu().numpy()
        assert np.array_equal(got2[:2], got[:2]) and np.array_equal(got2[2:], out[2:])


# ---------------------------------------------------------------- attention side ---

def _attn_problem(seed, B, S, heads, dtype, holes=False, weird_mask=False, d=64):
    rng = np.random.RandomState(seed)
    if holes:
        mask = (rng.random_sample((B, S)) < 0.6).astype(np.int32)
        mask[0] = 0                                  # an empty sequence
        mask[1] = 1
    else:
        lens = rng.randint(1, S + 1, size=B)
        mask = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
    _, T, bi, wi, _ = o.input_op_fast(np.zeros((B, S, 1), np.float32), mask)
    H = heads * d
    q, kk, v = (o.rnd(rng.randn(T, H), dtype) for _ in range(3))
    bq, bk, bv = (o.rnd(0.5 * rng.randn(H), dtype) for _ in range(3))
    if weird_mask:
        attr = (rng.random_sample((B, S, S)) < 0.7).astype(np.float32)
        attr[:, 0, :] = 0                            # fully masked query rows
    else:
        attr = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (B, S, S))).astype(np.float32)
    return dict(B=B, S=S, heads=heads, d=d, mask=mask, T=T, bi=bi, wi=wi, q=q, k=kk, v=v, bq=bq, bk=bk, bv=bv,
                attr=o.rnd(attr, dtype))


def _idx_dev(p):
    n = p["B"] * p["S"]
    bi = np.full(n, -1, np.int32); bi[:p["T"]] = p["bi"]
    wi = np.full(n, -1, np.int32); wi[:p["T"]] = p["wi"]
    return dev(bi), dev(wi), torch.tensor([p["T"]], dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("holes", [False, True])
def test_qkv_bias_padding_and_unpad(k, dtype, holes):
    p = _attn_problem(11, 6, 13, 3, dtype, holes=holes)
    bi, wi, vwn = _idx_dev(p)
    want = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], p["T"], p["B"], p["S"],
                                  p["heads"], p["d"], p["bi"], p["wi"], dtype)
    got = k.add_qkv_bias_padding(dev(p["q"]), dev(p["bq"]), dev(p["k"]), dev(p["bk"]), dev(p["v"]), dev(p["bv"]), vwn,
                                 p["B"], p["S"], p["heads"], p["d"], bi, wi)
    for g, w_ in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w_)          # one correctly rounded add per element: bit-exact
    un = k.transpose_rm_padding(got[0], vwn, bi, wi).cpu().numpy()
    assert np.array_equal(un[:p["T"]], o.transpose_rm_padding(want[0], p["T"], p["bi"], p["wi"]))
    assert np.all(un[p["T"]:] == 0)                          # rows beyond T untouched


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("S", [1, 7, 32, 64, 100, 128, 300, 513, 600, 1024])
def test_softmax(k, dtype, S):
    rng = np.random.RandomState(S)
    B, heads = 3, 2
    qk = o.rnd(6 * rng.randn(B, heads, S, S), dtype)
    attr = (rng.random_sample((B, S, S)) < 0.7).astype(np.float32)
    attr[0, 0] = 0
    attr = o.rnd(attr, dtype)
    want = o.softmax(qk, attr, 0.125, dtype)
    got = k.softmax(dev(qk), dev(attr), 0.125).cpu().numpy()
    if dtype == "fp32":
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-7)
    else:
        assert_half_close(got, want, ulps=1.0, frac=0.02, what="softmax")
    if S < 1024:
        assert np.all(got[0, :, 0, :] == 0)                  # fully masked row -> zeros (maximum clamped at 0)
    else:
        assert np.all(got[0, :, 0, :] > 0)                   # 1024 keys: no clamp, a fully masked row stays a distribution


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("S,holes,weird", [(5, False, False), (32, False, False), (64, False, False),
                                           (64, True, True), (100, True, False), (128, False, True), (21, True, True),
                                           # beyond 128 positions: fp32 the chunked kernel (K and V in 128-key chunks),
                                           # fp16 the kernel that keeps K and V of a sequence in LDS
                                           (129, False, False), (200, True, True), (256, False, False),
                                           (300, True, False), (384, False, True), (512, False, False), (509, True, True)])
def test_fused_attention_both_layouts(k, dtype, S, holes, weird):
    print("attention", dtype, S, holes, weird, flush=True)
    p = _attn_problem(S + 1, 5, S, 2, dtype, holes=holes, weird_mask=weird)
    bi, wi, vwn = _idx_dev(p)
    T, B, heads, d = p["T"], p["B"], p["heads"], p["d"]
    H = heads * d
    qp, kp, vp = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], T, B, S, heads, d, p["bi"],
                                        p["wi"], dtype)
    want = o.attention(qp, kp, vp, p["attr"], T, p["bi"], p["wi"], dtype)
    # layout 0: padded buffers
    got0 = k.attention(dev(qp), dev(kp), dev(vp), 0, 0, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    # layout 1: packed [T,3H] rows with the bias already added
    add = (lambda a, b: (a.astype(np.float32) + b.astype(np.float32)).astype(np.float32)) if dtype == "fp32" else o.hadd
    packed = np.zeros((B * S, 3 * H), o._np_dtype(dtype))
    packed[:T, :H] = add(p["q"], p["bq"]); packed[:T, H:2 * H] = add(p["k"], p["bk"]); packed[:T, 2 * H:] = add(p["v"], p["bv"])
    pk = dev(packed)
    got1 = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    assert np.array_equal(got0, got1)
    assert np.all(got0[T:] == 0)
    # the same call with the batch's sequence start table handed in (et_attention_with_starts)
    from effective_transformer_amd import ops as _ops
    starts = _ops.sequence_starts(vwn, bi, B, S)
    got2 = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(p["attr"]), vwn, B, S, heads, d, bi, wi,
                       seq_start=starts).cpu().numpy()
    assert np.array_equal(got0, got2)
    if dtype == "fp32":
        np.testing.assert_allclose(got0[:T], want, rtol=1e-4, atol=2e-5)
    else:
        # fp32 accumulation vs the oracle's exact sums, three roundings to half on the way
        np.testing.assert_allclose(got0[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)


# fp16, 128 < seq_len <= 512: K and V of a sequence stay in LDS for all of its query tiles, which are dealt to one, two
# or four workgroups per (head, sequence) depending on how many such pairs the batch has (on a 256-CU part: 288, 144
# and 12 pairs here).
@pytest.mark.parametrize("B,heads,S,holes,weird", [(24, 12, 200, True, False), (12, 12, 300, False, True),
                                                   (3, 4, 500, True, True), (22, 12, 130, False, False)])
def test_fused_attention_with_resident_keys(k, B, heads, S, holes, weird):
    print("attention resident", B, heads, S, holes, weird, flush=True)
    p = _attn_problem(B + S, B, S, heads, "fp16", holes=holes, weird_mask=weird)
    bi, wi, vwn = _idx_dev(p)
    T, d = p["T"], p["d"]
    H = heads * d
    qp, kp, vp = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], T, B, S, heads, d, p["bi"],
                                        p["wi"], "fp16")
    want = o.attention(qp, kp, vp, p["attr"], T, p["bi"], p["wi"], "fp16")
    got0 = k.attention(dev(qp), dev(kp), dev(vp), 0, 0, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    packed = np.zeros((B * S, 3 * H), np.float16)
    packed[:T, :H] = o.hadd(p["q"], p["bq"]); packed[:T, H:2 * H] = o.hadd(p["k"], p["bk"])
    packed[:T, 2 * H:] = o.hadd(p["v"], p["bv"])
    pk = dev(packed)
    got1 = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    assert np.array_equal(got0, got1)
    assert np.all(got0[T:] == 0)
    np.testing.assert_allclose(got0[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("S,d,holes,weird", [(40, 32, False, False), (70, 128, True, True), (33, 8, True, False),
                                             (16, 256, False, True), (600, 64, False, False), (513, 64, True, True),
                                             (1024, 64, False, True), (1000, 32, True, False),
                                             (1023, 64, True, False), (768, 64, False, True), (900, 64, True, True)])
def test_fused_attention_other_head_sizes_and_long_sequences(k, dtype, S, d, holes, weird):
    """size_per_head other than 64 (the reference op takes any, tf_op/bert_transformer_op.cc:53-57) and 512 < seq_len <= 1024
    (its softmax launcher's last branch, cuda/attention.cu:345-356; no clamp of the maximum at 1024 keys)."""
    print("attention generic", dtype, S, d, holes, weird, flush=True)
    if dtype == "fp32" and d == 8:
        d = 12                                             # rows move in 16-byte pieces
    B, heads = 3, 2
    p = _attn_problem(S + d, B, S, heads, dtype, holes=holes, weird_mask=weird, d=d)
    bi, wi, vwn = _idx_dev(p)
    T = p["T"]
    H = heads * d
    qp, kp, vp = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], T, B, S, heads, d, p["bi"],
                                        p["wi"], dtype)
    want = o.attention(qp, kp, vp, p["attr"], T, p["bi"], p["wi"], dtype)
    got0 = k.attention(dev(qp), dev(kp), dev(vp), 0, 0, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    add = (lambda a, b: (a.astype(np.float32) + b.astype(np.float32)).astype(np.float32)) if dtype == "fp32" else o.hadd
    packed = np.zeros((B * S, 3 * H), o._np_dtype(dtype))
    packed[:T, :H] = add(p["q"], p["bq"]); packed[:T, H:2 * H] = add(p["k"], p["bk"]); packed[:T, 2 * H:] = add(p["v"], p["bv"])
    pk = dev(packed)
    got1 = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    assert np.array_equal(got0, got1)
    assert np.all(got0[T:] == 0)
    if dtype == "fp32":
        np.testing.assert_allclose(got0[:T], want, rtol=1e-4, atol=2e-5)
    else:
        np.testing.assert_allclose(got0[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("S", [300, 712])
def test_fused_attention_long_sequences_same_bits_in_any_batch(k, dtype, S):
    """A sequence's attention output does not depend on what else is in the batch or where it stands in it: the same
    five sequences in two orders, and one of them alone, give the same bits (kernels that split a sequence's queries
    or keys over workgroups and wavefronts: keys resident in LDS up to 512 positions, key halves beyond)."""
    print("attention batch independence", dtype, S, flush=True)
    heads, d = 3, 64
    H = heads * d
    rng = np.random.RandomState(S)
    lens = [S, 1, S // 2 + 3, 17, S - 9]
    rows = [o.rnd(rng.randn(n, 3 * H), dtype) for n in lens]
    attr_seq = [o.rnd((rng.random_sample((S, S)) < 0.8).astype(np.float32), dtype) for _ in lens]

    def run(order):
        B = len(order)
        mask = np.zeros((B, S), np.int32)
        for i, j in enumerate(order):
            mask[i, :lens[j]] = 1
        _, T, bi, wi, _ = o.input_op_fast(np.zeros((B, S, 1), np.float32), mask)
        packed = np.zeros((B * S, 3 * H), o._np_dtype(dtype))
        packed[:T] = np.concatenate([rows[j] for j in order])
        attr = np.stack([attr_seq[j] for j in order])
        p = dict(B=B, S=S, T=T, bi=bi, wi=wi)
        bi_d, wi_d, vwn = _idx_dev(p)
        pk = dev(packed)
        out = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(attr), vwn, B, S, heads, d, bi_d, wi_d).cpu().numpy()
        starts = np.concatenate([[0], np.cumsum([lens[j] for j in order])])
        return {j: out[starts[i]:starts[i + 1]] for i, j in enumerate(order)}

    a = run([0, 1, 2, 3, 4])
    b = run([3, 4, 0, 2, 1])
    c = run([2])
    for j in range(5):
        assert np.array_equal(a[j], b[j]), j
    assert np.array_equal(a[2], c[2])


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("S", [40, 64, 100, 128])
@pytest.mark.parametrize("layout", [1, 0])
def test_fused_attention_mixed_lengths_same_bits_in_any_batch(k, dtype, S, layout):
    """The kernel for up to 128 positions on a batch of very different sequences: every sequence must give the bits it
    gives alone in a batch of one, whatever stands beside it, and match the oracle: short and long sequences,
    token-less ones, a short one whose tokens sit at late positions, holes, and masks that attend to padded keys
    (their zero scores count in the softmax of the sequence they belong to)."""
    print("attention mixed lengths", dtype, S, layout, flush=True)
    heads, d = 4, 64
    H = heads * d
    rng = np.random.RandomState(S + layout)
    half = 32 if S <= 64 else 64
    masks = []
    for n in [1, 5, half, half - 1, half + 1, S, 0, 17, 3, S - 2, 9, half, 2, 30, 0, 12, 7]:
        m = np.zeros(S, np.int32)
        m[:min(n, S)] = 1
        masks.append(m)
    late = np.zeros(S, np.int32); late[[0, S // 2 + 3, S - 1]] = 1                # three tokens, the last position in use
    holes = np.zeros(S, np.int32); holes[[1, 4, 5, half - 1]] = 1                  # fits a half
    holes2 = (rng.random_sample(S) < 0.3).astype(np.int32); holes2[half:] = 0      # fits a half
    masks += [late, holes, holes2]
    n_seq = len(masks)
    lens = [int(m.sum()) for m in masks]
    rows = [o.rnd(rng.randn(n, 3 * H), dtype) for n in lens]
    attr_seq = [o.rnd((rng.random_sample((S, S)) < 0.7).astype(np.float32), dtype) for _ in masks]

    def run(order):
        B = len(order)
        mask = np.stack([masks[j] for j in order])
        _, T, bi, wi, _ = o.input_op_fast(np.zeros((B, S, 1), np.float32), mask)
        packed = np.zeros((B * S, 3 * H), o._np_dtype(dtype))
        if T:
            packed[:T] = np.concatenate([rows[j] for j in order])
        attr = np.stack([attr_seq[j] for j in order])
        p = dict(B=B, S=S, T=T, bi=bi, wi=wi)
        bi_d, wi_d, vwn = _idx_dev(p)
        z = np.zeros(H, o._np_dtype(dtype))
        qp, kp, vp = o.add_qkv_bias_padding(packed[:T, :H], z, packed[:T, H:2 * H], z, packed[:T, 2 * H:], z, T, B, S, heads,
                                            d, bi, wi, dtype)
        if layout == 1:
            pk = dev(packed)
            out = k.attention(pk, pk[:, H:], pk[:, 2 * H:], 1, 3 * H, dev(attr), vwn, B, S, heads, d, bi_d, wi_d).cpu().numpy()
        else:
            out = k.attention(dev(qp), dev(kp), dev(vp), 0, 0, dev(attr), vwn, B, S, heads, d, bi_d, wi_d).cpu().numpy()
        want = o.attention(qp, kp, vp, attr, T, bi, wi, dtype)
        if dtype == "fp32":
            np.testing.assert_allclose(out[:T], want, rtol=1e-4, atol=2e-5)
        else:
            np.testing.assert_allclose(out[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)
        starts = np.concatenate([[0], np.cumsum([lens[j] for j in order])])
        return {j: out[starts[i]:starts[i + 1]] for i, j in enumerate(order)}

    a = run(list(range(n_seq)))
    b = run(list(rng.permutation(n_seq)))
    for j in range(n_seq):
        assert np.array_equal(a[j], b[j]), j
    for j in [0, 2, 4, 5, n_seq - 3, n_seq - 2, n_seq - 1]:
        assert np.array_equal(a[j], run([j])[j]), j


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_fused_attention_many_sequences_head_groups(k, dtype):
    """A batch large enough that one workgroup serves a group of 4 heads (shared mask registers, positions and
    zero fill across heads, next head prefetched): holes in the mask, an attention mask unrelated to it."""
    S, heads, B = 16, 12, 720
    p = _attn_problem(99, B, S, heads, dtype, holes=True, weird_mask=True)
    bi, wi, vwn = _idx_dev(p)
    T, d = p["T"], p["d"]
    H = heads * d
    qp, kp, vp = o.add_qkv_bias_padding(p["q"], p["bq"], p["k"], p["bk"], p["v"], p["bv"], T, B, S, heads, d, p["bi"],
                                        p["wi"], dtype)
    want = o.attention(qp, kp, vp, p["attr"], T, p["bi"], p["wi"], dtype)
    got0 = k.attention(dev(qp), dev(kp), dev(vp), 0, 0, dev(p["attr"]), vwn, B, S, heads, d, bi, wi).cpu().numpy()
    assert np.all(got0[T:] == 0)
    if dtype == "fp32":
        np.testing.assert_allclose(got0[:T], want, rtol=1e-4, atol=2e-5)
    else:
        np.testing.assert_allclose(got0[:T].astype(np.float32), want.astype(np.float32), rtol=4e-3, atol=4e-3)


# ---------------------------------------------------------------------------- GEMM ---

@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("m,n,k_", [(1, 768, 768), (134, 768, 768), (257, 3072, 768), (300, 768, 3072),
                                    (1000, 1024, 1024), (100, 200, 64), (70, 264, 128), (2000, 2304, 768),
                                    (5000, 3072, 96), (40, 136, 64)])
def test_gemm(k, dtype, m, n, k_):
    print("gemm", dtype, m, n, k_, flush=True)
    rng = np.random.RandomState(m + n + k_)
    a = o.rnd(rng.randn(m, k_), dtype)
    b = o.rnd(0.05 * rng.randn(k_, n), dtype)
    bias = o.rnd(rng.randn(n), dtype)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    got = k.gemm(dev(a), dev(b)).cpu().numpy()
    scale = np.abs(exact).max()
    if dtype == "fp32":
        assert np.abs(got - exact).max() <= 1e-5 * scale
    else:
        assert np.all(np.abs(got.astype(np.float64) - exact) <= 0.51 * half_ulp(exact) + 1e-5 * scale)
    # bias epilogue: element-type add on the rounded product
    gotb = k.gemm(dev(a), dev(b), bias=dev(bias)).cpu().numpy()
    if dtype == "fp32":
        np.testing.assert_allclose(gotb, got + bias, rtol=1e-6, atol=1e-6)
    else:
        assert np.array_equal(gotb, o.hadd(got, bias))
    # device-side row bound
    if m > 10:
        md = torch.tensor([m - 5], dtype=torch.int32, device="cuda")
        got2 = k.gemm(dev(a), dev(b), m_dev=md).cpu().numpy()
        assert np.array_equal(got2[:m - 5], got[:m - 5]) and np.all(got2[m - 5:] == 0)


# The k-contiguous-B kernels: the persistent 256x256 one from 128 such tiles on (first six shapes; the last two of
# those leave a last round that keeps at most half of the workgroups busy, so those tiles are shared by two
# workgroups, one per 128-column half, one of them with a ragged last column tile; the next three run on tiles of
# 160, 192 and 224 rows, which fill the chip's single round better), below that one tile per workgroup
# of 32 .. 128 rows by 64 .. 256 columns, with ragged last tiles in both directions and a single pair of k-steps.  The
# last eighteen shapes reach, on a 256-CU part, every tile of that kernel in both of its ring depths: 32x64, 64x64,
# 64x128, 96x64, 96x128, 96x192, 128x64, 128x128, 128x192 with a CU per workgroup and with two workgroups per CU, and
# 128x256; three of the 192-column ones have a ragged last column tile.  The last shape is large enough (A and C
# together above 96 MB) for the persistent kernel's non-temporal C stores; the persistent shapes before it take its
# plain stores.  The oracle product is taken on the CPU in float64 for a sample of rows.
@pytest.mark.parametrize("m,n,k_", [(11000, 768, 768), (8200, 1032, 128), (4100, 2304, 768), (10900, 776, 3072),
                                    (23301, 768, 768), (14000, 1032, 128),
                                    (13097, 768, 3072), (15866, 768, 768), (13097, 1024, 1024),
                                    (6000, 776, 768), (4000, 768, 3072), (3000, 1032, 128), (2000, 768, 768),
                                    (1001, 776, 3072), (500, 768, 64), (302, 40, 192),
                                    (2308, 392, 128), (722, 768, 192), (2491, 776, 128), (2064, 768, 128),
                                    (5419, 768, 128), (1393, 768, 192), (3467, 776, 128), (2735, 768, 128),
                                    (6151, 768, 128), (5480, 768, 192), (9348, 776, 128), (1881, 776, 128),
                                    (4626, 776, 128), (4077, 768, 128), (8225, 776, 64), (3849, 1032, 192),
                                    (9803, 776, 128), (8225, 768, 128), (40000, 1032, 640)])
def test_gemm_bt(k, m, n, k_):
    print("gemm_bt", m, n, k_, flush=True)
    rng = np.random.RandomState(m + n + k_)
    a = o.rnd(rng.randn(m, k_), "fp16")
    b = o.rnd(0.05 * rng.randn(k_, n), "fp16")
    bias = o.rnd(rng.randn(n), "fp16")
    bt = k.transpose_weight(dev(b))
    assert np.array_equal(bt.cpu().numpy(), b.T)                       # the transpose is a pure copy
    got = k.gemm_bt(dev(a), bt).cpu().numpy()
    # the same rows through the untransposed kernel: both accumulate k in the same order
    assert np.array_equal(got, k.gemm(dev(a), dev(b)).cpu().numpy())
    rows = np.unique(np.concatenate([np.arange(0, min(m, 300)), np.arange(max(m - 300, 0), m), rng.randint(0, m, 400)]))
    exact = a[rows].astype(np.float64) @ b.astype(np.float64)
    assert np.all(np.abs(got[rows].astype(np.float64) - exact) <= 0.51 * half_ulp(exact) + 1e-5 * np.abs(exact).max())
    gotb = k.gemm_bt(dev(a), bt, bias=dev(bias)).cpu().numpy()
    assert np.array_equal(gotb, o.hadd(got, bias))
    md = torch.tensor([m - 301], dtype=torch.int32, device="cuda")
    got2 = k.gemm_bt(dev(a), bt, m_dev=md).cpu().numpy()
    assert np.array_equal(got2[:m - 301], got[:m - 301]) and np.all(got2[m - 301:] == 0)


# A sequence gives the same bits in a batch of any size: every fp16 kernel accumulates k in the same order, so the
# rows of a small problem (64x128 tiles), a middle one (128x256 tiles) and a large one (persistent 256x256 tiles, B in
# either storage order) agree bit for bit, and so do the one-tile-per-workgroup kernels for k-contiguous B
# (tiles from 32x64 to 128x256); the two fp32 tiles likewise.
@pytest.mark.parametrize("n,k_", [(768, 768), (768, 3072), (3072, 768)])
def test_gemm_same_bits_in_every_kernel(k, n, k_):
    print("gemm same bits", n, k_, flush=True)
    rng = np.random.RandomState(n + k_)
    m = 11000
    a = dev(o.rnd(rng.randn(m, k_), "fp16"))
    b = dev(o.rnd(0.05 * rng.randn(k_, n), "fp16"))
    big = k.gemm(a, b).cpu().numpy()
    bt = k.transpose_weight(b)
    assert np.array_equal(k.gemm_bt(a, bt).cpu().numpy(), big)
    for rows in (6000, 2500, 300, 1):
        part = k.gemm(a[:rows].contiguous(), b).cpu().numpy()
        assert np.array_equal(part, big[:rows]), rows
    for rows in (9000, 8200, 6000, 5400, 4000, 2700, 2000, 1400, 1000, 500, 130, 1):
        part = k.gemm_bt(a[:rows].contiguous(), bt).cpu().numpy()
        assert np.array_equal(part, big[:rows]), rows
    a32, b32 = a.float(), b.float()
    big32 = k.gemm(a32, b32).cpu().numpy()
    for rows in (1500, 100):
        assert np.array_equal(k.gemm(a32[:rows].contiguous(), b32).cpu().numpy(), big32[:rows]), rows


# every GEMM kernel behind et_gemm: fp32 128x128 and 64x64 tiles, fp16 64x128 and 128x256 tiles, fp16 persistent
@pytest.mark.parametrize("dtype,m,n,k_", [("fp32", 700, 256, 64), ("fp32", 3000, 3072, 96), ("fp16", 300, 512, 64),
                                           ("fp16", 2000, 2304, 64), ("fp16", 5000, 3072, 96),
                                           ("fp16", 11000, 1032, 160)])
def test_gemm_bias_gelu_equals_the_two_passes(k, dtype, m, n, k_):
    print("gemm_bias_gelu", dtype, m, n, k_, flush=True)
    rng = np.random.RandomState(m + n + k_ + 2)
    a = o.rnd(rng.randn(m, k_), dtype)
    b = o.rnd(0.05 * rng.randn(k_, n), dtype)
    bias = o.rnd(rng.randn(n), dtype)
    two = k.add_bias_act(k.gemm(dev(a), dev(b)), dev(bias)).cpu().numpy()
    one = k.gemm(dev(a), dev(b), bias=dev(bias), gelu=True).cpu().numpy()
    assert np.array_equal(one, two) and one.tobytes() == two.tobytes()       # same rounding points, bit for bit
    md = torch.tensor([m - 77], dtype=torch.int32, device="cuda")
    part = k.gemm(dev(a), dev(b), bias=dev(bias), m_dev=md, gelu=True).cpu().numpy()
    assert np.array_equal(part[:m - 77], one[:m - 77]) and np.all(part[m - 77:] == 0)
    with pytest.raises(Exception, match="null bias"):
        k.gemm(dev(a), dev(b), gelu=True)


# (the four shapes before the last: 192-column tiles, whose lanes store a group of four and a group of two columns;
# the last one: the persistent kernel's non-temporal stores behind the GELU)
@pytest.mark.parametrize("m,n,k_", [(11000, 768, 768), (8200, 1032, 128), (5000, 3072, 768), (2000, 3072, 768),
                                    (1000, 776, 128), (400, 768, 768), (350, 200, 64),
                                    (5480, 768, 128), (3849, 1032, 64), (9803, 776, 64), (1288, 3080, 64),
                                    (36000, 1032, 768)])
def test_gemm_bt_bias_gelu_equals_the_two_passes(k, m, n, k_):
    print("gemm_bt_bias_gelu", m, n, k_, flush=True)
    rng = np.random.RandomState(m + n + k_ + 1)
    a = o.rnd(rng.randn(m, k_), "fp16")
    b = o.rnd(0.05 * rng.randn(k_, n), "fp16")
    bias = o.rnd(rng.randn(n), "fp16")
    bt = k.transpose_weight(dev(b))
    two = k.add_bias_act(k.gemm_bt(dev(a), bt), dev(bias)).cpu().numpy()
    one = k.gemm_bt(dev(a), bt, bias=dev(bias), gelu=True).cpu().numpy()
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16))        # same rounding points, bit for bit
    # against the oracle's bias + GELU on the product the kernel produced
    prod = k.gemm_bt(dev(a), bt).cpu().numpy()
    want = o.add_bias_act(prod, bias, "fp16")
    assert np.max(np.abs(one.astype(np.float32) - want.astype(np.float32))) <= 2e-3 * max(1.0, np.abs(want).max())
    md = torch.tensor([m - 301], dtype=torch.int32, device="cuda")
    part = k.gemm_bt(dev(a), bt, bias=dev(bias), m_dev=md, gelu=True).cpu().numpy()
    assert np.array_equal(part[:m - 301], one[:m - 301]) and np.all(part[m - 301:] == 0)
    with pytest.raises(Exception, match="null bias"):
        k.gemm_bt(dev(a), bt, gelu=True)


def test_gemm_bt_refuses_k_that_is_no_multiple_of_64(k):
    a = torch.zeros(1000, 96, dtype=torch.float16, device="cuda")
    bt = torch.zeros(768, 96, dtype=torch.float16, device="cuda")
    with pytest.raises(Exception, match="k % 64"):
        k.gemm_bt(a, bt)


# The measurement aid: a launch returns its floating-point operation count (CUs x 8 waves x iters x 64 MFMAs x 16384),
# fills the sink with finite sums (zero for zero operands) and refuses a sink that is too small.
def test_calibrate_mfma(ops):
    import ctypes as C
    from effective_transformer_amd import _lib
    lib = _lib.load()
    h = ops.handle(torch.device("cuda:0"))
    nbytes = lib.et_calibrate_mfma_sink_bytes(h)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert nbytes == cus * 512 * 4
    sink = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    fl = C.c_double(0.0)
    for rnd in (0, 1):
        _lib.check(lib.et_calibrate_mfma(h, rnd, 10, C.c_void_p(sink.data_ptr()), nbytes, C.byref(fl), st), h)
        torch.cuda.synchronize()
        assert fl.value == cus * 8 * 10 * 64 * 16384.0
        assert bool(torch.isfinite(sink).all())
        assert bool((sink == 0).all()) == (rnd == 0)
    assert lib.et_calibrate_mfma(h, 0, 10, C.c_void_p(sink.data_ptr()), nbytes - 4, C.byref(fl), st) == 2   # ET_WORKSPACE_TOO_SMALL
    assert lib.et_calibrate_mfma(h, 0, 0, C.c_void_p(sink.data_ptr()), nbytes, C.byref(fl), st) == 1         # ET_INVALID_ARGUMENT
