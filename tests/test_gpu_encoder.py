"""Parity of the three ops (Input -> L x Layer -> Output through the C ABI) against the CPU
oracle on the seeded workloads, plus size-independent properties at the full benchmark sizes."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import et_oracle as o
from gpu_util import TDT, dev, run_encoder, subset_workload

pytestmark = pytest.mark.gpu


def _oracle(w, layers=None):
    wl = w["wl"]
    weights = w["weights"] if layers is None else w["weights"][:16 * layers]
    return o.encoder(w["x"], w["mask"], w["attr_mask"], weights, wl.heads, wl.d, wl.dtype)


def _check(got, want, mask, dtype):
    valid = mask.astype(bool)
    assert np.all(got[~valid] == 0)                              # the Output op zero-fills padding
    g, w_ = got[valid].astype(np.float64), want[valid].astype(np.float64)
    if dtype == "fp32":
        # fp32 bar: 1e-4 relative error of every token's output row, ||got - want|| / ||want|| (a LayerNorm output row
        # has norm ~ sqrt(H), so no floor is needed), and 5e-5 absolute on every element.  Measured after 12 layers:
        # 4e-6 relative per row, 1.2e-5 absolute; a drift towards the bars shows up here long before the contract breaks.
        rel = np.linalg.norm(g - w_, axis=-1) / np.linalg.norm(w_, axis=-1)
        assert rel.max() < 1e-4, rel.max()
        assert np.abs(g - w_).max() < 5e-5, np.abs(g - w_).max()
    else:
        # fp16 bar: 2e-2 max-abs after 12 layers
        assert np.abs(g - w_).max() < 2e-2, np.abs(g - w_).max()
    return np.abs(g - w_).max()


@pytest.mark.parametrize("random_affine", [False, True])
def test_cfg1_single_layer_fp32(random_affine):
    w = o.make_workload("cfg1", random_affine=random_affine)
    got = run_encoder(w)
    print("cfg1 max abs diff", _check(got, _oracle(w), w["mask"], "fp32"), flush=True)
    # and the reference's own check: agreement with the standard BERT graph on valid tokens
    std = o.tf_graph_encoder(w["x"], w["attr_mask"], w["weights"], w["wl"].heads, w["wl"].d)
    valid = w["mask"].astype(bool)
    assert np.abs(got[valid] - std[valid]).max() < 1e-4


def test_cfg1_fp16_variant():
    w = o.make_workload("cfg1", random_affine=True)
    w16 = dict(w, wl=o.Workload(**{**w["wl"].__dict__, "dtype": "fp16"}), x=w["x"].astype(np.float16),
               attr_mask=w["attr_mask"].astype(np.float16), weights=[a.astype(np.float16) for a in w["weights"]])
    got = run_encoder(w16)
    print("cfg1/fp16 max abs diff", _check(got, _oracle(w16), w16["mask"], "fp16"), flush=True)


def test_cfg2_twelve_layers_fp16():
    w = o.make_workload("cfg2")
    got = run_encoder(w)
    print("cfg2 max abs diff", _check(got, _oracle(w), w["mask"], "fp16"), flush=True)
    # device-side token count (no host hint) gives the same bits
    got2 = run_encoder(w, hint=False)
    assert np.array_equal(got, got2)


def test_cfg2_random_affine_fp32_twelve_layers():
    w = o.make_workload("cfg2", random_affine=True)
    w32 = dict(w, wl=o.Workload(**{**w["wl"].__dict__, "dtype": "fp32"}), x=w["x"].astype(np.float32),
               attr_mask=w["attr_mask"].astype(np.float32), weights=[a.astype(np.float32) for a in w["weights"]])
    sub = subset_workload(w32, np.arange(24))
    got = run_encoder(sub)
    print("cfg2/fp32 12 layers max abs diff", _check(got, _oracle(sub), sub["mask"], "fp32"), flush=True)


@pytest.mark.parametrize("name,nsub,layers", [("cfg3", 24, 12), ("cfg4", 12, 12), ("cfg5", 8, 24)])
def test_full_size_properties_and_subset_oracle(name, nsub, layers):
    """At the benchmark sizes the oracle is too slow, so: (1) sequences are independent, hence a
    run on a subset of the sequences must reproduce the full run's rows bit for bit, and the
    subset is small enough for the oracle; (2) permuting the batch permutes the output;
    (3) padding is zero."""
    print("full-size", name, flush=True)
    w = o.make_workload(name)
    wl = w["wl"]
    full = run_encoder(w)
    assert np.all(full[~w["mask"].astype(bool)] == 0)
    assert np.isfinite(full.astype(np.float32)).all()
    rng = np.random.RandomState(1)
    idx = np.sort(rng.choice(wl.B, nsub, replace=False))
    sub = subset_workload(w, idx)
    got_sub = run_encoder(sub)
    assert np.array_equal(got_sub, full[idx])
    print(name, "subset max abs diff vs oracle", _check(got_sub, _oracle(sub), sub["mask"], wl.dtype), flush=True)
    perm = rng.permutation(wl.B)
    wp = subset_workload(w, perm)
    assert np.array_equal(run_encoder(wp), full[perm])
    if name == "cfg3":
        # batches in between run other GEMM kernels (128 x 256 tiles for the narrow projections, the persistent kernel
        # for the wide ones): the same sequences still give the same bits
        for n in (150, 420):
            assert np.array_equal(run_encoder(subset_workload(w, np.arange(n))), full[:n]), n


@pytest.mark.parametrize("name,layers", [("cfg3", 2), ("cfg2", 3), ("cfg4", 1)])
def test_prepared_weights_and_shared_start_table_change_nothing(name, layers):
    """et_layer_with_prepared (transposed kernels made once, one sequence start table per batch) against plain et_layer
    calls: the same bits, with the wide projections' kernels prepared and with all six."""
    print("prepared", name, flush=True)
    w = o.make_workload(name)
    plain = run_encoder(w, layers=layers, prepare=False)
    assert np.array_equal(run_encoder(w, layers=layers, prepare=True), plain)
    assert np.array_equal(run_encoder(w, layers=layers, prepare=True, every_kernel=False), plain)
    assert np.array_equal(run_encoder(w, layers=layers, prepare=True, hint=False), plain)


def test_prepared_q_k_v_go_together():
    from effective_transformer_amd import _lib, ops
    w = o.make_workload("cfg2")
    wl = w["wl"]
    enc = ops.EffectiveTransformerEncoder(1, wl.heads, wl.d, w["weights"][:16], torch.float16, "cuda")
    enc.layers[0].prepared.attr_kernel_K_t = None
    with pytest.raises(_lib.EtError, match="go together"):
        enc(dev(w["x"], torch.float16), dev(w["mask"].astype(np.int32)), dev(w["attr_mask"], torch.float16))


def _packed(w, x_np, dt):
    """Input op on x_np with the workload's mask: packed tensor + the index tensors."""
    from effective_transformer_amd import ops
    wl = w["wl"]
    return ops.effective_transformer_input(dev(x_np, dt), dev(w["mask"].astype(np.int32)), wl.B, wl.S, wl.S, wl.heads,
                                           wl.d, return_host_count=True)


@pytest.mark.parametrize("name,nseq", [("cfg1", None), ("cfg2", None), ("cfg3", 110), ("cfg4", 40)])
@pytest.mark.parametrize("prepared", [False, True])
@pytest.mark.parametrize("hint", [True, False])
def test_layer_with_distinct_from_and_to_tensors(name, nseq, prepared, hint):
    """Q comes from from_tensor, K and V from to_tensor, and the residual of the first LayerNorm is from_tensor
    (tf_op/bert_transformer_op.cu.cc:110-141, 210): one layer with two different packed tensors against the oracle,
    through et_layer and et_layer_with_prepared, with and without the host-side token count.  cfg3's subset is large
    enough for the persistent large-M GEMMs (grouped Q/K/V launch with two different A operands)."""
    from effective_transformer_amd import ops
    print("from != to", name, "prepared", prepared, "hint", hint, flush=True)
    w = o.make_workload(name, layers=1, random_affine=True)
    if nseq is not None:
        w = subset_workload(w, np.arange(nseq))
    wl = w["wl"]
    dt = TDT[wl.dtype]
    rng = np.random.RandomState(99)
    x_to = o.rnd(rng.randn(*w["x"].shape), wl.dtype)
    frm, vwn, bidx, widx, T = _packed(w, w["x"], dt)
    to = _packed(w, x_to, dt)[0]
    lw = ops.LayerWeights.from_slots(frm.device, dt, w["weights"][:16])
    if prepared:
        lw.prepare()
    starts = ops.sequence_starts(vwn, bidx, wl.B, wl.S) if prepared else None
    attr = dev(w["attr_mask"], dt)
    run = lambda a, b: ops.effective_transformer(a, b, attr, vwn, bidx, widx, lw, wl.B, wl.S, wl.S, wl.heads, wl.d,
                                                 valid_word_num_hint=T if hint else -1, seq_start=starts)
    got = run(frm, to).reshape(wl.B * wl.S, wl.H)[:T].cpu().numpy().astype(np.float64)
    bi, wi_ = bidx.cpu().numpy().ravel(), widx.cpu().numpy().ravel()
    pf = frm.reshape(wl.B * wl.S, wl.H).cpu().numpy()
    pt = to.reshape(wl.B * wl.S, wl.H).cpu().numpy()
    want = o.layer(pf, pt, w["attr_mask"], T, bi, wi_, w["weights"][:16], wl.B, wl.S, wl.heads, wl.d,
                   wl.dtype).astype(np.float64)
    err = np.abs(got - want).max()
    print("  max abs diff", err, flush=True)
    # one layer: fp32 2e-5 absolute (measured 3e-6); fp16 8e-3 absolute (measured 4.9e-3: a rounding of an intermediate
    # that falls the other way than the oracle's moves an output of magnitude 2..8 by one or two of its half-ulps)
    assert err < (2e-5 if wl.dtype == "fp32" else 8e-3), err
    # the check can tell the operands apart: swapped, or the same tensor twice, is far from the oracle
    for a, b in ((to, frm), (frm, frm), (to, to)):
        other = run(a, b).reshape(wl.B * wl.S, wl.H)[:T].cpu().numpy().astype(np.float64)
        assert np.abs(other - want).max() > 0.1


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_get_sequence_output_is_the_encoder(dtype):
    """The one name the reference's Python package exports (python/effective_transformer/__init__.py:32-84), with its
    argument list and a BertConfig-like object: same result as the encoder object, and oracle parity."""
    from types import SimpleNamespace
    from effective_transformer_amd import get_sequence_output
    print("get_sequence_output", dtype, flush=True)
    w = o.make_workload("cfg1" if dtype == "fp32" else "cfg2", layers=2, random_affine=True)
    wl = w["wl"]
    dt = TDT[dtype]
    config = SimpleNamespace(num_attention_heads=wl.heads, hidden_size=wl.H, num_hidden_layers=2)
    x = dev(w["x"], dt); mask = dev(w["mask"].astype(np.int32)); attr = dev(w["attr_mask"], dt)
    got = get_sequence_output(config=config, max_batch_size=wl.B, max_seq_length=wl.S, attention_mask=attr,
                              input_mask=mask, from_tensor=x, weights_value=w["weights"][:32])
    assert tuple(got.shape) == (wl.B, wl.S, wl.H)
    assert np.array_equal(got.cpu().numpy(), run_encoder(w, layers=2))
    _check(got.cpu().numpy(), _oracle(w, layers=2), w["mask"], dtype)


def test_empty_batch_of_tokens_and_holes():
    w = o.make_workload("cfg1", random_affine=True)
    wl = w["wl"]
    zero = dict(w, mask=np.zeros_like(w["mask"]), attr_mask=np.zeros_like(w["attr_mask"]))
    out = run_encoder(zero)
    assert np.all(out == 0)
    out = run_encoder(zero, hint=False)
    assert np.all(out == 0)
    # a mask with holes and an attention mask that is not tied to it
    rng = np.random.RandomState(5)
    mask = (rng.random_sample(w["mask"].shape) < 0.6).astype(np.int32)
    attr = (rng.random_sample(w["attr_mask"].shape) < 0.8).astype(np.float32)
    hol = dict(w, mask=mask, attr_mask=attr)
    got = run_encoder(hol)
    print("holes max abs diff", _check(got, _oracle(hol), mask, "fp32"), flush=True)


def test_hip_graph_replays_match_eager():
    """The whole stack captured in one HIP graph: several replays with eager work and synchronisations between
    them, each checked bit for bit against the eager run; a replay with a different mask adapts on the device."""
    from effective_transformer_amd import ops
    w = o.make_workload("cfg2", layers=3)
    wl = w["wl"]
    dt = TDT[wl.dtype]
    enc = ops.EffectiveTransformerEncoder(3, wl.heads, wl.d, w["weights"], dt, "cuda")
    x = dev(w["x"], dt); mask = dev(w["mask"]); attr = dev(w["attr_mask"], dt)
    eager = enc(x, mask, attr).clone()
    g = enc.make_graph(x, mask, attr)
    for rep in range(4):
        got = g().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), rep
        junk = enc(x * 0.5, mask, attr)              # eager work on the same workspaces between replays
        torch.cuda.synchronize()
        assert not torch.equal(junk, eager)
    # other lengths through the same graph
    rng = np.random.RandomState(3)
    lens = rng.randint(1, wl.S + 1, size=wl.B)
    mask2 = (np.arange(wl.S)[None, :] < lens[:, None]).astype(np.int32)
    attr2 = np.ascontiguousarray(np.broadcast_to(mask2[:, None, :], (wl.B, wl.S, wl.S))).astype(np.float16)
    want2 = enc(x, dev(mask2), dev(attr2)).clone()
    got2 = g(None, dev(mask2), dev(attr2)).clone()
    torch.cuda.synchronize()
    assert torch.equal(got2, want2)
    w2 = dict(w, mask=mask2, attr_mask=attr2, weights=w["weights"][:48])
    print("graph/new mask max abs diff", _check(got2.cpu().numpy(), _oracle(w2), mask2, "fp16"), flush=True)


def test_hip_graph_sized_for_a_token_bound():
    """A graph captured with max_valid_tokens sizes its launches for that many rows instead of B*S: replays with the
    capture mask, with a shorter one and with one that reaches the bound exactly equal the eager runs bit for bit, and a
    mask beyond the bound is refused."""
    from effective_transformer_amd import ops
    w = o.make_workload("cfg2", layers=2)
    wl = w["wl"]
    dt = TDT[wl.dtype]
    enc = ops.EffectiveTransformerEncoder(2, wl.heads, wl.d, w["weights"], dt, "cuda")
    x = dev(w["x"], dt); mask = dev(w["mask"]); attr = dev(w["attr_mask"], dt)
    tokens = int(w["mask"].sum())
    bound = tokens + 37
    assert bound < wl.B * wl.S
    g = enc.make_graph(x, mask, attr, max_valid_tokens=bound)
    assert torch.equal(g().clone(), enc(x, mask, attr))
    rng = np.random.RandomState(5)
    for case in ("shorter", "at the bound"):
        lens = w["mask"].sum(axis=1)
        if case == "shorter":
            lens = np.maximum(lens - rng.randint(0, 8, size=wl.B), 0)
        else:
            room = wl.S - lens
            add = np.zeros_like(lens)
            left = 37
            for b in range(wl.B):
                add[b] = min(room[b], left)
                left -= add[b]
            assert left == 0
            lens = lens + add
        mask2 = (np.arange(wl.S)[None, :] < lens[:, None]).astype(np.int32)
        assert mask2.sum() <= bound and (case == "shorter" or mask2.sum() == bound)
        attr2 = np.ascontiguousarray(np.broadcast_to(mask2[:, None, :], (wl.B, wl.S, wl.S))).astype(np.float16)
        want = enc(x, dev(mask2), dev(attr2)).clone()
        got = g(None, dev(mask2), dev(attr2)).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), case
    full = dev(np.ones((wl.B, wl.S), np.int32))
    with pytest.raises(ValueError, match="max_valid_tokens"):
        g(None, full, None)
    with pytest.raises(ValueError, match="max_valid_tokens"):
        enc.make_graph(x, full, attr, max_valid_tokens=bound)


def test_error_paths():
    from effective_transformer_amd import _lib, ops
    lib = _lib.load()
    h = ops.handle(torch.device("cuda", 0))
    w = o.make_workload("cfg1")
    wl = w["wl"]
    x = dev(w["x"]); mask = dev(w["mask"]); attr = dev(w["attr_mask"])
    to, vwn, bidx, widx = ops.effective_transformer_input(x, mask, wl.B, wl.S, wl.S, wl.heads, wl.d)
    lw = ops.LayerWeights.from_slots(x.device, torch.float32, w["weights"][:16])
    with pytest.raises(_lib.EtError) as e:       # from_seq_len != to_seq_len
        ops.effective_transformer(to, to, attr, vwn, bidx, widx, lw, wl.B, wl.S, wl.S + 1, wl.heads, wl.d)
    assert e.value.status == 1 and "from_seq_len == to_seq_len" in str(e.value)
    with pytest.raises(_lib.EtError) as e:       # a head size beyond what the attention kernels hold
        ops.effective_transformer(to, to, attr, vwn, bidx, widx, lw, wl.B, wl.S, wl.S, 1, 257)
    assert e.value.status == 3
    out = torch.empty_like(to)
    st = lib.et_layer(h, 0, C.byref(lw.struct), to.data_ptr(), to.data_ptr(), attr.data_ptr(), vwn.data_ptr(),
                      bidx.data_ptr(), widx.data_ptr(), out.data_ptr(), wl.B, wl.S, wl.S, wl.heads, wl.d, -1,
                      out.data_ptr(), 1024, None)
    assert st == 2 and b"ET_WORKSPACE_TOO_SMALL" in lib.et_last_error(h)
    st = lib.et_layer(h, 0, C.byref(lw.struct), to.data_ptr(), to.data_ptr(), attr.data_ptr(), vwn.data_ptr(),
                      bidx.data_ptr(), widx.data_ptr(), to.data_ptr(), wl.B, wl.S, wl.S, wl.heads, wl.d, -1,
                      out.data_ptr(), 1 << 30, None)
    assert st == 1 and b"alias" in lib.et_last_error(h)
    # one sequence more than the attention grid holds: refused before anything is launched (the declared workspace
    # size only has to pass the size check)
    st = lib.et_layer(h, 0, C.byref(lw.struct), to.data_ptr(), to.data_ptr(), attr.data_ptr(), vwn.data_ptr(),
                      bidx.data_ptr(), widx.data_ptr(), out.data_ptr(), 65536, 1, 1, wl.heads, wl.d, -1,
                      out.data_ptr(), 1 << 40, None)
    assert st == 3 and b"65535" in lib.et_last_error(h)
    with pytest.raises(TypeError):
        ops.effective_transformer_input(x.to(torch.bfloat16), mask, wl.B, wl.S, wl.S, wl.heads, wl.d)
    # a sequence table of B + 1 words (2 B + 1 are needed) is refused wherever one is handed in or asked for
    small = torch.zeros(wl.B + 1, dtype=torch.int32, device="cuda")
    nsmall = small.numel() * 4
    st = lib.et_sequence_starts(h, bidx.data_ptr(), vwn.data_ptr(), wl.B, wl.S, small.data_ptr(), nsmall, None)
    assert st == 2 and b"et_seq_workspace_bytes" in lib.et_last_error(h)
    prep = _lib.LayerPrepared()
    prep.seq_start, prep.seq_start_bytes = small.data_ptr(), nsmall
    ws = torch.empty(lib.et_layer_workspace_bytes(0, wl.B, wl.S, wl.heads, wl.d), dtype=torch.uint8, device="cuda")
    st = lib.et_layer_with_prepared(h, 0, C.byref(lw.struct), C.byref(prep), to.data_ptr(), to.data_ptr(), attr.data_ptr(),
                                    vwn.data_ptr(), bidx.data_ptr(), widx.data_ptr(), out.data_ptr(), wl.B, wl.S, wl.S,
                                    wl.heads, wl.d, -1, ws.data_ptr(), ws.numel(), None)
    assert st == 2 and b"seq_start" in lib.et_last_error(h)
    qkv = torch.zeros(wl.B * wl.S, 3 * wl.H, device="cuda")
    st = lib.et_attention_with_starts(h, 0, qkv.data_ptr(), qkv.data_ptr(), qkv.data_ptr(), 1, 3 * wl.H, attr.data_ptr(),
                                      out.data_ptr(), vwn.data_ptr(), wl.B, wl.S, wl.heads, wl.d, bidx.data_ptr(),
                                      widx.data_ptr(), small.data_ptr(), None, nsmall, None)
    assert st == 2 and b"et_seq_workspace_bytes" in lib.et_last_error(h)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_long_sequences_layer_against_oracle(dtype):
    """seq_len 256 (beyond the 128 positions the resident-K/V attention kernel holds): two layers against the oracle."""
    print("encoder S=256", dtype, flush=True)
    wl = o.Workload("long", 77, dtype, 2, 6, 256, 4, 64, 1024, 40, 257)
    rng = np.random.RandomState(wl.seed)
    lens, mask, attr = o.make_masks(wl, rng)
    x = o.rnd(rng.randn(wl.B, wl.S, wl.H), dtype)
    weights = []
    for _ in range(2):
        weights.extend(o.make_layer_weights(wl, rng, True))
    w = dict(wl=wl, lens=lens, mask=mask, attr_mask=attr, x=x, weights=weights)
    got = run_encoder(w)
    _check(got, _oracle(w), mask, dtype)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("B,S,heads,d", [(4, 48, 4, 32), (3, 40, 2, 128), (2, 600, 2, 64), (1, 1024, 1, 64), (2, 520, 4, 32),
                                         (5, 40, 3, 32),       # hidden size 96: no multiple of 64, the weights stay [k][n]
                                         (3, 384, 2, 64), (2, 512, 12, 64), (4, 250, 3, 64)])  # keys resident in LDS (fp16)
def test_other_head_sizes_and_sequences_beyond_512(dtype, B, S, heads, d):
    """The reference op takes any size_per_head (tf_op/bert_transformer_op.cc:53-57) and sequences up to the 1024 keys
    its softmax launcher covers (cuda/attention.cu:345-356): one layer against the oracle."""
    print("encoder other shapes", dtype, B, S, heads, d, flush=True)
    wl = o.Workload("odd", 500 + S + d, dtype, 1, B, S, heads, d, 4 * heads * d, max(1, S // 3), S + 1)
    rng = np.random.RandomState(wl.seed)
    lens, mask, attr = o.make_masks(wl, rng)
    lens[0] = S; mask[0] = 1; attr[0] = 1                   # one sequence of full length
    x = o.rnd(rng.randn(B, S, wl.H), dtype)
    w = dict(wl=wl, lens=lens, mask=mask, attr_mask=o.rnd(attr, dtype), x=x, weights=o.make_layer_weights(wl, rng, True))
    got = run_encoder(w)
    _check(got, _oracle(w), mask, dtype)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_largest_batch_the_attention_grid_holds(dtype):
    """65535 sequences (one more is refused, see test_error_paths): a subset of the sequences against the oracle, and the
    full run reproduces the subset's rows bit for bit."""
    print("encoder B=65535", dtype, flush=True)
    B, S, heads, d = 65535, 4, 2, 64
    wl = o.Workload("wide-batch", 65535, dtype, 1, B, S, heads, d, 4 * heads * d, 0, S + 1)
    rng = np.random.RandomState(wl.seed)
    lens, mask, attr = o.make_masks(wl, rng)
    x = o.rnd(rng.randn(B, S, wl.H), dtype)
    w = dict(wl=wl, lens=lens, mask=mask, attr_mask=o.rnd(attr, dtype), x=x, weights=o.make_layer_weights(wl, rng, True))
    full = run_encoder(w)
    assert np.all(full[~mask.astype(bool)] == 0)
    idx = np.sort(np.concatenate([np.arange(20), B - 1 - np.arange(20), rng.choice(np.arange(20, B - 20), 40, replace=False)]))
    sub = subset_workload(w, idx)
    got_sub = run_encoder(sub)
    assert np.array_equal(got_sub, full[idx])
    _check(got_sub, _oracle(sub), sub["mask"], dtype)


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_against_oracle(seed):
    """One layer on randomly drawn shapes (sequence lengths that are not multiples of 4 or 16, one head, holes in the
    mask, empty sequences, both element types) against the oracle."""
    rng = np.random.RandomState(1000 + seed)
    dtype = ["fp32", "fp16"][seed % 2]
    B = int(rng.randint(1, 9))
    S = int(rng.choice([1, 3, 7, 16, 17, 33, 50, 64, 65, 96, 127, 130, 200]))
    heads = int(rng.choice([1, 2, 3, 12]))
    print("random shape", seed, dtype, "B", B, "S", S, "heads", heads, flush=True)
    wl = o.Workload("rnd", 1000 + seed, dtype, 1, B, S, heads, 64, 4 * heads * 64, 1, S + 1)
    if seed % 3 == 0:
        mask = (rng.rand(B, S) < 0.7).astype(np.int32)
        if B > 1:
            mask[rng.randint(0, B)] = 0                       # an empty sequence
        attr = (rng.rand(B, S, S) < 0.8).astype(np.float32)   # an attention mask unrelated to the input mask
    else:
        lens = rng.randint(1, S + 1, size=B)
        mask = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
        attr = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (B, S, S))).astype(np.float32)
    attr = o.rnd(attr, dtype)
    x = o.rnd(rng.randn(B, S, wl.H), dtype)
    weights = o.make_layer_weights(wl, rng, True)
    w = dict(wl=wl, lens=None, mask=mask, attr_mask=attr, x=x, weights=weights)
    got = run_encoder(w)
    if mask.sum() == 0:
        assert np.all(got == 0)
        return
    _check(got, _oracle(w), mask, dtype)


@pytest.mark.parametrize("seed", range(10))
def test_random_long_shapes_against_oracle(seed):
    """One layer on randomly drawn shapes around the borders between the attention kernels (128, 256, 384, 512 keys)
    and up to the 1024 keys the reference's softmax launch covers (cuda/attention.cu:345-356): holes in the mask, empty
    sequences, attention masks unrelated to the input mask, both element types, against the oracle."""
    rng = np.random.RandomState(2000 + seed)
    dtype = ["fp16", "fp32"][seed % 2]
    B = int(rng.randint(1, 5))
    S = int(rng.choice([129, 255, 257, 300, 383, 384, 385, 511, 512, 513, 640, 777, 1000, 1024]))
    heads = int(rng.choice([1, 2, 3]))
    print("random long shape", seed, dtype, "B", B, "S", S, "heads", heads, flush=True)
    wl = o.Workload("rndlong", 2000 + seed, dtype, 1, B, S, heads, 64, 4 * heads * 64, 1, S + 1)
    if seed % 3 == 0:
        mask = (rng.rand(B, S) < 0.7).astype(np.int32)
        if B > 1:
            mask[rng.randint(0, B)] = 0                       # an empty sequence
        attr = (rng.rand(B, S, S) < 0.8).astype(np.float32)   # an attention mask unrelated to the input mask
    else:
        lens = rng.randint(1, S + 1, size=B)
        lens[0] = S                                           # one sequence of full length
        mask = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
        attr = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (B, S, S))).astype(np.float32)
    attr = o.rnd(attr, dtype)
    x = o.rnd(rng.randn(B, S, wl.H), dtype)
    weights = o.make_layer_weights(wl, rng, True)
    w = dict(wl=wl, lens=None, mask=mask, attr_mask=attr, x=x, weights=weights)
    got = run_encoder(w)
    if mask.sum() == 0:
        assert np.all(got == 0)
        return
    _check(got, _oracle(w), mask, dtype)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_cpp_host_gives_the_same_bits(tmp_path, dtype):
    """The C++ sample (csrc/encoder_example.cpp on include/et.hpp) against the Python mirror on the same problem."""
    import os
    import subprocess
    from effective_transformer_amd import build as b
    print("C++ host", dtype, flush=True)
    if not os.path.exists(b.EXAMPLE):
        pytest.fail("lib/et_encoder_example has not been built (python -m effective_transformer_amd.build)")
    w = o.make_workload("cfg1" if dtype == "fp32" else "cfg2", layers=2, random_affine=True)
    wl = w["wl"]
    npdt = np.float32 if dtype == "fp32" else np.float16
    prob, outp = str(tmp_path / "problem.bin"), str(tmp_path / "out.bin")
    with open(prob, "wb") as f:
        np.array([0 if dtype == "fp32" else 1, wl.B, wl.S, wl.heads, wl.d, 2], np.int32).tofile(f)
        w["mask"].astype(np.int32).tofile(f)
        w["x"].astype(npdt).tofile(f)
        w["attr_mask"].astype(npdt).tofile(f)
        for a in w["weights"][:32]:
            np.ascontiguousarray(a).astype(npdt).tofile(f)
    r = subprocess.run([b.EXAMPLE, prob, outp], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert "valid tokens %d of %d" % (int(w["mask"].sum()), wl.B * wl.S) in r.stdout
    got = np.fromfile(outp, dtype=npdt).reshape(wl.B, wl.S, wl.H)
    want = run_encoder(w, layers=2)
    assert np.array_equal(got, want)
