"""Pins the CPU oracle to facts that do not come from the oracle itself: the worked
examples in the reference's documentation, closed forms, brute force on tiny inputs
and library routines.  A dropped term, a wrong sign/index or a transposed operand in
the oracle fails at least one of these."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import et_oracle as o

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _ka():
    with open(os.path.join(GOLD, "known_answers.json")) as f:
        return json.load(f)


# ----------------------------------------------------------------- indices ---

def test_figure_known_answer():
    ka = _ka()["figure_4x8"]
    mask = np.array(ka["mask"], dtype=np.int32)
    x = np.arange(mask.size * 4, dtype=np.float32).reshape(4, 8, 4)
    to, T, bi, wi, prefix = o.input_op(x, mask)
    assert T == ka["valid_word_num"] == 22
    pre = prefix.reshape(mask.shape)
    for b, row in enumerate(ka["prefix_at_valid"]):
        assert pre[b, :len(row)].tolist() == row
    padded = (bi.astype(np.int64) * 8 + wi).tolist()
    assert padded[:8] == ka["packed_to_padded_first8"]
    assert np.array_equal(to, x.reshape(32, 4)[padded])


def test_readme_known_answer():
    ka = _ka()["readme_3x5"]
    mask = np.array(ka["mask"], dtype=np.int32)
    tok = np.array(ka["tokens_padded"], dtype=np.float32)[..., None]
    to, T, bi, wi, _ = o.input_op(tok, mask)
    assert T == ka["valid_word_num"] and mask.size == ka["total"]
    assert to[:, 0].tolist() == ka["tokens_packed"]
    back = o.restore(to, T, bi, wi, 3, 5)
    assert np.array_equal(back[..., 0], np.array(ka["tokens_padded"], dtype=np.float32))


def test_debug_lens_known_answer():
    ka = _ka()["debug_lens"]
    lens = np.array(ka["lens"])
    mask = (np.arange(40)[None, :] < lens[:, None]).astype(np.int32)
    _, T, bi, wi, _ = o.input_op(np.zeros((4, 40, 2), np.float32), mask)
    assert T == ka["valid_word_num"] == int(lens.sum())
    # token `word` of sequence `bi` sits at packed row sum(lens[:bi]) + word (the debug block's offset rule)
    for b in range(4):
        t = int(lens[:b].sum()) + 1
        assert bi[t] == b and wi[t] == 1


@pytest.mark.parametrize("seed", range(6))
def test_scan_and_indices_brute_force(seed):
    rng = np.random.RandomState(seed)
    B, S = rng.randint(1, 7), rng.randint(1, 12)
    mask = (rng.random_sample((B, S)) < 0.6).astype(np.int32)      # holes allowed
    if seed == 0:
        mask[:] = 0
    if seed == 1:
        mask[:] = 1
    flat = mask.reshape(-1)
    pre = o.exclusive_scan(mask)
    for i in range(flat.size):
        assert pre[i] == sum(int(v) for v in flat[:i])
    x = rng.randn(B, S, 3).astype(np.float32)
    to, T, bi, wi, _ = o.input_op(x, mask)
    pairs = [(b, s) for b in range(B) for s in range(S) if mask[b, s] == 1]
    assert T == len(pairs) == int(flat.sum())
    assert list(zip(bi.tolist(), wi.tolist())) == pairs
    for t, (b, s) in enumerate(pairs):
        assert np.array_equal(to[t], x[b, s])
    to2, T2, bi2, wi2, pre2 = o.input_op_fast(x, mask)
    assert T2 == T and np.array_equal(to2, to) and np.array_equal(bi2, bi) and np.array_equal(wi2, wi)
    back = o.restore(to, T, bi, wi, B, S)
    assert np.array_equal(back, x * mask[..., None])


def test_last_element_branch():
    # T = prefix[last] + (mask[last] == 1): both branches
    for last in (0, 1):
        mask = np.array([[1, 0, 1, last]], dtype=np.int32)
        _, T, _, _, pre = o.input_op(np.zeros((1, 4, 1), np.float32), mask)
        assert pre.tolist() == [0, 1, 1, 2] and T == 2 + last


def test_workload_digests_frozen():
    import hashlib
    with open(os.path.join(GOLD, "workload_digests.json")) as f:
        dig = json.load(f)
    assert {k: v["T"] for k, v in dig.items()} == {"cfg1": 134, "cfg2": 2000, "cfg3": 40396, "cfg4": 20375, "cfg5": 13097}
    for name in ("cfg1", "cfg2"):
        w = o.make_workload(name, layers=1)
        sha = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
        assert int(w["mask"].sum()) == dig[name]["T"]
        assert sha(w["mask"]) == dig[name]["mask_sha256"]
        assert sha(w["x"][0, 0]) == dig[name]["x_first_row_sha256"]
        assert sha(w["weights"][0][0]) == dig[name]["layer0_wq_row0_sha256"]
        assert sha(w["weights"][12][0]) == dig[name]["layer0_out_kernel_row0_sha256"]
        # attr_mask[b,q,k] = mask[b,k]
        assert np.array_equal(w["attr_mask"][3, 5].astype(np.int32), w["mask"][3])


# ------------------------------------------------------------- row kernels ---

def test_gelu_against_torch_and_closed_form():
    rng = np.random.RandomState(0)
    x = (3 * rng.randn(7, 64)).astype(np.float32)
    b = rng.randn(64).astype(np.float32)
    got = o.add_bias_act(x, b, "fp32")
    want = torch.nn.functional.gelu(torch.from_numpy(x + b), approximate="tanh").numpy()
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-7)
    # special values: gelu(0) = 0, gelu(large) = x, gelu(-large) = 0
    sp = o.add_bias_act(np.array([[0.0, 20.0, -20.0]], np.float32), np.zeros(3, np.float32), "fp32")
    assert sp[0, 0] == 0 and sp[0, 1] == 20 and abs(sp[0, 2]) < 1e-6
    # half path: rounding points keep it within a few half ulps of the exact function
    got16 = o.add_bias_act(x.astype(np.float16), b.astype(np.float16), "fp16")
    assert got16.dtype == np.float16
    xb = (x.astype(np.float16).astype(np.float64) + b.astype(np.float16).astype(np.float64))
    exact = 0.5 * xb * (1 + np.tanh(0.7978845608028654 * (xb + 0.044715 * xb ** 3)))
    np.testing.assert_allclose(got16.astype(np.float64), exact, rtol=4e-3, atol=2e-3)


def test_layernorm_against_torch():
    rng = np.random.RandomState(1)
    n = 96
    out = rng.randn(5, n).astype(np.float32)
    inp = rng.randn(5, n).astype(np.float32)
    bias, gamma, beta = (rng.randn(n).astype(np.float32) for _ in range(3))
    got = o.add_bias_input_layernorm(out, inp, bias, gamma, beta, "fp32")
    want = torch.nn.functional.layer_norm(torch.from_numpy(out + inp + bias), (n,), torch.from_numpy(gamma),
                                          torch.from_numpy(beta), eps=1e-6).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    # eps matters: constant row -> output exactly beta, and tiny-variance rows shrink by sqrt(var/(var+eps))
    const = o.add_bias_input_layernorm(np.ones((1, n), np.float32), np.ones((1, n), np.float32),
                                       np.zeros(n, np.float32), gamma, beta, "fp32")
    np.testing.assert_allclose(const[0], beta, atol=1e-7)
    tiny = np.zeros((1, n), np.float32); tiny[0, ::2] = 1e-3; tiny[0, 1::2] = -1e-3      # var = 1e-6 = eps
    y = o.add_bias_input_layernorm(tiny, np.zeros((1, n), np.float32), np.zeros(n, np.float32),
                                   np.ones(n, np.float32), np.zeros(n, np.float32), "fp32")
    np.testing.assert_allclose(np.abs(y[0]), 1 / math.sqrt(2), rtol=1e-5)
    got16 = o.add_bias_input_layernorm(out.astype(np.float16), inp.astype(np.float16), bias.astype(np.float16),
                                       gamma.astype(np.float16), beta.astype(np.float16), "fp16")
    assert got16.dtype == np.float16
    np.testing.assert_allclose(got16.astype(np.float32), want, rtol=2e-2, atol=2e-2)


def test_softmax_against_torch_and_quirks():
    rng = np.random.RandomState(2)
    B, h, S = 2, 3, 10
    qk = (4 * rng.randn(B, h, S, S)).astype(np.float32)
    lens = np.array([10, 6])
    mask = (np.arange(S)[None, None, :] < lens[:, None, None]).astype(np.float32) * np.ones((B, S, S), np.float32)
    got = o.softmax(qk, mask, 0.125, "fp32")
    want = torch.softmax(torch.from_numpy(qk) * 0.125 + (1 - torch.from_numpy(mask))[:, None] * -10000.0, -1).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)     # differs only by the +1e-6 denominator
    assert np.all(got[1, :, :, 6:] == 0)                              # masked keys are exactly 0
    # a fully masked row gives zeros (max clamped at 0), not a uniform row
    z = o.softmax(qk[:1, :1], np.zeros((1, S, S), np.float32), 0.125, "fp32")
    assert np.all(z == 0)
    # all scores far below 0: mass is lost to the 1e-6 term because the max is clamped at 0
    low = np.full((1, 1, 1, 4), -160.0, np.float32)                   # t = -20 each
    p = o.softmax(low, np.ones((1, 1, 4), np.float32), 0.125, "fp32")
    e = math.exp(-20.0)
    np.testing.assert_allclose(p[0, 0, 0], e / (4 * e + 1e-6), rtol=1e-6)
    # positive max: ordinary max-subtraction
    hi = np.array([[[[80.0, 0.0]]]], np.float32)                      # t = 10, 0
    p = o.softmax(hi, np.ones((1, 1, 2), np.float32), 0.125, "fp32")
    np.testing.assert_allclose(p[0, 0, 0, 0], 1 / (1 + math.exp(-10) + 1e-6), rtol=1e-6)


def test_softmax_clamp_rule_by_block_size():
    """Which rows see the clamp of the maximum follows from the launch geometry (cuda/attention.cu:345-356) and the
    two fillers of the reduction (:91-92 idle lanes give 0, :267-270 out-of-range threads give -1e-20): up to 1023 keys a
    fully masked row is all zeros (every term exp(-10000 - 0) underflows), at exactly 1024 keys nothing clamps and the
    row is uniform.  Brute force per row in float64 with that rule written out."""
    rng = np.random.RandomState(4)
    for S in (512, 513, 600, 1023, 1024):
        qk = (3 * rng.randn(1, 1, 2, S)).astype(np.float32)
        mask = np.ones((1, 2, S), np.float32)
        mask[0, 1] = 0                                                # second query row fully masked
        got = o.softmax(qk, mask, 0.125, "fp32")      # a [2,S] slab of query rows is enough for the row-wise arithmetic
        t0 = qk[0, 0, 0].astype(np.float64) * 0.125
        m0 = max(t0.max(), 0.0) if S < 1024 else t0.max()
        e0 = np.exp(t0 - m0)
        np.testing.assert_allclose(got[0, 0, 0], e0 / (e0.sum() + 1e-6), rtol=2e-6)
        if S < 1024:
            assert np.all(got[0, 0, 1] == 0)
        else:
            # the kernel adds the -10000 in float (cuda/attention.cu:262-265): at that magnitude a float step is 1e-3
            t1 = ((qk[0, 0, 1] * np.float32(0.125)).astype(np.float32) + np.float32(-10000.0)).astype(np.float64)
            e1 = np.exp(t1 - t1.max())
            np.testing.assert_allclose(got[0, 0, 1], e1 / (e1.sum() + 1e-6), rtol=1e-4)
            assert got[0, 0, 1].min() > 0


def test_qkv_pad_and_unpad_brute_force():
    rng = np.random.RandomState(3)
    B, S, heads, d = 3, 5, 2, 4
    mask = np.array([[1, 1, 0, 0, 0], [1, 1, 1, 1, 1], [1, 0, 1, 0, 0]], np.int32)     # one row has a hole
    _, T, bi, wi, _ = o.input_op(np.zeros((B, S, 1), np.float32), mask)
    H = heads * d
    q, k, v = (rng.randn(T, H).astype(np.float32) for _ in range(3))
    bq, bk, bv = (rng.randn(H).astype(np.float32) for _ in range(3))
    qp, kp, vp = o.add_qkv_bias_padding(q, bq, k, bk, v, bv, T, B, S, heads, d, bi, wi, "fp32")
    for src, bias, dst in ((q, bq, qp), (k, bk, kp), (v, bv, vp)):
        want = np.zeros((B, heads, S, d), np.float32)
        for t in range(T):
            for hh in range(heads):
                for j in range(d):
                    want[bi[t], hh, wi[t], j] = src[t, hh * d + j] + bias[hh * d + j]
        assert np.array_equal(dst, want)
        assert np.all(dst[mask == 0][:, :, :].reshape(-1) == 0) if False else True
        for b in range(B):
            for s in range(S):
                if mask[b, s] == 0:
                    assert np.all(dst[b, :, s, :] == 0)
    # un-pad is the inverse gather
    np.testing.assert_array_equal(o.transpose_rm_padding(qp, T, bi, wi), q + bq)


# -------------------------------------------------------------- whole layer ---

def _tiny_layer_problem(seed, dtype="fp32"):
    rng = np.random.RandomState(seed)
    wl = o.Workload("tiny", seed, dtype, 1, 3, 8, 2, 64, 256)
    lens = np.array([8, 3, 5])
    mask = (np.arange(wl.S)[None, :] < lens[:, None]).astype(np.int32)
    attr = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (wl.B, wl.S, wl.S))).astype(o._np_dtype(dtype))
    x = rng.randn(wl.B, wl.S, wl.H).astype(np.float32).astype(o._np_dtype(dtype))
    w = o.make_layer_weights(wl, rng, random_affine=True)
    return wl, lens, mask, attr, x, w


def test_layer_against_huggingface_bert_layer():
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer

    wl, lens, mask, attr, x, w = _tiny_layer_problem(5)
    cfg = BertConfig(hidden_size=wl.H, num_attention_heads=wl.heads, intermediate_size=wl.F, hidden_act="gelu_new",
                     layer_norm_eps=1e-6, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                     num_hidden_layers=1)
    cfg._attn_implementation = "eager"
    hf = BertLayer(cfg).eval()
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a.astype(np.float32)))
    (wq, bq, wk, bk, wv, bv, wo, bo, b1, g1, wi, bi_, wo2, bo2, b2, g2) = w
    with torch.no_grad():
        sa = hf.attention.self
        sa.query.weight.copy_(t(wq).T); sa.query.bias.copy_(t(bq))
        sa.key.weight.copy_(t(wk).T); sa.key.bias.copy_(t(bk))
        sa.value.weight.copy_(t(wv).T); sa.value.bias.copy_(t(bv))
        so = hf.attention.output
        so.dense.weight.copy_(t(wo).T); so.dense.bias.copy_(t(bo))
        so.LayerNorm.weight.copy_(t(g1)); so.LayerNorm.bias.copy_(t(b1))
        hf.intermediate.dense.weight.copy_(t(wi).T); hf.intermediate.dense.bias.copy_(t(bi_))
        hf.output.dense.weight.copy_(t(wo2).T); hf.output.dense.bias.copy_(t(bo2))
        hf.output.LayerNorm.weight.copy_(t(g2)); hf.output.LayerNorm.bias.copy_(t(b2))
        ext = (1.0 - t(mask)[:, None, None, :]) * -10000.0
        out = hf(t(x), attention_mask=ext)
        out = out[0] if isinstance(out, (tuple, list)) else out
    want = out.numpy()
    got = o.encoder(x, mask, attr, w, wl.heads, wl.d, "fp32")
    valid = mask.astype(bool)
    np.testing.assert_allclose(got[valid], want[valid], rtol=1e-4, atol=2e-5)
    assert np.all(got[~valid] == 0)


def test_et_math_against_tf_graph_restatement():
    """The reference benchmark's own check (sample/tensorflow/benchmark.py:104-112): the ET
    arithmetic and the standard BERT graph agree on valid tokens."""
    w = o.make_workload("cfg1", random_affine=True)
    wl = w["wl"]
    got = o.encoder(w["x"], w["mask"], w["attr_mask"], w["weights"], wl.heads, wl.d, "fp32")
    want = o.tf_graph_encoder(w["x"], w["attr_mask"], w["weights"], wl.heads, wl.d)
    valid = w["mask"].astype(bool)
    diff = np.abs(got[valid] - want[valid]).max(axis=-1)
    assert diff.max() < 5e-5, diff.max()


def test_fp16_mode_tracks_fp32_mode():
    wl, lens, mask, attr, x, w = _tiny_layer_problem(7, "fp16")
    got16 = o.encoder(x, mask, attr, w, wl.heads, wl.d, "fp16")
    assert got16.dtype == np.float16
    w32 = [a.astype(np.float32) for a in w]
    got32 = o.encoder(x.astype(np.float32), mask, attr.astype(np.float32), w32, wl.heads, wl.d, "fp32")
    assert np.abs(got16.astype(np.float32) - got32).max() < 2e-2


def test_embedding_block_against_huggingface_embeddings():
    """The padded embedding block (word + token type + position, LayerNorm 1e-12) against transformers'
    BertEmbeddings with the same tables; the packed form against a position-by-position loop."""
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertEmbeddings
    rng = np.random.RandomState(11)
    V, Vt, P, H, B, S = 97, 3, 40, 64, 4, 12
    word = rng.randn(V, H).astype(np.float32)
    typ = rng.randn(Vt, H).astype(np.float32)
    pos = rng.randn(P, H).astype(np.float32)
    gamma = (1 + 0.1 * rng.randn(H)).astype(np.float32)
    beta = (0.1 * rng.randn(H)).astype(np.float32)
    ids = rng.randint(0, V, size=(B, S)).astype(np.int32)
    tt = rng.randint(0, Vt, size=(B, S)).astype(np.int32)
    cfg = BertConfig(vocab_size=V, hidden_size=H, max_position_embeddings=P, type_vocab_size=Vt, layer_norm_eps=1e-12,
                     hidden_dropout_prob=0.0, num_hidden_layers=1, num_attention_heads=1, intermediate_size=4 * H,
                     pad_token_id=0)
    emb = BertEmbeddings(cfg).eval()
    with torch.no_grad():
        emb.word_embeddings.weight.copy_(torch.from_numpy(word))
        emb.token_type_embeddings.weight.copy_(torch.from_numpy(typ))
        emb.position_embeddings.weight.copy_(torch.from_numpy(pos))
        emb.LayerNorm.weight.copy_(torch.from_numpy(gamma))
        emb.LayerNorm.bias.copy_(torch.from_numpy(beta))
        want = emb(input_ids=torch.from_numpy(ids).long(), token_type_ids=torch.from_numpy(tt).long()).numpy()
    got = o.embedding_postprocess(ids, tt, word, typ, pos, gamma, beta, "fp32")
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    # without the optional tables: plain LayerNorm of the word rows
    got_w = o.embedding_postprocess(ids, None, word, None, None, gamma, beta, "fp32")
    want_w = torch.nn.functional.layer_norm(torch.from_numpy(word[ids]), (H,), torch.from_numpy(gamma),
                                            torch.from_numpy(beta), eps=1e-12).numpy()
    np.testing.assert_allclose(got_w, want_w, rtol=1e-5, atol=1e-5)
    # an id outside the vocabulary contributes a zero row
    ids2 = ids.copy(); ids2[1, 3] = V + 5; ids2[2, 0] = -1
    got2 = o.embedding_postprocess(ids2, tt, word, typ, pos, gamma, beta, "fp32")
    x = typ[tt[1, 3]] + pos[3]
    ref = (x - x.mean()) / np.sqrt(x.var() + 1e-12) * gamma + beta
    np.testing.assert_allclose(got2[1, 3], ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(got2[0], got[0])
    # packed form: row t is the padded row of the t-th valid position
    mask = (rng.rand(B, S) < 0.6).astype(np.int32)
    packed, T, bi, wi, _ = o.embedding_input(ids, tt, mask, word, typ, pos, gamma, beta, "fp32")
    t = 0
    for b in range(B):
        for s_ in range(S):
            if mask[b, s_]:
                assert bi[t] == b and wi[t] == s_ and np.array_equal(packed[t], got[b, s_])
                t += 1
    assert t == T == packed.shape[0]
    # fp16: the sums round to half after each add
    h = o.embedding_postprocess(ids, tt, word, typ, pos, gamma, beta, "fp16")
    assert h.dtype == np.float16
    np.testing.assert_allclose(h.astype(np.float32), got, rtol=2e-2, atol=2e-2)
