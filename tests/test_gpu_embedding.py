"""Embedding block fused with the input op (et_embedding_input) against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import et_oracle as o
from gpu_util import TDT, dev, assert_half_close

pytestmark = pytest.mark.gpu


def _tables(rng, V, Vt, P, H, dtype):
    word = o.rnd(rng.randn(V, H), dtype)
    typ = o.rnd(rng.randn(Vt, H), dtype)
    pos = o.rnd(rng.randn(P, H), dtype)
    gamma = o.rnd(1 + 0.1 * rng.randn(H), dtype)
    beta = o.rnd(0.1 * rng.randn(H), dtype)
    return word, typ, pos, gamma, beta


def _run(ids, tt, mask, word, typ, pos, gamma, beta, dtype, heads):
    from effective_transformer_amd import ops
    emb = ops.EmbeddingWeights("cuda", TDT[dtype], word, gamma, beta, token_type_embeddings=typ, position_embeddings=pos)
    r = ops.effective_transformer_embedding_input(dev(ids), None if tt is None else dev(tt), dev(mask), emb, heads,
                                                  word.shape[1] // heads, return_host_count=True)
    torch.cuda.synchronize()
    return [x.cpu().numpy() if isinstance(x, torch.Tensor) else x for x in r]


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("B,S,heads,holes", [(8, 32, 12, False), (5, 17, 2, True), (64, 128, 16, False), (1, 1, 1, False)])
def test_embedding_input_matches_oracle(dtype, B, S, heads, holes):
    print("embedding_input", dtype, B, S, heads, holes, flush=True)
    rng = np.random.RandomState(B * 131 + S)
    H = heads * 64
    V, Vt, P = 1000, 2, max(S, 130)
    word, typ, pos, gamma, beta = _tables(rng, V, Vt, P, H, dtype)
    ids = rng.randint(0, V, size=(B, S)).astype(np.int32)
    tt = rng.randint(0, Vt, size=(B, S)).astype(np.int32)
    if holes:
        mask = (rng.rand(B, S) < 0.6).astype(np.int32)
        ids[0, 0] = V + 3          # outside the vocabulary: zero word row
        ids[B - 1, S - 1] = -7
        mask[0, 0] = mask[B - 1, S - 1] = 1
    else:
        lens = rng.randint(1, S + 1, size=B)
        mask = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
    want, T, bi, wi, _ = o.embedding_input(ids, tt, mask, word, typ, pos, gamma, beta, dtype)
    to, vwn, gbi, gwi, gT = _run(ids, tt, mask, word, typ, pos, gamma, beta, dtype, heads)
    assert gT == T and int(vwn[0]) == T
    assert np.array_equal(gbi.reshape(-1)[:T], bi) and np.array_equal(gwi.reshape(-1)[:T], wi)
    got = to.reshape(B * S, H)[:T]
    if dtype == "fp32":
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    else:
        assert_half_close(got, want, ulps=1, atol=1e-6, frac=0.02, what="embedding")


def test_embedding_input_equals_padded_embedding_then_input_op():
    """Same packed rows as LayerNorm on the padded tensor followed by et_input (the reference's order)."""
    from effective_transformer_amd import ops
    print("embedding_input vs et_input", flush=True)
    rng = np.random.RandomState(3)
    B, S, heads, dtype = 16, 64, 12, "fp16"
    H = heads * 64
    word, typ, pos, gamma, beta = _tables(rng, 500, 2, 64, H, dtype)
    ids = rng.randint(0, 500, size=(B, S)).astype(np.int32)
    tt = rng.randint(0, 2, size=(B, S)).astype(np.int32)
    lens = rng.randint(16, S + 1, size=B)
    mask = (np.arange(S)[None, :] < lens[:, None]).astype(np.int32)
    to, vwn, gbi, gwi, T = _run(ids, tt, mask, word, typ, pos, gamma, beta, dtype, heads)
    # all-valid mask gives the padded block itself; compress it with the real mask
    full = np.ones_like(mask)
    padded = _run(ids, tt, full, word, typ, pos, gamma, beta, dtype, heads)[0]
    to2, vwn2, bi2, wi2 = ops.effective_transformer_input(dev(padded), dev(mask), B, S, S, heads, 64)
    torch.cuda.synchronize()
    assert int(vwn2.cpu()[0]) == T
    assert np.array_equal(to2.cpu().numpy().reshape(B * S, H)[:T], to.reshape(B * S, H)[:T])


def test_embedding_input_without_optional_tables_and_errors():
    from effective_transformer_amd import ops, _lib
    print("embedding_input optional tables", flush=True)
    rng = np.random.RandomState(9)
    B, S, heads = 4, 16, 2
    H = heads * 64
    word, typ, pos, gamma, beta = _tables(rng, 50, 2, 16, H, "fp32")
    ids = rng.randint(0, 50, size=(B, S)).astype(np.int32)
    mask = np.ones((B, S), np.int32)
    emb = ops.EmbeddingWeights("cuda", torch.float32, word, gamma, beta)
    to = ops.effective_transformer_embedding_input(dev(ids), None, dev(mask), emb, heads, 64)[0].cpu().numpy()
    want = o.embedding_postprocess(ids, None, word, None, None, gamma, beta, "fp32")
    np.testing.assert_allclose(to, want, rtol=1e-4, atol=1e-5)
    # type ids without a type table, and a sequence longer than the position table
    with pytest.raises(_lib.EtError, match="go together"):
        ops.effective_transformer_embedding_input(dev(ids), dev(ids), dev(mask), emb, heads, 64)
    emb2 = ops.EmbeddingWeights("cuda", torch.float32, word, gamma, beta, position_embeddings=pos[:8])
    with pytest.raises(_lib.EtError, match="max_position_embeddings"):
        ops.effective_transformer_embedding_input(dev(ids), None, dev(mask), emb2, heads, 64)


def test_encoder_from_ids_matches_encoder_on_padded_embeddings():
    from effective_transformer_amd import ops
    print("encoder forward_ids", flush=True)
    w = o.make_workload("cfg2", layers=2)
    wl = w["wl"]
    rng = np.random.RandomState(21)
    H = wl.heads * wl.d
    word, typ, pos, gamma, beta = _tables(rng, 300, 2, wl.S, H, "fp16")
    ids = rng.randint(0, 300, size=(wl.B, wl.S)).astype(np.int32)
    tt = rng.randint(0, 2, size=(wl.B, wl.S)).astype(np.int32)
    mask = w["mask"].astype(np.int32)
    emb = ops.EmbeddingWeights("cuda", torch.float16, word, gamma, beta, token_type_embeddings=typ, position_embeddings=pos)
    enc = ops.EffectiveTransformerEncoder(2, wl.heads, wl.d, w["weights"][:32], torch.float16)
    attr = dev(w["attr_mask"], torch.float16)
    got = enc.forward_ids(dev(ids), dev(tt), dev(mask), attr, emb)
    padded = o.embedding_postprocess(ids, tt, word, typ, pos, gamma, beta, "fp16")
    want = enc(dev(padded), dev(mask), attr)
    torch.cuda.synchronize()
    # the fused path rounds like the oracle up to the LayerNorm's last ulp; after two layers the outputs agree closely
    np.testing.assert_allclose(got.float().cpu().numpy(), want.float().cpu().numpy(), rtol=0, atol=2e-2)


@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
@pytest.mark.parametrize("case", ["prefix", "holes", "empty_sequences", "all_empty"])
def test_first_token_equals_restore_then_slice(dtype, case):
    from effective_transformer_amd import ops
    print("first_token", dtype, case, flush=True)
    rng = np.random.RandomState(17)
    B, S, H = 37, 24, 128
    x = o.rnd(rng.randn(B, S, H), dtype)
    if case == "prefix":
        mask = (np.arange(S)[None, :] < rng.randint(1, S + 1, size=B)[:, None]).astype(np.int32)
    elif case == "holes":
        mask = (rng.rand(B, S) < 0.5).astype(np.int32)
    elif case == "empty_sequences":
        mask = (np.arange(S)[None, :] < rng.randint(1, S + 1, size=B)[:, None]).astype(np.int32)
        mask[[0, 5, 6, 7, B - 1]] = 0
    else:
        mask = np.zeros((B, S), np.int32)
    to, vwn, bi, wi = ops.effective_transformer_input(dev(x), dev(mask), B, S, S, H // 64, 64)
    got = ops.effective_transformer_first_token(to, vwn, bi, wi).cpu().numpy()
    packed, T, obi, owi, _ = o.input_op_fast(x, mask)
    want = o.restore(packed, T, obi, owi, B, S)[:, 0, :]
    assert np.array_equal(got, want)
