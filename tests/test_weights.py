"""Checkpoint import into the 16-slot layout (CPU only)."""
import numpy as np
import pytest

from effective_transformer_amd import weights as W
from oracle import et_oracle as o


def _layers(n=3):
    w = o.make_workload("cfg1", layers=1, random_affine=True, with_inputs=False)
    wl = w["wl"]
    rng = np.random.RandomState(5)
    out = []
    for _ in range(n):
        out.extend(o.make_layer_weights(wl, rng, True))
    return out


@pytest.mark.parametrize("ext", ["npz", "safetensors"])
def test_round_trip_tf_names(tmp_path, ext):
    ws = _layers(12)                       # 12 layers: layer_1 vs layer_10/layer_11 must not be confused
    path = str(tmp_path / ("enc." + ext))
    W.save_weights(path, ws)
    got = W.load_weights(path)
    assert len(got) == len(ws)
    for a, b in zip(got, ws):
        assert a.dtype == b.dtype and np.array_equal(a, b)
    assert W.count_layers(W.read_tensors(path)) == 12
    assert len(W.load_weights(path, num_layers=2)) == 32


def test_hugging_face_names_are_transposed(tmp_path):
    ws = _layers(2)
    named = {}
    for n, a in enumerate(ws):
        tf_tail, hf_tail, is_kernel = W.SLOTS[n % 16]
        named["bert.encoder.layer.%d.%s" % (n // 16, hf_tail)] = np.ascontiguousarray(a.T) if is_kernel else a
    path = str(tmp_path / "hf.npz")
    np.savez(path, **named)
    got = W.load_weights(path)
    for a, b in zip(got, ws):
        assert np.array_equal(a, b) and a.flags["C_CONTIGUOUS"]


def test_tf_variable_suffix_and_prefix(tmp_path):
    ws = _layers(1)
    named = {}
    for n, a in enumerate(ws):
        named["model_a/layer_0/%s:0" % W.SLOTS[n][0]] = a
        named["model_b/layer_0/%s:0" % W.SLOTS[n][0]] = a + 1
    with pytest.raises(ValueError, match="ambiguous"):
        W.weights_from_tensors(named)
    got = W.weights_from_tensors(named, prefix="model_b/")
    assert np.array_equal(got[3], ws[3] + 1)


def test_missing_tensor_and_bad_shapes():
    ws = _layers(1)
    named = {"layer_0/%s" % W.SLOTS[n][0]: a for n, a in enumerate(ws)}
    del named["layer_0/output/dense/bias"]
    with pytest.raises(KeyError, match="output/dense/bias"):
        W.weights_from_tensors(named)
    named = {"layer_0/%s" % W.SLOTS[n][0]: a for n, a in enumerate(ws)}
    named["layer_0/output/dense/kernel"] = named["layer_0/output/dense/kernel"].T
    with pytest.raises(ValueError, match="not an encoder layer"):
        W.weights_from_tensors(named)
    with pytest.raises(ValueError, match="unsupported"):
        W.read_tensors("weights.ckpt")


def test_slot_order_is_the_oracles_and_fused_qkv():
    ws = _layers(2)
    wl = o.WORKLOADS["cfg1"]
    H, F = wl.heads * wl.d, 4 * wl.heads * wl.d
    shapes = [(H, H), (H,), (H, H), (H,), (H, H), (H,), (H, H), (H,), (H,), (H,), (H, F), (F,), (F, H), (H,), (H,), (H,)]
    assert [a.shape for a in ws[:16]] == shapes
    k, b = W.fuse_qkv(ws, 1)
    x = np.random.RandomState(0).randn(5, H).astype(np.float32)
    want = np.concatenate([x @ ws[16] + ws[17], x @ ws[18] + ws[19], x @ ws[20] + ws[21]], axis=1)
    np.testing.assert_allclose(x @ k + b, want, rtol=1e-6, atol=1e-6)
