"""torch.library registration of the three ops: schemas and fake kernels on the CPU, the real kernels on the GPU."""
import numpy as np
import pytest
import torch

from effective_transformer_amd import torch_ops


def _meta_inputs(B=3, S=16, heads=2, d=64, dtype=torch.float16):
    H = heads * d
    x = torch.empty(B, S, H, device="meta", dtype=dtype)
    mask = torch.empty(B, S, device="meta", dtype=torch.int32)
    attr = torch.empty(B, S, S, device="meta", dtype=dtype)
    w = [torch.empty(1, device="meta", dtype=dtype) for _ in range(16)]
    return x, mask, attr, w


def test_ops_are_registered_with_fake_kernels():
    x, mask, attr, w = _meta_inputs()
    to, vwn, bidx, widx = torch.ops.effective_transformer.input(x, mask, 2, 64)
    assert to.shape == x.shape and to.dtype == x.dtype
    assert vwn.shape == (1,) and vwn.dtype == torch.int32
    assert bidx.shape == mask.shape and widx.shape == mask.shape and bidx.dtype == torch.int32
    y = torch.ops.effective_transformer.layer(to, to, attr, vwn, bidx, widx, w, 2, 64)
    assert y.shape == x.shape and y.dtype == x.dtype
    z = torch.ops.effective_transformer.output(y, vwn, bidx, widx, 2, 64)
    assert z.shape == x.shape
    out = torch_ops.encoder(x, mask, attr, [w, w, w], 2, 64)
    assert out.shape == x.shape and out.device.type == "meta"


def test_layer_needs_16_weights():
    x, mask, attr, w = _meta_inputs()
    to, vwn, bidx, widx = torch.ops.effective_transformer.input(x, mask, 2, 64)
    with pytest.raises(Exception, match="16 weight"):
        torch.ops.effective_transformer.layer(to, to, attr, vwn, bidx, widx, w[:15], 2, 64)


def test_schemas():
    s = str(torch.ops.effective_transformer.layer.default._schema)
    assert "Tensor[] weights" in s and "head_num" in s and "size_per_head" in s
    s = str(torch.ops.effective_transformer.input.default._schema)
    assert s.count("Tensor") >= 6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp32", "fp16"])
def test_custom_ops_equal_the_encoder(dtype):
    from oracle import et_oracle as o
    from effective_transformer_amd import EffectiveTransformerEncoder
    print("torch custom ops", dtype, flush=True)
    w = o.make_workload("cfg1" if dtype == "fp32" else "cfg2", layers=2, random_affine=True)
    wl = w["wl"]
    tdt = torch.float32 if dtype == "fp32" else torch.float16
    x = torch.from_numpy(np.ascontiguousarray(w["x"])).cuda().to(tdt)
    mask = torch.from_numpy(w["mask"].astype(np.int32)).cuda()
    attr = torch.from_numpy(np.ascontiguousarray(w["attr_mask"])).cuda().to(tdt)
    enc = EffectiveTransformerEncoder(2, wl.heads, wl.d, w["weights"][:32], tdt)
    want = enc(x, mask, attr)
    lw = [[torch.from_numpy(np.ascontiguousarray(a)).cuda().to(tdt).contiguous() for a in w["weights"][16 * l:16 * l + 16]]
          for l in range(2)]
    got = torch_ops.encoder(x, mask, attr, lw, wl.heads, wl.d)
    assert torch.equal(got, want)
    # traceable: one graph, no breaks, same result
    fn = torch.compile(torch_ops.encoder, backend="aot_eager", fullgraph=True)
    got2 = fn(x, mask, attr, lw, wl.heads, wl.d)
    assert torch.equal(got2, want)


@pytest.mark.gpu
def test_encoder_from_checkpoint_file(tmp_path):
    from oracle import et_oracle as o
    from effective_transformer_amd import EffectiveTransformerEncoder, weights as W
    print("encoder from checkpoint", flush=True)
    w = o.make_workload("cfg1", layers=2, random_affine=True)
    wl = w["wl"]
    path = str(tmp_path / "enc.safetensors")
    W.save_weights(path, w["weights"][:32])
    x = torch.from_numpy(np.ascontiguousarray(w["x"])).cuda()
    mask = torch.from_numpy(w["mask"].astype(np.int32)).cuda()
    attr = torch.from_numpy(np.ascontiguousarray(w["attr_mask"])).cuda()
    a = EffectiveTransformerEncoder(2, wl.heads, wl.d, w["weights"][:32], torch.float32)(x, mask, attr)
    b = EffectiveTransformerEncoder.from_checkpoint(path, wl.heads, wl.d, torch.float32)(x, mask, attr)
    assert torch.equal(a, b)
