"""Bert performance measuring sample -- the counterpart of the reference's
sample/tensorflow/benchmark.py (same flags, same input recipe, same printed lines).

    python -m effective_transformer_amd.sample.benchmark -p fp16 -b 1000 -m 64 -a 40

The "standard" model it is compared with is the padded BERT encoder (the graph of the reference's
modeling.transformer_model, sample/tensorflow/modeling.py:755-893) written with plain torch ops on the same GPU;
it plays the role TF-XLA plays in the reference's benchmark: parity on valid tokens and a timing to compare with.
"""
import argparse
import json
import math
import os
from datetime import datetime
from types import SimpleNamespace

import numpy as np
import torch

from .. import ops


def standard_transformer(x, attention_mask, weights, num_layers, heads, size_per_head):
    """Padded [B*S,H] encoder: dense Q/K/V, scores/sqrt(d) + (1-mask)*-10000, softmax, dense + residual +
    LayerNorm, dense + tanh-GELU, dense + residual + LayerNorm (modeling.py:558-893).  eps 1e-12."""
    B, S, H = x.shape
    h = x.reshape(B * S, H)
    adder = ((1.0 - attention_mask.float()) * -10000.0).to(x.dtype)[:, None]
    scale = 1.0 / math.sqrt(float(size_per_head))
    for l in range(num_layers):
        (wq, bq, wk, bk, wv, bv, wo, bo, b1, g1, wi, bi, wo2, bo2, b2, g2) = weights[16 * l:16 * l + 16]
        q = (h @ wq + bq).reshape(B, S, heads, size_per_head).permute(0, 2, 1, 3)
        k = (h @ wk + bk).reshape(B, S, heads, size_per_head).permute(0, 2, 1, 3)
        v = (h @ wv + bv).reshape(B, S, heads, size_per_head).permute(0, 2, 1, 3)
        p = torch.softmax(torch.matmul(q, k.transpose(-1, -2)) * scale + adder, dim=-1)
        ctx = torch.matmul(p, v).permute(0, 2, 1, 3).reshape(B * S, H)
        y1 = torch.nn.functional.layer_norm(ctx @ wo + bo + h, (H,), g1, b1, eps=1e-12)
        u = y1 @ wi + bi
        inter = u * 0.5 * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * u * u * u)))
        h = torch.nn.functional.layer_norm(inter @ wo2 + bo2 + y1, (H,), g2, b2, eps=1e-12)
    return h.reshape(B, S, H)


def make_weights(cfg, dtype, device, rng):
    """16 tensors per layer in the order of the reference's `weights_value`
    (python/effective_transformer/__init__.py:55-74): kernels N(0, initializer_range), biases 0, beta 0, gamma 1."""
    H, F = cfg.hidden_size, cfg.intermediate_size
    out = []

    def kern(i, o):
        return torch.from_numpy((cfg.initializer_range * rng.randn(i, o)).astype(np.float32)).to(device=device, dtype=dtype)

    def vec(n, v):
        return torch.full((n,), v, device=device, dtype=dtype)

    for _ in range(cfg.num_hidden_layers):
        for _ in range(3):
            out += [kern(H, H), vec(H, 0.0)]
        out += [kern(H, H), vec(H, 0.0), vec(H, 0.0), vec(H, 1.0)]
        out += [kern(H, F), vec(F, 0.0), kern(F, H), vec(H, 0.0), vec(H, 0.0), vec(H, 1.0)]
    return out


def main(args):
    with open(args.config) as f:
        cfg = SimpleNamespace(**json.load(f))
    batch_size, avg_seq_len, max_seq_len = args.batch_size, args.avg_seq_length, args.max_seq_length
    dtype = torch.float16 if args.precision == "fp16" else torch.float32
    dev = torch.device("cuda", 0)
    rng = np.random.RandomState(args.seed)

    # fake input array length (benchmark.py:38-41)
    input_len = rng.randint(low=2 * avg_seq_len - max_seq_len, high=max_seq_len + 1, size=batch_size).astype(np.int32)
    input_mask = (np.arange(max_seq_len)[None, :] < input_len[:, None]).astype(np.int32)
    embed_output = rng.randn(batch_size, max_seq_len, cfg.hidden_size).astype(np.float32)
    att_mask = np.tile(input_mask, max_seq_len).reshape(batch_size, max_seq_len, max_seq_len)   # benchmark.py:59-61
    valid_word_num = int(input_len.sum())
    print("Valid word num : {}/{}, avg sequence length : {:.6} ".format(
        valid_word_num, batch_size * max_seq_len, valid_word_num / batch_size))

    x = torch.from_numpy(embed_output).to(device=dev, dtype=dtype)
    mask = torch.from_numpy(input_mask).to(dev)
    attention_mask = torch.from_numpy(att_mask).to(device=dev, dtype=dtype)
    weights = make_weights(cfg, dtype, dev, rng)
    heads = cfg.num_attention_heads
    size_per_head = cfg.hidden_size // heads

    std = lambda: standard_transformer(x, attention_mask, weights, cfg.num_hidden_layers, heads, size_per_head)
    enc = ops.EffectiveTransformerEncoder(cfg.num_hidden_layers, heads, size_per_head, weights, dtype, dev)
    et = lambda: enc(x, mask, attention_mask)

    with torch.no_grad():
        val1 = std().float().cpu().numpy().reshape(-1, cfg.hidden_size)
        val2 = et().float().cpu().numpy().reshape(-1, cfg.hidden_size)
        diff = []
        for b_idx, s_len in enumerate(input_len):
            rows = slice(b_idx * max_seq_len, b_idx * max_seq_len + int(s_len))
            diff.append(np.fabs(val1[rows] - val2[rows]).max(axis=1))
        diff = np.concatenate(diff)
        print("max diff : {:.6}, avg diff : {:.6}.".format(float(diff.max()), float(diff.mean())))

        def time_inference(fn):
            iter_num = getattr(args, "iters", 128)            # benchmark.py:114-124: 10 warm-ups, 128 timed runs
            for _ in range(getattr(args, "warmup", 10)):
                fn()
            torch.cuda.synchronize()
            beg = datetime.now()
            for _ in range(iter_num):
                fn()
            torch.cuda.synchronize()
            return (datetime.now() - beg).total_seconds() * 1000 / iter_num

        print("std cost : {:.6} ms".format(time_inference(std)))
        print("et  cost : {:.6} ms".format(time_inference(et)))


def build_parser() -> argparse.ArgumentParser:
    """The reference's flags with its defaults (sample/tensorflow/benchmark.py:129-141); --seed, --iters and --warmup
    are additions (the reference hard-codes 128 timed runs after 10 warm-ups and draws from an unseeded generator)."""
    here = os.path.dirname(os.path.abspath(__file__))
    parser = argparse.ArgumentParser(description="Bert performance measuring sample.")
    parser.add_argument("-c", "--config", type=str, default=os.path.join(here, "bert_config.json"), help="Bert config file.")
    parser.add_argument("-p", "--precision", type=str, default="fp16", choices=["fp32", "fp16"], help="Weight precision.")
    parser.add_argument("-b", "--batch_size", type=int, default=128, help="Batch size.")
    parser.add_argument("-m", "--max_seq_length", type=int, default=32, help="Max sequence length.")
    parser.add_argument("-a", "--avg_seq_length", type=int, default=20, help="Average sequence length.")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--iters", type=int, default=128, help="Timed runs per model.")
    parser.add_argument("--warmup", type=int, default=10, help="Untimed runs in front of them.")
    return parser


if __name__ == "__main__":
    main(build_parser().parse_args())
