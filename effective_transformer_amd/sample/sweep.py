"""Regenerates the tables the reference publishes (Readme.md:62-107: 12-layer BERT-base encoder, ms per batch over
batch size for fp16 max_seq 32 / avg 20, fp16 max_seq 64 / avg 40 and fp32 max_seq 64 / avg 40) on this GPU, with the
input recipe and timing protocol of the benchmark sample, and prints them as markdown beside the published
EffectiveTransformer numbers (Tesla V100).

    python -m effective_transformer_amd.sample.sweep [--std] [--iters 128]

`--long` prints a second table instead, for sequence lengths beyond the published ones (128 ... 1024 positions, the
reach of the reference's softmax launch, cuda/attention.cu:345-356), beside the padded torch encoder.
"""
import argparse
import json
import os
import time
from types import SimpleNamespace

import numpy as np
import torch

from .. import ops
from .benchmark import make_weights, standard_transformer

# (precision, max_seq, avg_seq, [(batch, ms the reference publishes for its own kernels on V100, Readme line)])
TABLES = (
    ("fp16", 32, 20, [(100, 8.75, 65), (200, 15.32, 66), (300, 22.18, 67), (400, 28.31, 68), (500, 33.08, 69), (1000, 64.34, 70)]),
    ("fp16", 64, 40, [(100, 16.03, 75), (200, 30.15, 76), (300, 41.27, 77), (400, 54.12, 78), (500, 65.92, 79), (1000, 133.61, 80)]),
    ("fp32", 64, 40, [(100, 67.45, 85), (200, 125.44, 86), (300, 197.07, 87), (400, 247.39, 88), (500, 325.37, 89)]),
)


# (precision, max_seq, avg_seq, batch): no published figures for these
LONG_ROWS = (("fp16", 128, 96, 128), ("fp16", 256, 160, 64), ("fp16", 384, 256, 64), ("fp16", 512, 384, 32),
             ("fp16", 1024, 700, 16), ("fp32", 384, 256, 16), ("fp32", 1024, 700, 4))


def time_ms(fn, iters, warm=10):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    beg = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - beg) * 1e3 / iters


def main(args):
    with open(args.config) as f:
        cfg = SimpleNamespace(**json.load(f))
    dev = torch.device("cuda", 0)
    heads = cfg.num_attention_heads
    d = cfg.hidden_size // heads
    print("| precision | max_seq | avg_seq | batch | valid tokens | reference on V100 ms | this GPU ms%s | speed-up | valid tokens/s |"
          % (" | padded torch ms" if args.std else ""))
    print("|---|---|---|---|---|---|---|%s---|---|" % ("---|" if args.std else ""))
    for precision, max_seq, avg_seq, rows in TABLES:
        if args.precision and precision != args.precision:
            continue
        if args.max_batch:
            rows = [r for r in rows if r[0] <= args.max_batch]
        dtype = torch.float16 if precision == "fp16" else torch.float32
        rng = np.random.RandomState(args.seed)
        weights = make_weights(cfg, dtype, dev, rng)
        enc = ops.EffectiveTransformerEncoder(cfg.num_hidden_layers, heads, d, weights, dtype, dev)
        for batch, published, line in rows:
            lens = rng.randint(low=2 * avg_seq - max_seq, high=max_seq + 1, size=batch).astype(np.int32)
            mask_np = (np.arange(max_seq)[None, :] < lens[:, None]).astype(np.int32)
            x = torch.from_numpy(rng.randn(batch, max_seq, cfg.hidden_size).astype(np.float32)).to(device=dev, dtype=dtype)
            mask = torch.from_numpy(mask_np).to(dev)
            att = torch.from_numpy(np.tile(mask_np, max_seq).reshape(batch, max_seq, max_seq)).to(device=dev, dtype=dtype)
            with torch.no_grad():
                ms = time_ms(lambda: enc(x, mask, att), args.iters)
                std = ""
                if args.std:
                    std = " | %.2f" % time_ms(lambda: standard_transformer(x, att, weights, cfg.num_hidden_layers, heads, d),
                                              max(args.iters // 8, 4), warm=2)
            T = int(lens.sum())
            print("| %s | %d | %d | %d | %d | %.2f (Readme.md:%d) | %.3f%s | %.1fx | %.3g |"
                  % (precision, max_seq, avg_seq, batch, T, published, line, ms, std, published / ms, T / ms * 1e3), flush=True)
        del enc, weights


def main_long(args):
    with open(args.config) as f:
        cfg = SimpleNamespace(**json.load(f))
    dev = torch.device("cuda", 0)
    heads = cfg.num_attention_heads
    d = cfg.hidden_size // heads
    print("| precision | max_seq | avg_seq | batch | valid tokens | this GPU ms | padded torch ms | speed-up | valid tokens/s |")
    print("|---|---|---|---|---|---|---|---|---|")
    for precision, max_seq, avg_seq, batch in LONG_ROWS:
        if (args.precision and precision != args.precision) or (args.max_seq and max_seq > args.max_seq):
            continue
        dtype = torch.float16 if precision == "fp16" else torch.float32
        rng = np.random.RandomState(args.seed)
        weights = make_weights(cfg, dtype, dev, rng)
        enc = ops.EffectiveTransformerEncoder(cfg.num_hidden_layers, heads, d, weights, dtype, dev)
        lens = rng.randint(low=2 * avg_seq - max_seq, high=max_seq + 1, size=batch).astype(np.int32)
        mask_np = (np.arange(max_seq)[None, :] < lens[:, None]).astype(np.int32)
        x = torch.from_numpy(rng.randn(batch, max_seq, cfg.hidden_size).astype(np.float32)).to(device=dev, dtype=dtype)
        mask = torch.from_numpy(mask_np).to(dev)
        att = torch.from_numpy(np.tile(mask_np, max_seq).reshape(batch, max_seq, max_seq)).to(device=dev, dtype=dtype)
        with torch.no_grad():
            ms = time_ms(lambda: enc(x, mask, att), args.iters)
            std = time_ms(lambda: standard_transformer(x, att, weights, cfg.num_hidden_layers, heads, d),
                          max(args.iters // 8, 4), warm=2)
        T = int(lens.sum())
        print("| %s | %d | %d | %d | %d | %.3f | %.2f | %.1fx | %.3g |"
              % (precision, max_seq, avg_seq, batch, T, ms, std, std / ms, T / ms * 1e3), flush=True)
        del enc, weights


def build_parser() -> argparse.ArgumentParser:
    here = os.path.dirname(os.path.abspath(__file__))
    parser = argparse.ArgumentParser(description="Sweep over the reference's published benchmark tables.")
    parser.add_argument("-c", "--config", type=str, default=os.path.join(here, "bert_config.json"))
    parser.add_argument("--iters", type=int, default=128)
    parser.add_argument("--std", action="store_true", help="also time the padded torch encoder")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--precision", choices=["fp16", "fp32"], default=None, help="only the tables of this precision")
    parser.add_argument("--max-batch", type=int, default=0, help="only rows up to this batch size (0 = all)")
    parser.add_argument("--long", action="store_true", help="the table of longer sequences (128 ... 1024 positions)")
    parser.add_argument("--max-seq", type=int, default=0, help="with --long: only rows up to this max_seq (0 = all)")
    return parser


if __name__ == "__main__":
    _args = build_parser().parse_args()
    (main_long if _args.long else main)(_args)
