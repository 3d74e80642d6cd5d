"""The benchmark sample keeps the command line and the printed lines of the reference's
sample/tensorflow/benchmark.py (:63-66 `Valid word num`, :112 `max diff`, :126-127 the two cost lines, :129-141 the
flags), and the sweep regenerates rows of the tables in the reference's Readme.md:62-107."""
import re
from types import SimpleNamespace

import numpy as np
import pytest

from effective_transformer_amd.sample import benchmark, sweep


def test_parser_has_the_reference_flags_and_defaults():
    p = benchmark.build_parser()
    a = p.parse_args([])
    # defaults of benchmark.py:129-141 (the config default points at the copy beside the sample)
    assert a.config.endswith("bert_config.json")
    assert (a.precision, a.batch_size, a.max_seq_length, a.avg_seq_length) == ("fp16", 128, 32, 20)
    a = p.parse_args("-c x.json -p fp32 -b 8 -m 64 -a 40".split())
    assert (a.config, a.precision, a.batch_size, a.max_seq_length, a.avg_seq_length) == ("x.json", "fp32", 8, 64, 40)
    a = p.parse_args("--config y.json --precision fp16 --batch_size 3 --max_seq_length 16 --avg_seq_length 9".split())
    assert (a.config, a.precision, a.batch_size, a.max_seq_length, a.avg_seq_length) == ("y.json", "fp16", 3, 16, 9)
    with pytest.raises(SystemExit):
        p.parse_args(["-p", "bf16"])                     # choices = fp32 / fp16 (:133)
    short = {s for act in p._actions for s in act.option_strings if len(s) == 2}
    assert short == {"-h", "-c", "-p", "-b", "-m", "-a"}
    # the protocol of :114-124 unless told otherwise
    assert (a.iters, a.warmup) == (128, 10)


def test_bert_config_is_bert_base():
    import json
    cfg = json.load(open(benchmark.build_parser().parse_args([]).config))
    assert (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_hidden_layers"], cfg["intermediate_size"]) == \
        (768, 12, 12, 3072)


def test_sweep_tables_are_the_published_ones():
    """Row keys and published times of Readme.md:62-107 (V100, EffectiveTransformer column)."""
    t = {(p, m, a): rows for p, m, a, rows in sweep.TABLES}
    assert set(t) == {("fp16", 32, 20), ("fp16", 64, 40), ("fp32", 64, 40)}
    assert (1000, 133.61, 80) in t[("fp16", 64, 40)]
    assert (100, 8.75, 65) in t[("fp16", 32, 20)]
    assert [r[0] for r in t[("fp32", 64, 40)]] == [100, 200, 300, 400, 500]


def _run_benchmark(capsys, precision):
    args = benchmark.build_parser().parse_args(["-p", precision, "-b", "8", "-m", "32", "-a", "20", "--iters", "4",
                                                "--warmup", "2"])
    capsys.readouterr()                                  # drop what the test itself printed
    benchmark.main(args)
    return capsys.readouterr().out


@pytest.mark.gpu
@pytest.mark.parametrize("precision,tol", [("fp32", 1e-4), ("fp16", 2e-2)])
def test_benchmark_prints_the_reference_lines(capsys, precision, tol):
    print("sample benchmark", precision, flush=True)
    out = _run_benchmark(capsys, precision)
    lines = out.strip().splitlines()
    m = re.match(r"Valid word num : (\d+)/(\d+), avg sequence length : ([0-9.]+) $", lines[0])
    assert m, lines[0]
    lens = np.random.RandomState(0).randint(low=2 * 20 - 32, high=33, size=8)        # benchmark.py:38-41
    assert (int(m.group(1)), int(m.group(2))) == (int(lens.sum()), 8 * 32)
    m = re.match(r"max diff : ([0-9.e+-]+), avg diff : ([0-9.e+-]+)\.$", lines[1])
    assert m, lines[1]
    assert float(m.group(1)) < tol and float(m.group(2)) <= float(m.group(1))
    assert re.match(r"std cost : [0-9.]+ ms$", lines[2]), lines[2]
    assert re.match(r"et  cost : [0-9.]+ ms$", lines[3]), lines[3]
    assert len(lines) == 4


@pytest.mark.gpu
def test_sweep_prints_one_row_per_published_row(capsys):
    print("sample sweep", flush=True)
    args = sweep.build_parser().parse_args(["--iters", "3", "--precision", "fp16", "--max-batch", "100"])
    capsys.readouterr()
    sweep.main(args)
    rows = [l for l in capsys.readouterr().out.splitlines() if l.startswith("| fp16")]
    assert len(rows) == 2
    for row, (max_seq, avg, published, line) in zip(rows, [(32, 20, 8.75, 65), (64, 40, 16.03, 75)]):
        cells = [c.strip() for c in row.strip("|").split("|")]
        assert cells[:4] == ["fp16", str(max_seq), str(avg), "100"]
        assert cells[5] == "%.2f (Readme.md:%d)" % (published, line)
        ms, T = float(cells[6]), int(cells[4])
        assert ms > 0 and abs(float(cells[8]) - T / ms * 1e3) <= 0.01 * T / ms * 1e3


def test_sweep_long_rows_stay_within_the_reach_of_the_reference():
    """The second table's rows: precisions of the reference, max_seq up to the 1024 positions its softmax launch
    covers (cuda/attention.cu:345-356), and the benchmark's length recipe needs 2 * avg - max >= 1."""
    assert sweep.build_parser().parse_args(["--long", "--max-seq", "256"]).long
    for precision, max_seq, avg_seq, batch in sweep.LONG_ROWS:
        assert precision in ("fp16", "fp32") and 64 < max_seq <= 1024 and batch >= 1
        assert 2 * avg_seq - max_seq >= 1 and avg_seq <= max_seq


@pytest.mark.gpu
def test_sweep_long_prints_its_rows(capsys):
    print("sample sweep --long", flush=True)
    args = sweep.build_parser().parse_args(["--long", "--iters", "2", "--precision", "fp16", "--max-seq", "256"])
    capsys.readouterr()
    sweep.main_long(args)
    rows = [l for l in capsys.readouterr().out.splitlines() if l.startswith("| fp16")]
    assert [r.split("|")[2].strip() for r in rows] == ["128", "256"]
    for row in rows:
        cells = [c.strip() for c in row.strip("|").split("|")]
        ms, std, T = float(cells[5]), float(cells[6]), int(cells[4])
        assert ms > 0 and std > 0 and abs(float(cells[8]) - T / ms * 1e3) <= 0.01 * T / ms * 1e3


def test_profile_summary_cuts_encoder_steps_out_of_a_dispatch_sequence(tmp_path):
    """The tables under profiles/ give every launch of a layer its own row: the seven layer kernels between an input
    op and an output op, whatever else (table build, read-back copy, stand-alone loops) the trace holds."""
    from effective_transformer_amd.sample import profile_summary as ps
    layer = ["gemm_f16_pair_kernel<a>", "attention_kernel<b>", "gemm_f16_pair_kernel<a>", "bias_residual_layernorm_kernel<c>",
             "gemm_f16_pair_kernel<d>", "gemm_f16_pair_kernel<a>", "bias_residual_layernorm_kernel<c>"]
    step = ["scan_index_kernel", "compress_rows_kernel<x>", "seq_start_kernel", "seq_order_kernel",
            "__amd_rocclr_copyBuffer"] + 2 * layer + ["restore_rows_kernel<x>"]
    names = ["bias_gelu_kernel<h>"] * 3 + step + ["attention_kernel<b>"] * 4 + step + ["compress_rows_kernel<x>"] + layer
    path = tmp_path / "t_kernel_trace.csv"
    with open(path, "w") as f:
        f.write("Kernel_Name,Start_Timestamp,End_Timestamp\n")
        for i, n in enumerate(names):
            f.write('"%s",%d,%d\n' % (n, 1000 * i, 1000 * i + 100 + i))
    trace = ps.load_trace(str(path))
    steps = ps.encoder_steps([t["kind"] for t in trace], layers=2)
    assert len(steps) == 2 and all(len(b) == 14 for b in steps)          # the unfinished third step is left out
    assert [names[i] for i in steps[0]] == 2 * layer
    agg, short_names, n = ps.role_durations(trace, layers=2, skip=1)
    assert n == 2 and set(agg) == set(ps.ROLES) and all(len(v) == 2 for v in agg.values())
    first_qkv = steps[1][0]
    assert agg["QKV"][0] == pytest.approx((100 + first_qkv) / 1e3)
    assert ps.encoder_steps([t["kind"] for t in trace], layers=3) == []  # a different layer count matches nothing


def test_profile_summary_prices_launches_with_the_documented_formulas():
    from effective_transformer_amd.sample import profile_summary as ps
    from effective_transformer_amd.sample.workloads import WORKLOADS
    wl = WORKLOADS["cfg3"]
    T, H, F, B, S, e = 40396, wl.H, wl.F, wl.B, wl.S, 2
    assert ps.valid_tokens("cfg3") == T
    a = ps.algorithmic("cfg3", T)
    assert a["QKV"]["flops"] == 2.0 * T * 3 * H * H and a["FFN up + GELU"]["flops"] == 2.0 * T * F * H
    assert a["attention"]["read"] + a["attention"]["write"] == 4 * T * H * e + B * S * S * e + 8 * T
    assert a["LayerNorm 1"]["read"] + a["LayerNorm 1"]["write"] == 3 * T * H * e + 3 * H * e
