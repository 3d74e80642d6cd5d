"""Benchmark of the padding-free BERT encoder on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3] [--no-cpu] [--no-calibrate]

A step is one pass Input -> L x Layer -> Output over one synthetic batch that is already
resident in HBM.  Prints ONE JSON line: valid tokens/s (whole job), ms/step, the roofline of the
dominant kernel measured live with HIP events (inside the layer's launch sequence, and in a launch loop of the
kernel alone), per-kernel rooflines, and the CPU baseline (the
standard padded BERT encoder graph on the host cores, on a bounded sample of the same batch).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch come from profiles/hbm_traffic.json when it holds an entry for the workload and kernel: two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch) folded in by
# `bench.py --fold-traffic`, each counter scaled by what it reads for the plain device copy of --calibrate-copy.  The
# file names the commit it was measured on; without an entry `traffic` is null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
# kernel name in the counter files -> key in `kernels`, for the kernels one name identifies (the FFN-up projection is the
# only launch of the GELU instance of the large-M GEMM; the other three projections share one instance)
TRAFFIC_KERNELS = (("gemm_f16_pair_kernel<true,", "gemm_ffn_up"), ("gemm_f16_pair_kernelILb1", "gemm_ffn_up"),
                   ("attention_kernel", "attention"), ("attention_long_kernel", "attention"),
                   ("bias_residual_layernorm_kernel", "bias_residual_layernorm"), ("bias_gelu_kernel", "bias_gelu"),
                   ("restore_rows_kernel", "output_restore"))
COPY_BYTES = 256 << 20


def measured_traffic(workload, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            d = json.load(f)
        e = d["workloads"][workload][kernel]
        return {"bytes": e["read_bytes"] + e["write_bytes"], "read_bytes": e["read_bytes"], "write_bytes": e["write_bytes"],
                "source": "profiles/hbm_traffic.json", "measured_on_commit": d["workloads"][workload].get("commit")}
    except (OSError, KeyError, ValueError):
        return None


def fold_traffic(workload, fetch_csv, write_csv, commit, command):
    """Folds two counter files (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --calibrate-copy`) into
    profiles/hbm_traffic.json."""
    import collections
    import csv

    def load(path):
        agg = collections.defaultdict(list)
        for r in csv.DictReader(open(path)):
            agg[r["Kernel_Name"]].append(float(r["Counter_Value"]) * 1024.0)      # KiB per dispatch
        return agg

    fe, wr = load(fetch_csv), load(write_csv)

    def mean_of(agg, sub):
        v = [x for k, vals in agg.items() if sub in k for x in vals]
        return (sum(v) / len(v), len(v)) if v else (None, 0)

    # the copy of --calibrate-copy is the largest device copy of the run
    cf = max([x for k, vals in fe.items() if "copyBuffer" in k for x in vals], default=0)
    cw = max([x for k, vals in wr.items() if "copyBuffer" in k for x in vals], default=0)
    if not cf or not cw:
        sys.exit("no device copy in the counter files: run bench.py with --calibrate-copy under rocprofv3")
    scale_f, scale_w = COPY_BYTES / cf, COPY_BYTES / cw
    entry = {"commit": commit, "command": command,
             "scale": {"FETCH_SIZE": round(scale_f, 3), "WRITE_SIZE": round(scale_w, 3),
                       "from": "device copy of %d bytes in the same runs" % COPY_BYTES}}
    for sub, key in TRAFFIC_KERNELS:
        f, n = mean_of(fe, sub)
        w, _ = mean_of(wr, sub)
        if f is None or w is None or key in entry:
            continue
        entry[key] = {"read_bytes": round(f * scale_f), "write_bytes": round(w * scale_w), "dispatches": n}
    try:
        with open(TRAFFIC_FILE) as fh:
            d = json.load(fh)
    except (OSError, ValueError):
        d = {"workloads": {}}
    d["workloads"][workload] = entry
    with open(TRAFFIC_FILE, "w") as fh:
        json.dump(d, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print(json.dumps(entry, indent=1))


# ms/batch the reference publishes for the same model/batch/sequence recipe (Tesla V100, Readme.md:65-89 of the
# reference); vs_baseline = published ms / measured ms.
PUBLISHED_MS = {"cfg2": (8.75, "Readme.md:65"), "cfg3": (133.61, "Readme.md:80"), "cfg4": (325.37, "Readme.md:89")}
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"fp16": 2500.0, "fp32": 157.3}


def _time_kernel(fn, iters, warm=3):
    import torch
    for _ in range(warm):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters          # ms per launch


def mfma_ceiling(iters=4000):
    """The MFMA rate this GPU sustains under the instruction mix of the large fp16 GEMM's inner loop (MFMAs + LDS
    operand reads, no global memory), with zero and with random operands: et_calibrate_mfma, timed with HIP events.
    Switching activity costs clock, so the rate on random data, not the data-sheet peak, is the ceiling the GEMMs run
    under on this part."""
    import ctypes as C
    import torch
    from effective_transformer_amd import _lib, ops
    lib = _lib.load()
    h = ops.handle(torch.device("cuda:0"))
    sink = torch.empty(lib.et_calibrate_mfma_sink_bytes(h), dtype=torch.uint8, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    fl = C.c_double(0.0)
    out = {}
    for name, rnd in (("zero_operands", 0), ("random_operands", 1)):
        def run():
            _lib.check(lib.et_calibrate_mfma(h, rnd, iters, C.c_void_p(sink.data_ptr()), sink.numel(), C.byref(fl), st), h)
        ms = min(_time_kernel(run, 5, warm=2) for _ in range(2))
        out[name + "_tflops"] = round(fl.value / ms / 1e9, 1)
    out["unit"] = "TFLOP/s"
    out["what"] = "8 waves per CU, per wave and k-step 32 v_mfma_f32_16x16x32_f16 + 12 ds_read_b128, no global memory"
    return out


def per_kernel(wl, T, mask_np, iters=20, vendor_gemm=False):
    """Times every kernel of the path in isolation at the workload's real shapes and prices it
    against its roofline with ALGORITHMIC bytes / flops.  vendor_gemm: also time the vendor library's GEMM
    (torch.matmul) on the same operands in the same kind of launch loop, as a calibration point."""
    import numpy as np
    import torch
    from effective_transformer_amd import kernel_ops as k, ops

    dt = torch.float16 if wl.dtype == "fp16" else torch.float32
    e = 2 if wl.dtype == "fp16" else 4
    B, S, H, F, heads, d = wl.B, wl.S, wl.H, wl.F, wl.heads, wl.d
    g = torch.Generator(device="cuda").manual_seed(0)
    rnd = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float32, generator=g).to(dt)
    x = rnd(B, S, H)
    mask = torch.from_numpy(mask_np).cuda()
    attr = mask[:, None, :].expand(B, S, S).to(dt).contiguous()
    to, vwn, bidx, widx = ops.effective_transformer_input(x, mask, B, S, S, heads, d)
    res = {}

    def add(name, ms, bound, work):
        if bound == "hbm":
            ach, peak, unit = work / ms / 1e6, HBM_PEAK_GBS, "GB/s"
        else:
            ach, peak, unit = work / ms / 1e9, MFMA_PEAK_TFLOPS[wl.dtype], "TFLOP/s"
        res[name] = {"ms": round(ms, 5), "bound": bound, "achieved": round(ach, 2), "peak": peak, "unit": unit,
                     "frac": round(ach / peak, 4)}

    # input op = scan + index build + compress; output op = restore.  Called through the C ABI with preallocated
    # outputs so that the host side of the loop stays shorter than the kernels.
    import ctypes as C
    from effective_transformer_amd import _lib
    lib = _lib.load()
    h = ops.handle(x.device)
    code = _lib.ET_FP16 if wl.dtype == "fp16" else _lib.ET_FP32
    ws = torch.empty(lib.et_input_workspace_bytes(B, S), dtype=torch.uint8, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: C.c_void_p(t.data_ptr())
    back = torch.empty_like(x)

    def run_input():
        _lib.check(lib.et_input(h, code, P(x), P(mask), P(to), P(vwn), P(bidx), P(widx), B, S, heads, d, P(ws),
                                ws.numel(), st, None), h)

    def run_output():
        _lib.check(lib.et_output(h, code, P(to), P(vwn), P(bidx), P(widx), P(back), B, S, heads, d, st), h)

    ms = _time_kernel(run_input, iters)
    add("input_scan_compress", ms, "hbm", 2 * T * H * e + 4 * B * S + 8 * T + 4)
    ms = _time_kernel(run_output, iters)
    add("output_restore", ms, "hbm", T * H * e + B * S * H * e + 8 * T)
    # the step in front of the path: BERT-base embedding block fused with the input op (ids -> packed rows)
    V, Vt, Pmax = 30522, 2, 512
    emb = ops.EmbeddingWeights(x.device, dt, rnd(V, H), rnd(H), rnd(H), token_type_embeddings=rnd(Vt, H),
                               position_embeddings=rnd(Pmax, H))
    ids = torch.randint(0, V, (B, S), dtype=torch.int32, device="cuda")
    tts = torch.randint(0, Vt, (B, S), dtype=torch.int32, device="cuda")
    to_e = torch.empty_like(x)

    def run_embed():
        _lib.check(lib.et_embedding_input(h, code, C.byref(emb.struct), P(ids), P(tts), P(mask), P(to_e), P(vwn), P(bidx),
                                          P(widx), B, S, heads, d, P(ws), ws.numel(), st, None), h)

    ms = _time_kernel(run_embed, iters)
    add("embedding_input", ms, "hbm", 2 * T * H * e + 12 * B * S + 16 * T + 4)
    run_input()      # leaves the index arrays of the activation path in place
    # row kernels
    a = rnd(T, H); r = rnd(T, H); bias = rnd(H); gam = rnd(H); bet = rnd(H)
    ms = _time_kernel(lambda: k.add_bias_input_layernorm(a, r, bias, gam, bet), iters)
    add("bias_residual_layernorm", ms, "hbm", 3 * T * H * e + 3 * H * e)
    inter = rnd(T, F) * 0.1; bF = rnd(F)
    ms = _time_kernel(lambda: k.add_bias_act(inter, bF), iters)
    add("bias_gelu", ms, "hbm", 2 * T * F * e + F * e)
    res["bias_gelu"]["on_path"] = False       # et_add_bias_act on its own; the layer fuses it into the FFN-up GEMM
    # fused attention on packed rows
    qkv = rnd(B * S, 3 * H)
    ctx = torch.empty(B * S, H, device="cuda", dtype=dt)
    starts = ops.sequence_starts(vwn, bidx, B, S)          # one table per batch, as the encoder builds it
    ms = _time_kernel(lambda: k.attention(qkv, qkv[:, H:], qkv[:, 2 * H:], 1, 3 * H, attr, vwn, B, S, heads, d, bidx,
                                          widx, dst=ctx, seq_start=starts), iters)
    lens = mask_np.sum(axis=1).astype(np.float64)
    add("attention", ms, "hbm", 4 * T * H * e + B * S * S * e + 8 * T)
    res["attention"]["valid_tflops"] = round(4 * H * float((lens ** 2).sum()) / ms / 1e9, 2)
    # the four projections; the first FFN projection carries bias + GELU in its epilogue, as in the layer
    for name, n, kk in (("gemm_qkv", 3 * H, H), ("gemm_attn_out", H, H), ("gemm_ffn_up", F, H), ("gemm_ffn_down", H, F)):
        A = rnd(T, kk); Bm = rnd(kk, n) * 0.02
        Cm = torch.empty(T, n, device="cuda", dtype=dt)
        kw = {"bias": bF, "gelu": True} if name == "gemm_ffn_up" else {}
        fn = lambda: k.gemm(A, Bm, out=Cm, **kw)
        plain = lambda: k.gemm(A, Bm, out=Cm)
        if dt == torch.float16:
            # the encoder object hands k-contiguous copies of its (constant) weights to the layer op, which runs them
            # on the large-M kernel once the batch fills the chip
            Bt = k.transpose_weight(Bm)
            try:
                k.gemm_bt(A, Bt, out=Cm, **kw)
                fn = lambda: k.gemm_bt(A, Bt, out=Cm, **kw)
                plain = lambda: k.gemm_bt(A, Bt, out=Cm)
            except Exception:
                pass
        ms = _time_kernel(fn, iters)
        add(name, ms, "mfma", 2.0 * T * n * kk)
        if kw:
            res[name]["epilogue"] = "bias+gelu"
        if vendor_gemm:
            # calibration only, never on the path: the plain product (no bias, no GELU) by the vendor library, with the
            # weights in TF's [k][n] order and in the k-contiguous [n][k] order
            Bnk = Bm.t().contiguous()
            try:
                v_kn = _time_kernel(lambda: torch.matmul(A, Bm, out=Cm), iters)
                v_nk = _time_kernel(lambda: torch.matmul(A, Bnk.t(), out=Cm), iters)
                res[name]["vendor"] = {"library": "torch.matmul (hipBLASLt / rocBLAS), plain product",
                                       "ms_weights_kn": round(v_kn, 5), "ms_weights_nk": round(v_nk, 5)}
                if kw:      # the own kernel without the epilogue, for a like-for-like number
                    res[name]["ms_plain_product"] = round(_time_kernel(plain, iters), 5)
            except Exception as ex:       # a library failure must not take the benchmark line down
                res[name]["vendor"] = {"error": str(ex)[:200]}
    if dt == torch.float16:
        Wall = rnd(H, 7 * H)                          # Q, K, V and FFN-up kernels
        Wt = torch.empty(7 * H, H, device="cuda", dtype=dt)
        ms = _time_kernel(lambda: k.transpose_weight(Wall, out=Wt), iters)
        add("weight_transpose", ms, "hbm", 2 * 7 * H * H * e)
        res["weight_transpose"]["on_path"] = False   # per call only for callers of plain et_layer; the encoder object prepares once
    return res


def in_layer_kernels(wl, T, mask_np, reps=4):
    """The kernels of one layer launched in the layer's own order on the layer's own data flow (each kernel reads what
    the one before it wrote, as inside et_layer), with a HIP event between every two launches: the duration a kernel
    has on the path, where its input is still in the last-level cache.  Returns ms per launch by kernel name and the
    sum over one layer."""
    import torch
    from effective_transformer_amd import kernel_ops as k, ops

    dt = torch.float16 if wl.dtype == "fp16" else torch.float32
    B, S, H, F, heads, d = wl.B, wl.S, wl.H, wl.F, wl.heads, wl.d
    g = torch.Generator(device="cuda").manual_seed(1)
    rnd = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float32, generator=g).to(dt)
    mask = torch.from_numpy(mask_np).cuda()
    attr = mask[:, None, :].expand(B, S, S).to(dt).contiguous()
    x, vwn, bidx, widx = ops.effective_transformer_input(rnd(B, S, H), mask, B, S, S, heads, d)
    x = x.reshape(B * S, H)[:T]
    weights = {"gemm_qkv": rnd(H, 3 * H) * 0.02, "gemm_attn_out": rnd(H, H) * 0.02, "gemm_ffn_up": rnd(H, F) * 0.02,
               "gemm_ffn_down": rnd(F, H) * 0.02}
    bias = {n: rnd(w.shape[1]) * 0.02 for n, w in weights.items()}
    gam, bet = torch.ones(H, device="cuda", dtype=dt), torch.zeros(H, device="cuda", dtype=dt)
    mm = {}
    for n, w in weights.items():          # the kernel the encoder object runs this projection on
        mm[n] = (k.gemm, w)
        if dt == torch.float16:
            wt = k.transpose_weight(w)
            try:
                k.gemm_bt(rnd(T, w.shape[0]), wt)
                mm[n] = (k.gemm_bt, wt)
            except Exception:
                pass
    qkv = torch.empty(T, 3 * H, device="cuda", dtype=dt)
    ctx, ao, spare = (torch.empty(T, H, device="cuda", dtype=dt) for _ in range(3))
    inter = torch.empty(T, F, device="cuda", dtype=dt)
    names = ("gemm_qkv", "attention", "gemm_attn_out", "bias_residual_layernorm", "gemm_ffn_up", "gemm_ffn_down",
             "bias_residual_layernorm")
    starts = ops.sequence_starts(vwn, bidx, B, S)          # one table per batch, as the encoder builds it

    def layer(ev):
        cur, down = x, spare
        for l in range(wl.layers):
            e = ev[l] if ev else None
            f, w = mm["gemm_qkv"]
            if e: e[0].record()
            f(cur, w, bias=bias["gemm_qkv"], out=qkv)
            if e: e[1].record()
            k.attention(qkv, qkv[:, H:], qkv[:, 2 * H:], 1, 3 * H, attr, vwn, B, S, heads, d, bidx, widx, dst=ctx,
                        seq_start=starts)
            if e: e[2].record()
            f, w = mm["gemm_attn_out"]
            f(ctx, w, out=ao)
            if e: e[3].record()
            k.add_bias_input_layernorm(ao, cur, bias["gemm_attn_out"], gam, bet)
            if e: e[4].record()
            f, w = mm["gemm_ffn_up"]
            f(ao, w, bias=bias["gemm_ffn_up"], gelu=True, out=inter)
            if e: e[5].record()
            f, w = mm["gemm_ffn_down"]
            f(inter, w, out=down)
            if e: e[6].record()
            k.add_bias_input_layernorm(down, ao, bias["gemm_ffn_down"], gam, bet)
            if e: e[7].record()
            cur, down = down, cur      # the layer's output feeds the next layer

    layer(None)
    tot = {n: 0.0 for n in names}
    for _ in range(reps):
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(8)] for _ in range(wl.layers)]
        torch.cuda.synchronize()
        layer(ev)
        torch.cuda.synchronize()
        for e in ev:
            for i, n in enumerate(names):
                tot[n] += e[i].elapsed_time(e[i + 1])
    calls = {n: reps * wl.layers * names.count(n) for n in tot}
    per = {n: tot[n] / calls[n] for n in tot}
    return per, sum(per[n] * names.count(n) for n in per)


def cpu_baseline(w, nseq=0, budget_s=12.0):
    """The standard padded BERT encoder graph (the reference's comparison path) in fp32 on the host cores, all
    layers, on the first `nseq` sequences of the batch.  nseq = 0: as many sequences as fit about `budget_s`
    seconds, judged from a short probe."""
    import numpy as np
    import torch
    from oracle import et_oracle as o
    wl = w["wl"]
    weights = [a.astype(np.float32) for a in w["weights"]]

    def run(n):
        x = w["x"][:n].astype(np.float32)
        attr = w["attr_mask"][:n].astype(np.float32)
        t0 = time.perf_counter()
        o.tf_graph_encoder(x, attr, weights, wl.heads, wl.d)
        return time.perf_counter() - t0

    probe = min(wl.B, 16)
    run(min(wl.B, 4))                                   # warm-up
    t_probe = run(probe)
    if nseq <= 0:
        nseq = int(max(probe, min(wl.B, budget_s / (t_probe / probe))))
    dtm = run(nseq)
    tokens = int(w["mask"][:nseq].sum())
    return {"value": round(tokens / dtm, 1), "unit": "valid tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": round(dtm, 2), "ms_per_batch_extrapolated": round(dtm * 1e3 * wl.B / nseq, 1),
            "sample": "first %d of %d sequences (%d valid tokens), all %d layers, fp32, padded [B*S,H] graph"
                      % (nseq, wl.B, tokens, wl.layers)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)       # the reference's 128 timed iterations
    ap.add_argument("--warmup", type=int, default=10)       # ... after 10 warm-ups
    ap.add_argument("--workload", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"])
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--cpu-seqs", type=int, default=0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy (reference point for the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--no-calibrate", action="store_true",
                    help="skip the measurement of the MFMA rate the GPU sustains on zero and on random operands "
                         "(fp16, about 0.3 s), which otherwise goes into `mfma_ceiling`")
    ap.add_argument("--calibrate-mfma", action="store_true", help="kept for old command lines: the measurement is on by default")
    ap.add_argument("--calibrate-gemm", action="store_true",
                    help="also time the vendor library's GEMM (torch.matmul) on the four projection shapes")
    ap.add_argument("--fold-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: fold two rocprofv3 --pmc counter files into profiles/hbm_traffic.json")
    ap.add_argument("--commit", default="unknown", help="with --fold-traffic: the commit the counters were measured on")
    a = ap.parse_args()
    if a.fold_traffic:
        fold_traffic(a.workload, a.fold_traffic[0], a.fold_traffic[1], a.commit,
                     "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -d out -o fetch|write -- python3 bench.py "
                     "--workload %s --steps 2 --warmup 1 --no-cpu --calibrate-copy" % a.workload)
        return
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every box here has one); --gpus %d is not supported" % a.gpus)

    import numpy as np
    import torch
    from effective_transformer_amd import _lib, ops
    from effective_transformer_amd.sample import workloads

    _lib.load()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    w = workloads.make_workload(a.workload)
    wl = w["wl"]
    dt = torch.float16 if wl.dtype == "fp16" else torch.float32
    enc = ops.EffectiveTransformerEncoder(wl.layers, wl.heads, wl.d, w["weights"], dt, "cuda:0")
    x = torch.from_numpy(w["x"]).cuda()
    mask = torch.from_numpy(w["mask"]).cuda()
    attr = torch.from_numpy(w["attr_mask"]).cuda()
    T = int(w["mask"].sum())

    for _ in range(a.warmup):
        enc(x, mask, attr)
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    s.record()
    for _ in range(a.steps):
        out = enc(x, mask, attr)
    e.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    ms = s.elapsed_time(e) / a.steps

    if a.calibrate_copy:
        src = torch.empty(COPY_BYTES, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
    # the same step replayed from one HIP graph (valid-token count kept on the device, no host read-back)
    graph_ms = None
    if not a.no_graph:
        g = enc.make_graph(x, mask, attr)
        for _ in range(3):
            g()
        torch.cuda.synchronize()
        s.record()
        for _ in range(a.steps):
            g()
        e.record()
        torch.cuda.synchronize()
        graph_ms = s.elapsed_time(e) / a.steps
        del g
    kernels = {} if a.no_kernels else per_kernel(wl, T, w["mask"], vendor_gemm=a.calibrate_gemm)
    roof = None
    layer_sum = None
    if kernels:
        # the same kernels inside the layer's launch sequence: what each costs on the path
        per, layer_sum = in_layer_kernels(wl, T, w["mask"])
        # launches shorter than the host's time per call space the events by the host, not by the GPU: then the sum
        # over the layers exceeds the measured step and the launch loop of the kernel alone is the better clock
        host_bound = layer_sum * wl.layers > 1.05 * ms
        for n, ms_l in per.items():
            kd = kernels[n]
            kd["ms_in_layer"] = round(ms_l, 5)
            kd["achieved_in_layer"] = round(kd["achieved"] * kd["ms"] / ms_l, 2)
            kd["frac_in_layer"] = round(kd["achieved_in_layer"] / kd["peak"], 4)
        # dominant kernel = the largest share of a layer's time; its roofline is priced at its duration on the path
        # (the `ms` a launch loop of the kernel alone gives, with cold inputs, stays beside it)
        share = {n: (kernels[n]["ms"] if host_bound else per[n]) * (2 if n == "bias_residual_layernorm" else 1)
                 for n in per}
        dom = max(share, key=share.get)
        kd = kernels[dom]
        alone = {"ms": kd["ms"], "achieved": kd["achieved"], "frac": kd["frac"]}
        if host_bound:
            roof = {"kernel": dom, "bound": kd["bound"], "achieved": kd["achieved"], "peak": kd["peak"],
                    "unit": kd["unit"], "frac": kd["frac"], "ms": kd["ms"],
                    "measured": "HIP events around a launch loop of the kernel alone (the layer replica is host-bound at this size)",
                    "traffic": measured_traffic(wl.name, dom)}
        else:
            roof = {"kernel": dom, "bound": kd["bound"], "achieved": kd["achieved_in_layer"], "peak": kd["peak"],
                    "unit": kd["unit"], "frac": kd["frac_in_layer"], "ms": kd["ms_in_layer"],
                    "measured": "HIP events around the kernel inside the layer's launch sequence, %d launches" % (4 * wl.layers),
                    "alone": alone, "traffic": measured_traffic(wl.name, dom)}
    ceiling = None
    if not a.no_calibrate and wl.dtype == "fp16":
        try:
            ceiling = mfma_ceiling()
            if roof is not None and roof["bound"] == "mfma" and wl.dtype == "fp16":
                roof["frac_of_sustained_on_random_operands"] = round(roof["achieved"] / ceiling["random_operands_tflops"], 4)
        except Exception as ex:      # a failed calibration must not take the benchmark line down
            ceiling = {"error": str(ex)[:200]}
    cpu = None
    if not a.no_cpu:
        cpu = cpu_baseline(w, a.cpu_seqs)

    print(json.dumps({
        "metric": "valid_tokens_per_s", "value": round(T / (ms / 1e3), 1), "unit": "valid tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "wall_ms_per_step": round(wall_ms, 4),
        "hip_graph_ms_per_step": None if graph_ms is None else round(graph_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(PUBLISHED_MS[wl.name][0] / ms, 3) if wl.name in PUBLISHED_MS else None,
        "baseline": ({"ms_per_batch": PUBLISHED_MS[wl.name][0], "hardware": "Tesla V100 (reference's own kernels)",
                      "source": PUBLISHED_MS[wl.name][1]} if wl.name in PUBLISHED_MS else None),
        "dtype": wl.dtype, "data": "synthetic",
        "config": {"workload": "%s: BERT %d layers, hidden %d, %d heads x %d, FFN %d, batch %d, max_seq %d, %d valid tokens"
                               % (wl.name, wl.layers, wl.H, wl.heads, wl.d, wl.F, wl.B, wl.S, T),
                   "valid_tokens": T, "padded_tokens": wl.B * wl.S},
        "roofline": roof, "layer_ms_sum_of_kernels": None if layer_sum is None else round(layer_sum, 4),
        "kernels": kernels, "cpu_baseline": cpu, "mfma_ceiling": ceiling,
    }))


if __name__ == "__main__":
    main()
