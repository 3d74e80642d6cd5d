"""Turns rocprofv3 CSV output of `bench.py` runs into the short markdown summaries kept under profiles/.

    python -m effective_transformer_amd.sample.profile_summary kernels  <dir> <name> <workload> [bench.json]
    python -m effective_transformer_amd.sample.profile_summary traffic  <fetch_counter_collection.csv> <write_counter_collection.csv> <workload>
    python -m effective_transformer_amd.sample.profile_summary counters <counter_collection.csv> <kernel_trace.csv> <workload>
    python -m effective_transformer_amd.sample.profile_summary vendor   <bench json of --calibrate-gemm> [<bench json> ...]
    python -m effective_transformer_amd.sample.profile_summary ceiling  <bench json> [<bench json> ...]

`kernels` reads <dir>/<name>_kernel_stats.csv and <dir>/<name>_kernel_trace.csv (rocprofv3 --kernel-trace --stats
--output-format csv -d <dir> -o <name>).  All three cut the launches of the encoder's own steps out of the dispatch
sequence (input op, L x 7 layer kernels, output op), so that every projection of a layer gets its own row although three
of them run the same kernel instance.  Everything is printed to stdout.
"""
from __future__ import annotations

import collections
import csv
import json
import re
import sys

from .workloads import WORKLOADS

ROLES = ["QKV", "attention", "attention out", "LayerNorm 1", "FFN up + GELU", "FFN down", "LayerNorm 2"]
SIDE = ("scan_index", "compress_rows", "embed_layernorm", "seq_start", "seq_order", "restore_rows")
LAYER_KINDS = ("attention", "bias_residual_layernorm", "gemm_f16_pair", "gemm_f16_bt", "gemm_f16_persistent", "gemm_f16_kernel",
               "gemm_f32")


def describe(workload: str) -> str:
    wl = WORKLOADS[workload]
    return "%d-layer encoder, hidden %d, %d heads x %d, FFN %d, %s, batch %d, max_seq %d" % (
        wl.layers, wl.H, wl.heads, wl.d, wl.F, wl.dtype, wl.B, wl.S)


def short(name: str) -> str:
    n = re.sub(r"\(anonymous namespace\)::", "", name)
    n = re.sub(r"^void ", "", n)
    m = re.match(r"_ZN2et12_GLOBAL__N_1\d+([a-z_0-9]+)I(.*?)EEv", n)
    if m:
        n = "et::%s<%s>" % (m.group(1), m.group(2).replace("DF16_", "half,").replace("Li", "").replace("Lb", "b").replace("E", ","))
    return n.split("(")[0][:70]


def kind(name: str) -> str:
    """What a dispatch is, by its kernel name."""
    for k in SIDE + ("attention", "bias_residual_layernorm", "bias_gelu", "layer_prologue", "gemm_f16_pair", "gemm_f16_bt",
                     "gemm_f16_persistent", "gemm_f16_kernel", "gemm_f32", "mfma_ceiling", "copyBuffer"):
        if k in name:
            return k
    return name[:30]


def encoder_steps(kinds, layers):
    """Index lists of the 7 x layers layer kernels of every complete encoder step (input op ... output op) in a
    dispatch sequence."""
    steps, i = [], 0
    while i < len(kinds):
        if kinds[i] in ("compress_rows", "embed_layernorm"):
            j = i + 1
            while j < len(kinds) and kinds[j] not in ("restore_rows", "compress_rows", "embed_layernorm", "scan_index"):
                j += 1
            if j < len(kinds) and kinds[j] == "restore_rows":
                # the layer kernels only: no table build, no prologue, no runtime copy kernel (read-back of the count)
                body = [q for q in range(i + 1, j) if kinds[q] in LAYER_KINDS]
                if len(body) == 7 * layers:
                    steps.append(body)
            i = j
        else:
            i += 1
    return steps


def load_trace(path):
    rows = list(csv.DictReader(open(path)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    return [dict(name=r["Kernel_Name"], kind=kind(r["Kernel_Name"]),
                 us=(int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3) for r in rows]


def role_durations(trace, layers, skip=3):
    """role -> list of durations (us) over the encoder steps of a kernel trace, the first `skip` steps left out."""
    steps = encoder_steps([t["kind"] for t in trace], layers)
    agg, names = collections.defaultdict(list), {}
    for body in steps[min(skip, max(0, len(steps) - 1)):]:
        for q, idx in enumerate(body):
            agg[ROLES[q % 7]].append(trace[idx]["us"])
            names[ROLES[q % 7]] = short(trace[idx]["name"])
    return agg, names, len(steps)


def load_counters(path):
    """Dispatches in order: list of dict(name, kind, counters{name: value})."""
    by_id = collections.OrderedDict()
    for r in csv.DictReader(open(path)):
        d = by_id.setdefault(int(r["Dispatch_Id"]), dict(name=r["Kernel_Name"], kind=kind(r["Kernel_Name"]), counters={}))
        d["counters"][r["Counter_Name"]] = d["counters"].get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    return [by_id[k] for k in sorted(by_id)]


def role_counters(disp, layers):
    """role -> counter -> list of values over the encoder steps; plus the same for the kernels outside the layers."""
    steps = encoder_steps([d["kind"] for d in disp], layers)
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for body in steps:
        for q, idx in enumerate(body):
            for c, v in disp[idx]["counters"].items():
                agg[ROLES[q % 7]][c].append(v)
    side = collections.defaultdict(lambda: collections.defaultdict(list))
    for d in disp:
        if d["kind"] in SIDE + ("bias_gelu", "copyBuffer", "layer_prologue"):
            for c, v in d["counters"].items():
                side[d["kind"]][c].append(v)
    return agg, side, len(steps)


def mean(v):
    return sum(v) / len(v) if v else float("nan")


def algorithmic(workload, tokens):
    """Algorithmic FLOPs / bytes per launch of the layer kernels for `tokens` valid tokens."""
    wl = WORKLOADS[workload]
    e = 2 if wl.dtype == "fp16" else 4
    T, H, F, B, S = tokens, wl.H, wl.F, wl.B, wl.S
    return {"QKV": dict(flops=2.0 * T * 3 * H * H, read=(T * H + 3 * H * H) * e, write=3 * T * H * e),
            "attention out": dict(flops=2.0 * T * H * H, read=(T * H + H * H) * e, write=T * H * e),
            "FFN up + GELU": dict(flops=2.0 * T * F * H, read=(T * H + H * F) * e, write=T * F * e),
            "FFN down": dict(flops=2.0 * T * F * H, read=(T * F + H * F) * e, write=T * H * e),
            "attention": dict(read=3 * T * H * e + B * S * S * e + 8 * T, write=T * H * e),
            "LayerNorm 1": dict(read=2 * T * H * e + 3 * H * e, write=T * H * e),
            "LayerNorm 2": dict(read=2 * T * H * e + 3 * H * e, write=T * H * e)}


def valid_tokens(workload):
    from .workloads import make_masks
    import numpy as np
    wl = WORKLOADS[workload]
    return int(make_masks(wl, np.random.RandomState(wl.seed))[1].sum())


def cmd_kernels(d, name, workload, bench_json=None):
    wl = WORKLOADS[workload]
    out = ["# rocprofv3 kernel summary: %s (%s)\n" % (workload, describe(workload))]
    out.append("Commands (repository root, one MI355X; `cd /tmp && export TMPDIR=/tmp` first, paths made absolute):\n")
    out.append("    rocprofv3 --kernel-trace --stats --output-format csv -d out -o %s -- python3 bench.py --workload %s --steps 10 --warmup 3 --no-cpu --no-graph --no-calibrate > out/bench.json" % (name, workload))
    out.append("    python3 -m effective_transformer_amd.sample.profile_summary kernels out %s %s out/bench.json\n" % (name, workload))
    if bench_json:
        try:
            b = json.loads(open(bench_json).read().strip().splitlines()[-1])
            out.append("The same (profiled) run printed %.4f ms per batch = %.3g valid tokens/s.\n" % (b["ms_per_step"], b["value"]))
        except (OSError, ValueError, KeyError, IndexError):
            pass
    out.append("## kernel_stats (rocprofv3 --stats), kernels of this library\n")
    out.append("| kernel | calls | total ms | avg us | min us | max us | % |")
    out.append("|---|---|---|---|---|---|---|")
    for r in csv.DictReader(open("%s/%s_kernel_stats.csv" % (d, name))):
        if "et::" not in r["Name"] and "_ZN2et" not in r["Name"]:
            continue
        out.append("| %s | %s | %.3f | %.2f | %.2f | %.2f | %s |" % (
            short(r["Name"]), r["Calls"], float(r["TotalDurationNs"]) / 1e6, float(r["AverageNs"]) / 1e3,
            float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3, r["Percentage"]))
    out.append("\nThe counts include `bench.py`'s per-kernel loops and its replica of the layer's launch sequence; `bias_gelu_kernel`,")
    out.append("`layer_prologue_kernel` and `embed_layernorm_kernel` only run there (the layer applies bias + GELU in the FFN-up GEMM's")
    out.append("epilogue and, with prepared weights, launches no prologue).  `seq_start_kernel` + `seq_order_kernel` build the sequence")
    out.append("table once per batch.\n")
    trace = load_trace("%s/%s_kernel_trace.csv" % (d, name))
    agg, names, nsteps = role_durations(trace, wl.layers)
    if agg:
        T = valid_tokens(workload)
        alg = algorithmic(workload, T)
        peak = 2500.0 if wl.dtype == "fp16" else 157.3
        used = len(agg[ROLES[0]]) // wl.layers
        out.append("## the kernels of one layer (same trace; launches taken in layer order from the last %d of %d encoder steps)\n" % (used, nsteps))
        out.append("| launch | kernel | calls | avg us | min us | max us | algorithmic work | achieved | of peak |")
        out.append("|---|---|---|---|---|---|---|---|---|")
        tot = 0.0
        for role in ROLES:
            v = agg[role]
            a = mean(v)
            tot += a
            w = alg[role]
            if "flops" in w:
                work = "%.1f GFLOP" % (w["flops"] / 1e9)
                ach = "%.0f TFLOP/s" % (w["flops"] / a / 1e6)
                frac = w["flops"] / a / 1e6 / peak
            else:
                work = "%.1f MB" % ((w["read"] + w["write"]) / 1e6)
                ach = "%.2f TB/s" % ((w["read"] + w["write"]) / a / 1e6)
                frac = (w["read"] + w["write"]) / a / 1e6 / 8.0
            out.append("| %s | `%s` | %d | %.1f | %.1f | %.1f | %s | %s | %.3f |" % (role, names[role], len(v), a, min(v), max(v), work, ach, frac))
        side = {}
        for k in SIDE:
            v = [t["us"] for t in trace if t["kind"] == k]
            if v:
                side[k] = mean(v)
        out.append("\nPeaks: %s MFMA %.1f TFLOP/s, HBM 8 TB/s.  Sum per layer: %.1f us; x %d layers + input / output ops and the sequence table (%s) = %.3f ms per batch."
                   % (wl.dtype, peak, tot, wl.layers, ", ".join("%s %.1f" % kv for kv in side.items() if kv[0] != "embed_layernorm"),
                      (tot * wl.layers + sum(v for k, v in side.items() if k != "embed_layernorm")) / 1e3))
    print("\n".join(out))


def cmd_traffic(fetch_csv, write_csv, workload):
    wl = WORKLOADS[workload]
    fe, wr = load_counters(fetch_csv), load_counters(write_csv)
    fagg, fside, nf = role_counters(fe, wl.layers)
    wagg, wside, nw = role_counters(wr, wl.layers)
    copy_f = max([v for d in fe if d["kind"] == "copyBuffer" for v in d["counters"].values()], default=0.0)
    copy_w = max([v for d in wr if d["kind"] == "copyBuffer" for v in d["counters"].values()], default=0.0)
    if not copy_f or not copy_w:
        sys.exit("no device copy in the counter files: run bench.py with --calibrate-copy under rocprofv3")
    copy_mib = 256.0
    sf, sw = copy_mib * 1024.0 / copy_f, copy_mib * 1024.0 / copy_w
    T = valid_tokens(workload)
    alg = algorithmic(workload, T)
    out = ["# HBM traffic per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): %s (%s)\n" % (workload, describe(workload))]
    out.append("Commands (two runs, one counter each; repository root, one MI355X, after `cd /tmp && export TMPDIR=/tmp`, paths made absolute):\n")
    for c, o in (("FETCH_SIZE", "fetch"), ("WRITE_SIZE", "write")):
        out.append("    rocprofv3 --pmc %s --output-format csv -d out -o %s -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu --no-calibrate --calibrate-copy" % (c, o, workload))
    out.append("    python3 -m effective_transformer_amd.sample.profile_summary traffic out/fetch_counter_collection.csv out/write_counter_collection.csv %s\n" % workload)
    out.append("Counters are KiB per dispatch.  Scale: the 256 MiB device copy of `--calibrate-copy` reads and writes 256 MiB and reports")
    out.append("FETCH_SIZE %.1f MiB, WRITE_SIZE %.1f MiB, so FETCH_SIZE is scaled by **%.2f** and WRITE_SIZE by **%.2f**.  The layer's launches are" % (copy_f / 1024, copy_w / 1024, sf, sw))
    out.append("taken in layer order from the %d encoder steps of each run (eager and replayed from the HIP graph).  `python bench.py --workload %s" % (min(nf, nw), workload))
    out.append("--fold-traffic <fetch csv> <write csv> --commit <id>` folds the two files into `profiles/hbm_traffic.json`, where `bench.py`")
    out.append("takes `roofline.traffic` from.\n")
    out.append("| launch | dispatches | read MiB | write MiB | algorithmic read / write MiB | read / algorithmic | total / algorithmic |")
    out.append("|---|---|---|---|---|---|---|")
    for role in ROLES:
        f = mean(fagg[role].get("FETCH_SIZE", [])) * sf / 1024.0
        w = mean(wagg[role].get("WRITE_SIZE", [])) * sw / 1024.0
        a = alg[role]
        ar, aw = a["read"] / 1048576.0, a["write"] / 1048576.0
        out.append("| %s | %d | %.1f | %.1f | %.1f / %.1f | %.2f | %.2f |" % (
            role, len(fagg[role].get("FETCH_SIZE", [])), f, w, ar, aw, f / ar, (f + w) / (ar + aw)))
    for k in ("compress_rows", "restore_rows", "embed_layernorm", "bias_gelu", "scan_index", "layer_prologue"):
        if k in fside:
            out.append("| %s (outside the layers) | %d | %.1f | %.1f |  |  |  |" % (
                k, len(fside[k].get("FETCH_SIZE", [])), mean(fside[k].get("FETCH_SIZE", [])) * sf / 1024.0,
                mean(wside[k].get("WRITE_SIZE", [])) * sw / 1024.0))
    print("\n".join(out))


def cmd_counters(counter_csv, trace_csv, workload):
    wl = WORKLOADS[workload]
    disp = load_counters(counter_csv)
    agg, _, n = role_counters(disp, wl.layers)
    dur, _, _ = role_durations(load_trace(trace_csv), wl.layers)
    T = valid_tokens(workload)
    alg = algorithmic(workload, T)
    mops = "SQ_INSTS_VALU_MFMA_MOPS_F16" if wl.dtype == "fp16" else "SQ_INSTS_VALU_MFMA_MOPS_F32"
    out = ["# MFMA utilisation and LDS conflicts per launch (rocprofv3 --pmc): %s (%s)\n" % (workload, describe(workload))]
    out.append("Commands (one pass, 5 SQ + 1 GRBM counter; repository root, one MI355X, after `cd /tmp && export TMPDIR=/tmp`, paths made absolute;")
    out.append("the durations come from the kernel trace of the same job, `profiles/encoder_%s_kernel_stats.md`):\n" % workload)
    out.append("    rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES %s SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_BUSY_CYCLES GRBM_GUI_ACTIVE --output-format csv -d out -o mfma -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu --no-graph --no-calibrate" % (mops, workload))
    out.append("    python3 -m effective_transformer_amd.sample.profile_summary counters out/mfma_counter_collection.csv out/%s_kernel_trace.csv %s\n" % (workload, workload))
    out.append("Per dispatch, averaged over the launches of the %d encoder steps, taken in layer order.  `GRBM_GUI_ACTIVE` comes back summed over" % n)
    out.append("the 8 XCDs and is shown per XCD; MFMA busy %% is rocprofv3's `MfmaUtil` expression, `SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE")
    out.append("per XCD x 1024 SIMDs)`; MFMA GFLOP = `%s x 512`.\n" % mops)
    out.append("| launch | dispatches | GUI active cycles per XCD | avg duration us (kernel trace) | cycles / duration (GHz) | MFMA busy % | MFMA GFLOP per launch | algorithmic GFLOP | LDS bank-conflict cycles / LDS active cycles |")
    out.append("|---|---|---|---|---|---|---|---|---|")
    for role in ROLES:
        c = agg[role]
        if not c:
            continue
        gui = mean(c.get("GRBM_GUI_ACTIVE", [])) / 8.0
        busy = mean(c.get("SQ_VALU_MFMA_BUSY_CYCLES", []))
        us = mean(dur.get(role, []))
        lds_a = mean(c.get("SQ_LDS_IDX_ACTIVE", []))
        out.append("| %s | %d | %.0f | %.1f | %.2f | %.1f | %.1f | %s | %.3f |" % (
            role, len(c.get("GRBM_GUI_ACTIVE", [])), gui, us, gui / us / 1e3, 100.0 * busy / (gui * 1024.0),
            mean(c.get(mops, [])) * 512.0 / 1e9, "%.1f" % (alg[role]["flops"] / 1e9) if "flops" in alg[role] else "-",
            mean(c.get("SQ_LDS_BANK_CONFLICT", [])) / lds_a if lds_a else 0.0))
    print("\n".join(out))


def last_json_line(path):
    return json.loads(open(path).read().strip().splitlines()[-1])


def cmd_vendor(paths):
    out = ["# Vendor GEMM calibration: the four projections of a layer, own kernels against `torch.matmul` (hipBLASLt / rocBLAS)\n"]
    out.append("Commands (one MI355X, repository root), one bench run per workload:\n")
    out.append("    python3 bench.py --workload cfgN --no-cpu --no-graph --no-calibrate --calibrate-gemm > cal_cfgN.json")
    out.append("    python3 -m effective_transformer_amd.sample.profile_summary vendor cal_cfg3.json cal_cfg5.json cal_cfg4.json\n")
    out.append("Each number is the average of a loop of 20 launches of one kernel on the workload's shapes, HIP events around the loop")
    out.append("(`kernels[*].ms`, `kernels[*].vendor` in the JSON line). The vendor product is the plain product (no bias, no GELU) with")
    out.append("the weights in TF's `[k][n]` order and in the k-contiguous `[n][k]` order; the own kernel includes the bias (QKV) or")
    out.append("bias + GELU (FFN up; `plain` = the same kernel without the epilogue). `in layer` = the own kernel inside the layer's")
    out.append("launch sequence (its input still in the last-level cache). TFLOP/s of the fastest vendor variant and of the own kernel")
    out.append("alone are given for the roofline (fp16 peak 2500, fp32 157.3).\n")
    for path in paths:
        d = last_json_line(path)
        T = d["config"]["valid_tokens"]
        name = d["config"]["workload"].split(":")[0]
        wl = WORKLOADS[name]
        H, F = wl.H, wl.F
        fl = {"gemm_qkv": 2.0 * T * 3 * H * H, "gemm_attn_out": 2.0 * T * H * H, "gemm_ffn_up": 2.0 * T * F * H,
              "gemm_ffn_down": 2.0 * T * H * F}
        out.append("## %s (T = %d, H = %d, F = %d, %s), whole step %.2f ms\n" % (name, T, H, F, wl.dtype, d["ms_per_step"]))
        out.append("| projection | own us (alone) | own plain us | own us in layer | vendor `[k][n]` us | vendor `[n][k]` us | own / best vendor | own TFLOP/s | best vendor TFLOP/s |")
        out.append("|---|---|---|---|---|---|---|---|---|")
        for kname in ("gemm_qkv", "gemm_attn_out", "gemm_ffn_up", "gemm_ffn_down"):
            kk = d["kernels"][kname]
            own = kk["ms"] * 1e3
            plain, inl, v = kk.get("ms_plain_product"), kk.get("ms_in_layer"), kk.get("vendor", {})
            vk = [x for x in (v.get("ms_weights_kn"), v.get("ms_weights_nk")) if x]
            best = min(vk) * 1e3 if vk else float("nan")
            cmp_own = plain * 1e3 if plain else own
            out.append("| %s | %.1f | %s | %s | %s | %s | %.2f | %.0f | %.0f |" % (
                kname[5:], own, "%.1f" % (plain * 1e3) if plain else "", "%.1f" % (inl * 1e3) if inl else "",
                "%.1f" % (v["ms_weights_kn"] * 1e3) if v.get("ms_weights_kn") else "",
                "%.1f" % (v["ms_weights_nk"] * 1e3) if v.get("ms_weights_nk") else "",
                cmp_own / best, fl[kname] / (cmp_own * 1e-6) / 1e12, fl[kname] / (best * 1e-6) / 1e12))
        out.append("")
    print("\n".join(out))


def cmd_ceiling(paths):
    out = ["# MFMA rate the part sustains under the GEMM's inner-loop instruction mix, zero against random operands\n"]
    out.append("Commands (one MI355X, repository root; the measurement is part of every default `bench.py` run):\n")
    out.append("    python3 bench.py --no-cpu --no-graph > bench.json")
    out.append("    python3 -m effective_transformer_amd.sample.profile_summary ceiling bench.json [more runs ...]\n")
    out.append("`bench.py` times `et_calibrate_mfma` (`effective_transformer_amd/csrc/calibrate.hip`) with HIP events: 8 wavefronts on")
    out.append("every CU repeat one k-step of a 128 x 64 wave tile, 32 `v_mfma_f32_16x16x32_f16` on one operand register set while 12")
    out.append("`ds_read_b128` refill the other set from LDS, as `gemm_f16_pair_kernel` does, with no global memory traffic, no barrier")
    out.append("and nothing to wait for but the LDS; 4000 k-steps per launch, best of 2 x 5 launches. One row per run (each on a box of")
    out.append("its own):\n")
    out.append("| run | zero operands TFLOP/s | random halves TFLOP/s | random / 2500 peak | step ms | dominant kernel in the layer | achieved | of peak | of the rate on random operands |")
    out.append("|---|---|---|---|---|---|---|---|---|")
    for path in paths:
        d = last_json_line(path)
        c, r = d["mfma_ceiling"], d["roofline"]
        of_random = r.get("frac_of_sustained_on_random_operands")      # only where the dominant kernel is MFMA-bound
        out.append("| %s | %.0f | %.0f | %.3f | %.3f | %s | %.0f %s | %.3f | %s |" % (
            d["config"]["workload"].split(":")[0], c["zero_operands_tflops"], c["random_operands_tflops"],
            c["random_operands_tflops"] / 2500.0, d["ms_per_step"], r["kernel"], r["achieved"], r["unit"], r["frac"],
            "%.3f" % of_random if of_random is not None else "-"))
    out.append("\nReading: instruction issue is not what limits the loop (0.96 of peak with operands that do not toggle). With operands")
    out.append("that look like data the same instruction stream runs about 30 % slower: the switching activity costs power and the part")
    out.append("lowers its clock (the counter runs show about 2.0 GHz under the GEMMs against the 2.4 GHz of the data-sheet peak). The rate on")
    out.append("random operands, not 2500 TFLOP/s, is the ceiling an fp16 GEMM on real data has on this part before it moves a byte from")
    out.append("memory; it differs from box to box by a few per cent, and the step time follows it.")
    print("\n".join(out))


def main(argv):
    if len(argv) >= 4 and argv[0] == "kernels":
        cmd_kernels(argv[1], argv[2], argv[3], argv[4] if len(argv) > 4 else None)
    elif len(argv) == 4 and argv[0] == "traffic":
        cmd_traffic(argv[1], argv[2], argv[3])
    elif len(argv) == 4 and argv[0] == "counters":
        cmd_counters(argv[1], argv[2], argv[3])
    elif len(argv) >= 2 and argv[0] == "vendor":
        cmd_vendor(argv[1:])
    elif len(argv) >= 2 and argv[0] == "ceiling":
        cmd_ceiling(argv[1:])
    else:
        sys.exit(__doc__)


if __name__ == "__main__":
    main(sys.argv[1:])
