#!/usr/bin/env python3
"""Benchmark of the speculative-decoding verify step on one MI355X.

A "step" is one verify step: the target forward over the k+1 fed rows, device-side acceptance
and the KV truncation (`HipVerifier.verify_accept`), on a Llama-3-8B-shaped random-init Q4_K
target with a 4096-token fp16 KV cache, chain draft k=4, rejection sampling at T=0.8 -- the
configuration the headline metric is quoted on.  Inputs (weights, KV cache, drafter logits,
proposals) are resident in HBM before the timed region.  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
os.environ.setdefault("TSV_MEASUREMENT_HOOKS", "1")   # the per-class timing and repeated launches answer only under this

WORKLOADS = {
    # the headline configuration: 8B-shaped Q4_K target, chain k = 4, 4096-token context, T = 0.8
    "llama3_8b_q4_k_k4_ctx4096": dict(model="llama3_8b_q4_k", ctx=4096, k=4, temperature=0.8),
    # the reference's CPU-runnable plumbing case, greedy
    "tiny_q8_0_k4_ctx256": dict(model="tiny_q8_0", ctx=256, k=4, temperature=0.0),
    "small_q4_k_k4_ctx256": dict(model="small_q4_k", ctx=256, k=4, temperature=0.8),
    # configuration 4: routed experts (MXFP4) + Q8_0 attention, chain k=8, greedy
    "qwen3_30b_a3b_mxfp4_k8_ctx8192": dict(model="qwen3_30b_a3b", ctx=8192, k=8, temperature=0.0),
    "moe_small_k8_ctx256": dict(model="moe_small", ctx=256, k=8, temperature=0.0),
    # configuration 5: gpt-oss arrangement (bf16 + MXFP4 experts top-4, window / full layers), T = 1.0
    "gptoss_120b_mxfp4_k8_ctx32768": dict(model="gptoss_120b", ctx=32768, k=8, temperature=1.0),
    "gptoss_small_k8_ctx256": dict(model="gptoss_small", ctx=256, k=8, temperature=1.0),
    # configuration 3: the 16-node tree (root, four children, chains below them), 16 384-token
    # context, multi-branch rejection at T = 1.0
    "llama3_8b_q4_k_tree16_ctx16384": dict(model="llama3_8b_q4_k", ctx=16384, k=15, temperature=1.0, tree=True),
    "small_q4_k_tree16_ctx256": dict(model="small_q4_k", ctx=256, k=15, temperature=1.0, tree=True),
}
TREE16 = [-1, 0, 0, 0, 0, 1, 5, 6, 2, 8, 9, 3, 11, 12, 4, 14]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(cfg, ctx, m, union=None, kv_bits=None):
    """Bytes one verify step has to move: every quantized weight once, the KV rows [0, ctx+m)
    once per layer, m embedding rows, m x vocab fp16 logits, m new KV rows.  Routed experts: an
    expert's matrices count once per layer in which any row chose it; `union` is the mean number of
    distinct experts per layer actually routed (read back from the device), None the expectation
    under independent uniform routing.  kv_bits = (key bits, value bits): the layers the reference's policy
    quantizes (full attention, all but the last of a stack of more than two) cost a norm and packed indices per
    kv head instead of fp16 rows."""
    from turbospark_amd import ffi
    H, F, V, L = cfg["hidden"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    qd, kvd = cfg["n_q_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    rb = lambda rows, cols, dt=None: rows * ffi.row_bytes(cfg["dtype"] if dt is None else dt, cols)
    E = cfg.get("n_experts", 0)
    if E:
        # routed experts: an expert's matrices are read once if any of the m rows chose it; with
        # independent uniform routing the expected number of distinct experts per layer is
        # E * (1 - (1 - k/E)^m)
        if union is None:
            union = E * (1.0 - (1.0 - cfg["top_k"] / E) ** m)
        xd = cfg.get("expert_dtype", cfg["dtype"])
        per_layer = dict(qkv=rb(qd + 2 * kvd, H), wo=rb(H, qd), gate_up=int(union * rb(2 * F, H, xd)) + rb(E, H),
                         down=int(union * rb(H, F, xd)))
    else:
        per_layer = dict(qkv=rb(qd + 2 * kvd, H), wo=rb(H, qd), gate_up=rb(2 * F, H), down=rb(H, F))
    head = rb(V, H)
    weights = L * sum(per_layer.values()) + head
    fp16_row = kvd * 2 * 2
    kv = 0
    for l in range(L):
        windowed = bool(cfg.get("gptoss")) and l % 2 == 0      # even layers read only their window
        positions = min(cfg["gptoss"]["window"] + m, ctx + m) if windowed else ctx + m
        row = fp16_row
        if kv_bits and not windowed and (L <= 2 or l + 1 < L):
            row = sum(cfg["n_kv_heads"] * (4 + 4 * ((cfg["head_dim"] * b + 31) // 32)) for b in kv_bits)
        kv += positions * row
    small = m * ffi.row_bytes(cfg["dtype"], H) + m * V * 2 + L * m * kvd * 2 * 2
    return dict(per_layer=per_layer, head=head, weights=weights, kv=kv, total=weights + kv + small)


def trace_summary(path, first="k_clear_result"):
    """Per-kernel statistics of the verify STEPS in a `rocprofv3 --kernel-trace --output-format csv`
    trace of this script: only dispatches from the first acceptance kernel on are counted,
    which leaves out weight re-tiling and the prompt passes that build the KV cache (--trace-from
    k_embed counts from the first pass on instead: the prompt passes of a --prefill-bench run).
    Kernels are keyed by name and grid size, so the five matmul shapes show up separately."""
    import csv
    rows = list(csv.DictReader(open(path)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    start = next(i for i, r in enumerate(rows) if first in r["Kernel_Name"])
    stats = {}
    for r in rows[start:]:
        name = r["Kernel_Name"].replace("tsv::", "").replace("(anonymous namespace)::", "")
        name = name.split("(")[0].replace("void ", "")
        key = (name, int(r["Grid_Size_X"]) // max(int(r["Workgroup_Size_X"]), 1), int(r["LDS_Block_Size"]))
        d = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        st = stats.setdefault(key, [0, 0, 10**12, 0])
        st[0] += 1
        st[1] += d
        st[2] = min(st[2], d)
        st[3] = max(st[3], d)
    total = sum(v[1] for v in stats.values())
    print(f"{'kernel':44s} {'wgs':>6s} {'lds':>7s} {'calls':>7s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'share':>7s}")
    for (name, wgs, lds), v in sorted(stats.items(), key=lambda kv: -kv[1][1]):
        print(f"{name[:44]:44s} {wgs:6d} {lds:7d} {v[0]:7d} {v[1] / v[0] / 1e3:9.2f} {v[2] / 1e3:9.2f} {v[3] / 1e3:9.2f} "
              f"{100.0 * v[1] / total:6.2f}%")
    what = "verify steps" if first == "k_clear_result" else f"dispatches from the first {first} on"
    print(f"total kernel time in {what}: {total / 1e6:.3f} ms over the traced steps")


# Figures read from the committed counter / trace summaries under profiles/ (a bench run does not collect counters).
# For each workload: the kernels `achieved` counts (the dominant launch: the gate/up matmul; for the routed workloads
# router matmul + ranking + grouped gate/up together), named as the tables name them with the workgroup count that
# tells same-named launches apart (None: the name is unique).  `traffic`: their HBM bytes per launch from
# `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`, each counter scaled by the copy kernel of known size (the rows of
# `bench.py --step-traffic`); `trace_avg_us`: the same kernels in the rocprofv3 kernel trace of this script;
# `step_traffic`: bytes read + written per verify pass over all its kernels, to set beside `step_algorithmic_bytes`.
_TRAFFIC = "profiles/verify_step_hbm_traffic_by_kernel_all_workloads.txt"
PROFILED = {
    "llama3_8b_q4_k_k4_ctx4096": dict(
        trace="profiles/verify_step_llama3_8b_q4k_ctx4096_kernels.txt", kernels=[("k_gemm<Q4K, 1, 2>", 448, 448)]),
    "llama3_8b_q4_k_tree16_ctx16384": dict(
        trace="profiles/verify_step_llama3_8b_q4k_tree16_ctx16384_kernels.txt", kernels=[("k_gemm16<1>", 448, 448)]),
    "qwen3_30b_a3b_mxfp4_k8_ctx8192": dict(
        trace="profiles/verify_step_qwen3_30b_a3b_mxfp4_ctx8192_kernels.txt",
        kernels=[("k_gemm<Q80, 0, 4>", 8, 8), ("k_route_rank", None, None), ("k_moe_gemm<MX4, 1, 2>", None, None)]),
    "gptoss_120b_mxfp4_k8_ctx32768": dict(
        trace="profiles/verify_step_gptoss_120b_mxfp4_ctx32768_kernels.txt",
        kernels=[("k_gemm<BF16W, 0, 4>", 16, 16), ("k_route_rank", None, None), ("k_moe_gemm<MX4, 1, 1>", None, None)]),
}


def _table_rows(lines, n_numbers):
    """(kernel name, [numbers]) of every table line: the name, then `n_numbers` right-aligned numeric columns."""
    import re
    pat = re.compile(r"^(\S.*?)" + r"\s+(-?[\d.]+)%?" * n_numbers + r"\s*$")
    for l in lines:
        m = pat.match(l.rstrip("\n"))
        if m and not l.startswith(("#", "kernel ")):
            yield m.group(1), [float(g) for g in m.groups()[1:]]


def recorded(workload):
    """The workload's figures out of profiles/ (see PROFILED), or {} where a summary is missing or names none of the kernels."""
    spec = PROFILED.get(workload)
    if not spec:
        return {}
    try:
        out = {}
        trace = list(_table_rows(open(os.path.join(ROOT, spec["trace"])), 7))   # wgs lds calls avg min max share
        section, per_pass = [], None
        inside = False
        for l in open(os.path.join(ROOT, _TRAFFIC)):
            if l.startswith("## "):
                inside = l[3:].strip() == workload
            elif inside:
                section.append(l)
                if l.startswith("all dispatches from the first"):
                    w = l.split()
                    per_pass = int(w[w.index("B") - 1]) + int(w[w.index("written") - 2])
        traffic = list(_table_rows(section, 4))                                   # wgs calls read written
        us, nbytes = 0.0, 0
        for name, trace_wgs, traffic_wgs in spec["kernels"]:
            t = [v for n, v in trace if n == name and (trace_wgs is None or v[0] == trace_wgs)]
            b = [v for n, v in traffic if n == name and (traffic_wgs is None or v[0] == traffic_wgs)]
            if len(t) != 1 or len(b) != 1:
                return {}
            us += t[0][3]
            nbytes += int(b[0][2] + b[0][3])
        names = " + ".join(n for n, _, _ in spec["kernels"])
        out.update(trace_avg_us=us, trace_source=f"recorded: {spec['trace']} ({names})", traffic=nbytes,
                   traffic_source=f"recorded: {_TRAFFIC} ({names})")
        if per_pass:
            out.update(step_traffic=per_pass, step_traffic_source=f"recorded: {_TRAFFIC}")
        return out
    except (OSError, ValueError):
        return {}


GATE_UP_8B = dict(dtype=12, rows=28672, cols=4096, m=5, epi=1)   # the dominant kernel of the headline workload
COPY_BYTES = 256 << 20
# What a counter run can be pointed at (--probe): `match` picks the kernel's dispatches out of the
# collection, `alg` is its algorithmic bytes per launch.
ATTN_8B = dict(m=5, nq=32, nkv=8, hd=128, base=4096)             # one layer's attention of the headline workload
PROBES = {
    "gate_up": dict(match="k_gemm<", what="gate/up matmul, 28672 x 4096 Q4_K, M = 5", **GATE_UP_8B),
    # the same weights under sixteen rows (the 16-node tree): the 16x16x32 MFMA form
    "gemm16": dict(match="k_gemm16<", what="gate/up matmul, 28672 x 4096 Q4_K, M = 16", **dict(GATE_UP_8B, m=16)),
    # the same weights in a 64-row prompt pass (counters over a --prefill-bench run; --counter-summary only)
    "gemm_wide": dict(match="k_gemm_wide<1>", what="gate/up matmul, 28672 x 4096 Q4_K, 64-row prompt pass",
                      **dict(GATE_UP_8B, m=64)),
    "attention": dict(match="k_attn_partial", what="attention partial pass, 32 q / 8 kv heads x 128, M = 5, 4096-token context",
                      **ATTN_8B),
    # the same pass over TurboQuant rows, four bits for keys and values: norms and packed indices instead of fp16 rows
    "attention_tq": dict(match="k_attn_partial_tq", what="attention partial pass over 4-bit KV rows, 32 q / 8 kv heads x 128, "
                                                         "M = 5, 4096-token context", kv_bits=4, **ATTN_8B),
}


def probe_bytes(pr):
    from turbospark_amd import ffi
    if "rows" in pr:
        return pr["rows"] * ffi.row_bytes(pr["dtype"], pr["cols"])
    if "kv_bits" in pr:   # per position and kv head and side: an f32 norm and head_dim * bits / 8 bytes of indices
        return (pr["base"] + pr["m"]) * pr["nkv"] * 2 * (4 + pr["hd"] * pr["kv_bits"] // 8)
    return (pr["base"] + pr["m"]) * pr["nkv"] * pr["hd"] * 2 * 2    # K and V rows [0, base + m), fp16, read once


def traffic_probe(which):
    """What `rocprofv3 --pmc ...` is pointed at: the plain copy kernel of known size (COPY_BYTES
    read, COPY_BYTES written per launch), then the probed kernel at the headline workload's shape
    (matmuls: on weights cycled through HBM; attention: fresh seeded K/V per launch)."""
    import numpy as np
    from turbospark_amd import ffi
    pr = PROBES[which]
    us = ffi.copy_time(COPY_BYTES, iters=10)
    log(f"[traffic-probe] copy kernel {COPY_BYTES >> 20} MiB: {us:.1f} us, {2 * COPY_BYTES / us / 1e3:.0f} GB/s read+write")
    if "rows" in pr:
        us = ffi.matmul_time(pr["dtype"], pr["rows"], pr["cols"], pr["m"], pr["epi"], 0, 20, 4)
        log(f"[traffic-probe] {pr['what']}: {us:.2f} us, {probe_bytes(pr) / us / 1e3:.0f} GB/s of weight bytes")
        return
    rng = np.random.default_rng(1)
    for it in range(8):
        q = rng.standard_normal((pr["m"], pr["nq"], pr["hd"]), np.float32)
        k = rng.standard_normal((pr["base"] + pr["m"], pr["nkv"], pr["hd"]), np.float32)
        v = rng.standard_normal((pr["base"] + pr["m"], pr["nkv"], pr["hd"]), np.float32)
        if "kv_bits" in pr:
            out = ffi.attention_quantized(q, k, v, pr["base"], pr["kv_bits"], pr["kv_bits"])[0]
        else:
            out = ffi.attention(q, k, v, pr["base"])
        assert np.isfinite(out).all()
    log(f"[traffic-probe] {pr['what']}: 8 launches, {probe_bytes(pr)} algorithmic bytes each")


def per_kernel_counters(path, which):
    """{counter: {"copy" | "kernel": [value per dispatch]}} from a counter-collection CSV of --traffic-probe."""
    import csv
    match = PROBES[which]["match"]
    acc = {}
    for r in csv.DictReader(open(path)):
        key = "copy" if "k_copy_probe" in r["Kernel_Name"] else "kernel" if match in r["Kernel_Name"] else None
        if key:
            acc.setdefault(r["Counter_Name"], {}).setdefault(key, []).append(float(r["Counter_Value"]))
    return acc


def traffic_summary(fetch_csv, write_csv, which):
    """HBM bytes per launch of the probed kernel from two counter-collection CSVs of
    `bench.py --traffic-probe` (FETCH_SIZE and WRITE_SIZE, KiB-like units per dispatch), each
    scaled by what the same counter reads for the copy kernel of known size."""
    alg = probe_bytes(PROBES[which])
    out = {"kernel": PROBES[which]["what"], "algorithmic_bytes_per_launch": alg}
    for name, path, counter in (("read", fetch_csv, "FETCH_SIZE"), ("write", write_csv, "WRITE_SIZE")):
        acc = per_kernel_counters(path, which)[counter]
        avg = {k: sum(v) / len(v) for k, v in acc.items()}
        factor = COPY_BYTES / avg["copy"]          # bytes per counter unit, from the copy kernel
        out[name] = dict(counter=counter, copy_kernel_reading=round(avg["copy"], 1), bytes_per_unit=round(factor, 2),
                         kernel_reading=round(avg["kernel"], 1), kernel_bytes=int(avg["kernel"] * factor),
                         dispatches={k: len(v) for k, v in acc.items()})
    out["traffic_bytes_per_launch"] = out["read"]["kernel_bytes"] + out["write"]["kernel_bytes"]
    out["traffic_over_algorithmic"] = round(out["traffic_bytes_per_launch"] / alg, 3)
    print(json.dumps(out, indent=1))


def step_traffic(fetch_csv, write_csv, first="k_clear_result"):
    """HBM bytes per launch of every kernel of the verify passes, from two `rocprofv3 --pmc` collections (FETCH_SIZE,
    then WRITE_SIZE) of `bench.py --copy-probe ...`: dispatches from the first acceptance kernel on, keyed by kernel
    name and grid like --trace-summary, each counter scaled by what it reads for the copy kernel of known size that
    --copy-probe launches in the same process.  The last line is the whole run's bytes over its passes (one k_embed
    each)."""
    import csv
    tables, passes = {}, 0
    for side, path, counter in (("read", fetch_csv, "FETCH_SIZE"), ("write", write_csv, "WRITE_SIZE")):
        rows = [r for r in csv.DictReader(open(path)) if r["Counter_Name"] == counter]
        rows.sort(key=lambda r: int(r["Dispatch_Id"]))
        copies = [float(r["Counter_Value"]) for r in rows if "k_copy_probe" in r["Kernel_Name"]]
        factor = COPY_BYTES / (sum(copies) / len(copies))
        start = next(i for i, r in enumerate(rows) if first in r["Kernel_Name"])
        passes = sum("k_embed" in r["Kernel_Name"] for r in rows[start:])
        for r in rows[start:]:
            name = r["Kernel_Name"].replace("tsv::", "").replace("(anonymous namespace)::", "").split("(")[0].replace("void ", "")
            key = (name, int(r["Grid_Size"]) // max(int(r["Workgroup_Size"]), 1))
            st = tables.setdefault(key, {"read": [0, 0.0], "write": [0, 0.0]})[side]
            st[0] += 1
            st[1] += float(r["Counter_Value"]) * factor
        print(f"# {counter}: {factor:.2f} bytes per unit ({len(copies)} copy launches of {COPY_BYTES} B)")
    print(f"{'kernel':44s} {'wgs':>6s} {'calls':>7s} {'read_B/launch':>14s} {'written_B/launch':>17s}")
    tot = [0.0, 0.0]
    for (name, wgs), v in sorted(tables.items(), key=lambda kv: -(kv[1]["read"][1] + kv[1]["write"][1])):
        rd, wr = v["read"], v["write"]
        tot[0] += rd[1]
        tot[1] += wr[1]
        print(f"{name[:44]:44s} {wgs:6d} {rd[0]:7d} {rd[1] / max(rd[0], 1):14.0f} {wr[1] / max(wr[0], 1):17.0f}")
    print(f"all dispatches from the first {first} on: {tot[0] / passes:.0f} B read + {tot[1] / passes:.0f} B written per pass "
          f"({passes} passes)")


def counter_summary(path, which):
    """Per-dispatch averages of every counter in a `rocprofv3 --pmc ... --output-format csv` collection of
    `bench.py --traffic-probe`, for the probed kernel's launches (the copy kernel is left out)."""
    acc = {c: d["kernel"] for c, d in per_kernel_counters(path, which).items() if "kernel" in d}
    print(json.dumps({"kernel": PROBES[which]["what"]} | {k: round(sum(v) / len(v), 1) for k, v in sorted(acc.items())} |
                     {"dispatches": len(next(iter(acc.values())))}, indent=1))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--trace-summary", default=None, metavar="CSV",
                    help="summarise a rocprofv3 kernel-trace CSV of this script (verify steps only) and exit")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="run the copy kernel of known size and the dominant matmul (for rocprofv3 --pmc) and exit")
    ap.add_argument("--counter-summary", default=None, metavar="CSV",
                    help="per-dispatch averages of the counters a rocprofv3 --pmc run of --traffic-probe collected")
    ap.add_argument("--traffic-summary", nargs=2, default=None, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="HBM bytes per launch of the dominant matmul from two --pmc runs of --traffic-probe")
    ap.add_argument("--step-traffic", nargs=2, default=None, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="HBM bytes per launch of every kernel of the verify passes from two --pmc runs of this script "
                         "with --copy-probe")
    ap.add_argument("--copy-probe", action="store_true",
                    help="for a --pmc run: launch the copy kernel of known size before the workload (it calibrates the "
                         "counters) and leave out the per-kernel timing, whose passes launch one kernel class twice")
    ap.add_argument("--probe", default="gate_up", choices=sorted(PROBES),
                    help="which kernel --traffic-probe runs and the two summaries read")
    ap.add_argument("--trace-from", default="k_clear_result", metavar="KERNEL",
                    help="--trace-summary counts dispatches from the first one of this kernel on")
    ap.add_argument("--prefill-bench", type=int, default=0, metavar="TOKENS",
                    help="time tsv_prefill over a prompt of this many tokens (after one untimed run of the same), print one "
                         "JSON line and exit")
    ap.add_argument("--weights-dtype", default=None, choices=["q4_k", "q8_0", "bf16", "q4_k_m", "q5_k_m"],
                    help="--prefill-bench: the dense workload's shape with its matrices in this storage type")
    ap.add_argument("--loop-bench", type=int, default=0, metavar="NEW_TOKENS",
                    help="end to end instead of one step: generate this many tokens with the library's loop and its "
                         "drafter head (one decoder layer of the workload's shape, draft cost inside the timed region); "
                         "prints verified tokens/s with the acceptance the synthetic weights give")
    ap.add_argument("--weak-layers", type=float, default=1.0,
                    help="--loop-bench: scale of what each layer adds to the stream; below 1 the target's picks follow "
                         "the last token's embedding, which the synthetic head predicts (sets the acceptance rate)")
    ap.add_argument("--embed-scale", type=float, default=1.0,
                    help="--loop-bench: scale of the embedding rows, to the same end (the final norm removes it)")
    ap.add_argument("--greedy", action="store_true", help="--loop-bench: temperature 0 (block drafts chained on the device)")
    ap.add_argument("--step-drafts", action="store_true", help="--loop-bench: draft step by step even when greedy")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="llama3_8b_q4_k_k4_ctx4096", choices=sorted(WORKLOADS))
    ap.add_argument("--layers", type=int, default=None, help="debug: build only this many layers")
    ap.add_argument("--routing", default="model", choices=["model", "independent"],
                    help="routed-expert workloads: 'independent' forces every row of every layer onto top_k experts drawn "
                         "uniformly and independently (tsv_force_route) instead of the synthetic router's own, nearly "
                         "row-independent choice; a secondary measurement, labelled in the line")
    ap.add_argument("--kv-bits", default="off", choices=["off", "2", "3", "3.5", "4"],
                    help="TurboQuant KV rows on the layers the reference's policy names (crates/model-io/src/kv_quant.rs); "
                         "a secondary measurement, labelled in the line -- the headline workloads keep fp16 rows")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seed", type=int, default=20261125)
    args = ap.parse_args()
    if args.trace_summary:
        trace_summary(args.trace_summary, args.trace_from)
        return
    if args.traffic_probe:
        traffic_probe(args.probe)
        return
    if args.counter_summary:
        counter_summary(args.counter_summary, args.probe)
        return
    if args.traffic_summary:
        traffic_summary(*args.traffic_summary, args.probe)
        return
    if args.step_traffic:
        step_traffic(*args.step_traffic, args.trace_from)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the verify step on ONE GPU; --gpus N with N > 1 is not "
                 "supported: every number here is one GPU's throughput.")

    import turbospark_amd as ts
    from turbospark_amd import hip, synth

    wl = WORKLOADS[args.workload]
    cfg = dict(synth.CONFIGS[wl["model"]])
    if args.layers:
        cfg["n_layers"] = args.layers
    k, ctx, T = wl["k"], wl["ctx"], wl["temperature"]
    m = k + 1
    cfg["max_context"] = ctx + 32
    V = cfg["vocab"]

    if args.weights_dtype:
        if not args.prefill_bench or cfg.get("n_experts"):
            sys.exit("bench.py: --weights-dtype goes with --prefill-bench at a dense workload")
        cfg["dtype"] = {"q4_k": ts.ffi.Q4_K, "q8_0": ts.ffi.Q8_0, "bf16": ts.ffi.BF16, "q4_k_m": ts.ffi.Q4_K,
                        "q5_k_m": ts.ffi.Q5_K}[args.weights_dtype]
        if args.weights_dtype.endswith("_m"):
            # the tensor mix of a *_K_M file: value and down projections in Q6_K in the first and last eighth of the
            # layers and every third layer between, and the output head
            n = cfg["n_layers"]
            more = [i for i in range(n) if i < n // 8 or i >= 7 * n // 8 or (i - n // 8) % 3 == 2]
            cfg["overrides"] = {"lm_head": ts.ffi.Q6_K}
            for i in more:
                cfg["overrides"][(i, "wv")] = cfg["overrides"][(i, "w_down")] = ts.ffi.Q6_K
    if args.loop_bench and args.weak_layers != 1.0:
        cfg["weak_layers"] = args.weak_layers
    if args.loop_bench and args.embed_scale != 1.0:
        cfg["embed_scale"] = args.embed_scale
    t0 = time.time()
    weights = synth.make_weights(cfg, seed=args.seed)
    log(f"[bench] synthetic {wl['model']} weights ({cfg['n_layers']} layers) in {time.time() - t0:.1f}s")
    t0 = time.time()
    kv_bits = ts.producer.parse_kv_bits(args.kv_bits)
    eng = ts.HipVerifier(cfg, weights, kv_bits=kv_bits)
    log(f"[bench] upload + re-tile in {time.time() - t0:.1f}s")
    rng = np.random.default_rng(args.seed)
    if args.prefill_bench:
        n = args.prefill_bench
        if n >= cfg["max_context"]:
            sys.exit(f"bench.py: --prefill-bench takes at most {cfg['max_context'] - 1} tokens at this workload")
        prompt = rng.integers(0, V, n).astype(np.int32)
        eng.prefill(prompt, 0, want_logits=False)     # untimed: first-use allocations, code objects
        eng.reset()
        t0 = time.perf_counter()
        eng.prefill(prompt, 0, want_logits=False)     # returns after the stream has drained
        dt = time.perf_counter() - t0
        wide = cfg["dtype"] in (ts.ffi.Q4_K, ts.ffi.Q5_K, ts.ffi.Q8_0, ts.ffi.BF16) and not (cfg.get("n_experts") and os.environ.get("TSV_MOE_FP4"))
        rows = 64 if wide and os.environ.get("TSV_WIDE_PREFILL") != "0" else 16
        print(json.dumps({"metric": "prefill tokens/s", "value": round(n / dt, 1), "unit": "tokens/s", "n_gpus": 1,
                          "higher_is_better": True, "dtype": "f16", "data": "synthetic", "seconds": round(dt, 4),
                          "config": {"workload": args.workload, "weights": args.weights_dtype or "as the workload names",
                                     "layers": cfg["n_layers"], "prompt_tokens": n,
                                     "rows_per_pass": rows, "logits": "none (headless passes)"}}))
        return
    if args.loop_bench:
        loop_bench(args, ts, synth, cfg, weights, eng, wl, rng)
        return
    prompt = rng.integers(0, V, ctx).astype(np.int32)
    t0 = time.time()
    if args.copy_probe:
        # a counter run: the prompt goes one pass per call, each ending with the stream drained (with a few thousand
        # launches queued ahead of the device the counter collection has crashed inside the profiler)
        step = 64 if eng.cfg["dtype"] == ts.ffi.Q4_K and not eng.cfg.get("n_experts") else 16
        for i in range(0, ctx - 1, step):
            eng.prefill(prompt[i:min(i + step, ctx - 1)], i, want_logits=False)
    else:
        eng.prefill(prompt[:-1], 0, want_logits=False)   # the last prompt token is the round's confirmed token
    if args.copy_probe:
        us = ts.ffi.copy_time(COPY_BYTES, iters=3)
        log(f"[bench] copy kernel {COPY_BYTES >> 20} MiB: {us:.1f} us")
    prefill_s = time.time() - t0                      # first use: includes one-time allocations (--prefill-bench times it properly)
    log(f"[bench] prefill of {ctx - 1} tokens in {prefill_s:.2f}s")
    base = eng.position
    point = eng.checkpoint()
    anchor = int(prompt[-1])
    if args.routing == "independent":
        if not cfg.get("n_experts"):
            sys.exit("bench.py: --routing independent needs a routed-expert workload")
        forced = np.full((cfg["n_layers"], 16, 8), -1, np.int32)
        for l in range(cfg["n_layers"]):
            for r in range(16):
                forced[l, r, :cfg["top_k"]] = rng.permutation(cfg["n_experts"])[:cfg["top_k"]]
        eng.force_route(forced)

    # drafter logits N(0,1) per round, resident on the device; proposals drawn on the device
    rounds = args.warmup + args.steps
    shaping = [ts.shaping(T, seed=args.seed + r) if T > 0 else ts.shaping(0.0) for r in range(rounds)]
    tree = TREE16 if wl.get("tree") else None
    drows = m if tree else k      # a tree round needs the drafter's row of every node
    draft_host = rng.standard_normal((rounds, drows, V)).astype(np.float16)
    draft_dev = hip.DeviceBuffer(draft_host.nbytes).upload(draft_host)
    row_bytes = drows * V * 2
    feeds, draw_steps = [], []
    for r in range(rounds):
        if tree:   # node tokens uniform over the vocabulary
            feeds.append([anchor] + [int(t) for t in rng.integers(0, V, k)])
            draw_steps.append(0)
            continue
        props, ds = eng.draft_chain((draft_dev.address(r * row_bytes), k), shaping[r], 0)
        feeds.append([anchor] + [int(t) for t in props])
        draw_steps.append(ds)

    def step(r):
        res = eng.verify_accept(feeds[r], base, shaping[r], parent=tree,
                                draft_logits=draft_dev.address(r * row_bytes) if T > 0 else None,
                                draw_step=draw_steps[r])
        eng.rollback(point)   # every step verifies at exactly `ctx` tokens of context
        return res

    for r in range(args.warmup):
        step(r)
    stream = eng.stream
    e0, e1 = hip.Event(), hip.Event()
    hip.check(hip.rt().hipStreamSynchronize(stream), "sync")
    e0.record(stream)
    t0 = time.perf_counter()
    results = [step(args.warmup + i) for i in range(args.steps)]
    hip.check(hip.rt().hipStreamSynchronize(stream), "sync")
    wall = time.perf_counter() - t0
    e1.record(stream)
    e1.sync()
    gpu_ms = e1.ms_since(e0)
    verified = sum(r.accepted + 1 for r in results)
    mean_acc = float(np.mean([r.accepted for r in results]))
    min_margin = min(r.min_margin for r in results)
    ms_per_step = wall * 1000.0 / args.steps

    # Per-kernel durations inside the pipeline, with HIP events on the engine's stream around
    # whole timed regions only: a region in which every launch of one kernel class is issued
    # twice (same inputs, same outputs) takes longer than the plain region by exactly that
    # class's launches.  (An event pair around each single launch adds ~2 us to a 5-20 us
    # kernel; those readings are kept as profile_ms_per_step for the coarse breakdown.)
    def timed_region(n):
        hip.check(hip.rt().hipStreamSynchronize(stream), "sync")
        a, b = hip.Event(), hip.Event()
        a.record(stream)
        for i in range(n):
            step(args.warmup + (i % args.steps))
        b.record(stream)
        b.sync()
        return b.ms_since(a) / n

    nrep = min(10, args.steps)
    plain_ms = timed_region(nrep)
    # routed experts: the experts the timed steps actually chose, read back from the device in a pass
    # of their own (the same feeds route the same way: the pass is deterministic)
    union = None
    if cfg.get("n_experts"):
        per_step = []
        for i in range(min(args.steps, 20)):
            step(args.warmup + i)
            sel = eng.route_selected()[:, :m, :cfg["top_k"]]
            per_step.append(np.mean([len(np.unique(sel[l])) for l in range(sel.shape[0])]))
        union = float(np.mean(per_step))
    ab = algorithmic_bytes(cfg, ctx, m, union, kv_bits)
    L = cfg["n_layers"]
    kern = {}
    for name, nbytes, count in (("qkv", ab["per_layer"]["qkv"], L), ("wo", ab["per_layer"]["wo"], L),
                                ("gate_up", ab["per_layer"]["gate_up"], L), ("down", ab["per_layer"]["down"], L),
                                ("head", ab["head"], 1), ("attention", ab["kv"] // L, L), ("rope_kv", 0, L)):
        if args.copy_probe:   # a counter run: every pass plain, so that the collection divides evenly by its passes
            avg_ms = 0.0
        else:
            eng.set_repeat(name, 2)
            twice_ms = timed_region(nrep)
            eng.set_repeat(name, 1)
            avg_ms = (twice_ms - plain_ms) / count
        kern[name] = dict(avg_us=round(avg_ms * 1000, 2), bytes=int(nbytes), launches_per_step=count,
                          GBps=round(nbytes / (avg_ms * 1e-3) / 1e9, 1) if nbytes and avg_ms > 0 else None)
    gemm_ms = sum(kern[n]["avg_us"] * kern[n]["launches_per_step"] for n in ("qkv", "wo", "gate_up", "down", "head")) / 1000.0

    # coarse breakdown: an event pair around every launch
    eng.set_profile(True)
    nprof = min(5, args.steps)
    for i in range(nprof):
        step(args.warmup + i)
    prof = eng.get_profile()
    eng.set_profile(False)
    if prof.get("rope_kv", (0.0, 0))[1] == 0:  # the q/k/v projection rotates and stores its own rows: no such launch
        kern.pop("rope_kv", None)
        prof.pop("rope_kv", None)
        kern["qkv"]["epilogue"] = "bias + rotation + fp16 q / KV-cache stores"
    dom = kern.get("gate_up", {})
    peak = 8000.0
    # the recorded figures are the workload's as named: not a variant's (other KV rows, forced routing, fewer layers)
    rec = {} if (kv_bits or args.routing != "model" or args.layers) else recorded(args.workload)
    roofline = dict(bound="hbm",
                    kernel=f"router + grouped expert gate/up matmuls (experts actually routed: {union:.1f} of {cfg['n_experts']} per layer)"
                    if cfg.get("n_experts")
                    else "k_gemm<Q4_K> gate/up (silu-mul epilogue)" if cfg["dtype"] == 12 else "k_gemm<Q8_0> gate/up",
                    achieved=dom.get("GBps"), peak=peak, unit="GB/s",
                    frac=round((dom.get("GBps") or 0.0) / peak, 4),
                    timing="live: HIP events on the engine's stream around timed regions, the region with this kernel class "
                           "launched twice minus the plain region, per launch",
                    traffic=rec.get("traffic"), traffic_source=rec.get("traffic_source", "not measured for this workload"),
                    # the same kernel in the committed rocprofv3 kernel trace (begin-to-end of the dispatch, which
                    # includes what overlaps with its neighbours in the pipeline): the lower of the two fractions
                    trace_avg_launch_us=round(rec["trace_avg_us"], 2) if rec.get("trace_avg_us") else None, trace_source=rec.get("trace_source"),
                    trace_frac=round(dom["bytes"] / (rec["trace_avg_us"] * 1e-6) / 1e9 / peak, 4) if rec.get("trace_avg_us") and dom.get("bytes") else None,
                    algorithmic_bytes_per_launch=dom.get("bytes"), avg_launch_us=dom.get("avg_us"),
                    all_matmuls_GBps=round(ab["weights"] / (gemm_ms * 1e-3) / 1e9, 1) if gemm_ms else None,
                    step_algorithmic_bytes=int(ab["total"]),
                    step_traffic=rec.get("step_traffic"), step_traffic_source=rec.get("step_traffic_source"),
                    step_frac_of_hbm_roofline=round(ab["total"] / (ms_per_step * 1e-3) / 1e9 / peak, 4),
                    per_kernel=kern,
                    profile_ms_per_step={n: round(v[0] / nprof, 4) for n, v in prof.items()})

    cpu = None
    if not args.no_cpu_baseline and not kv_bits:   # the baseline leg is the headline workloads' (fp16 rows)
        cpu = cpu_baseline(cfg, weights, eng, base, feeds[args.warmup], mean_acc, tree)

    out = {
        "metric": "verified tokens/s + verify-step latency (8B Q4_K, k=4, 4K ctx); % HBM roofline",
        "value": round(verified / wall, 2), "unit": "verified tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16",
        "dtype_detail": {12: "q4_k", 8: "q8_0", 30: "bf16"}[cfg["dtype"]] +
                        " weight codes as exact f16 x f16 activations on MFMA, f32 accumulate" +
                        ("" if not cfg.get("n_experts") else
                         "; mxfp4 experts as f16 x f16 too" if os.environ.get("TSV_MOE_FP4", "0") not in ("2", "3") else
                         "; mxfp4 experts as stored on the block-scaled fp4 x fp8 MFMA (TSV_MOE_FP4), activations as " +
                         ("three" if os.environ.get("TSV_MOE_FP4") == "3" else "two") + " block-scaled e4m3 terms") +
                        "; f64 acceptance",
        "data": "synthetic",
        "config": {"workload": args.workload, "layers": cfg["n_layers"], "rows": m, "context": ctx,
                   "temperature": T, "mean_accepted": round(mean_acc, 3), "min_margin": min_margin,
                   **({"kv_rows": f"TurboQuant K{kv_bits[0]}/V{kv_bits[1]} on every full-attention layer but the last"} if kv_bits else {}),
                   **({"experts_routed_per_layer": round(union, 2),
                       "routing": "the synthetic router's own" if args.routing == "model" else
                                  "forced: top_k experts per row drawn uniformly and independently"} if union is not None else {})},
        "roofline": roofline, "cpu_baseline": cpu,
        # outside the timed region: how the cache the steps read was filled
        "prefill": {"tokens": ctx - 1, "seconds": round(prefill_s, 3), "tokens_per_s": round((ctx - 1) / prefill_s, 1)},
    }
    print(json.dumps(out), flush=True)


def loop_bench(args, ts, synth, cfg, weights, eng, wl, rng):
    """Verified tokens/s of the whole loop: prompt of ctx - NEW tokens, then NEW tokens generated by
    tsv_run_speculative with the drafter head inside the library (chain rounds of the workload's k).  The timed
    region is the difference of two runs of the same prompt, one generating 1 token and one 1 + NEW: every
    draft step, verify pass, acceptance and truncation of the NEW tokens, and nothing of the prompt."""
    k, ctx, V = wl["k"], wl["ctx"], cfg["vocab"]
    T = 0.0 if args.greedy else wl["temperature"]
    new = args.loop_bench
    hcfg, hw = synth.make_mtp_weights(cfg, weights, seed=args.seed + 1, follow=256.0, norm_jitter=0.0)
    head = ts.MtpHead(eng, hcfg, hw)
    prompt = rng.integers(0, V, ctx - new).astype(np.int32)
    sh = ts.shaping(T, seed=args.seed) if T > 0 else ts.shaping(0.0)

    def run(n_new):
        t0 = time.perf_counter()
        r = eng.run_speculative(prompt, head, sh, n_new, k, block_drafts=not args.step_drafts)
        return time.perf_counter() - t0, r

    run(k + 2)   # untimed: first-use allocations, code objects
    t_a, _ = run(1)
    t_b, r = run(1 + new)
    dt = t_b - t_a
    log(f"[bench] prompt of {prompt.size} tokens + 1 token: {t_a:.2f}s; + {new} more: {t_b:.2f}s")
    # the draft side alone: the block of k chained steps (plus the row-only step) from where the run ended
    pos = eng.position
    reps = 20
    head.draft_block(r["tokens"][-1], pos, k)
    t0 = time.perf_counter()
    for _ in range(reps):
        head.rewind(pos - 1)
        head.draft_block(r["tokens"][-1], pos, k)
    draft_ms = (time.perf_counter() - t0) * 1e3 / reps
    head.rewind(pos - 1)
    # plain decoding on the same handle at the same context: one-row rounds (pass, device arg-max, no draft)
    tok, plain_n = int(r["tokens"][-1]), min(64, eng.cfg["max_context"] - pos - 1)
    greedy = ts.shaping(0.0)
    t0 = time.perf_counter()
    for i in range(plain_n):
        tok = eng.verify_accept([tok], pos + i, greedy).next
    plain_s = time.perf_counter() - t0
    print(json.dumps({
        "metric": "verified tokens/s, end to end (drafter head inside the library)", "value": round(new / dt, 1),
        "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "f16", "data": "synthetic",
        "new_tokens": new, "seconds": round(dt, 4), "rounds": r["rounds"], "offered": r["offered"],
        "accepted": r["accepted"], "tokens_per_round": round(new / max(r["rounds"], 1), 3),
        "ms_per_round": round(dt * 1e3 / max(r["rounds"], 1), 3),
        "prompt_tokens_per_s": round(prompt.size / t_a, 1), "draft_ms_per_block": round(draft_ms, 3),
        "plain_decode_tokens_per_s": round(plain_n / plain_s, 1), "vs_plain_decode": round(new / dt / (plain_n / plain_s), 2),
        "config": {"workload": args.workload, "layers": cfg["n_layers"], "block": k, "temperature": T,
                   "drafts": "step by step" if args.step_drafts else "block, chained on the device" + (" (drawn there)" if T > 0 else ""),
                   "weak_layers": args.weak_layers, "embed_scale": args.embed_scale, "prompt_tokens": int(prompt.size)}}))


def cpu_baseline(cfg, weights, eng, base, feed, mean_acc, parent=None):
    """The oracle (the CPU restatement of the reference path) timed on this host, one thread, on
    a bounded sample: the first two layers plus the output head of the same verify step, and
    the head alone; the full-stack time is extrapolated linearly in the layer count."""
    from oracle import binding as ob
    L = cfg["n_layers"]
    sample_layers = min(2, L)

    def timed(threads):
        cpu = ob.Model(cfg, weights, round_kv_f16=True, threads=threads)
        for layer in range(sample_layers):
            kg, vg = eng.read_kv(layer, 0, base)
            kc, vc = cpu.kv(layer)
            kc[:base] = kg.astype(np.float32)
            vc[:base] = vg.astype(np.float32)
        cpu.rewind_to(base)
        t0 = time.perf_counter()
        cpu.verify(feed, base, parent=parent, n_layers_run=0)
        t_head = time.perf_counter() - t0
        cpu.rewind_to(base)
        t0 = time.perf_counter()
        cpu.verify(feed, base, parent=parent, n_layers_run=sample_layers)
        t_sample = time.perf_counter() - t0
        return t_head, t_sample, t_head + (t_sample - t_head) * L / sample_layers

    # the same sample with the oracle's rows spread over the host cores this process may use (the
    # reference itself is single-threaded: `value` stays the one-thread figure)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores) or cores)))
    many = None
    if cores > 1:
        _, _, t_many = timed(cores)
        many = {"value": round((mean_acc + 1.0) / t_many, 4), "cores": cores, "seconds_per_step_extrapolated": round(t_many, 3)}
    t_head, t_sample, t_full = timed(1)
    return {"all_cores": many, "value": round((mean_acc + 1.0) / t_full, 4), "unit": "verified tokens/s", "cores": 1, "kind": "port",
            "sample": f"oracle forward of the same verify step, {sample_layers} of {L} layers + output head "
                      f"({t_sample:.2f}s) and head alone ({t_head:.2f}s), extrapolated to {L} layers = {t_full:.2f}s; "
                      "acceptance excluded (ms-scale)",
            "seconds_per_step_extrapolated": round(t_full, 3)}


if __name__ == "__main__":
    main()
