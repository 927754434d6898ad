"""bench.py's own arithmetic, on the CPU: the algorithmic bytes of a verify step against a count by hand, the refusal
of more than one GPU, and the three summaries (kernel trace, dominant-kernel traffic, per-kernel step traffic) on
small hand-written rocprofv3 CSVs whose answers are known."""
import csv
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_algorithmic_bytes_of_the_headline_step_counted_by_hand():
    from turbospark_amd import synth
    b = _bench()
    cfg = synth.CONFIGS["llama3_8b_q4_k"]
    ab = b.algorithmic_bytes(cfg, 4096, 5)
    q4k = lambda rows, cols: rows * (cols // 256) * 144          # a Q4_K superblock: 256 weights in 144 bytes
    assert ab["per_layer"] == dict(qkv=q4k(4096 + 2 * 1024, 4096), wo=q4k(4096, 4096), gate_up=q4k(2 * 14336, 4096),
                                   down=q4k(4096, 14336))
    assert ab["per_layer"]["gate_up"] == 66060288 and ab["head"] == q4k(128256, 4096) == 295501824
    weights = 32 * (14155776 + 9437184 + 66060288 + 33030144) + 295501824
    kv = 32 * (4096 + 5) * 1024 * 2 * 2                          # K and V rows [0, ctx + m), fp16, once per layer
    small = 5 * (4096 // 256) * 144 + 5 * 128256 * 2 + 32 * 5 * 1024 * 2 * 2
    assert ab["weights"] == weights and ab["kv"] == kv and ab["total"] == weights + kv + small == 4760846080
    # quantized rows: a norm and packed indices per kv head and side, on every layer but the last
    tq = b.algorithmic_bytes(cfg, 4096, 5, kv_bits=(4, 4))
    assert tq["kv"] == 31 * (4096 + 5) * 2 * 8 * (4 + 64) + (4096 + 5) * 4096
    # routed experts: an expert counts once per layer in which a row chose it
    moe = dict(cfg, n_experts=128, top_k=8, expert_dtype=cfg["dtype"])
    assert b.algorithmic_bytes(moe, 64, 9, union=10.0)["per_layer"]["gate_up"] == 10 * q4k(2 * 14336, 4096) + q4k(128, 4096)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr


def _write(path, header, rows):
    with open(path, "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(header)
        w.writerows(rows)


def test_trace_summary_counts_from_the_first_acceptance_kernel(tmp_path, capsys):
    b = _bench()
    head = ["Kernel_Name", "Start_Timestamp", "End_Timestamp", "Grid_Size_X", "Workgroup_Size_X", "LDS_Block_Size"]
    rows = [("tsv::k_embed(int)", 0, 5000, 256, 256, 0),                 # a prompt pass: left out
            ("tsv::k_clear_result(int*)", 10000, 11000, 64, 64, 0),
            ("void tsv::k_gemm<1, 2>(float*)", 12000, 28000, 448 * 64, 64, 0),
            ("void tsv::k_gemm<1, 2>(float*)", 30000, 48000, 448 * 64, 64, 0),
            ("void tsv::k_gemm<1, 2>(float*)", 50000, 56000, 96 * 64, 64, 0)]   # same name, other grid: its own line
    p = tmp_path / "t.csv"
    _write(p, head, rows)
    b.trace_summary(str(p))
    out = capsys.readouterr().out.splitlines()
    line = next(l for l in out if l.startswith("k_gemm<1, 2>") and " 448 " in l).split()
    assert line[-7:-1] == ["448", "0", "2", "17.00", "16.00", "18.00"]   # workgroups, lds, calls, avg, min, max (us)
    assert any(l.startswith("k_gemm<1, 2>") and " 96 " in l and "6.00" in l for l in out)
    assert "k_embed" not in "\n".join(out)
    assert out[-1].startswith("total kernel time in verify steps: 0.041 ms")


def _counter_rows(counter, copy_reading, kernel_name, kernel_readings, grid=448 * 64, first=None):
    head = ["Dispatch_Id", "Kernel_Name", "Grid_Size", "Workgroup_Size", "Counter_Name", "Counter_Value"]
    rows, d = [], 1
    for _ in range(3):
        rows.append((d, "tsv::k_copy_probe(void*)", 1024 * 256, 256, counter, copy_reading))
        d += 1
    if first:
        rows.append((d, first, 64, 64, counter, 0.0))
        d += 1
    for v in kernel_readings:
        rows.append((d, kernel_name, grid, 64, counter, v))
        d += 1
    return head, rows


def test_traffic_summary_scales_each_counter_by_the_copy_kernel(tmp_path, capsys):
    import json
    b = _bench()
    f, w = tmp_path / "f.csv", tmp_path / "w.csv"
    # the copy kernel moves COPY_BYTES each way: here one FETCH unit is 2048 bytes, one WRITE unit 1024
    _write(f, *_counter_rows("FETCH_SIZE", b.COPY_BYTES / 2048, "void tsv::k_gemm<Q4K, 1, 2>(x)", [32000.0, 33000.0]))
    _write(w, *_counter_rows("WRITE_SIZE", b.COPY_BYTES / 1024, "void tsv::k_gemm<Q4K, 1, 2>(x)", [250.0, 254.0]))
    b.traffic_summary(str(f), str(w), "gate_up")
    out = json.loads(capsys.readouterr().out)
    assert out["algorithmic_bytes_per_launch"] == 66060288
    assert out["read"]["kernel_bytes"] == 32500 * 2048 and out["write"]["kernel_bytes"] == 252 * 1024
    assert out["traffic_bytes_per_launch"] == 32500 * 2048 + 252 * 1024
    assert out["traffic_over_algorithmic"] == round((32500 * 2048 + 252 * 1024) / 66060288, 3)


def test_step_traffic_gives_bytes_per_launch_and_per_pass(tmp_path, capsys):
    b = _bench()
    f, w = tmp_path / "f.csv", tmp_path / "w.csv"
    def rows(counter, unit, a, c):
        head, r = _counter_rows(counter, b.COPY_BYTES / unit, "void tsv::k_gemm<Q4K, 1, 2>(x)", a, first="tsv::k_clear_result(int*)")
        d = len(r) + 1
        for v in c:   # two passes, one k_embed each
            r.append((d, "tsv::k_embed(int)", 5 * 256, 256, counter, v))
            d += 1
        return head, r
    _write(f, *rows("FETCH_SIZE", 2048, [1000.0, 3000.0], [10.0, 30.0]))
    _write(w, *rows("WRITE_SIZE", 1024, [100.0, 300.0], [1.0, 3.0]))
    b.step_traffic(str(f), str(w))
    out = capsys.readouterr().out.splitlines()
    gemm = next(l for l in out if l.startswith("k_gemm<Q4K, 1, 2>")).split()
    assert gemm[-4:] == ["448", "2", str(2000 * 2048), str(200 * 1024)]
    embed = next(l for l in out if l.startswith("k_embed")).split()
    assert embed[-4:] == ["5", "2", str(20 * 2048), str(2 * 1024)]
    assert out[-1].startswith(f"all dispatches from the first k_clear_result on: {(4000 + 40) * 2048 // 2} B read + "
                              f"{(400 + 4) * 1024 // 2} B written per pass (2 passes)")


def test_the_recorded_figures_come_out_of_the_committed_profiles():
    """bench.py reads the dominant launch's trace duration and HBM traffic from the tables under profiles/: every
    measured workload finds its kernels there, the traffic is the algorithmic bytes plus a little, and a pass moves
    more than its algorithmic bytes and less than half as much again."""
    from turbospark_amd import synth
    b = _bench()
    assert set(b.PROFILED) == {"llama3_8b_q4_k_k4_ctx4096", "llama3_8b_q4_k_tree16_ctx16384",
                               "qwen3_30b_a3b_mxfp4_k8_ctx8192", "gptoss_120b_mxfp4_k8_ctx32768"}
    for w in b.PROFILED:
        r = b.recorded(w)
        assert r, w
        assert 5.0 < r["trace_avg_us"] < 80.0 and r["trace_source"].startswith("recorded: profiles/")
        wl = b.WORKLOADS[w]
        cfg = synth.CONFIGS[wl["model"]]
        if not cfg.get("n_experts"):
            gate_up = b.algorithmic_bytes(cfg, wl["ctx"], wl["k"] + 1)["per_layer"]["gate_up"]
            assert 1.0 <= r["traffic"] / gate_up < 1.05, (w, r["traffic"], gate_up)
        assert r["step_traffic"] > 3e9
    assert b.recorded("tiny_q8_0_k4_ctx256") == {}
