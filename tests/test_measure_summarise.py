"""The rocprofv3 summariser behind profiles/ on small synthetic CSV files (no GPU, no profiler needed)."""
import csv

from llm_reproducibility_amd.measure import summarise


def _write(path, header, rows):
    path.parent.mkdir(parents=True, exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(header)
        w.writerows(rows)


def _trace(tmp_path, rows):
    """rows: (kernel, start ns, end ns)"""
    _write(tmp_path / "pid" / "r_kernel_trace.csv", ["Kernel_Name", "Start_Timestamp", "End_Timestamp"], rows)


def test_kernels_table_and_dispatch_order_sequence(tmp_path, capsys):
    rows = [("void tbik::big(int)", 1000 * i, 1000 * i + 200_000 + 1000 * (30 - i)) for i in range(30)]
    rows += [("void tbik::small(int)", 50_000_000 + 10 * i, 50_000_000 + 10 * i + 5000) for i in range(4)]
    rows += [("at::native::other", 60_000_000, 60_010_000)]
    _trace(tmp_path, rows)
    assert summarise.main(["kernels", str(tmp_path), "--only", "tbik::", "--sequence", "big"]) == 0
    out = capsys.readouterr().out
    lines = out.splitlines()
    assert lines[1].startswith("tbik::big(int)") and " 30 " in lines[1]          # sorted by total time, `void ` dropped
    assert lines[2].startswith("tbik::small(int)") and "5.0" in lines[2]
    assert "other" not in out
    assert "30 dispatches, 30 of them above 60 % of the longest" in out
    assert "last 20: mean 210.5 us, min 201.0, max 220.0" in out


def test_counters_scaled_by_the_largest_copy_dispatch(tmp_path, capsys):
    head = ["Kernel_Name", "Counter_Name", "Counter_Value", "Grid_Size", "Workgroup_Size"]
    rows = [("__amd_rocclr_copyBuffer", "FETCH_SIZE", 24576.0, 131072, 256),     # the calibration copy: 49152 KiB
            ("__amd_rocclr_copyBuffer", "FETCH_SIZE", 8.0, 512, 256),            # a small copy of the runtime's own
            ("tbik::k(int)", "FETCH_SIZE", 1000.0, 1024, 256), ("tbik::k(int)", "FETCH_SIZE", 3000.0, 1024, 256),
            ("tbik::k(int)", "FETCH_SIZE", 10.0, 64, 256)]
    _write(tmp_path / "pid" / "r_counter_collection.csv", head, rows)
    assert summarise.main(["counters", str(tmp_path), "--kernel", "tbik::", "--copy-kib", "49152", "--by-grid"]) == 0
    out = capsys.readouterr().out
    assert "FETCH_SIZE reads 24576 -> scale factor 2.000" in out
    assert "[grid 1024 x wg 256]" in out and "[grid 64 x wg 256]" in out
    assert "2000  (2 dispatches)   x 2.000 KiB = 4.1 MB per dispatch" in out     # mean 2000 KiB x 2 = 4096000 B
    assert summarise.main(["counters", str(tmp_path), "--kernel", "tbik::", "--largest", "1"]) == 0
    assert "3000  (1 dispatches)" in capsys.readouterr().out


def test_decode_breakdown_finds_the_steps_from_the_attention_launches(tmp_path, capsys):
    t = [0]

    def k(name, us):
        t[0] += 1000
        start = t[0]
        t[0] += int(us * 1000)
        return (name, start, t[0])
    rows = [k("warmup_kernel", 50.0)]
    for _step in range(3):
        rows.append(k("embedding_lookup", 2.0))
        for _layer in range(2):
            rows += [k("tbik::gemm_single_acc_stream_rows_kernel<3>", 10.0), k("tbik::qk_norm_rope_cache_kernel", 3.0),
                     k("tbik::attention_group_kernel<4, true>", 5.0), k("tbik::gemm_tree_strip_kernel<2, 4>", 7.0)]
        rows.append(k("tbik::argmax_rows_kernel", 1.0))
    _trace(tmp_path, rows)
    assert summarise.main(["decode", str(tmp_path), "--layers", "2", "--steps", "2"]) == 0
    out = capsys.readouterr().out
    # a step = 2 us of library kernels + 2 x 25 us + 1 us = 53 us, 26.5 us per layer, (1 + 8 + 1) / 2 launches per layer
    assert "kernels   26.5 us per layer (   53.0 us per step), 5.0 launches per layer" in out
    assert "attention" in out and "5.0 us per layer" in out
    assert "batch-invariant mm (streaming kernels" in out and "10.0 us per layer" in out
