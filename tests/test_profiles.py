"""The counter figure bench.py reports as roofline.traffic is the one the committed counter summary holds, every sweep shape
has rows of its own in the committed profiler summaries, and the summaries name kernels that exist."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _shape_rows(text, header_starts_with):
    """The rows of the markdown table whose header starts with the given cell, as lists of cells."""
    lines = text.splitlines()
    start = next(i for i, l in enumerate(lines) if l.startswith("| " + header_starts_with))
    rows = []
    for line in lines[start + 2:]:
        if not line.startswith("|"):
            break
        rows.append([c.strip() for c in line.strip().strip("|").split("|")])
    return rows


def _bench():
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    return bench


def test_bench_traffic_constant_is_the_figure_of_the_committed_counter_summary():
    """roofline.traffic is recomputed here from the per-shape counter readings of profiles/gemv_sweep_pmc.md."""
    bench = _bench()
    text = open(os.path.join(ROOT, "profiles", "gemv_sweep_pmc.md")).read()
    # calibration stated in the same file: FETCH_SIZE x 2.0 = KiB read, WRITE_SIZE x 1.0 = KiB written
    assert re.search(r"FETCH_SIZE x 2\.0 = KiB read", text) and re.search(r"WRITE_SIZE x 1\.0 = KiB written", text)
    rows = {r[0]: r for r in _shape_rows(text, "shape (out x in)")}
    assert set(rows) == {f"{n}x{k}" for n, k in bench.SWEEP}          # every shape of the sweep has a row of its own
    per_shape = {}
    for n, k in bench.SWEEP:
        r = rows[f"{n}x{k}"]
        fetch, write = float(r[2]), float(r[4])
        traffic = (fetch * 2.0 + write) * 1024
        assert abs(traffic - float(r[5])) <= 1 and int(r[6]) == bench.gemv_bytes(n, k)
        assert 1.0 <= traffic / bench.gemv_bytes(n, k) <= 1.011        # no re-reads: the counters see the algorithmic bytes
        per_shape[(n, k)] = traffic
    dominant = [per_shape[s] for s in bench.SWEEP if s[1] >= 4096]     # the three in >= 4096 shapes: gemv_mv_f16_kernel<2,4,4,4>
    traffic = sum(dominant) / len(dominant)
    assert abs(bench.DOMINANT_KERNEL_TRAFFIC_BYTES - traffic) <= 0.0005 * traffic, (bench.DOMINANT_KERNEL_TRAFFIC_BYTES, traffic)


def test_every_sweep_shape_has_its_own_kernel_trace_row():
    """Per-shape fractions can be recomputed from profiles/: median duration per shape, of the GEMV and of the read-only
    kernel on the same matrices, one profiler run per shape."""
    bench = _bench()
    text = open(os.path.join(ROOT, "profiles", "gemv_sweep_per_shape_kernel_trace.md")).read()
    rows = {r[0]: r for r in _shape_rows(text, "shape (out x in)")}
    assert set(rows) == {f"{n}x{k}" for n, k in bench.SWEEP}
    for n, k in bench.SWEEP:
        r = rows[f"{n}x{k}"]
        median_ns, gbs, frac, probe_ns = float(r[5]), float(r[7]), float(r[8]), float(r[9])
        assert abs(bench.gemv_bytes(n, k) / median_ns - gbs) <= 0.1 and abs(gbs / bench.HBM_PEAK_GBS - frac) <= 0.001
        assert 0.5 <= frac <= 1.0 and 0.85 <= probe_ns / median_ns <= 1.1
        # the table of the shape's own run is in the file too
        assert f"## {n}x{k}" in text


def test_profile_summaries_name_the_kernels_the_library_builds():
    """Every pimhip kernel named in profiles/ exists in the sources (names drift when a kernel is re-templated)."""
    src = "".join(open(os.path.join(ROOT, "pimaicompiler_amd", "csrc", f)).read() for f in os.listdir(os.path.join(ROOT, "pimaicompiler_amd", "csrc")))
    for name in os.listdir(os.path.join(ROOT, "profiles")):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        for kernel in set(re.findall(r"pimhip::?(\w+_kernel)", text)) | set(re.findall(r"_ZN6pimhip\d+(\w+?_kernel)", text)):
            assert re.search(r"\b" + kernel + r"\b", src), (name, kernel)
    trace = open(os.path.join(ROOT, "profiles", "gemv_sweep_and_lstm_kernel_trace.md")).read()
    for kernel in ("lstm_seq_f16_kernel<2, true, 4, 16>", "decoder_step_f16_kernel<4, true>", "lstm_xcd_f16_kernel<true>", "moe_ffn_step_f16_kernel",
                   "rnnt_step_f16_kernel", "rnnt_greedy_f16_kernel"):
        assert kernel in trace, kernel
