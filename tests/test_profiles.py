"""The counter figure bench.py reports as roofline.traffic is the one the committed counter summary holds."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _rows(section_text, needle):
    rows = []
    for line in section_text.splitlines():
        if needle in line and line.startswith("|"):
            cells = [c.strip() for c in line.strip("|").split("|")]
            rows.append(dict(grid=int(cells[1]), calls=int(cells[2]), avg=float(cells[3]), min=float(cells[4]), max=float(cells[6])))
    return rows


def test_bench_traffic_constant_is_the_figure_of_the_committed_counter_summary():
    text = open(os.path.join(ROOT, "profiles", "gemv_sweep_pmc.md")).read()
    fetch = text[text.index("## FETCH_SIZE"):text.index("## WRITE_SIZE")]
    write = text[text.index("## WRITE_SIZE"):]
    needle = "gemv_mv_f16_kernelILi2ELi4ELi4ELi4"          # the dominant kernel: the three in >= 4096 shapes

    def per_shape(section):
        rows = {r["grid"]: r for r in _rows(section, needle)}
        big, two = rows[2097152], rows[524288]              # 16384x4096 alone; 4096x4096 (min) and 4096x16384 (max) together
        return big["avg"], two["min"], two["max"]
    f_big, f_small, f_wide = per_shape(fetch)
    w_big, w_small, w_wide = per_shape(write)
    # calibration stated in the same file: FETCH_SIZE x 2.0 = KiB read, WRITE_SIZE x 1.0 = KiB written
    assert re.search(r"FETCH_SIZE x 2\.0 = KiB read", text) and re.search(r"WRITE_SIZE x 1\.0 = KiB written", text)
    traffic = ((f_big + f_small + f_wide) * 2.0 + (w_big + w_small + w_wide)) / 3 * 1024
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert abs(bench.DOMINANT_KERNEL_TRAFFIC_BYTES - traffic) <= 0.0005 * traffic, (bench.DOMINANT_KERNEL_TRAFFIC_BYTES, traffic)
    algorithmic = sum(bench.gemv_bytes(n, k) for n, k in bench.SWEEP if k >= 4096) / 3
    assert 1.0 <= traffic / algorithmic <= 1.01       # no re-reads: the counters see the algorithmic bytes


def test_profile_summaries_name_the_kernels_the_library_builds():
    """Every pimhip kernel named in profiles/ exists in the sources (names drift when a kernel is re-templated)."""
    src = "".join(open(os.path.join(ROOT, "pimaicompiler_amd", "csrc", f)).read() for f in os.listdir(os.path.join(ROOT, "pimaicompiler_amd", "csrc")))
    for name in os.listdir(os.path.join(ROOT, "profiles")):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        for kernel in set(re.findall(r"pimhip::?(\w+_kernel)", text)) | set(re.findall(r"_ZN6pimhip\d+(\w+?_kernel)", text)):
            assert re.search(r"\b" + kernel + r"\b", src), (name, kernel)
    trace = open(os.path.join(ROOT, "profiles", "gemv_sweep_and_lstm_kernel_trace.md")).read()
    assert "lstm_seq_f16_kernel<2, true, 4, 16>" in trace and "decoder_step_f16_kernel<4, true>" in trace
