"""Tables from rocprofv3's CSV output for the kernels of libpimhip.so: durations per kernel and grid from a kernel trace
(`*_kernel_trace.csv`), counter values per dispatch from a counter run (`*_counter_collection.csv`).

    python -m pimaicompiler_amd.profile_tables trace out/bench_kernel_trace.csv
    python -m pimaicompiler_amd.profile_tables pmc out/p_counter_collection.csv

The summaries under profiles/ are made of these tables."""
import collections
import csv
import sys

# kernels of other libraries that the summaries keep: the copy kernel that calibrates the counters
KEEP = ("CUDAFunctorOnSelf_add",)
WIDTH = 70


def _ours(name):
    return "pimhip" in name or any(k in name for k in KEEP)


def _stats(values):
    v = sorted(values)
    return dict(calls=len(v), avg=sum(v) / len(v), min=v[0], median=v[len(v) // 2], max=v[-1])


def trace_rows(path):
    """[(kernel name cut to WIDTH, grid in work-items, stats of End - Start in ns)] sorted by name and grid."""
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        if _ours(r["Kernel_Name"]):
            agg[(r["Kernel_Name"][:WIDTH], int(r["Grid_Size_X"]) * int(r.get("Grid_Size_Y", 1) or 1) * int(r.get("Grid_Size_Z", 1) or 1))].append(
                int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    return [(k[0], k[1], _stats(v)) for k, v in sorted(agg.items())]


def pmc_rows(path):
    """[(kernel name cut to WIDTH, grid in work-items, stats of the counter value per dispatch)] sorted by name and grid."""
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        if _ours(r["Kernel_Name"]):
            agg[(r["Kernel_Name"][:WIDTH], int(r["Grid_Size"]))].append(float(r["Counter_Value"]))
    return [(k[0], k[1], _stats(v)) for k, v in sorted(agg.items())]


def table(rows, unit):
    out = [f"| kernel | grid (work-items) | calls | avg {unit} | min | median | max |", "|---|---|---|---|---|---|---|"]
    for name, grid, s in rows:
        out.append(f"| `{name}` | {grid} | {s['calls']} | {s['avg']:.1f} | {s['min']:.1f} | {s['median']:.1f} | {s['max']:.1f} |")
    return "\n".join(out)


def main(argv):
    if len(argv) != 3 or argv[1] not in ("trace", "pmc"):
        print(__doc__, file=sys.stderr)
        return 2
    print(table(trace_rows(argv[2]), "ns") if argv[1] == "trace" else table(pmc_rows(argv[2]), "KiB"))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
