"""The driver's entry points on the CPU: every global name that bench.py and __graft_entry__.py refer to inside their
functions exists (a name that only a GPU run would reach must not wait for one to be found missing), bench.py refuses
more than one GPU, and the default sections are the documented ones."""
import builtins
import os
import subprocess
import symtable
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def unresolved_globals(path):
    src = open(path).read()
    top = symtable.symtable(src, path, "exec")
    defined = {s.get_name() for s in top.get_symbols() if s.is_assigned() or s.is_imported() or s.is_namespace()}
    defined |= set(dir(builtins)) | {"__file__", "__name__", "__doc__"}
    missing = []

    def walk(table):
        for child in table.get_children():
            for s in child.get_symbols():
                if s.is_global() and s.is_referenced() and s.get_name() not in defined:
                    missing.append((child.get_name(), s.get_name()))
            walk(child)
    walk(top)
    return missing


def test_every_global_name_of_the_entry_points_resolves():
    for name in ("__graft_entry__.py", "bench.py"):
        assert unresolved_globals(os.path.join(ROOT, name)) == [], name
    for name in ("ops.py", "executor.py", "rewrite.py", "workloads.py", "io.py", "_lib.py", "build.py"):
        assert unresolved_globals(os.path.join(ROOT, "pimaicompiler_amd", name)) == [], name


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""
