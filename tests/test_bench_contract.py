"""What the driver relies on without a GPU: bench.py refuses more than one GPU with one line and exit
status 2, and the entry module exposes build() and smoke()."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_several_gpus():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout


def test_entry_module_has_build_and_smoke():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry

    assert callable(entry.build) and callable(entry.smoke)
