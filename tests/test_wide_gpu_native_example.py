"""The C ABI driven by a compiled C++ program instead of ctypes: examples/collectives_threads.cc, one host
thread per rank with its own stream, blocking calls outside any group -- the calling pattern of the reference's
examples/02_collectives.  The binary is built by `make -C examples` (part of __graft_entry__.build())."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "examples", "bin", "collectives_threads")


@pytest.mark.parametrize("ranks,count", [(8, 100003), (3, 1), (16, 4096), (1, 77)])
def test_native_thread_per_rank_program(ranks, count):
    assert os.path.exists(BINARY), "run `make -C examples` (or __graft_entry__.build()) first"
    done = subprocess.run([BINARY, str(ranks), str(count)], capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.startswith("PASS"), done.stdout


def test_native_latency_program_runs_and_reports_every_size():
    binary = os.path.join(ROOT, "examples", "bin", "allreduce_latency")
    assert os.path.exists(binary), "run `make -C examples` (or __graft_entry__.build()) first"
    done = subprocess.run([binary, "8"], capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stdout + done.stderr
    rows = [line.split() for line in done.stdout.splitlines()[2:]]
    assert [int(r[0]) for r in rows] == [1, 1024, 65536, 1 << 18, 1 << 20, 1 << 22]
    assert all(float(r[1]) > 0 for r in rows)
