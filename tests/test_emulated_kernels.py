"""CPU tier: the GPU parity tests, run against the library's own sources built for the host.

tests/emu compiles hccl_amd/csrc (host layer and gfx950 kernels, inline assembly replaced by its plain meaning)
against a stand-in HIP runtime that runs every launch workgroup by workgroup and lane by lane on the CPU.  The
parity tests of a dozen GPU test files then run unchanged in a pytest process of their own with
HCCL_AMD_TEST_EMU=1:
tests/gpu_util.py hands out host buffers, tests/conftest.py points the Python mirror at the emulation library.

What this checks without a GPU: the kernels' index arithmetic, fold interpreter, heads / tails, tile tables and the
host layer's launch geometry give the oracle's bits, touch no byte outside the 16-byte granules of the buffers
they were given (AddressSanitizer) and do nothing the language leaves undefined, such as an overflowing signed
product or a misaligned vector access (the undefined-behaviour checks of the same build).  It is how a kernel change is tried before it goes to the GPU.
It says nothing about timing or about what the GPU compiler makes of the code: the `-m gpu` run stays the
parity gate.  The emulation is test infrastructure; the package never loads it.
"""
import glob
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
import build_emu  # noqa: E402

FILES = ["tests/test_gpu_parity.py", "tests/test_gpu_copies.py", "tests/test_wide_gpu_copy_sweep.py",
         "tests/test_wide_gpu_two_level.py", "tests/test_wide_gpu_three_level.py",
         "tests/test_wide_gpu_rooted_sweep.py", "tests/test_gpu_rooted_and_v_ops.py",
         "tests/test_gpu_random_sweep.py", "tests/test_gpu_point_to_point.py",
         "tests/test_gpu_reference_python_suites.py", "tests/test_wide_gpu_reference_st_shapes.py",
         "tests/test_wide_gpu_reference_st_reduce_shapes.py", "tests/test_zz_no_alloc.py"]
# Left out: tests that allocate or compute with torch on the GPU themselves (graphs, own streams, device-side
# generators) and tests whose size is meant for the GPU.
DESELECT = [
    "tests/test_gpu_parity.py::test_two_kernel_all_reduce_can_be_captured_into_a_graph",
    "tests/test_gpu_parity.py::test_warmed_up_collectives_can_be_captured_into_a_graph_and_replayed",
    "tests/test_gpu_parity.py::test_all_reduce_larger_than_a_million_workgroups",
    "tests/test_gpu_parity.py::test_reduce_scatter_into_the_own_slice_of_the_send_buffer",
    "tests/test_gpu_parity.py::test_config2_reduce_scatter_bf16_n8",
    "tests/test_gpu_parity.py::test_config3_all_reduce_int32_n16_max_and_prod",
    "tests/test_gpu_copies.py::test_one_host_thread_per_rank_with_own_streams",
    "tests/test_gpu_copies.py::test_all_gather_with_the_send_buffer_inside_the_receive_buffer",
    "tests/test_gpu_copies.py::test_broadcast_and_all_gather_of_half_a_gigabyte",
    "tests/test_gpu_rooted_and_v_ops.py::test_rooted_ops_with_one_blocking_thread_per_rank",
    "tests/test_gpu_point_to_point.py::test_blocking_calls_from_one_thread_per_rank_on_streams_of_their_own",
    "tests/test_gpu_point_to_point.py::test_barrier_orders_the_streams_of_all_ranks",
    "tests/test_zz_no_alloc.py::test_ranks_on_their_own_streams",
    "tests/test_zz_no_alloc.py::test_it_can_be_captured_into_a_graph_and_replayed",
]


def asan_runtime():
    found = glob.glob("/opt/rocm/llvm/lib/clang/*/lib/linux/libclang_rt.asan-x86_64.so")
    assert found, "the sanitizer runtime of the ROCm clang is missing"
    return found[0]


def emu_env(lib, asan_log=None):
    env = dict(os.environ)
    env["HCCL_AMD_TEST_EMU"] = "1"
    env["HCCL_AMD_TEST_EMU_LIB"] = lib
    if asan_log is not None:
        # The sanitizer's runtime has to be in the process before Python allocates; whatever is preloaded already stays.
        env["LD_PRELOAD"] = ":".join(x for x in (env.get("LD_PRELOAD", ""), asan_runtime()) if x)
        env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:log_path=" + asan_log
    return env


def run_gpu_tests(env, files=FILES, workers=None):
    workers = workers or max(2, min(8, os.cpu_count() or 2))
    cmd = [sys.executable, "-m", "pytest", "-m", "gpu", "-q", "-x", "-p", "no:cacheprovider", "-n", str(workers),
           "--timeout", "900"] + files
    for name in DESELECT:
        cmd += ["--deselect", name]
    proc = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    tail = proc.stdout[-6000:]
    m = re.search(r"(\d+) passed", proc.stdout)
    return proc.returncode, int(m.group(1)) if m else 0, tail


def test_gpu_parity_tests_pass_on_the_emulation_and_touch_no_byte_outside_their_buffers(tmp_path):
    """One run for both: the tests compare with the oracle, AddressSanitizer watches every access.  (Without the
    sanitizer, for a quick look while working on a kernel: run_gpu_tests(emu_env(build_emu.build())).)"""
    lib = build_emu.build(asan=True)
    log = str(tmp_path / "asan")
    rc, passed, tail = run_gpu_tests(emu_env(lib, log))
    reports = "".join(open(f).read()[:3000] for f in sorted(glob.glob(log + "*"))[:2])
    assert rc == 0 and not reports, tail + reports
    assert passed >= 780, tail   # a shrinking selection would hide what no longer runs


OVERRUN = r"""
import ctypes, sys
sys.path.insert(0, %r)
import hccl_amd
from gpu_util import HostBuf
comms = hccl_amd.comm_init_all(2)
count = 1000                                   # fp32 elements per rank
sends = [HostBuf(4 * count), HostBuf(4 * count - 64)]   # the second send buffer is 64 bytes short
recvs = [HostBuf(8 * count), HostBuf(8 * count)]
with hccl_amd.group():
    for r in range(2):
        hccl_amd.all_gather(comms[r], sends[r], recvs[r], count, hccl_amd.HcclDataType.FP32, 0x1000)
print("not caught")
"""


def test_the_sanitizer_run_does_catch_a_kernel_that_leaves_its_buffer(tmp_path):
    """The check checks: a collective over a buffer that is too short must end the process with a report."""
    lib = build_emu.build(asan=True)
    log = str(tmp_path / "asan")
    script = tmp_path / "overrun.py"
    script.write_text(OVERRUN % os.path.join(ROOT, "tests"))
    env = emu_env(lib, log)
    env["PYTHONPATH"] = os.pathsep.join([ROOT, os.path.join(ROOT, "tests"), env.get("PYTHONPATH", "")])
    boot = ("import ctypes, os, hccl_amd; hccl_amd._lib = hccl_amd._bind(ctypes.CDLL(os.environ['HCCL_AMD_TEST_EMU_LIB']));"
            "exec(open(%r).read())" % str(script))
    proc = subprocess.run([sys.executable, "-c", boot], cwd=ROOT, env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    reports = "".join(open(f).read()[:2000] for f in glob.glob(log + "*"))
    assert proc.returncode != 0 and "not caught" not in proc.stdout, proc.stdout[-2000:]
    assert "heap-buffer-overflow" in reports, reports


def run_native(name, sanitizer, *args, **extra_env):
    exe = build_emu.build_example(name, sanitizer)
    env = dict(os.environ, **extra_env)
    env["LD_LIBRARY_PATH"] = os.pathsep.join(x for x in (os.path.dirname(asan_runtime()), env.get("LD_LIBRARY_PATH", "")) if x)
    return subprocess.run([exe] + [str(a) for a in args], cwd=ROOT, env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=900)


def test_host_layer_has_no_data_race_under_thread_sanitizer():
    """tests/emu/host_stress.cc: two worlds with a thread per rank (blocking collectives, point-to-point rings,
    batches), a world driven through groups by one thread and a world that a rank leaves while its peers are parked,
    all at once, against the emulation build under ThreadSanitizer."""
    proc = run_native("host_stress", "tsan", 600)
    assert proc.returncode == 0 and "PASS" in proc.stdout, proc.stdout[-4000:]
    assert "ThreadSanitizer" not in proc.stdout, proc.stdout[-4000:]


def test_wavefronts_that_share_a_tiles_stores_do_not_race():
    """The same driver with the reduce kernel's shared-store form forced: the folding wavefront parks a tile in one of
    two LDS slots, one barrier per tile, the storing wavefronts read it.  Lanes are OS threads here, so
    ThreadSanitizer sees a slot that is written again before every reader is through."""
    proc = run_native("host_stress", "tsan", 120, HCCL_AMD_REDUCE_STORE_WAVES="3")
    assert proc.returncode == 0 and "PASS" in proc.stdout, proc.stdout[-4000:]
    assert "ThreadSanitizer" not in proc.stdout, proc.stdout[-4000:]


@pytest.mark.parametrize("seed,sanitizer", [(1, "tsan"), (2, "tsan"), (3, "asan")])
def test_faulty_calls_reach_every_rank_and_leave_the_sequence_intact(seed, sanitizer):
    """tests/emu/host_fuzz.cc: seeded scripts of collectives in which, now and then, one rank passes a different count,
    a null buffer or a type the operator does not take.  Every rank must see the same code for such a step, the
    clean steps must give the right values and the calls after a fault must pair up as before; with a thread per
    rank in two worlds and through groups in a third, at once."""
    proc = run_native("host_fuzz", sanitizer, seed, 300, HCCL_EXEC_TIMEOUT="30", HCCL_AMD_LOG_LEVEL="0")
    assert proc.returncode == 0 and "PASS" in proc.stdout, proc.stdout[-4000:]
    assert "Sanitizer" not in proc.stdout, proc.stdout[-4000:]


def test_host_layer_frees_what_it_allocates():
    """The same driver under AddressSanitizer with its leak check: worlds, pending calls, events and plans are gone
    when their last communicator has been destroyed."""
    proc = run_native("host_stress", "asan", 300, ASAN_OPTIONS="detect_leaks=1")
    assert proc.returncode == 0 and "PASS" in proc.stdout, proc.stdout[-4000:]
    assert "Sanitizer" not in proc.stdout, proc.stdout[-4000:]


@pytest.mark.parametrize("ranks,count", [(8, 100003), (3, 1), (16, 4096), (1, 77), (7, 1001)])
def test_native_thread_per_rank_example_runs_on_the_emulation(ranks, count):
    """examples/collectives_threads.cc, the thirteen operators of the reference's own examples with a thread per rank,
    under ThreadSanitizer and under AddressSanitizer (the first four cases are the ones the GPU test runs)."""
    for sanitizer in ("tsan", "asan"):
        proc = run_native("collectives_threads", sanitizer, ranks, count)
        assert proc.returncode == 0 and proc.stdout.startswith("PASS"), sanitizer + "\n" + proc.stdout[-4000:]
        assert "Sanitizer" not in proc.stdout, proc.stdout[-4000:]


def test_the_package_never_loads_the_emulation():
    """The emulation is a checker.  Nothing under hccl_amd/, bench.py or __graft_entry__.py may name it."""
    offenders = []
    for path in glob.glob(os.path.join(ROOT, "hccl_amd", "**", "*"), recursive=True) + [
            os.path.join(ROOT, "bench.py"), os.path.join(ROOT, "__graft_entry__.py")]:
        if os.path.isfile(path) and path.endswith((".py", ".cc", ".h", ".hip", "Makefile")) and "/build/" not in path:
            text = open(path, errors="replace").read()
            if "libhccl_amd_emu" in text or "tests/emu" in text or "TEST_EMU" in text:
                offenders.append(path)
    assert not offenders, offenders
