"""The library's Makefile must fail when a compile fails, also when an object of an earlier build is still
there: a stale object that links silently would ship a kernel that does not match its source."""
import os
import shutil
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hccl_amd", "csrc")


def test_a_failed_compile_fails_the_build_and_leaves_no_object(tmp_path):
    work = tmp_path / "csrc"
    work.mkdir()
    headers = [f for f in os.listdir(CSRC) if f.endswith(".h")]   # the rules name the headers as prerequisites
    for name in ["Makefile", "fold_plan.cc"] + headers:
        shutil.copy(os.path.join(CSRC, name), work / name)
    env = dict(os.environ)
    # the recipe includes ../../include relative to the source directory: point it at the real headers
    (tmp_path / "x").mkdir()
    src_dir = tmp_path / "x" / "y"
    shutil.move(str(work), str(src_dir))
    os.symlink(os.path.join(ROOT, "include"), tmp_path / "include")
    make = ["make", "-s", "-C", str(src_dir), "build/fold_plan.o"]
    good = subprocess.run(make, capture_output=True, text=True, env=env, timeout=300)
    assert good.returncode == 0, good.stdout + good.stderr
    obj = src_dir / "build" / "fold_plan.o"
    assert obj.exists()
    with open(src_dir / "fold_plan.cc", "a") as f:
        f.write("\n#error deliberately broken\n")
    bad = subprocess.run(make, capture_output=True, text=True, env=env, timeout=300)
    assert bad.returncode != 0, "a compile error must fail the build"
    assert "deliberately broken" in bad.stderr
    assert not obj.exists(), "the object of the earlier build must not survive a failed compile"
