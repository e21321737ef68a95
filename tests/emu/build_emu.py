"""Builds the CPU emulation of the library for the tests: test infrastructure only, never loaded by the package.

The sources of hccl_amd/csrc (host layer and kernels) are copied to tests/emu/build/src with their inline assembly
replaced by its plain C++ meaning, and compiled for the host against the stand-in HIP header of this directory
(hip/hip_runtime.h) and the execution engine (emu_runtime.cc):

    build/libhccl_amd_emu.so        the whole library with the hccl.h entry points, kernels run by the engine
    build/libhccl_amd_emu_asan.so   the same, instrumented by AddressSanitizer (loaded by build/asan_sweep)

Any inline assembly the rules below do not know stops the build: a kernel that gains a new instruction has to get
its emulation here before the CPU tests run again.
"""
import hashlib
import os
import re
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "hccl_amd", "csrc")
BUILD = os.path.join(HERE, "build")
SRC = os.path.join(BUILD, "src")
CLANG = "/opt/rocm/llvm/bin/clang++"

KERNEL_UNITS = ["reduce_i8", "reduce_i16", "reduce_i32", "reduce_i64", "reduce_u64", "reduce_f16", "reduce_bf16",
                "reduce_f32", "reduce_f64", "reduce_launch", "copy_kernels"]
HOST_UNITS = ["api", "host_world", "launch_reduce", "launch_copy", "rendezvous", "fold_plan", "algo_config"]

# inline assembly with a meaning -> that meaning
ASM_RULES = [
    # 16-byte store written through at system scope (dataplane.h StoreStream16); the address may be unaligned
    ('asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" : : "v"(p), "v"(v) : "memory");',
     "__builtin_memcpy(p, &v, 16);"),
    # 1.0f the optimiser cannot see through (reduce_kernel_impl.h OpaqueOne)
    ('asm volatile("v_mov_b32 %0, 1.0" : "=v"(one));', "one = 1.0f;"),
]
# empty assembly statements only pin values in registers at a point of the instruction stream
EMPTY_ASM = re.compile(r'asm volatile\(""\s*:[^;]*\);', re.S)


def transform(text, name):
    for old, new in ASM_RULES:
        text = text.replace(old, new)
    text = EMPTY_ASM.sub("", text)
    text = text.replace("extern __shared__", "extern")
    if re.search(r"\basm\b", re.sub(r"//[^\n]*", "", text)):
        raise RuntimeError("%s: inline assembly without an emulation rule in tests/emu/build_emu.py" % name)
    return text


def prepare_sources():
    os.makedirs(SRC, exist_ok=True)
    digest = hashlib.sha256()
    for fn in sorted(os.listdir(CSRC)):
        path = os.path.join(CSRC, fn)
        if not os.path.isfile(path) or not fn.endswith((".h", ".hip", ".cc")):
            continue
        text = transform(open(path).read(), fn)
        out = os.path.join(SRC, fn[:-4] + ".cc" if fn.endswith(".hip") else fn)
        digest.update(fn.encode() + b"\0" + text.encode())
        if not os.path.exists(out) or open(out).read() != text:
            open(out, "w").write(text)
    for fn in ("emu_runtime.cc", os.path.join("hip", "hip_runtime.h"), "build_emu.py"):
        digest.update(open(os.path.join(HERE, fn), "rb").read())
    return digest.hexdigest()


# "asan" is AddressSanitizer together with the undefined-behaviour checks (one runtime serves both); a finding of
# either kind ends the process.
SANITIZE = {"": [], "asan": ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"],
            "tsan": ["-fsanitize=thread", "-fno-omit-frame-pointer"]}


def flags(asan):
    f = [CLANG, "-x", "c++", "-std=c++17", "-O1", "-gline-tables-only", "-fPIC", "-ffp-contract=off", "-mf16c", "-pthread",
         "-Wno-unknown-attributes", "-Wno-ignored-attributes",
         "-I" + HERE, "-I" + os.path.join(ROOT, "include"), "-I" + SRC,
         "-D__builtin_amdgcn_readfirstlane=emu::ReadFirstLane", "-D__builtin_amdgcn_update_dpp=emu::UpdateDpp",
         "-D__builtin_amdgcn_alignbyte=emu::AlignByte", "-D__builtin_amdgcn_s_waitcnt=emu::WaitCnt",
         "-Daddress_space(x)="]
    f += SANITIZE["asan" if asan is True else (asan or "")]
    return f


def build(asan=False, jobs=8):
    """Returns the path of the emulation library (built if its sources changed)."""
    stamp = prepare_sources()
    tag = "_asan" if asan is True else ("_" + asan if asan else "")
    lib = os.path.join(BUILD, "libhccl_amd_emu%s.so" % tag)
    stamp_file = lib + ".stamp"
    if os.path.exists(lib) and os.path.exists(stamp_file) and open(stamp_file).read() == stamp:
        return lib
    objdir = os.path.join(BUILD, "obj" + tag)
    shutil.rmtree(objdir, ignore_errors=True)
    os.makedirs(objdir)
    jobs_list = []
    for unit in KERNEL_UNITS:
        jobs_list.append((os.path.join(SRC, unit + ".cc"), os.path.join(objdir, unit + ".o"), ["-D__HIPCC__=1"]))
    for unit in HOST_UNITS:
        jobs_list.append((os.path.join(SRC, unit + ".cc"), os.path.join(objdir, unit + ".o"), []))
    jobs_list.append((os.path.join(HERE, "emu_runtime.cc"), os.path.join(objdir, "emu_runtime.o"), []))
    running = []
    for src, obj, extra in jobs_list:
        running.append((src, subprocess.Popen(flags(asan) + extra + ["-c", src, "-o", obj], stderr=subprocess.PIPE)))
        if len(running) >= jobs:
            _reap(running.pop(0))
    while running:
        _reap(running.pop(0))
    link = [CLANG, "-shared", "-pthread", "-o", lib] + [obj for _, obj, _ in jobs_list]
    if asan:
        link += SANITIZE["asan" if asan is True else asan][:1] + ["-shared-libsan"]
    subprocess.check_call(link)
    open(stamp_file, "w").write(stamp)
    return lib


def build_example(name, sanitizer=""):
    """One of the native callers of examples/ (a .cc file) linked against the emulation library, optionally under a
    sanitizer ("asan" or "tsan"); returns the path of the executable."""
    lib = build(asan=sanitizer or False)
    exe = os.path.join(BUILD, name + ("_" + sanitizer if sanitizer else ""))
    src = os.path.join(ROOT, "examples", name + ".cc")
    if not os.path.exists(src) and os.path.exists(os.path.join(ROOT, "examples", name + ".hip")):
        # an example with kernels of its own: same treatment as the library's kernels
        os.makedirs(SRC, exist_ok=True)
        src = os.path.join(SRC, "example_" + name + ".cc")
        text = transform(open(os.path.join(ROOT, "examples", name + ".hip")).read(), name + ".hip")
        if not os.path.exists(src) or open(src).read() != text:
            open(src, "w").write(text)
    if not os.path.exists(src):
        src = os.path.join(HERE, name + ".cc")   # a driver of the tests' own
    if os.path.exists(exe) and os.path.getmtime(exe) >= max(os.path.getmtime(lib), os.path.getmtime(src)):
        return exe
    cmd = flags(sanitizer or False)[:1] + [f for f in flags(sanitizer or False)[3:] if f != "-fPIC"] + [
        "-D__HIPCC__=1", src, lib, "-Wl,-rpath," + BUILD, "-o", exe]
    if sanitizer:
        cmd += ["-shared-libsan"]
    subprocess.check_call(cmd)
    return exe


def _reap(job):
    src, proc = job
    _, err = proc.communicate()
    if proc.returncode != 0:
        raise RuntimeError("emulation build failed for %s:\n%s" % (src, err.decode()[-4000:]))


if __name__ == "__main__":
    print(build())
