"""CPU tier: what the compiler made of the kernels, read from the built library's own code objects.

Every kernel of hccl_amd/libhccl_amd.so carries a metadata note (registers, spills, private memory).  The fold
interpreter lives on the edge of the scalar register file: a change that looks harmless in the source can push a
few uniform values into vector registers or into private memory, and the launch then runs at a fraction of its rate
without any test failing.  This test fails instead.  Nothing runs on a GPU here; the note is written by hipcc when
the library is built.
"""
import os
import re
import subprocess

import pytest

import hccl_amd

LLVM = "/opt/rocm/llvm/bin"
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def kernel_notes(tmp_path):
    """[{name, vgpr, sgpr, sgpr_spills, vgpr_spills, private_bytes, lds_bytes}] for every kernel of the library."""
    fat = tmp_path / "fat.bin"
    subprocess.check_call([LLVM + "/llvm-objcopy", "--dump-section", ".hip_fatbin=%s" % fat, hccl_amd.LIB_PATH,
                           str(tmp_path / "unused.so")])
    data = fat.read_bytes()
    starts = [m.start() for m in re.finditer(re.escape(MAGIC), data)]   # one bundle per translation unit
    kernels = []
    for i, at in enumerate(starts):
        bundle = tmp_path / ("bundle%d.bin" % i)
        bundle.write_bytes(data[at:starts[i + 1] if i + 1 < len(starts) else len(data)])
        obj = tmp_path / ("code%d.o" % i)
        subprocess.check_call([LLVM + "/clang-offload-bundler", "--unbundle", "--type=o",
                               "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", "--input=%s" % bundle, "--output=%s" % obj])
        notes = subprocess.run([LLVM + "/llvm-readelf", "--notes", str(obj)], stdout=subprocess.PIPE, text=True,
                               check=True).stdout
        for block in re.split(r"\n\s+- \.agpr_count:", notes)[1:]:
            def field(key, block=block):
                m = re.search(r"\.%s:\s+(\S+)" % key, block)
                return m.group(1) if m else None
            kernels.append({"name": field("name"), "vgpr": int(field("vgpr_count")), "sgpr": int(field("sgpr_count")),
                            "sgpr_spills": int(field("sgpr_spill_count")), "vgpr_spills": int(field("vgpr_spill_count")),
                            "private_bytes": int(field("private_segment_fixed_size")),
                            "lds_bytes": int(field("group_segment_fixed_size"))})
    return kernels


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    if not os.path.exists(hccl_amd.LIB_PATH):
        pytest.fail("%s is missing: build the library first" % hccl_amd.LIB_PATH)
    return kernel_notes(tmp_path_factory.mktemp("notes"))


def test_every_translation_unit_is_there(kernels):
    reduce_kernels = [k for k in kernels if "ReduceKernel" in k["name"]]
    # 34 combinations of element type and operation, each with the eight-leaf and the sixteen-leaf load batch and
    # with the eight-leaf batch over two tiles per wavefront
    assert len(reduce_kernels) == 102, sorted(k["name"] for k in reduce_kernels)
    # and five times as the kernel that is launched from its arguments alone (any counts and eight of everything,
    # each with one and with two tiles per wavefront; up to sixteen leaves and destinations)
    direct_kernels = [k for k in kernels if "DirectFold" in k["name"]]
    assert len(direct_kernels) == 170, sorted(k["name"] for k in direct_kernels)
    # the copy, fan-out (two load flavours) and AlltoAllV kernels, and the copy that is launched from its arguments alone
    assert len(kernels) - len(reduce_kernels) - len(direct_kernels) == 23


def test_no_kernel_spills_or_uses_private_memory(kernels):
    bad = [k for k in kernels if k["sgpr_spills"] or k["vgpr_spills"] or k["private_bytes"]]
    assert not bad, bad


def test_register_budgets(kernels):
    """Vector registers: at most 96 for a fold kernel, so that five wavefronts fit a SIMD (512 / 96) whatever the
    type and batch; at most 24 for the copy kernels.  Scalar registers cannot exceed what the hardware has; what is
    checked for them is that the compiler did not have to spill (above)."""
    for k in kernels:
        # (the kernel launched from its arguments: at most 64, so that the eight wavefronts a SIMD can hold all fit;
        # with sixteen loaded vectors, two tiles per wavefront or sixteen leaves, 96 like the fold kernels)
        two_tiles = re.search(r"DirectFoldExactKernel.*Li2EEEv|DirectFoldTwoTileKernel|DirectFoldWideKernel", k["name"]) is not None
        limit = (96 if "ReduceKernel" in k["name"] or two_tiles else 64 if "DirectFold" in k["name"] else 24)
        assert k["vgpr"] <= limit, k


def test_uniform_values_are_uniform_for_the_compiler_too(kernels, tmp_path_factory):
    """The kernels pin launch scalars, program words and leaf addresses in scalar registers (the "+s" operands of
    their empty assembly statements).  Had one of them been computed per lane, the compiler would satisfy the
    constraint by taking the first lane's value, silently: a v_readfirstlane in the code.  The only one the sources
    ask for themselves are the wavefront index of the fan-out kernel (two instantiations of that kernel) and of the
    fold kernels that are launched from their arguments alone (one per instantiation)."""
    tmp = tmp_path_factory.mktemp("code")
    kernel_notes(tmp)
    counts = {}
    for obj in sorted(tmp.glob("code*.o")):
        text = subprocess.run([LLVM + "/llvm-objdump", "-d", "--mcpu=gfx950", str(obj)], stdout=subprocess.PIPE,
                              text=True, check=True).stdout
        assert "s_endpgm" in text                       # the listing is real
        direct = len(re.findall(r"^[0-9a-f]+ <[^>+]*DirectFold(Exact|TwoTile|Wide)?Kernel[^>+]*>:$", text, re.M))
        counts[obj.name] = text.count("v_readfirstlane") - direct
    assert sorted(counts.values()) == [0] * (len(counts) - 1) + [2], counts   # the fan-out kernel's two load flavours
