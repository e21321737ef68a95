"""CPU tier: the launch-policy table (hccl_amd/csrc/launch_policy.h) compiled on its own and walked over a grid of
shapes.  What is checked is the shape of the table, not its figures: a form that a threshold switches on stays on for
every longer message of the same world (the two-kernel forms), the forms that exist for a window of sizes have one
window, every count the launchers cannot take (more wavefronts than the workgroup limit, a batch other than 8 or 16)
is never returned, and the thresholds the documentation quotes are the ones compiled in."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = r"""
#include "launch_policy.h"
#include <cstdio>
using namespace hccl_amd::policy;
int main()
{
    const unsigned long long sizes[] = {1ull << 10, 1ull << 16, 1ull << 20, 3ull << 19, 2ull << 20, 5ull << 19, 3ull << 20,
        4ull << 20, 5ull << 20, 6ull << 20, (6ull << 20) + 1, 7ull << 20, (7ull << 20) + 1, 8ull << 20, (8ull << 20) + 1, 16ull << 20, 24ull << 20, 48ull << 20, 64ull << 20, 128ull << 20,
        160ull << 20, 256ull << 20, 1ull << 30, 8ull << 30};
    for (unsigned n = 1; n <= 64; ++n) {
        for (unsigned long long b : sizes) {
            std::printf("%u %llu %d %d %d %d %u %u %u %u %d %d %u %u %d %u\n", n, b, (int)FoldThenFanOut(n, b),
                        (int)GatherThenFanOut(n, b, true), (int)GatherThenFanOut(n, b, false), (int)PairTiles(n, false, b),
                        StoreWaves(n, b, 4), StoreWaves(n, b, 2), VecBatch(n, false, false), VecBatch(n, true, false),
                        (int)FanOutStreamLoad(n, false), (int)FanOutStreamLoad(n, true), AllFoldWaves(n, b),
                        DirectFoldWaves(n < 8 ? n : 8, n < 8 ? n : 8, b), (int)DirectFoldTwoTiles(n, n, b),
                        DirectFoldWideWaves(n, n, b));
        }
    }
    return 0;
}
"""


@pytest.fixture(scope="module")
def table(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("policy")
    src = tmp / "probe.cc"
    src.write_text(PROBE)
    exe = tmp / "probe"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "hccl_amd", "csrc"), str(src), "-o", str(exe)])
    rows = {}
    for line in subprocess.check_output([str(exe)], text=True).splitlines():
        v = [int(x) for x in line.split()]
        rows[(v[0], v[1])] = dict(fold=v[2], gather=v[3], gather_general=v[4], pair=v[5], waves4=v[6], waves2=v[7],
                                  batch_many=v[8], batch_one=v[9], nt_single=v[10], nt_several=v[11], all_fold=v[12],
                                  direct=v[13], two_tiles=v[14], wide=v[15])
    return rows


def by_world(table):
    worlds = {}
    for (n, b), row in table.items():
        worlds.setdefault(n, []).append((b, row))
    return {n: sorted(rows) for n, rows in worlds.items()}


def test_two_kernel_forms_stay_on_for_longer_messages(table):
    for n, rows in by_world(table).items():
        for key in ("fold", "gather", "gather_general"):
            seen = False
            for b, row in rows:
                assert not (seen and not row[key]), (key, n, b)
                seen = seen or bool(row[key])


def test_small_worlds_never_split_into_two_kernels(table):
    for (n, b), row in table.items():
        if n < 5:
            assert not row["fold"], (n, b)
        if n < 6:
            assert not row["gather"] and not row["gather_general"], (n, b)
        if row["gather_general"]:
            assert row["gather"], (n, b)         # sources that share the destinations' alignment never fare worse


def test_the_all_fold_form_has_one_window_of_sizes_and_fits_the_workgroup(table):
    for n, rows in by_world(table).items():
        flags = [row["all_fold"] for _, row in rows]
        assert all(f in (0, 2, 3, 4) for f in flags), (n, flags)
        on = [bool(f) for f in flags]
        assert not on[0] and not on[-1], n
        assert sum(1 for a, b in zip(on, on[1:]) if a != b) in (0, 2), (n, flags)
        if n < 5 or n > 32:
            assert not any(on), n
    assert table[(8, 4 << 20)]["all_fold"] == 3 and table[(8, 7 << 20)]["all_fold"] == 2
    assert table[(8, 3 << 20)]["all_fold"] == 0 and table[(8, (7 << 20) + 1)]["all_fold"] == 0
    assert table[(16, 5 << 19)]["all_fold"] == 3 and table[(16, 2 << 20)]["all_fold"] == 0
    assert table[(6, 4 << 20)]["all_fold"] == 0 and table[(6, 5 << 20)]["all_fold"] == 3


def test_the_kernel_launched_from_its_arguments_covers_everything_up_to_its_limit(table):
    """From the shortest message up to 12 MiB per rank (16 MiB for up to four destinations), with a count of
    wavefronts the launcher takes for up to eight destinations; two where the launch is latency-bound, the count whose
    workgroups deal out evenly over the CUs in between (3 MiB = 3072 tiles: six, 4 MiB: eight, 5 MiB: four)."""
    for n, rows in by_world(table).items():
        if n < 2 or n > 8:
            continue
        limit = (16 if n <= 4 else 12) << 20
        for b, row in rows:
            assert (row["direct"] != 0) == (b <= limit), (n, b)
            assert row["direct"] in (0, 2, 3, 4, 6, 8), (n, b)
    assert table[(8, 1 << 20)]["direct"] == 2 and table[(8, 2 << 20)]["direct"] == 2
    assert table[(8, 3 << 20)]["direct"] == 6 and table[(8, 4 << 20)]["direct"] == 8
    assert table[(8, 5 << 20)]["direct"] == 4 and table[(8, 6 << 20)]["direct"] == 8
    assert table[(8, 8 << 20)]["direct"] == 8 and table[(8, (8 << 20) + 1)]["direct"] == 3
    assert table[(8, 16 << 20)]["direct"] == 0 and table[(4, 16 << 20)]["direct"] == 3


def test_two_tiles_per_wavefront_only_for_whole_workgroups_that_fill_the_cus(table):
    """A multiple of 16 KiB between 3.5 and 12 MiB per rank whose workgroups of sixteen tiles fill the CUs (4 MiB: 256
    workgroups; 5 MiB: 320, left to the one-tile forms)."""
    for (n, b), row in table.items():
        if row["two_tiles"]:
            assert b % (16 << 10) == 0 and (7 << 19) <= b <= (12 << 20), (n, b)
    assert table[(4, 8 << 20)]["two_tiles"] and table[(2, 4 << 20)]["two_tiles"]
    assert table[(8, 4 << 20)]["two_tiles"] and table[(8, 7 << 20)]["two_tiles"] and table[(8, 8 << 20)]["two_tiles"]
    assert table[(8, 6 << 20)]["two_tiles"]
    assert not table[(8, 5 << 20)]["two_tiles"] and not table[(8, 3 << 20)]["two_tiles"]
    assert not table[(8, (8 << 20) + 1)]["two_tiles"] and not table[(8, 16 << 20)]["two_tiles"]


def test_the_kernel_for_nine_to_sixteen_ranks_takes_the_short_messages(table):
    for n, rows in by_world(table).items():
        if n < 9 or n > 16:
            continue
        for b, row in rows:
            assert (row["wide"] != 0) == (b <= (3 << 20)), (n, b)
            assert row["wide"] in (0, 2, 8), (n, b)
    assert table[(16, 1 << 20)]["wide"] == 2 and table[(16, 2 << 20)]["wide"] == 8 and table[(12, 2 << 20)]["wide"] == 2
    assert table[(12, 3 << 20)]["wide"] == 8 and table[(16, 4 << 20)]["wide"] == 0


def test_the_pair_form_has_one_window_of_sizes(table):
    for n, rows in by_world(table).items():
        flags = [row["pair"] for _, row in rows]
        assert flags[0] == 0 and flags[-1] == 0, n
        changes = sum(1 for a, b in zip(flags, flags[1:]) if a != b)
        assert changes in (0, 2), (n, flags)
    assert table[(8, 4 << 20)]["pair"] and table[(8, 3 << 19)]["pair"] and table[(8, 6 << 20)]["pair"]
    assert not table[(8, 1 << 20)]["pair"] and not table[(8, (6 << 20) + 1)]["pair"]
    assert table[(2, 8 << 20)]["pair"] and not table[(2, (8 << 20) + 1)]["pair"]


def test_returned_counts_are_ones_the_launchers_take(table):
    for (n, b), row in table.items():
        assert row["waves4"] in (1, 2, 3) and row["waves2"] in (1, 2, 3), (n, b)
        assert row["waves4"] <= max(n, 1) and row["waves2"] <= max(n, 1), (n, b)
        assert row["batch_many"] in (8, 16) and row["batch_one"] in (8, 16), (n, b)
        if row["nt_single"]:
            assert row["nt_several"], (n, b)     # another piece behind the fan-out only adds reasons to stream
