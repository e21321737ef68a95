"""The launch forms the library picks by itself (hccl_amd/csrc/launch_policy.h) against the forms it could have
picked, timed on the same buffers in one process with hccl_amd.tune: on shapes that lie well inside a form's territory
the library's choice has to be within a few per cent of the fastest forced form.  A kernel change that moves a
crossover far enough shows up here; the rows next to the thresholds themselves are what `python -m hccl_amd.tune`
prints.  Timing only: what the forms compute is compared with the oracle elsewhere; collected behind the parity tests."""
import pytest

from gpu_util import require_library_on_gpu

pytestmark = pytest.mark.gpu

TOLERANCE = 0.92    # forms of a row repeat within 1 %; between the forms of these shapes lie 5 to 25 %


@pytest.fixture(scope="module", autouse=True)
def _native_library():
    require_library_on_gpu()


def behind_best(rows):
    out = []
    for label, fracs in rows:
        best = max(v for k, v in fracs.items() if k != "auto")
        if fracs["auto"] < TOLERANCE * best:
            out.append((label, fracs))
    return out


@pytest.mark.parametrize("ranks,mib", [(3, 64), (4, 256), (16, 64)])
def test_all_reduce_form(ranks, mib):
    import torch
    import hccl_amd
    from hccl_amd import tune
    assert behind_best(tune.all_reduce_rows(torch, hccl_amd, [ranks], [mib], 3)) == []


@pytest.mark.parametrize("ranks,kib", [(8, 4096), (8, 16384), (2, 4096)])
def test_small_all_reduce_form(ranks, kib):
    import torch
    import hccl_amd
    from hccl_amd import tune
    # (one form of each kind: the more forms are timed, the further the luckiest of them lies ahead of its own mean)
    forms = ("one", "pair", "fold3", "direct3", "direct8")
    assert behind_best(tune.all_reduce_small_rows(torch, hccl_amd, [ranks], [kib], 3, only=forms)) == []


@pytest.mark.parametrize("ranks,mib", [(4, 64), (16, 8)])
def test_all_gather_form(ranks, mib):
    import torch
    import hccl_amd
    from hccl_amd import tune
    assert behind_best(tune.all_gather_rows(torch, hccl_amd, [ranks], [mib], 3)) == []


@pytest.mark.parametrize("ranks,mib", [(6, 16), (16, 64)])
def test_broadcast_form(ranks, mib):
    import torch
    import hccl_amd
    from hccl_amd import tune
    assert behind_best(tune.broadcast_rows(torch, hccl_amd, [ranks], [mib], 3)) == []
