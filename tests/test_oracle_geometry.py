"""Pins the oracle's step geometry (rows a10, a11, a16) against the hand tables and invariants held by
the reference's own unit tests (tests/golden/rhd_nhr_tables.json lists the source lines)."""
import json
import os

import pytest

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "rhd_nhr_tables.json")))
INVALID = 0xFFFFFFFF


def _largest_pow2_le(p):
    hp = 1
    while hp <= p // 2:
        hp *= 2
    return hp


def _info_for_virtual(orc, p, v):
    r = p - _largest_pow2_le(p)
    carrier = v if v < r else v + r
    rc, info = orc.rhd_part1(p, carrier)
    assert rc == 0 and info.virtualRank == v
    return info


def test_step_counts(orc):
    for n, want in GOLD["rhd_step_num"]:
        assert orc.lib().orc_rhd_step_num(n) == want
    for n in range(1, 70):
        steps, covered = 0, 1
        while covered < n:
            covered <<= 1
            steps += 1
        assert orc.lib().orc_nhr_step_num(n) == steps


def test_nhr_steps_match_the_reference_golden_values(orc):
    """The step tables the reference's own unit test holds for 2, 3, 4, 5, 6 and 8 ranks
    (test/ut/reduce_scatter_nhr_dpu/test_nhr_geometry.cc:51-84), and its step counts (:226-236)."""
    for n, want in GOLD["nhr_step_num"]:
        assert orc.lib().orc_nhr_step_num(n) == want
    seen = 0
    for case in GOLD["nhr_golden_steps"]:
        n, rank = case["rankSize"], case["rank"]
        assert orc.lib().orc_nhr_step_num(n) == len(case["steps"])
        for step, want in enumerate(case["steps"]):
            rc, to, frm, tx, rx = orc.nhr_step_info(n, rank, step)
            assert rc == 0, (n, rank, step)
            assert (to, frm, len(tx), tx, rx) == (want["toRank"], want["fromRank"], want["nSlices"], want["tx"], want["rx"]), \
                (n, rank, step)
            seen += 1
    assert seen == 25


def test_round_up(orc):
    assert orc.lib().orc_round_up(10, 4) == 3
    assert orc.lib().orc_round_up(8, 4) == 2
    assert orc.lib().orc_round_up(0, 4) == 0
    assert orc.lib().orc_round_up(7, 0) == 7


def test_rs_and_ag_segment_tables_p8(orc):
    for key, fn in (("rs_segment_formula_p8", orc.rhd_rs_steps), ("ag_segment_formula_p8", orc.rhd_ag_steps)):
        for v, k, peer, txs, txe, rxs, rxe in GOLD[key]["rows"]:
            rc, steps = fn(_info_for_virtual(orc, 8, v))
            assert rc == 0 and len(steps) == 3
            s = steps[k]
            assert (s.step, s.peer, s.txSegStart, s.txSegEnd, s.rxSegStart, s.rxSegEnd) == (k, peer, txs, txe, rxs, rxe)
            assert s.nSlices == ((8 >> (k + 1)) if key.startswith("rs") else (1 << k))


def test_seg_bytes_uniform_table(orc):
    for us, ue, ss, ts, tu, off, ln in GOLD["seg_bytes_uniform"]["rows"]:
        assert orc.rhd_seg_bytes_uniform(us, ue, ss, ts, tu) == (off, ln)


def test_unit_start_sentinels_and_sigma(orc):
    for p, j, want in GOLD["unit_start_of_rank"]:
        assert orc.lib().orc_rhd_unit_start_of_rank(p, j) == want
    for p in (5, 6, 7, 13):
        r = p - _largest_pow2_le(p)
        starts = sorted(orc.lib().orc_rhd_unit_start_of_rank(p, j) for j in range(p))
        assert starts == list(range(p))                      # sigma is a permutation
        for t in range(r):                                   # pair members sit next to each other
            assert orc.lib().orc_rhd_unit_start_of_rank(p, t) == 2 * t
            assert orc.lib().orc_rhd_unit_start_of_rank(p, t + r) == 2 * t + 1
        for u in range(p):                                   # owner map inverts sigma
            assert orc.lib().orc_rhd_unit_start_of_rank(p, orc.lib().orc_rhd_owner_of_unit(p, u)) == u


def test_part1_partition(orc):
    for p in (2, 4, 8, 16):
        for j in range(p):
            rc, i = orc.rhd_part1(p, j)
            assert rc == 0 and i.isPowerOfTwo and i.r == 0 and i.effectiveRankSize == p and not i.inPart1
            assert i.pairedAlgRank == INVALID and i.virtualRank == j and i.unitStart == j and i.unitCount == 1
    for p in (5, 6, 7, 9, 13):
        r = p - _largest_pow2_le(p)
        for j in range(p):
            rc, i = orc.rhd_part1(p, j)
            assert rc == 0 and i.r == r and not i.isPowerOfTwo and i.effectiveRankSize == p - r
            assert bool(i.inPart1) == (j < 2 * r)
            assert i.virtualRank == ((j % r) if j < 2 * r else j - r)
            assert bool(i.isRepresentative) == (j < r)


def test_part1_roles_follow_root(orc):
    for p in (5, 7, 9, 13):
        r = p - _largest_pow2_le(p)
        for root in range(p):
            rep_low = (root < r) if root < 2 * r else True
            for j in range(p):
                rc, i = orc.rhd_part1(p, j, root)
                assert rc == 0
                if j >= 2 * r:
                    assert not i.inPart1 and i.unitStart == j and i.unitCount == 1
                    continue
                low, t = j < r, j % r
                assert i.pairedAlgRank == (t + r if low else t)
                assert bool(i.isRepresentative) == (low if rep_low else not low)
                if i.isRepresentative:
                    assert (i.unitStart, i.unitCount) == (2 * t, 2)
                else:
                    assert (i.unitStart, i.unitCount) == (2 * t if low else 2 * t + 1, 1)
            for v in range(p - r):
                carrier = orc.lib().orc_rhd_alg_rank_of_virtual(p, root, v)
                rc, ci = orc.rhd_part1(p, carrier, root)
                assert ci.virtualRank == v
                assert ci.isRepresentative if v < r else carrier == v + r


def test_part1_validation(orc):
    assert orc.rhd_part1(0, 0)[0] == 1
    assert orc.rhd_part1(4, 4, 0)[0] == 1
    assert orc.rhd_part1(4, 0, 4)[0] == 1
    rc, i = orc.rhd_part1(1, 0)
    assert rc == 0 and i.isPowerOfTwo and i.effectiveRankSize == 1
    assert orc.lib().orc_rhd_alg_rank_of_virtual(0, INVALID, 0) == INVALID
    assert orc.lib().orc_rhd_alg_rank_of_virtual(5, INVALID, 4) == INVALID


def test_prepost_seg_modes_p5(orc):
    for j, pre_full, post_full, pre_w, post_w in GOLD["prepost_seg_mode_p5"]["rows"]:
        rc, info = orc.rhd_part1(5, j)
        rc, pre, post = orc.rhd_prepost(info, pre_full, post_full)
        assert rc == 0
        assert [pre.nSlices, pre.txSegStart, pre.txSegEnd, pre.rxSegStart, pre.rxSegEnd] == pre_w
        assert [post.nSlices, post.txSegStart, post.txSegEnd, post.rxSegStart, post.rxSegEnd] == post_w
    for p in (2, 4, 8, 16):   # powers of two: both steps empty
        for j in range(p):
            rc, info = orc.rhd_part1(p, j)
            rc, pre, post = orc.rhd_prepost(info, True, True)
            assert rc == 0 and pre.nSlices == 0 and post.nSlices == 0 and pre.peer == INVALID


@pytest.mark.parametrize("p", [2, 3, 4, 5, 6, 7, 9, 17, 32, 48, 64])
def test_rs_steps_deliver_every_contribution_once(orc, p):
    """Counting simulation: every rank contributes +1 to every unit; after PRE(FULL) and the MAIN
    steps each unit holds exactly p at its owner (the invariant of the reference's RsFinalState)."""
    r = p - _largest_pow2_le(p)
    P = p - r
    L = orc.lib()
    hold = [[1] * p for _ in range(p)]
    for t in range(r):
        rc, minfo = orc.rhd_part1(p, t + r)
        rc, pre, post = orc.rhd_prepost(minfo, True, False)
        assert pre.peer == t and (pre.txSegStart, pre.txSegEnd) == (0, p)
        for u in range(p):
            hold[t][u] += hold[t + r][u]
            hold[t + r][u] = 0
    steps = [orc.rhd_rs_steps(_info_for_virtual(orc, p, v))[1] for v in range(P)]
    n_steps = L.orc_rhd_step_num(P)
    for k in range(n_steps):
        sent = [[0] * p for _ in range(p)]
        for v in range(P):
            s, phys = steps[v][k], L.orc_rhd_alg_rank_of_virtual(p, INVALID, v)
            ps = steps[s.peer][k]   # mirror: my tx is the peer's rx
            assert ps.peer == v and (ps.rxSegStart, ps.rxSegEnd) == (s.txSegStart, s.txSegEnd)
            for u in range(s.txSegStart, s.txSegEnd):
                sent[phys][u], hold[phys][u] = hold[phys][u], 0
        for v in range(P):
            s, phys = steps[v][k], L.orc_rhd_alg_rank_of_virtual(p, INVALID, v)
            peer = L.orc_rhd_alg_rank_of_virtual(p, INVALID, s.peer)
            for u in range(s.rxSegStart, s.rxSegEnd):
                hold[phys][u] += sent[peer][u]
    for u in range(p):
        v = u // 2 if u < 2 * r else u - r
        assert hold[L.orc_rhd_alg_rank_of_virtual(p, INVALID, v)][u] == p


@pytest.mark.parametrize("p", [2, 3, 5, 6, 7, 9, 17, 32])
def test_ag_steps_mirror_rs_steps(orc, p):
    r = p - _largest_pow2_le(p)
    P = p - r
    n = orc.lib().orc_rhd_step_num(P)
    for v in range(P):
        info = _info_for_virtual(orc, p, v)
        rs, ag = orc.rhd_rs_steps(info)[1], orc.rhd_ag_steps(info)[1]
        for k in range(n):
            a, s = ag[k], rs[n - 1 - k]
            assert a.peer == s.peer
            assert (a.txSegStart, a.txSegEnd, a.rxSegStart, a.rxSegEnd) == (s.rxSegStart, s.rxSegEnd, s.txSegStart, s.txSegEnd)


def test_step_validation(orc):
    import oracle
    info = oracle.RhdPart1()
    assert orc.rhd_rs_steps(info)[0] == 1
    info.effectiveRankSize, info.r, info.virtualRank = 4, 0, 4
    assert orc.rhd_rs_steps(info)[0] == 1 and orc.rhd_ag_steps(info)[0] == 1
    info.effectiveRankSize, info.r, info.virtualRank = 6, 1, 5
    assert orc.rhd_rs_steps(info)[0] == 1
    info.effectiveRankSize, info.r, info.virtualRank = 4, 4, 0
    assert orc.rhd_rs_steps(info)[0] == 1


def test_nhr_hand_table_and_totals(orc):
    for row in GOLD["nhr_steps_n4_rank0"]:
        rc, to, frm, tx, rx = orc.nhr_step_info(4, 0, row["step"])
        assert rc == 0 and (to, frm, tx, rx) == (row["toRank"], row["fromRank"], row["tx"], row["rx"])
    for n in (1, 2, 3, 4, 5, 6, 8, 9, 16, 33, 64):
        steps = orc.lib().orc_nhr_step_num(n)
        for me in range(n):
            total = 0
            for s in range(steps):
                rc, to, frm, tx, rx = orc.nhr_step_info(n, me, s)
                assert rc == 0 and to < n and frm < n and all(i < n for i in tx + rx)
                total += len(tx)
            assert total == n - 1


def test_rhd_tail_loop_plan(orc):
    g = GOLD["rhd_tail_one_mib_72_ranks"]
    sel = orc.lib().orc_rhd_select_loop_count
    processed, tail = 0, 0
    while processed < g["totalCount"]:
        c = sel(g["totalCount"] - processed, g["maxCountPerLoop"], g["rankAlign"])
        if c < g["rankAlign"]:
            tail = c
        processed += c
    assert processed == g["totalCount"] and tail == g["tailCount"]
    assert sel(144, 72, 12) == 72      # test/ut/common/hostdpu_inline_reduce/all_reduce_rhd_test.cc:88-94: a full loop, no tail
    for ranks in (2, 3, 6, 12, 16, 24, 72):       # every element processed exactly once
        cap = 3 * ranks
        for total in range(0, 300):
            done = 0
            while done < total:
                c = sel(total - done, cap, ranks)
                assert 0 < c <= cap
                assert c == total - done if c < ranks else c % ranks == 0
                done += c
            assert done == total


def test_local_copy_slices_merges_contiguous_runs(orc):
    # three contiguous slices then a gap then one more: two copies
    got = orc.local_copy_slices([0, 16, 32, 100], [64, 80, 96, 400], [16, 16, 16, 8])
    assert got == [(0, 64, 48), (100, 400, 8)]
    # source contiguous but destination not: no merge
    got = orc.local_copy_slices([0, 16], [0, 32], [16, 16])
    assert got == [(0, 0, 16), (16, 32, 16)]
    assert orc.local_copy_slices([5], [9], [7]) == [(5, 9, 7)]


def test_ccl_buffer_available_size_known_answers(orc):
    g = GOLD["ccl_buffer_available_size"]
    for env, want in g["valid"]:
        assert orc.ccl_buffer_available_size(env) == (0, want)
    for env in g["invalid"]:
        assert orc.ccl_buffer_available_size(env)[0] != 0, env


def test_rhd_tail_workspace_known_answers(orc):
    for count, align, esz, ws, rc, left, in_off, out_off in GOLD["rhd_tail_workspace"]["rows"]:
        got = orc.rhd_prepare_tail_workspace(count, align, esz, ws)
        assert got[0] == rc and got[1] == left, (count, align, esz, ws, got)
        if in_off is not None:
            assert got[2:] == (in_off, out_off)
            assert in_off % 128 == 0 and out_off % 128 == 0            # the reference's own assertions
            assert in_off + align * esz <= out_off and out_off + align * esz <= ws


def test_loop_limits_closed_forms(orc):
    """Sole executor: floor(ccl / multiple / 128) * 128 bytes, never above ccl, in whole elements.
    RHD sequence: the tail tiles come off first, then half, 128-byte floor, whole elements, multiple of p."""
    for ccl in (1 << 20, 199 << 20, 1000, 4096 + 17):
        for mult in (0, 1, 2, 6, 8):
            for esz in (1, 2, 4, 8):
                want = (ccl if mult == 0 else min(ccl, ccl // mult // 128 * 128)) // esz
                assert orc.sole_max_count_per_loop(ccl, mult, esz) == want
    for ccl, count, p, esz in ((4096, 144, 6, 4), (4096, 145, 6, 4), (1 << 20, 1000, 6, 2), (1 << 20, 1001, 7, 2)):
        left = ccl
        if count % p:
            slot = -(-p * esz // 128) * 128
            left = ccl - 2 * slot
        want = left // 2 // 128 * 128 // esz // p * p
        assert orc.rhd_max_count_per_loop(ccl, count, p, esz) == (0, want)
    assert orc.rhd_max_count_per_loop(512, 73, 72, 4)[0] == 4       # too small for the tail tiles
    assert orc.rhd_max_count_per_loop(200, 12, 6, 8)[0] == 4        # half of it, floored to 128 B, holds no whole frame


def test_all_to_all_v_var_area_layout_and_parse(orc):
    """[sendCounts | recvCounts | sdispls | rdispls]; parsing yields counts and byte lengths, displacements and
    byte offsets; the furthest touched byte of either buffer; the size rules of the parser."""
    import ctypes
    L = orc.lib()
    n = 3
    u64 = lambda v: (ctypes.c_uint64 * len(v))(*v)
    sc, rc_, sd, rd = [5, 0, 7], [1, 2, 3], [0, 5, 9], [4, 0, 10]
    var = (ctypes.c_uint64 * (4 * n))()
    L.orc_a2a_construct_var_data(ctypes.c_uint32(n), u64(sc), u64(rc_), u64(sd), u64(rd), var)
    assert list(var) == sc + rc_ + sd + rd
    out = (ctypes.c_uint64 * (8 * n))()
    assert L.orc_a2a_parse_var_data(var, ctypes.c_uint64(4 * n * 8), ctypes.c_uint64(n), ctypes.c_uint64(2), 0, out) == 0
    assert list(out) == sc + [2 * v for v in sc] + rc_ + [2 * v for v in rc_] + sd + [2 * v for v in sd] + rd + \
        [2 * v for v in rd]
    # exactly four vectors; AlltoAllVC may carry a fifth; a ragged size is refused
    for nbytes, vc, want in ((4 * n * 8, 0, 0), (4 * n * 8 - 8, 0, 1), (5 * n * 8, 0, 1), (5 * n * 8, 1, 0),
                             (4 * n * 8 + 8, 1, 1), (6 * n * 8, 1, 1)):
        big = (ctypes.c_uint64 * (6 * n))()
        assert L.orc_a2a_parse_var_data(big, ctypes.c_uint64(nbytes), ctypes.c_uint64(n), ctypes.c_uint64(2), vc,
                                        out) == want, (nbytes, vc)
    assert L.orc_a2a_parse_var_data(var, ctypes.c_uint64(0), ctypes.c_uint64(0), ctypes.c_uint64(2), 0, out) == 1
    i, o = ctypes.c_uint64(0), ctypes.c_uint64(0)
    L.orc_a2a_io_size(ctypes.c_uint32(n), u64(sc), u64(rc_), u64(sd), u64(rd), ctypes.c_uint64(2), ctypes.byref(i),
                      ctypes.byref(o))
    assert (i.value, o.value) == ((9 + 7) * 2, (10 + 3) * 2)
