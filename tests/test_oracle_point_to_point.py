"""Oracle for Send / Recv / BatchSendRecv: which send meets which receive (reference
src/ops/batch_send_recv/algorithm/executor/ins_v2_batch_send_recv_executor.cc:105-128, 137-200), pinned by
distinct byte patterns on tiny worlds."""
import numpy as np
import pytest

import oracle

F32, I8, F16 = oracle.FP32, oracle.INT8, oracle.FP16
SEND, RECV = 0, 1


@pytest.fixture(scope="module")
def orc():
    oracle.lib()
    return oracle


def pat(rank, tag, count, dt=np.float32):
    v = np.arange(count) + 1000 * rank + 100000 * tag
    if dt == np.int8:
        v = v % 101 + tag
    elif dt == np.float16:
        v = v % 1999 + tag
    return v.astype(dt)


def test_ring_exchange_is_a_permutation_of_buffers(orc):
    n, c = 5, 33
    outs = [np.zeros(c, dtype=np.float32) for _ in range(n)]
    items = [[(SEND, pat(r, 0, c), c, F32, (r + 1) % n), (RECV, outs[r], c, F32, (r - 1) % n)] for r in range(n)]
    assert orc.batch_send_recv(items) == 0
    for r in range(n):
        assert np.array_equal(outs[r], pat((r - 1) % n, 0, c))


def test_several_transfers_between_two_ranks_pair_by_count_then_type_not_by_position(orc):
    """Rank 0 lists its sends small-first, rank 1 its receives in yet another order: the larger count pairs
    first, equal counts pair by the larger data-type value (fp16 = 3 before int8 = 0)."""
    big, mid = pat(0, 1, 64), pat(0, 2, 16)
    half = pat(0, 3, 16, np.float16)                        # 16 elements of fp16
    bytes_ = pat(0, 4, 16, np.int8)                         # 16 elements of int8
    r_big, r_mid = np.zeros(64, np.float32), np.zeros(16, np.float32)
    r_half, r_bytes = np.zeros(16, np.float16), np.zeros(16, np.int8)
    items = [
        [(SEND, bytes_, 16, I8, 1), (SEND, mid, 16, F32, 1), (SEND, half, 16, F16, 1), (SEND, big, 64, F32, 1)],
        [(RECV, r_mid, 16, F32, 0), (RECV, r_big, 64, F32, 0), (RECV, r_bytes, 16, I8, 0), (RECV, r_half, 16, F16, 0)],
    ]
    assert orc.batch_send_recv(items) == 0
    assert np.array_equal(r_big, big) and np.array_equal(r_mid, mid)
    assert np.array_equal(r_half, half) and np.array_equal(r_bytes, bytes_)


def test_equal_transfers_keep_their_order_of_appearance(orc):
    a, b = pat(0, 5, 8), pat(0, 6, 8)
    ra, rb = np.zeros(8, np.float32), np.zeros(8, np.float32)
    assert orc.batch_send_recv([[(SEND, a, 8, F32, 1), (SEND, b, 8, F32, 1)],
                                [(RECV, ra, 8, F32, 0), (RECV, rb, 8, F32, 0)]]) == 0
    assert np.array_equal(ra, a) and np.array_equal(rb, b)


def test_own_rank_transfers_and_empty_items(orc):
    x, y = pat(2, 7, 12), np.zeros(12, np.float32)
    z = np.zeros(4, np.float32)
    items = [[], [(SEND, None, 0, F32, 0)], [(SEND, x, 12, F32, 2), (RECV, y, 12, F32, 2), (RECV, z, 0, F32, 0)]]
    assert orc.batch_send_recv(items) == 0
    assert np.array_equal(y, x) and np.all(z == 0)


def test_unmatched_or_unequal_transfers_are_rejected(orc):
    x, y = pat(0, 8, 8), np.zeros(8, np.float32)
    assert orc.batch_send_recv([[(SEND, x, 8, F32, 1)], []]) == 1                        # nobody receives
    assert orc.batch_send_recv([[(SEND, x, 8, F32, 1)], [(RECV, y, 4, F32, 0)]]) == 1    # counts differ
    assert orc.batch_send_recv([[(SEND, x, 8, F32, 1)], [(RECV, y, 8, I8, 0)]]) == 1     # types differ
    assert orc.batch_send_recv([[(SEND, x, 8, F32, 2)], [(RECV, y, 8, F32, 0)]]) == 1    # no such rank
    assert orc.batch_send_recv([[(SEND, x, 8, 12, 1)], [(RECV, y, 8, 12, 0)]]) == 5      # int128
    assert orc.batch_send_recv([[(SEND, None, 8, F32, 1)], [(RECV, y, 8, F32, 0)]]) == 2
    assert orc.batch_send_recv([[(2, x, 8, F32, 1)], [(RECV, y, 8, F32, 0)]]) == 1       # neither send nor receive


def test_all_pairs_exchange(orc):
    n, c = 4, 9
    outs = [[np.zeros(c + j, dtype=np.float32) for j in range(n)] for _ in range(n)]
    items = []
    for r in range(n):
        row = []
        for j in range(n):
            if j != r:
                row.append((SEND, pat(r, j, c + j), c + j, F32, j))        # r -> j carries c + j elements
                row.append((RECV, outs[r][j], c + r, F32, j))              # j -> r carries c + r elements
        items.append(row)
    for r in range(n):
        for j in range(n):
            outs[r][j] = np.zeros(c + r, dtype=np.float32)
            items[r] = [(k, (outs[r][j] if (k == RECV and rem == j) else b), cnt, dt, rem)
                        for (k, b, cnt, dt, rem) in items[r]]
    assert orc.batch_send_recv(items) == 0
    for r in range(n):
        for j in range(n):
            if j != r:
                assert np.array_equal(outs[r][j], pat(j, r, c + r)), (r, j)
