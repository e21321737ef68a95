"""Pins the oracle's pairwise reduce and half conversions (rows a1-a3 of the hot path).

The reference holds no numeric golden vector for these functions, so the checks are against what
the mathematics fixes: numpy's IEEE float16 conversion over every bit pattern / every rounding
boundary, two's-complement modular arithmetic over every int8 pair, single IEEE operations, and
hand-enumerated signed-zero / NaN / tie tables for MAX and MIN
(reference alg_data_trans_wrapper.cc:1082-1358).
"""
import numpy as np
import pytest

I8, I16, I32, F16, F32, I64, U64, F64, BF16 = 0, 1, 2, 3, 4, 5, 6, 10, 11
SUM, PROD, MAX, MIN = range(4)


# ---------------------------------------------------------------------------------------------
# a2: conversions
# ---------------------------------------------------------------------------------------------
def test_fp16_to_fp32_every_bit_pattern(orc):
    h = np.arange(65536, dtype=np.uint16)
    got = orc.fp16_to_fp32_bits(h)
    ref = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], ref[~nan])
    # NaN: sign, all-ones exponent, the 10 payload bits moved to the top of the fp32 mantissa
    hn = h[nan].astype(np.uint32)
    expect = ((hn >> 15) << 31) | (0xFF << 23) | ((hn & 0x3FF) << 13)
    assert np.array_equal(got[nan], expect)


def test_fp16_to_fp32_known_answers(orc):
    got = orc.fp16_to_fp32_bits(np.array([0x3C00, 0x0001, 0x8000, 0x7BFF, 0x0400, 0xFC00, 0x03FF], dtype=np.uint16))
    vals = got.view(np.float32)
    assert vals[0] == 1.0
    assert vals[1] == 2.0 ** -24
    assert got[2] == 0x80000000
    assert vals[3] == 65504.0
    assert vals[4] == 2.0 ** -14
    assert np.isneginf(vals[5])
    assert vals[6] == 1023 * 2.0 ** -24


def _f32_bits_corpus():
    rng = np.random.default_rng(1234)
    parts = [rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)]
    # every fp16 value, every midpoint between neighbours, and one fp32 ulp either side of each
    h = np.arange(0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    hi[-1] = np.float32(65536.0)  # the overflow boundary: 65520 is the tie that rounds to Inf
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    for base in (lo, mid):
        b = base.view(np.uint32)
        for d in (-1, 0, 1):
            v = (b.astype(np.int64) + d).clip(0, 0x7F7FFFFF).astype(np.uint32)
            parts.append(v)
            parts.append(v | np.uint32(0x80000000))
    # fp32 subnormals and the smallest normals
    parts.append(np.arange(0, 4096, dtype=np.uint32))
    parts.append(np.arange(0x007FF000, 0x00801000, dtype=np.uint32))
    # around 2^-25 (half of the smallest fp16 subnormal: ties to zero) and 2^-24
    for e in (-26, -25, -24, -15, -14):
        c = np.float32(2.0 ** e).view(np.uint32).astype(np.int64)
        parts.append(np.arange(c - 64, c + 64).astype(np.uint32))
    return np.concatenate(parts)


def test_fp32_to_fp16_matches_ieee_rne(orc):
    bits = _f32_bits_corpus()
    f = bits.view(np.float32)
    keep = ~np.isnan(f)
    got = orc.fp32_to_fp16_bits(bits[keep])
    with np.errstate(over="ignore"):
        ref = f[keep].astype(np.float16).view(np.uint16)
    bad = np.nonzero(got != ref)[0]
    assert bad.size == 0, (hex(int(bits[keep][bad[0]])), hex(int(got[bad[0]])), hex(int(ref[bad[0]])))


def test_fp32_to_fp16_known_answers(orc):
    # (fp32 bits, fp16 bits).  NaN: top 10 mantissa bits kept, forced to 1 when they are all zero.
    kat = [
        (0x3F802000, 0x3C01),  # 1.0009765625 -> tie? no: exactly representable + 0 -> 0x3C01
        (0x3F801000, 0x3C00),  # 1 + 2^-11: tie, rounds to even (down)
        (0x3F803000, 0x3C02),  # 1 + 3*2^-11: tie, rounds to even (up)
        (0x477FE000, 0x7BFF),  # 65504
        (0x477FF000, 0x7C00),  # 65520: tie -> Inf
        (0x477FEFFF, 0x7BFF),  # just below the tie
        (0x33800000, 0x0001),  # 2^-24
        (0x33000000, 0x0000),  # 2^-25: tie -> even (zero)
        (0x33000001, 0x0001),  # just above 2^-25
        (0x32FFFFFF, 0x0000),
        (0x387FE000, 0x0400),  # largest subnormal + half ulp ... rounds up to the smallest normal
        (0x00000001, 0x0000),  # fp32 subnormal -> +0
        (0x807FFFFF, 0x8000),  # negative fp32 subnormal -> -0
        (0x7F800000, 0x7C00), (0xFF800000, 0xFC00),
        (0x7FC00000, 0x7E00),  # quiet NaN
        (0x7F800001, 0x7C01),  # payload below bit 13 only -> forced non-zero
        (0x7F802000, 0x7C01),  # payload bit 13 -> mantissa 1
        (0xFFFFFFFF, 0xFFFF),
        (0x7FA00000, 0x7D00),
    ]
    bits = np.array([k for k, _ in kat], dtype=np.uint32)
    got = orc.fp32_to_fp16_bits(bits)
    for (k, want), g in zip(kat, got):
        assert int(g) == want, (hex(k), hex(int(g)), hex(want))


def test_fp16_round_trip_is_identity(orc):
    h = np.arange(65536, dtype=np.uint16)
    back = orc.fp32_to_fp16_bits(orc.fp16_to_fp32_bits(h))
    assert np.array_equal(back, h)  # includes every NaN payload


def test_bf16_narrow_is_rne_on_upper_half(orc):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    keep = ~np.isnan(f)
    got = orc.fp32_to_bf16_bits(bits[keep]).astype(np.uint32)
    # closed form: nearest multiple of 2^16 in the bit pattern, ties to the even upper half
    b = bits[keep].astype(np.uint64)
    low = b & 0xFFFF
    up = b >> 16
    expect = np.where(low > 0x8000, up + 1, np.where(low < 0x8000, up, up + (up & 1))).astype(np.uint32)
    assert np.array_equal(got, expect & 0xFFFF)
    # NaN stays NaN with the sign kept
    nan_bits = np.array([0x7FC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF], dtype=np.uint32)
    g = orc.fp32_to_bf16_bits(nan_bits)
    assert [hex(int(x)) for x in g] == ["0x7fc0", "0x7f81", "0xff81", "0x7fff"]
    assert np.array_equal(orc.np_fp32_to_bf16_bits(f), orc.fp32_to_bf16_bits(bits))


def test_bf16_round_trip_is_identity(orc):
    h = np.arange(65536, dtype=np.uint16)
    wide = (h.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(orc.bf16_bits_to_fp32(h).view(np.uint32), wide.view(np.uint32))
    assert np.array_equal(orc.fp32_to_bf16_bits(wide.view(np.uint32)), h)  # includes every NaN payload


# ---------------------------------------------------------------------------------------------
# a1: integers = two's-complement modular arithmetic
# ---------------------------------------------------------------------------------------------
def _int_expect(src, dst, op, bits):
    s = src.astype(object)
    d = dst.astype(object)
    mod = 1 << bits
    if op == SUM:
        r = [(int(a) + int(b)) % mod for a, b in zip(s, d)]
    elif op == PROD:
        r = [(int(a) * int(b)) % mod for a, b in zip(s, d)]
    elif op == MAX:
        r = [max(int(a), int(b)) % mod for a, b in zip(s, d)]
    else:
        r = [min(int(a), int(b)) % mod for a, b in zip(s, d)]
    return np.array(r, dtype=object)


def _as_unsigned(a, bits):
    return np.array([int(v) % (1 << bits) for v in a], dtype=object)


def test_int8_every_pair_every_op(orc):
    v = np.arange(-128, 128, dtype=np.int8)
    src = np.repeat(v, 256)
    dst0 = np.tile(v, 256)
    for op in (SUM, PROD, MAX, MIN):
        dst = dst0.copy()
        assert orc.pair_reduce(dst, src, I8, op) == 0
        s, d = src.astype(np.int32), dst0.astype(np.int32)
        if op == SUM:
            want = ((s + d) & 0xFF)
        elif op == PROD:
            want = ((s * d) & 0xFF)
        elif op == MAX:
            want = np.maximum(s, d) & 0xFF
        else:
            want = np.minimum(s, d) & 0xFF
        assert np.array_equal(dst.view(np.uint8).astype(np.int32), want), op


@pytest.mark.parametrize("dtype,npdt,bits", [(I16, np.int16, 16), (I32, np.int32, 32), (I64, np.int64, 64),
                                              (U64, np.uint64, 64)])
def test_wide_int_edges_and_random(orc, dtype, npdt, bits):
    info = np.iinfo(npdt)
    edge = [info.min, info.min + 1, -1 if info.min < 0 else 1, 0, 1, 2, 3, info.max - 1, info.max,
            info.max // 2, info.max // 2 + 1, 0x5555, 2 ** (bits // 2), 2 ** (bits // 2) + 1]
    edge = np.array([e for e in edge if info.min <= e <= info.max], dtype=npdt)
    rng = np.random.default_rng(bits)
    rnd = rng.integers(info.min, info.max, size=2000, dtype=npdt, endpoint=True)
    vals = np.concatenate([edge, rnd])
    src = np.repeat(edge, vals.size)
    dst0 = np.tile(vals, edge.size)
    for op in (SUM, PROD, MAX, MIN):
        if dtype == I16 and op == PROD:
            continue
        dst = dst0.copy()
        assert orc.pair_reduce(dst, src, dtype, op) == 0
        want = _int_expect(src, dst0, op, bits)
        assert np.array_equal(_as_unsigned(dst, bits), want), op


def test_int32_prod_wraparound_known_answers(orc):
    src = np.array([-2, 2_000_000_000, -2147483648, 65536], dtype=np.int32)
    dst = np.array([2, 2, -1, 65536], dtype=np.int32)
    orc.pair_reduce(dst, src, I32, PROD)
    assert dst.tolist() == [-4, -294967296, -2147483648, 0]


# ---------------------------------------------------------------------------------------------
# a1: floating point = one IEEE operation; MAX / MIN = compare-and-select with src on ties
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,npdt,udt", [(F32, np.float32, np.uint32), (F64, np.float64, np.uint64)])
def test_float_sum_prod_single_ieee_op(orc, dtype, npdt, udt):
    rng = np.random.default_rng(99)
    n = 200_000
    bits = 32 if npdt == np.float32 else 64
    src = rng.integers(0, 2 ** bits, size=n, dtype=np.uint64).astype(udt).view(npdt)
    dst0 = rng.integers(0, 2 ** bits, size=n, dtype=np.uint64).astype(udt).view(npdt)
    # also moderate values where rounding, cancellation and subnormal results occur
    src[: n // 2] = (rng.standard_normal(n // 2) * 10.0 ** rng.integers(-30, 30, n // 2)).astype(npdt)
    dst0[: n // 2] = (rng.standard_normal(n // 2) * 10.0 ** rng.integers(-30, 30, n // 2)).astype(npdt)
    ok = ~(np.isnan(src) | np.isnan(dst0))
    with np.errstate(all="ignore"):
        for op, fn in ((SUM, np.add), (PROD, np.multiply)):
            dst = dst0.copy()
            assert orc.pair_reduce(dst, src, dtype, op) == 0
            want = fn(src, dst0)
            m = ok & ~np.isnan(want)
            assert np.array_equal(dst.view(udt)[m], want.view(udt)[m])
            assert np.all(np.isnan(dst[~m]))


def test_fp32_max_min_truth_table(orc):
    nan = np.float32(np.nan)
    pz, nz, inf = np.float32(0.0), np.float32(-0.0), np.float32(np.inf)
    # (src, dst, max, min): std::max(src,dst) = (src<dst)?dst:src ; std::min(src,dst) = (dst<src)?dst:src
    table = [
        (1.0, 2.0, 2.0, 1.0), (2.0, 1.0, 2.0, 1.0), (3.0, 3.0, 3.0, 3.0),
        (nz, pz, nz, nz),      # equal compare -> src wins both ways
        (pz, nz, pz, pz),
        (nan, 1.0, nan, nan),  # unordered -> src (the NaN) is returned
        (1.0, nan, 1.0, 1.0),  # NaN already in dst is dropped
        (inf, 1.0, inf, 1.0), (-inf, 1.0, 1.0, -inf), (nan, nan, nan, nan),
    ]
    src = np.array([t[0] for t in table], dtype=np.float32)
    dst0 = np.array([t[1] for t in table], dtype=np.float32)
    for op, col in ((MAX, 2), (MIN, 3)):
        dst = dst0.copy()
        orc.pair_reduce(dst, src, F32, op)
        want = np.array([t[col] for t in table], dtype=np.float32)
        assert np.array_equal(dst.view(np.uint32), want.view(np.uint32)), (op, dst, want)


def test_max_min_return_src_bit_pattern_on_unordered(orc):
    # NaN payloads travel untouched because MAX / MIN only select.
    src = np.array([0x7FC12345, 0xFFC00001, 0x3F800000], dtype=np.uint32).view(np.float32)
    dst = np.array([0x3F800000, 0x7FC54321, 0x7FC54321], dtype=np.uint32).view(np.float32)
    d = dst.copy()
    orc.pair_reduce(d, src, F32, MAX)
    assert [hex(x) for x in d.view(np.uint32)] == ["0x7fc12345", "0xffc00001", "0x3f800000"]


def test_fp16_host_pattern_rounds_every_step(orc):
    """AicpuReduceFp16: widen, fp32 op, narrow -- equals numpy float16(float32(a) op float32(b))."""
    rng = np.random.default_rng(5)
    n = 300_000
    src = rng.integers(0, 65536, size=n, dtype=np.uint16)
    dst0 = rng.integers(0, 65536, size=n, dtype=np.uint16)
    sf, df = src.view(np.float16).astype(np.float32), dst0.view(np.float16).astype(np.float32)
    ok = ~(np.isnan(sf) | np.isnan(df))
    with np.errstate(all="ignore"):
        for op, fn in ((SUM, np.add), (PROD, np.multiply)):
            dst = dst0.copy()
            assert orc.pair_reduce(dst, src, F16, op) == 0
            want = fn(sf, df).astype(np.float16)
            m = ok & ~np.isnan(want)
            assert np.array_equal(dst[m], want.view(np.uint16)[m]), op
            assert np.all(np.isnan(dst.view(np.float16)[ok & ~m]))
        for op in (MAX, MIN):
            dst = dst0.copy()
            orc.pair_reduce(dst, src, F16, op)
            if op == MAX:
                want = np.where(sf < df, dst0, src)
            else:
                want = np.where(df < sf, dst0, src)
            assert np.array_equal(dst, want)


def test_fp16_prod_chain_rounds_after_every_step(orc):
    """A PROD chain narrows after every step; that is observably different from one final rounding."""
    rng = np.random.default_rng(11)
    n = 50_000
    xs = [(1.0 + rng.random(n)).astype(np.float16) for _ in range(4)]
    acc = xs[0].view(np.uint16).copy()
    emu = xs[0].copy()
    for x in xs[1:]:
        orc.pair_reduce(acc, x.view(np.uint16), F16, PROD)
        emu = (x.astype(np.float32) * emu.astype(np.float32)).astype(np.float16)
    assert np.array_equal(acc, emu.view(np.uint16))
    once = np.prod(np.stack([x.astype(np.float64) for x in xs]), axis=0).astype(np.float16)
    assert np.count_nonzero(once != emu) > n // 20


def test_aicpu_reduce_admission(orc):
    """Size mismatch and types without a host path return HCCL_E_INTERNAL (wrapper.cc:1264-1270, 1310-1313)."""
    a = np.zeros(8, dtype=np.int32)
    b = np.zeros(8, dtype=np.int32)
    assert orc.aicpu_reduce(a, b, I32, SUM) == 0
    assert orc.aicpu_reduce(a, b, I32, SUM, dst_bytes=32, src_bytes=16) == 4
    assert orc.aicpu_reduce(a, b, I16, SUM) == 4
    assert orc.aicpu_reduce(a, b, BF16, SUM) == 4
    assert orc.aicpu_reduce(a, b, 7, SUM) == 4
    for dt in (I8, I32, F16, F32, I64, U64, F64):
        assert orc.aicpu_reduce(a, b, dt, MAX) == 0


def test_chain_operand_roles(orc):
    """In acc = x_r (+) acc the new rank is src: ties resolve toward the later rank."""
    acc = np.array([0.0], dtype=np.float32)           # rank 0: +0
    orc.pair_reduce(acc, np.array([-0.0], dtype=np.float32), F32, MAX)   # rank 1: -0
    assert np.signbit(acc[0])
    orc.pair_reduce(acc, np.array([0.0], dtype=np.float32), F32, MAX)    # rank 2: +0
    assert not np.signbit(acc[0])


def test_local_reduce_routing(orc):
    """64-bit types and PROD are reduced on the host, everything else on the device: the same rule decides where
    the library falls back to the host-reduce mesh order."""
    L = orc.lib()
    host = {(t, op) for t in range(18) for op in range(4) if L.orc_local_reduce_runs_on_host(t, op)}
    want = {(t, op) for t in range(18) for op in range(4) if t in (5, 6, 10) or op == 1}
    assert host == want
