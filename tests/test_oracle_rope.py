"""Pins the oracle's rotary embedding (tables and rotation) before anything is checked against it.

1. bit-exact against the known answers written from the reference's compiled RotaryEmbedding
   (tests/golden/rope_kat.npz, made by tests/golden/make_fixtures.py);
2. live against oracle/_ref where that is built;
3. against what the mathematics fixes: the angle formula in float64, rotations preserve pair norms, the inverse
   undoes the forward rotation, position 0 is the identity, offsets and pack segments only re-index positions.
"""
import os

import numpy as np
import pytest

import oracle_lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rope_kat.npz")
TAGS = ["h3_d16_T40", "h2_d64_T130", "h1_d128_T33_base500k"]


@pytest.fixture(scope="module")
def kat():
    return np.load(GOLDEN)


@pytest.mark.parametrize("tag", TAGS)
def test_tables_and_rotation_match_reference_known_answers(kat, tag):
    heads, d, t, positions = (int(x) for x in kat[f"{tag}_geometry"])
    base = float(kat[f"{tag}_base"])
    cos, sin = oracle_lib.rope_tables(d, positions, base)
    assert np.array_equal(cos, kat[f"{tag}_cos"]) and np.array_equal(sin, kat[f"{tag}_sin"])
    x = kat[f"{tag}_x"]
    assert np.array_equal(oracle_lib.rope_rotate(x, heads, d, cos, sin), kat[f"{tag}_forward"])
    assert np.array_equal(oracle_lib.rope_rotate(x, heads, d, cos, sin, inverse=True), kat[f"{tag}_inverse"])


def test_live_against_compiled_reference():
    if oracle_lib.reference() is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    rng = np.random.default_rng(77)
    for heads, d, t, base in [(2, 8, 19, 10000.0), (5, 32, 64, 1000.0), (1, 128, 200, 10000.0)]:
        x = rng.standard_normal((heads * d, t)).astype(np.float32)
        cos, sin = oracle_lib.rope_tables(d, t, base)
        rcos, rsin = oracle_lib.rope_tables(d, t, base, lib="ref")
        assert np.array_equal(cos, rcos) and np.array_equal(sin, rsin)
        for inverse in (False, True):
            assert np.array_equal(oracle_lib.rope_rotate(x, heads, d, cos, sin, inverse=inverse),
                                  oracle_lib.ref_rope_rotate(x, heads, d, t, base, inverse=inverse))


def test_tables_follow_the_angle_formula():
    d, positions, base = 64, 300, 10000.0
    cos, sin = oracle_lib.rope_tables(d, positions, base)
    pair = np.arange(d // 2, dtype=np.float64)
    # angle = position * base ** (-2 pair / d) in float64; the tables carry the float32 error of the angle, which
    # grows with the position (a wrong exponent, sign or pairing is off by O(1))
    exact = np.arange(positions, dtype=np.float64)[:, None] * base ** (-2.0 * pair / d)[None, :]
    assert np.max(np.abs(cos - np.cos(exact))) < 1e-4
    assert np.max(np.abs(sin - np.sin(exact))) < 1e-4
    assert np.max(np.abs(cos[:8] - np.cos(exact[:8]))) < 1e-6 and np.max(np.abs(sin[:8] - np.sin(exact[:8]))) < 1e-6
    assert cos[0].tolist() == [1.0] * (d // 2) and sin[0].tolist() == [0.0] * (d // 2)


def test_rotation_invariants():
    rng = np.random.default_rng(5)
    heads, d, t = 3, 32, 50
    x = rng.standard_normal((heads * d, t)).astype(np.float32)
    cos, sin = oracle_lib.rope_tables(d, 128)
    y = oracle_lib.rope_rotate(x, heads, d, cos, sin)
    # a rotation of each (even, odd) pair: norms survive, the first column (position 0) is untouched
    nx = x.reshape(heads, d // 2, 2, t)
    ny = y.reshape(heads, d // 2, 2, t)
    assert np.allclose((nx ** 2).sum(2), (ny ** 2).sum(2), rtol=2e-6, atol=1e-6)
    assert np.array_equal(y[:, 0], x[:, 0])
    assert not np.allclose(y[:, 1:], x[:, 1:], atol=1e-3)
    back = oracle_lib.rope_rotate(y, heads, d, cos, sin, inverse=True)
    assert np.max(np.abs(back - x)) < 2e-6
    # explicit closed form for one element pair
    p, c, h = 5, 17, 2
    e, o = float(x[h * d + 2 * p, c]), float(x[h * d + 2 * p + 1, c])
    ang = c * 10000.0 ** (-2.0 * p / d)
    assert abs(y[h * d + 2 * p, c] - (e * np.cos(ang) - o * np.sin(ang))) < 1e-5
    assert abs(y[h * d + 2 * p + 1, c] - (e * np.sin(ang) + o * np.cos(ang))) < 1e-5


def test_offsets_segments_and_windows_only_reindex_positions():
    rng = np.random.default_rng(6)
    heads, d, t = 2, 16, 24
    cos, sin = oracle_lib.rope_tables(d, 64)
    x = rng.standard_normal((heads * d, 3 * t + 5)).astype(np.float32)
    # offset k == rotating with the table rows shifted by k
    off = oracle_lib.rope_rotate(x[:, :t], heads, d, cos, sin, position_offset=9)
    assert np.array_equal(off, oracle_lib.rope_rotate(x[:, :t], heads, d, np.ascontiguousarray(cos[9:]),
                                                       np.ascontiguousarray(sin[9:])))
    # segments: every pack of t columns is rotated like a sequence of its own; columns outside the window stay
    seg = oracle_lib.rope_rotate(x, heads, d, cos, sin, col_start=2, columns=3 * t, segment_length=t)
    for p in range(3):
        lo = 2 + p * t
        assert np.array_equal(seg[:, lo:lo + t], oracle_lib.rope_rotate(x[:, lo:lo + t], heads, d, cos, sin))
    assert np.array_equal(seg[:, :2], x[:, :2]) and np.array_equal(seg[:, 2 + 3 * t:], x[:, 2 + 3 * t:])


def test_positions_past_the_table_are_rejected():
    cos, sin = oracle_lib.rope_tables(8, 10)
    x = np.zeros((8, 12), dtype=np.float32)
    with pytest.raises(ValueError):
        oracle_lib.rope_rotate(x, 1, 8, cos, sin)                       # 12 columns, 10 positions
    with pytest.raises(ValueError):
        oracle_lib.rope_rotate(x[:, :6], 1, 8, cos, sin, position_offset=5)
    with pytest.raises(ValueError):
        oracle_lib.rope_rotate(x, 1, 8, cos, sin, segment_length=11)
    oracle_lib.rope_rotate(x, 1, 8, cos, sin, segment_length=6)         # 12 columns in segments of 6: fine
