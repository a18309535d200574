"""Pins the oracle's sliding-window / global-token mask before the device kernels are checked against it.

1. bit-exact against the known answers written from the reference's compiled dense masked path
   (tests/golden/sparse_kat.npz, preferSparseCompute = false), and to rounding against its sparse-compute path;
2. live against oracle/_ref where that is built;
3. against what the mask rule fixes: a float64 masked softmax built from index arithmetic, window 1 (every query
   sees only itself: O = V, dV = dO, dQ = dK = 0), a window at least as long as the sequence (plain causal),
   and the exact reach of one key (queries key .. key + window - 1, or every later query for a global token).
"""
import os

import numpy as np
import pytest

import oracle_lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sparse_kat.npz")
TAGS = ["smoke_h2_d16_T16_W4_G2", "gqa_4q2kv_d8_T50_W7_G0", "h1_d64_T140_W33_G5", "h2_d32_T70_W0_G9",
        "h1_d128_T130_W1_G0", "h1_d16_T40_W100_G3"]
KEYS = ("out", "lse", "dq", "dk", "dv")


@pytest.fixture(scope="module")
def kat():
    return np.load(GOLDEN)


def _run(kat, tag, **kw):
    hq, hkv, d, t, packs, window, global_tokens = (int(x) for x in kat[f"{tag}_geometry"])
    return oracle_lib.oracle_attention(kat[f"{tag}_q"], kat[f"{tag}_k"], kat[f"{tag}_v"], kat[f"{tag}_d_out"], q_heads=hq,
                                       kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs, window=window,
                                       global_tokens=global_tokens, **kw)


@pytest.mark.parametrize("tag", TAGS)
def test_matches_reference_dense_masked_path_bit_exactly(kat, tag):
    got = _run(kat, tag)
    for key in KEYS:
        assert np.array_equal(got[key], kat[f"{tag}_dense_{key}"]), key


@pytest.mark.parametrize("tag", TAGS)
def test_matches_reference_sparse_compute_path_to_rounding(kat, tag):
    got = _run(kat, tag)
    for key in KEYS:
        want = kat[f"{tag}_sparse_{key}"]
        assert np.max(np.abs(got[key] - want)) <= 1e-5 * max(1.0, np.max(np.abs(want))), key


def test_live_against_compiled_reference():
    if oracle_lib.reference() is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    rng = np.random.default_rng(123)
    for hq, hkv, d, t, packs, window, global_tokens in [(2, 1, 16, 37, 2, 5, 1), (3, 3, 8, 64, 1, 16, 0), (1, 1, 32, 90, 1, 64, 70)]:
        q, k, v, g = (rng.standard_normal((h * d, packs * t)).astype(np.float32) for h in (hq, hkv, hkv, hq))
        kw = dict(q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs, window=window, global_tokens=global_tokens)
        got = oracle_lib.oracle_attention(q, k, v, g, **kw)
        ref = oracle_lib.oracle_attention(q, k, v, g, lib="ref", prefer_sparse=False, **kw)
        for key in KEYS:
            assert np.array_equal(got[key], ref[key]), key


def _allowed(t, window, global_tokens):
    """[key, query] boolean matrix from index arithmetic (not the oracle's loop)."""
    key = np.arange(t)[:, None]
    query = np.arange(t)[None, :]
    inside = (query - key < window) if window > 0 else np.ones((t, t), dtype=bool)
    return (key <= query) & ((key < global_tokens) | inside)


def _float64(q, k, v, g, hq, hkv, d, t, window, global_tokens):
    allowed = _allowed(t, window, global_tokens)
    group = hq // hkv
    out, dq = np.zeros((hq * d, t)), np.zeros((hq * d, t))
    dk, dv = np.zeros((hkv * d, t)), np.zeros((hkv * d, t))
    lse = np.zeros((hq, t))
    for h in range(hq):
        kv = h // group
        qh, gh = (x[h * d:(h + 1) * d].astype(np.float64) for x in (q, g))
        kh, vh = (x[kv * d:(kv + 1) * d].astype(np.float64) for x in (k, v))
        s = np.where(allowed, (kh.T @ qh) / np.sqrt(d), -np.inf)  # [key, query]
        top = s.max(axis=0)
        e = np.exp(s - top)
        p = e / e.sum(axis=0)
        lse[h] = top + np.log(e.sum(axis=0))
        out[h * d:(h + 1) * d] = vh @ p
        dp = vh.T @ gh
        ds = p * (dp - (p * dp).sum(axis=0)) / np.sqrt(d)
        dq[h * d:(h + 1) * d] = kh @ ds
        dk[kv * d:(kv + 1) * d] += qh @ ds.T
        dv[kv * d:(kv + 1) * d] += gh @ p.T
    return dict(out=out, lse=lse, dq=dq, dk=dk, dv=dv)


@pytest.mark.parametrize("shape", [(2, 2, 16, 45, 6, 0), (4, 2, 8, 64, 9, 3), (1, 1, 32, 100, 40, 50), (2, 1, 16, 30, 0, 4)])
def test_against_float64_masked_softmax(shape):
    hq, hkv, d, t, window, global_tokens = shape
    rng = np.random.default_rng(sum(shape))
    q, k, v, g = (rng.standard_normal((h * d, t)).astype(np.float32) for h in (hq, hkv, hkv, hq))
    got = oracle_lib.oracle_attention(q, k, v, g, q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, window=window,
                                      global_tokens=global_tokens)
    want = _float64(q, k, v, g, hq, hkv, d, t, window, global_tokens)
    for key in KEYS:
        assert np.max(np.abs(got[key] - want[key])) <= 2e-5 * max(1.0, np.max(np.abs(want[key]))), key


def test_window_of_one_and_window_past_the_sequence():
    rng = np.random.default_rng(9)
    hq, hkv, d, t = 2, 1, 16, 33
    q, k, v, g = (rng.standard_normal((h * d, t)).astype(np.float32) for h in (hq, hkv, hkv, hq))
    kw = dict(q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t)
    one = oracle_lib.oracle_attention(q, k, v, g, window=1, **kw)
    assert np.array_equal(one["out"], np.concatenate([v, v]))          # P is the identity
    assert np.array_equal(one["dv"], g[:d] + g[d:])                    # both query heads of the group
    assert not one["dq"].any() and not one["dk"].any()                 # a softmax over one key has no gradient
    assert np.allclose(one["lse"], np.stack([(q[h * d:(h + 1) * d] * k).sum(0) / np.sqrt(d) for h in range(hq)]), atol=1e-5)
    plain = oracle_lib.oracle_attention(q, k, v, g, **kw)
    for window, global_tokens in [(t, 0), (t + 5, 0), (0, 7), (t, 3)]:
        wide = oracle_lib.oracle_attention(q, k, v, g, window=window, global_tokens=global_tokens, **kw)
        for key in KEYS:
            assert np.array_equal(wide[key], plain[key]), (window, global_tokens, key)


def test_reach_of_one_key():
    rng = np.random.default_rng(10)
    h, d, t, window, global_tokens = 1, 8, 40, 6, 2
    q, k, v, g = (rng.standard_normal((h * d, t)).astype(np.float32) for _ in range(4))
    kw = dict(q_heads=h, kv_heads=h, head_dim=d, seq_len=t, window=window, global_tokens=global_tokens)
    base = oracle_lib.oracle_attention(q, k, v, g, **kw)
    for key in (1, 10, 38):
        k2, v2 = k.copy(), v.copy()
        k2[:, key] += 1.0
        v2[:, key] -= 2.0
        moved = oracle_lib.oracle_attention(q, k2, v2, g, **kw)
        changed = np.any(moved["out"] != base["out"], axis=0)
        reach = np.zeros(t, dtype=bool)
        reach[key:(t if key < global_tokens else min(t, key + window))] = True
        assert np.array_equal(changed, reach), key
        assert np.array_equal(np.any(moved["dq"] != base["dq"], axis=0), reach), key


def test_sparse_mask_needs_the_causal_flag():
    x = np.zeros((8, 4), dtype=np.float32)
    with pytest.raises(ValueError):
        oracle_lib.oracle_attention(x, x, x, q_heads=1, kv_heads=1, head_dim=8, seq_len=4, causal=False, window=2)
    with pytest.raises(ValueError):
        oracle_lib.oracle_attention(x, x, x, q_heads=1, kv_heads=1, head_dim=8, seq_len=4, global_tokens=-1)
