"""The CPU oracle against the reference's own outputs.

Fixtures in tests/golden/*.npz were produced by the reference's compiled CPU sources
(tests/golden/make_fixtures.py).  The oracle restates the same loops, so fp32 results must agree bit for bit.
"""
import glob
import os

import numpy as np
import pytest

import oracle_lib

CASES = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))
               if not p.endswith("_kat.npz"))


def test_fixture_inventory():
    assert {"c1_tiny_fp32", "gqa_8q2kv_d8_T16", "d64_T132", "gqa_d128_T96_B2", "d64_T256_B2_window", "d32_T80_sharp"} <= set(CASES)


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("pack_parallel", [False, True])
def test_oracle_reproduces_reference_bits(golden_dir, name, pack_parallel):
    fx = np.load(os.path.join(golden_dir, name + ".npz"))
    hq, hkv, d, t, packs, col0, stride = (int(x) for x in fx["geometry"])
    res = oracle_lib.oracle_attention(fx["q"], fx["k"], fx["v"], fx["d_out"], q_heads=hq, kv_heads=hkv, head_dim=d,
                                      seq_len=t, pack_count=packs, col_start=col0, pack_parallel=pack_parallel)
    for key in ("out", "lse", "dq", "dk", "dv"):
        assert res[key].shape == fx[key].shape
        assert np.array_equal(res[key], fx[key], equal_nan=True), f"{name}:{key} differs from the reference's bits"
        inside = res[key][:, col0:col0 + packs * t]
        assert np.isfinite(inside).all()


def test_forward_only_matches_forward_of_full_call(golden_dir):
    fx = np.load(os.path.join(golden_dir, "d64_T132.npz"))
    hq, hkv, d, t, packs, col0, stride = (int(x) for x in fx["geometry"])
    res = oracle_lib.oracle_attention(fx["q"], fx["k"], fx["v"], None, q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t)
    assert np.array_equal(res["out"], fx["out"]) and np.array_equal(res["lse"], fx["lse"])


def test_gemm_and_softmax_known_answers(golden_dir):
    kat = np.load(os.path.join(golden_dir, "gemm_softmax_kat.npz"))
    tags = sorted({k[len("gemm_"):-2] for k in kat.files if k.startswith("gemm_") and k.endswith("_a")})
    assert len(tags) == 4
    for tag in tags:
        ta, tb = (bool(x) for x in kat[f"gemm_{tag}_flags"])
        got = oracle_lib.gemm(kat[f"gemm_{tag}_a"], kat[f"gemm_{tag}_b"], ta, tb)
        assert np.array_equal(got, kat[f"gemm_{tag}_c"]), tag
        # and the product itself is right (float64), not merely reproduced
        a = kat[f"gemm_{tag}_a"].astype(np.float64)
        b = kat[f"gemm_{tag}_b"].astype(np.float64)
        want = (a.T if ta else a) @ (b.T if tb else b)
        assert np.max(np.abs(got - want)) < 1e-4
    got = oracle_lib.softmax_columns(kat["softmax_in"])
    assert np.array_equal(got, kat["softmax_out"])
    assert np.allclose(got.sum(axis=0), 1.0, atol=1e-6)
    assert np.all(got[10:, 3] == 0.0)


def test_invalid_geometry_is_rejected():
    x = np.zeros((8, 8), dtype=np.float32)
    with pytest.raises(ValueError):
        oracle_lib.oracle_attention(x, x, x, None, q_heads=2, kv_heads=2, head_dim=4, seq_len=8, pack_count=2)
    y = np.zeros((12, 8), dtype=np.float32)
    with pytest.raises(ValueError):  # 3 query heads cannot share 2 kv heads
        oracle_lib.oracle_attention(y, x, x, None, q_heads=3, kv_heads=2, head_dim=4, seq_len=8)


@pytest.mark.skipif(oracle_lib.reference() is None, reason="oracle/_ref needs the reference checkout")
@pytest.mark.parametrize("shape", [(3, 1, 24, 77, 2), (4, 2, 16, 200, 1), (1, 1, 64, 300, 1)])
def test_oracle_vs_live_reference_build(shape):
    hq, hkv, d, t, packs = shape
    rng = np.random.default_rng(hash(shape) % (2 ** 32))
    stride = packs * t + 5
    q = rng.standard_normal((hq * d, stride)).astype(np.float32)
    k = rng.standard_normal((hkv * d, stride)).astype(np.float32)
    v = rng.standard_normal((hkv * d, stride)).astype(np.float32)
    g = rng.standard_normal((hq * d, stride)).astype(np.float32)
    kw = dict(q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs, col_start=3)
    a = oracle_lib.oracle_attention(q, k, v, g, **kw)
    for per_head in (False, True):
        b = oracle_lib.oracle_attention(q, k, v, g, lib="ref", per_head=per_head, **kw)
        for key in a:
            assert np.array_equal(a[key], b[key], equal_nan=True), (key, per_head)
