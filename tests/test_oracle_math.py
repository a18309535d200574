"""Pins the oracle by what the mathematics fixes, independently of the reference build:
closed forms, float64 autograd, central finite differences, and the relations the reference's own
GQA host smoke asserts (Layers/CausalSelfAttention.cpp:549-684)."""
import numpy as np
import pytest

import brute
import oracle_lib


def _rand(shape, seed, sigma=1.0):
    return (sigma * np.random.default_rng(seed).standard_normal(shape)).astype(np.float32)


def _run(q, k, v, g, hq, hkv, d, t, packs=1, **kw):
    return oracle_lib.oracle_attention(q, k, v, g, q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs, **kw)


@pytest.mark.parametrize("shape", [(4, 4, 16, 48, 4), (8, 2, 8, 16, 1), (2, 1, 128, 96, 2), (2, 2, 64, 132, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_matches_float64_autograd(shape, causal):
    hq, hkv, d, t, packs = shape
    q, k, v, g = (_rand((h * d, packs * t), s) for h, s in ((hq, 1), (hkv, 2), (hkv, 3), (hq, 4)))
    res = _run(q, k, v, g, hq, hkv, d, t, packs, causal=causal)
    want = brute.attention_autograd(brute.ref_to_bhtd(q, hq, d, t, packs), brute.ref_to_bhtd(k, hkv, d, t, packs),
                                    brute.ref_to_bhtd(v, hkv, d, t, packs), brute.ref_to_bhtd(g, hq, d, t, packs),
                                    causal=causal)
    for key, heads in (("out", hq), ("dq", hq), ("dk", hkv), ("dv", hkv)):
        assert brute.max_abs(brute.ref_to_bhtd(res[key], heads, d, t, packs), want[key]) < 2e-5, key
    assert brute.max_abs(brute.ref_to_bht(res["lse"], hq, t, packs), want["lse"]) < 2e-6
    delta = oracle_lib.oracle_delta(res["out"], g, q_heads=hq, head_dim=d, seq_len=t, pack_count=packs)
    assert brute.max_abs(brute.ref_to_bht(delta, hq, t, packs), want["delta"]) < 2e-5


def test_closed_forms_zero_queries():
    # Q = 0: every allowed key gets equal weight, so O[t] = mean(V[0..t]), LSE[t] = ln(t+1),
    # dV[j] = sum_{t>=j} dO[t]/(t+1), and dQ = scale * sum_j dS K with dS from uniform P.
    hq = hkv = 2
    d, t = 8, 40
    q = np.zeros((hq * d, t), dtype=np.float32)
    k, v, g = _rand((hkv * d, t), 5), _rand((hkv * d, t), 6), _rand((hq * d, t), 7)
    res = _run(q, k, v, g, hq, hkv, d, t)
    counts = np.arange(1, t + 1, dtype=np.float64)
    assert np.allclose(res["out"], np.cumsum(v.astype(np.float64), axis=1) / counts, atol=1e-6)
    assert np.allclose(res["lse"], np.log(counts)[None, :].repeat(hq, 0), atol=1e-6)
    want_dv = np.cumsum((g.astype(np.float64) / counts)[:, ::-1], axis=1)[:, ::-1]
    assert np.allclose(res["dv"], want_dv, atol=1e-5)
    assert np.allclose(res["dk"], 0.0, atol=1e-7)  # dK = sum_q Q dS^T with Q = 0


def test_closed_forms_constant_value_and_first_query():
    hq, hkv, d, t = 2, 1, 16, 33
    q, k, g = _rand((hq * d, t), 8), _rand((hkv * d, t), 9), _rand((hq * d, t), 10)
    v = np.tile(_rand((hkv * d, 1), 11), (1, t))
    res = _run(q, k, v, g, hq, hkv, d, t)
    # rows of P sum to one: constant V passes through, and then dP is constant per query so dS = 0
    assert np.allclose(res["out"], np.tile(v[:, :1], (hq, t)), atol=1e-6)
    assert np.allclose(res["dq"], 0.0, atol=1e-5) and np.allclose(res["dk"], 0.0, atol=1e-5)
    # query 0 only sees key 0
    v2 = _rand((hkv * d, t), 12)
    res2 = _run(q, k, v2, g, hq, hkv, d, t)
    scale = 1.0 / np.sqrt(d)
    for h in range(hq):
        assert np.allclose(res2["out"][h * d:(h + 1) * d, 0], v2[:, 0], atol=1e-6)
        want = scale * float(q[h * d:(h + 1) * d, 0].astype(np.float64) @ k[:, 0].astype(np.float64))
        assert abs(res2["lse"][h, 0] - want) < 1e-5


def test_lse_shift_and_key_constant_invariance():
    # adding the same vector to every key shifts all of a query's scores by q.c: P unchanged, LSE shifts
    hq = hkv = 1
    d, t = 8, 24
    q, k, v, g = _rand((d, t), 13), _rand((d, t), 14), _rand((d, t), 15), _rand((d, t), 16)
    c = _rand((d, 1), 17)
    a = _run(q, k, v, g, hq, hkv, d, t)
    b = _run(q, k + c, v, g, hq, hkv, d, t)
    scale = 1.0 / np.sqrt(d)
    shift = scale * (q.astype(np.float64) * c.astype(np.float64)).sum(0)
    assert np.allclose(b["lse"][0] - a["lse"][0], shift, atol=2e-5)
    assert np.allclose(a["out"], b["out"], atol=2e-5)
    assert np.allclose(a["dv"], b["dv"], atol=2e-5)
    # each query's dS sums to zero over keys  =>  sum_j dK[:, j] = scale * sum_q Q[:, q] * sum_j dS = 0
    assert np.allclose(a["dk"].astype(np.float64).sum(1), 0.0, atol=2e-5)


def test_central_finite_differences():
    # the reference's own recipe (Layers/CausalSelfAttention.cpp:474-494): eps = 1e-3 probes of a scalar loss;
    # here in float32 oracle calls with loss = sum(out * g)
    hq, hkv, d, t = 2, 1, 4, 10
    rng = np.random.default_rng(18)
    q, k, v, g = (rng.standard_normal((h * d, t)).astype(np.float32) for h in (hq, hkv, hkv, hq))
    base = _run(q, k, v, g, hq, hkv, d, t)
    eps = 1e-2

    def loss(qq, kk, vv):
        return float((_run(qq, kk, vv, None, hq, hkv, d, t)["out"].astype(np.float64) * g).sum())

    for name, arr, grad in (("dq", q, base["dq"]), ("dk", k, base["dk"]), ("dv", v, base["dv"])):
        for _ in range(6):
            i, j = rng.integers(arr.shape[0]), rng.integers(arr.shape[1])
            hi, lo = arr.copy(), arr.copy()
            hi[i, j] += eps
            lo[i, j] -= eps
            args_hi = [hi if x is arr else x for x in (q, k, v)]
            args_lo = [lo if x is arr else x for x in (q, k, v)]
            numeric = (loss(*args_hi) - loss(*args_lo)) / (2 * eps)
            assert abs(numeric - grad[i, j]) < 5e-3 * max(1.0, abs(numeric)), (name, i, j, numeric, grad[i, j])


def test_gqa_equals_mha_on_repeated_kv_with_group_summed_grads():
    # relation (2) of the reference's GQA host smoke, thresholds 1e-5 forward / 1e-4 backward
    hq, hkv, d, t = 8, 2, 8, 16
    group = hq // hkv
    q, k, v, g = _rand((hq * d, t), 19), _rand((hkv * d, t), 20), _rand((hkv * d, t), 21), _rand((hq * d, t), 22)
    gqa = _run(q, k, v, g, hq, hkv, d, t)
    kx = np.repeat(k.reshape(hkv, d, t), group, axis=0).reshape(hq * d, t)
    vx = np.repeat(v.reshape(hkv, d, t), group, axis=0).reshape(hq * d, t)
    mha = _run(q, kx, vx, g, hq, hq, d, t)
    assert brute.max_abs(gqa["out"], mha["out"]) <= 1e-5
    assert brute.max_abs(gqa["dq"], mha["dq"]) <= 1e-4
    for key in ("dk", "dv"):
        summed = mha[key].reshape(hkv, group, d, t).sum(axis=1).reshape(hkv * d, t)
        assert brute.max_abs(gqa[key], summed) <= 1e-4
    # relation (1): kv_heads == q_heads is plain MHA, bit for bit
    again = _run(q, kx, vx, g, hq, hq, d, t)
    assert all(np.array_equal(mha[key], again[key]) for key in mha)


def test_packs_equal_independent_sequences():
    hq, hkv, d, t, packs = 2, 2, 16, 20, 3
    q, k, v, g = (_rand((h * d, packs * t), s) for h, s in ((hq, 23), (hkv, 24), (hkv, 25), (hq, 26)))
    full = _run(q, k, v, g, hq, hkv, d, t, packs)
    for p in range(packs):
        sl = slice(p * t, (p + 1) * t)
        one = _run(*(np.ascontiguousarray(x[:, sl]) for x in (q, k, v, g)), hq, hkv, d, t)
        for key in full:
            assert np.array_equal(full[key][:, sl], one[key]), (p, key)
