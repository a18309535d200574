"""Pins the oracle's attention layer (projections, RoPE, causal attention, output projection and its backward).

1. bit-exact against known answers from the reference's compiled CausalSelfAttention (tests/golden/layer_kat.npz);
2. live against oracle/_ref where built;
3. against float64 autograd of the same layer written with torch primitives (shares no code with the oracle).
"""
import os

import numpy as np
import pytest
import torch

import oracle_lib

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layer_kat.npz")
TAGS = ["e64_h4_T48", "e48_gqa6q2kv_d8_T33", "e128_h2_d64_T70"]
OUTPUTS = ("y", "d_x", "d_wq", "d_wk", "d_wv", "d_wo")


@pytest.fixture(scope="module")
def kat():
    return np.load(GOLDEN)


@pytest.mark.parametrize("tag", TAGS)
def test_layer_matches_reference_known_answers(kat, tag):
    e, hq, hkv, d, t, positions = (int(v) for v in kat[f"{tag}_geometry"])
    args = [kat[f"{tag}_{n}"] for n in ("x", "wq", "wk", "wv", "wo", "d_y")]
    got = oracle_lib.layer(*args, q_heads=hq, kv_heads=hkv, head_dim=d, rope_base=float(kat[f"{tag}_base"]),
                           rope_positions=positions)
    for name in OUTPUTS:
        assert np.array_equal(got[name], kat[f"{tag}_{name}"]), name
    forward_only = oracle_lib.layer(*args[:5], q_heads=hq, kv_heads=hkv, head_dim=d, rope_base=float(kat[f"{tag}_base"]),
                                    rope_positions=positions)
    assert np.array_equal(forward_only["y"], kat[f"{tag}_y"])


def _random_layer(rng, e, hq, hkv, d, t):
    bound = 1.0 / np.sqrt(e)
    x = rng.standard_normal((e, t)).astype(np.float32)
    ws = [rng.uniform(-bound, bound, shape).astype(np.float32) for shape in ((hq * d, e), (hkv * d, e), (hkv * d, e), (e, hq * d))]
    return x, ws, rng.standard_normal((e, t)).astype(np.float32)


def test_live_against_compiled_reference():
    if oracle_lib.reference() is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    rng = np.random.default_rng(123)
    for e, hq, hkv, d, t in [(32, 2, 2, 16, 20), (40, 4, 1, 8, 37), (96, 3, 3, 32, 65)]:
        x, ws, d_y = _random_layer(rng, e, hq, hkv, d, t)
        got = oracle_lib.layer(x, *ws, d_y, q_heads=hq, kv_heads=hkv, head_dim=d)
        want = oracle_lib.layer(x, *ws, d_y, q_heads=hq, kv_heads=hkv, head_dim=d, lib="ref")
        for name in OUTPUTS:
            assert np.array_equal(got[name], want[name]), name


def _torch_layer(x, wq, wk, wv, wo, hq, hkv, d, base):
    """float64 layer from torch primitives: x [E, T] -> y [E, T]."""
    t = x.shape[1]
    pair = torch.arange(d // 2, dtype=torch.float64)
    ang = torch.arange(t, dtype=torch.float64)[:, None] * base ** (-2.0 * pair / d)[None, :]  # [T, d/2]
    cos, sin = torch.cos(ang).T, torch.sin(ang).T  # [d/2, T]

    def rope(m, heads):
        m = m.reshape(heads, d // 2, 2, t)
        even, odd = m[:, :, 0], m[:, :, 1]
        return torch.stack((even * cos - odd * sin, even * sin + odd * cos), dim=2).reshape(heads * d, t)

    q = rope(wq @ x, hq).reshape(hq, d, t)
    k = rope(wk @ x, hkv).reshape(hkv, d, t).repeat_interleave(hq // hkv, dim=0)
    v = (wv @ x).reshape(hkv, d, t).repeat_interleave(hq // hkv, dim=0)
    s = torch.einsum("hdq,hdk->hqk", q, k) / np.sqrt(d)
    s = s.masked_fill(~torch.ones(t, t, dtype=torch.bool).tril(), float("-inf"))
    a = torch.einsum("hqk,hdk->hdq", torch.softmax(s, dim=-1), v).reshape(hq * d, t)
    return wo @ a


@pytest.mark.parametrize("shape", [(24, 2, 2, 8, 13), (32, 4, 2, 8, 21)])
def test_layer_against_float64_autograd(shape):
    e, hq, hkv, d, t = shape
    rng = np.random.default_rng(sum(shape))
    x, ws, d_y = _random_layer(rng, e, hq, hkv, d, t)
    got = oracle_lib.layer(x, *ws, d_y, q_heads=hq, kv_heads=hkv, head_dim=d)
    tx, twq, twk, twv, two = (torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (x, *ws))
    y = _torch_layer(tx, twq, twk, twv, two, hq, hkv, d, 10000.0)
    (y * torch.tensor(d_y, dtype=torch.float64)).sum().backward()
    want = {"y": y.detach().numpy(), "d_x": tx.grad.numpy(), "d_wq": twq.grad.numpy(), "d_wk": twk.grad.numpy(),
            "d_wv": twv.grad.numpy(), "d_wo": two.grad.numpy()}
    for name in OUTPUTS:
        err = np.max(np.abs(got[name] - want[name]))
        assert err <= 2e-5 * max(1.0, np.max(np.abs(want[name]))), f"{name}: {err}"


def test_invalid_geometry_is_rejected():
    rng = np.random.default_rng(1)
    x, ws, _ = _random_layer(rng, 16, 2, 2, 8, 5)
    with pytest.raises(ValueError):
        oracle_lib.layer(x, *ws, q_heads=2, kv_heads=2, head_dim=8, rope_positions=4)   # sequence longer than the table
    with pytest.raises(ValueError):
        oracle_lib.layer(x, *ws, q_heads=3, kv_heads=2, head_dim=8)                     # heads not divisible
