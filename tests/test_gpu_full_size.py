"""The baseline configurations at their full sizes (C ABI, [B,H,T,d]).

The CPU oracle cannot run a whole configuration in seconds, so each case checks
  * three (batch, K/V head) slices, each with all query heads of its group, against the oracle at the full sequence
    length (heads are independent, so a slice sees exactly the long-sequence tiling of the full launch): the first
    head of the first batch entry and the last head of the last one are the two ends of the persistent grids' walk
    over the tiles, the third sits in the middle; every token's row is judged on its own (gpu_util.assert_close_lowp);
  * the same for the column-layout call Sentinel makes (fp32 matrices, 16-bit arithmetic) at the two largest shapes;
  * properties that hold at any size and that an indexing or synchronisation mistake breaks:
    - scaling dO by 2 scales dQ, dK, dV by exactly 2 (bitwise in bf16: powers of two commute with every rounding);
    - causality: changing Q, K, V, dO behind position t leaves O, LSE and dQ before t bit-identical;
    - constant V gives O = that constant; row sums of P are one;
    - permuting the batch entries permutes every output bit-identically.
"""
import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu

# name: (B, Hq, Hkv, T, d, dtype, sigma_qk)  -- the GPU configurations of the baseline and its target shape
CONFIGS = {
    "c2_gpt2_small": (8, 12, 12, 1024, 64, "bf16", 0.70710678),
    "c3_llama7b": (4, 32, 32, 2048, 128, "bf16", 1.0),
    "c4_gqa": (4, 32, 8, 4096, 128, "bf16", 1.0),
    "c5_long_fp16": (1, 16, 16, 16384, 64, "fp16", 3.0),
    "target_shape": (4, 32, 32, 4096, 128, "bf16", 1.0),
    # shapes whose persistent grids take the length-major deal of tiles (mfma_tile.h: plan_persistent_grid) in ways the
    # baseline configurations do not: key tiles dealt over three rounds; query tiles over 2.67 rounds (as C5, in bf16
    # with more heads per XCD); head_dim 128 query tiles dealt in one round
    "dealt_keys_d64_t2048": (8, 12, 12, 2048, 64, "bf16", 1.0),
    "dealt_queries_d64_t4096": (4, 16, 16, 4096, 64, "bf16", 1.0),
    "dealt_queries_d128_t2048": (1, 32, 32, 2048, 128, "bf16", 1.0),
}


def _inputs(name):
    b, hq, hkv, t, d, dtype, sigma = CONFIGS[name]
    tdt = gpu_util.TORCH_DTYPE[dtype]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234 + len(name))
    q = (sigma * torch.randn(b, hq, t, d, device="cuda", generator=gen)).to(tdt)
    k = (sigma * torch.randn(b, hkv, t, d, device="cuda", generator=gen)).to(tdt)
    v = torch.randn(b, hkv, t, d, device="cuda", generator=gen).to(tdt)
    g = torch.randn(b, hq, t, d, device="cuda", generator=gen).to(tdt)
    return q, k, v, g


def _run(q, k, v, g):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    out, lse = flash_attention_forward(q, k, v)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (q, k, v))
    flash_attention_backward(q, k, v, out, lse, g, dq=dq, dk=dk, dv=dv)
    torch.cuda.synchronize()
    return out, lse, dq, dk, dv


def _columns(x):
    """[H, T, d] device slice -> fp32 numpy [(h*d + c), T]"""
    h, t, d = x.shape
    return np.ascontiguousarray(x.float().cpu().numpy().transpose(0, 2, 1).reshape(h * d, t))


def _slice_of(where, b, hkv):
    """(batch, K/V head) of the slice: the two ends of the persistent grids' walk over the tiles and the middle."""
    return {"first": (0, 0), "middle": (b - 1, hkv // 2), "last": (b - 1, hkv - 1)}[where]


def _check_slice(name, where, out, lse, dq, dk, dv, q, k, v, g):
    b, hq, hkv, t, d, dtype, _ = CONFIGS[name]
    group = hq // hkv
    bi, kvh = _slice_of(where, b, hkv)
    hs = slice(kvh * group, (kvh + 1) * group)
    want = gpu_util.oracle(_columns(q[bi, hs]), _columns(k[bi, kvh:kvh + 1]), _columns(v[bi, kvh:kvh + 1]),
                           _columns(g[bi, hs]), group, 1, d, t, 1)
    tag = f"full-size {name} {where}"
    gpu_util.assert_close_lowp(_columns(out[bi, hs]), want["out"], tag + " out", d)
    got_lse = lse[bi, hs].float().cpu().numpy()
    assert np.max(np.abs(got_lse - want["lse"][:, :t])) <= 2e-3, "lse"
    gpu_util.assert_close_lowp(_columns(dq[bi, hs]), want["dq"], tag + " dq", d)
    gpu_util.assert_close_lowp(_columns(dk[bi, kvh:kvh + 1]), want["dk"], tag + " dk", d)
    gpu_util.assert_close_lowp(_columns(dv[bi, kvh:kvh + 1]), want["dv"], tag + " dv", d)


@pytest.mark.parametrize("where", ["first", "middle", "last"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_slice_matches_oracle_at_full_length(name, where):
    print(f"case {name} {where} slice vs oracle", flush=True)
    q, k, v, g = _inputs(name)
    out, lse, dq, dk, dv = _run(q, k, v, g)
    _check_slice(name, where, out, lse, dq, dk, dv, q, k, v, g)
    for x in (out, lse, dq, dk, dv):
        assert torch.isfinite(x.float()).all(), "non-finite value outside the checked slice"


@pytest.mark.parametrize("where", ["first", "last"])
@pytest.mark.parametrize("name", ["c4_gqa", "target_shape"])
def test_drop_in_column_layout_at_full_length(name, where):
    """The call Sentinel makes: fp32 [(head*d + dim), B*T] matrices through HipFlashAttention.forward_multi_head /
    backward_multi_head with 16-bit arithmetic (layout conversion passes around the MFMA kernels), at the full size;
    one (batch, K/V head) slice against the oracle."""
    from sentinel_amd import HipFlashAttention
    b, hq, hkv, t, d, dtype, _ = CONFIGS[name]
    print(f"case {name} {where} column layout vs oracle", flush=True)
    q, k, v, g = _inputs(name)  # 16-bit values, so the conversion pass rounds nothing on the way in

    def columns(x):  # [B, H, T, d] -> fp32 [(h*d + c), b*T + t]
        return x.float().permute(1, 3, 0, 2).reshape(x.shape[1] * d, b * t).contiguous()
    qc, kc, vc, gc = (columns(x) for x in (q, k, v, g))
    scale = 1.0 / np.sqrt(np.float32(d))
    args = (hq, d, scale, True, 0, t, b)
    kw = dict(kv_head_count=hkv, compute=dtype)
    out, lse = HipFlashAttention.forward_multi_head(qc, kc, vc, None, None, *args, **kw)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (qc, kc, vc))
    dq, dk, dv, _ = HipFlashAttention.backward_multi_head(qc, kc, vc, out, lse, gc, dq, dk, dv, None, *args, **kw)
    torch.cuda.synchronize()

    def bhtd(x, heads):  # back to [B, H, T, d]
        return x.reshape(heads, d, b, t).permute(2, 0, 3, 1)
    _check_slice(name, where, bhtd(out, hq), lse.reshape(hq, b, t).permute(1, 0, 2), bhtd(dq, hq), bhtd(dk, hkv),
                 bhtd(dv, hkv), q, k, v, g)
    for x in (out, lse, dq, dk, dv):
        assert torch.isfinite(x).all(), "non-finite value outside the checked slice"


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_size_independent_properties(name):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    b, hq, hkv, t, d, dtype, _ = CONFIGS[name]
    print(f"case {name} properties", flush=True)
    q, k, v, g = _inputs(name)
    out, lse, dq, dk, dv = _run(q, k, v, g)

    # gradients are linear in dO; a factor of two is exact in every rounding step
    dq2, dk2, dv2 = (torch.empty_like(x) for x in (q, k, v))
    flash_attention_backward(q, k, v, out, lse, g * 2, dq=dq2, dk=dk2, dv=dv2)
    torch.cuda.synchronize()
    for name2, a, a2 in (("dq", dq, dq2), ("dk", dk, dk2), ("dv", dv, dv2)):
        if dtype == "bf16":
            assert torch.equal(a * 2, a2), f"{name2} is not linear in dO"
        else:  # fp16 rounds tiny dS values on its subnormal grid, where doubling is no longer exact
            err = torch.max(torch.abs(a.float() * 2 - a2.float())).item()
            assert err <= 1e-3 * torch.max(torch.abs(a2.float())).item(), f"{name2} is not linear in dO"

    # causality: a change behind position cut cannot reach anything before it
    # (the cut sits on a wavefront boundary: the forward raises its running maximum per 32-query wavefront)
    cut = (t * 3 // 4) // 128 * 128
    qc, kc, vc, gc = (x.clone() for x in (q, k, v, g))
    for x in (qc, kc, vc, gc):
        x[:, :, cut:, :] = x[:, :, cut:, :].flip(2) * 0.5
    outc, lsec, dqc, _, _ = _run(qc, kc, vc, gc)
    assert torch.equal(out[:, :, :cut], outc[:, :, :cut]), "O before the cut changed"
    assert torch.equal(lse[:, :, :cut], lsec[:, :, :cut]), "LSE before the cut changed"
    # dQ of a query only sees keys before it (dK, dV of early keys do see the late queries and may change)
    assert torch.equal(dq[:, :, :cut], dqc[:, :, :cut]), "dQ before the cut changed"

    # softmax rows sum to one: a constant V comes back unchanged (P is rounded to 16 bit, hence the tolerance)
    vone = torch.full_like(v, 0.75)
    oone, _ = flash_attention_forward(q, k, vone)
    assert torch.max(torch.abs(oone.float() - 0.75)).item() <= 0.75 * 8e-3, "row sums of P differ from one"

    # batch entries are independent: a permutation of the batch permutes the results bit for bit
    if b > 1:
        perm = torch.roll(torch.arange(b, device="cuda"), 1)
        outp, lsep, dqp, dkp, dvp = _run(q[perm].contiguous(), k[perm].contiguous(), v[perm].contiguous(),
                                         g[perm].contiguous())
        for name2, a, ap in (("out", out, outp), ("lse", lse, lsep), ("dq", dq, dqp), ("dk", dk, dkp), ("dv", dv, dvp)):
            assert torch.equal(a[perm], ap), f"{name2} depends on the position in the batch"
