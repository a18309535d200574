"""Sliding-window + global-token mask on the device (C ABI through the Python mirror) against the pinned oracle.

fp32 arithmetic on Sentinel's column layout at the 1e-4 bar (including the reference's own known answers), bf16 / fp16
MFMA kernels on [B,H,T,d] at the 2e-2 bar with windows and global ranges that start, end and straddle the 64- and
128-wide tiles, the fused-rotation column path, and properties that hold at any size: a window that covers the
sequence is the plain causal result bit for bit, and one key reaches exactly the queries the mask rule names.
"""
import os

import numpy as np
import pytest
import torch

import gpu_util
import oracle_lib

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sparse_kat.npz")
KAT_TAGS = ["smoke_h2_d16_T16_W4_G2", "gqa_4q2kv_d8_T50_W7_G0", "h1_d64_T140_W33_G5", "h2_d32_T70_W0_G9",
            "h1_d128_T130_W1_G0", "h1_d16_T40_W100_G3"]


def _columns_fp32(q, k, v, g, hq, hkv, d, t, packs, window, global_tokens, col0=0, compute="fp32", rope=None):
    from sentinel_amd import HipFlashAttention
    qd, kd, vd, gd = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    sentinel = 777.0
    out = torch.full_like(qd, sentinel)
    lse = torch.full((hq, q.shape[1]), sentinel, device="cuda")
    scale = 1.0 / np.sqrt(np.float32(d))
    kw = dict(kv_head_count=hkv, compute=compute, window_size=window, global_token_count=global_tokens, rope=rope)
    out, lse = HipFlashAttention.forward_multi_head(qd, kd, vd, out, lse, hq, d, scale, True, col0, t, packs, **kw)
    dq, dk, dv = (torch.full_like(x, sentinel) for x in (qd, kd, vd))
    dq, dk, dv, _ = HipFlashAttention.backward_multi_head(qd, kd, vd, out, lse, gd, dq, dk, dv, None, hq, d, scale, True, col0,
                                                          t, packs, **kw)
    torch.cuda.synchronize()
    return {key: x.cpu().numpy() for key, x in dict(out=out, lse=lse, dq=dq, dk=dk, dv=dv).items()}, sentinel


@pytest.mark.parametrize("tag", KAT_TAGS)
def test_fp32_matches_reference_known_answers(tag):
    kat = np.load(GOLDEN)
    hq, hkv, d, t, packs, window, global_tokens = (int(x) for x in kat[f"{tag}_geometry"])
    print(f"case sparse kat {tag}", flush=True)
    got, _ = _columns_fp32(kat[f"{tag}_q"], kat[f"{tag}_k"], kat[f"{tag}_v"], kat[f"{tag}_d_out"], hq, hkv, d, t, packs, window,
                           global_tokens)
    for key in ("out", "lse", "dq", "dk", "dv"):
        gpu_util.assert_close_fp32(got[key], kat[f"{tag}_dense_{key}"], key)


# (q_heads, kv_heads, head_dim, seq_len, packs, col0, pad, window, global_tokens)
FP32_SHAPES = [
    (4, 4, 16, 48, 4, 0, 0, 8, 2),
    (8, 2, 8, 100, 2, 3, 5, 33, 0),
    (2, 1, 64, 200, 1, 0, 0, 64, 40),
    (2, 2, 128, 150, 1, 4, 0, 17, 70),
    (3, 3, 24, 130, 2, 0, 1, 1, 0),
    (1, 1, 32, 300, 1, 0, 0, 65, 129),
    (2, 2, 16, 90, 1, 0, 0, 0, 5),       # no window: plain causal
    (2, 2, 16, 90, 1, 0, 0, 500, 5),     # window past the sequence: plain causal
]


@pytest.mark.parametrize("shape", FP32_SHAPES)
def test_fp32_columns_match_oracle(shape):
    hq, hkv, d, t, packs, col0, pad, window, global_tokens = shape
    print(f"case sparse fp32 {shape}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape), col0=col0, pad=pad)
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, col0=col0, window=window, global_tokens=global_tokens)
    got, sentinel = _columns_fp32(q, k, v, g, hq, hkv, d, t, packs, window, global_tokens, col0=col0)
    for key in ("out", "lse", "dq", "dk", "dv"):
        outside = np.isnan(want[key])
        assert np.all(got[key][outside] == sentinel), f"{key}: wrote outside the pack window"
        gpu_util.assert_close_fp32(np.where(outside, np.nan, got[key]), want[key], key)


# (q_heads, kv_heads, head_dim, seq_len, packs, window, global_tokens): windows and global ranges that end on, before and
# after the 64-key / 128-query tile edges, windows shorter than a tile and longer than several
MFMA_SHAPES = [
    (2, 2, 64, 256, 1, 64, 0),
    (2, 2, 128, 256, 1, 64, 0),
    (2, 1, 128, 300, 2, 17, 3),
    (4, 2, 64, 513, 1, 100, 64),
    (2, 2, 128, 640, 1, 128, 70),
    (1, 1, 64, 700, 1, 333, 130),
    (2, 1, 128, 1024, 1, 200, 1),
    (1, 1, 128, 777, 1, 1, 0),
    (3, 3, 64, 450, 1, 65, 449),
    (2, 2, 128, 130, 3, 129, 0),
    (1, 1, 64, 1, 1, 5, 0),
]


def _bhtd(dtype, shape, seed_extra=0):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    hq, hkv, d, t, packs, window, global_tokens = shape
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape) + 11 + seed_extra, dtype=dtype)
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, window=window, global_tokens=global_tokens)
    qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, dtype)
                      for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
    kw = dict(window_size=window, global_token_count=global_tokens)
    out, lse = flash_attention_forward(qd, kd, vd, **kw)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (qd, kd, vd))
    flash_attention_backward(qd, kd, vd, out, lse, gd, dq=dq, dk=dk, dv=dv, **kw)
    torch.cuda.synchronize()
    gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(out, q, 0), want["out"], "out", d)
    got_lse = gpu_util.bht_to_columns(lse, hq, q.shape[1], 0)
    assert np.nanmax(np.abs(got_lse - want["lse"])) <= 2e-3, "lse"
    for name, got, like in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(got, like, 0), want[name], name, d)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("shape", MFMA_SHAPES)
def test_mfma_matches_oracle(dtype, shape):
    print(f"case sparse {dtype} {shape}", flush=True)
    _bhtd(dtype, shape)


@pytest.mark.parametrize("shape", [(8, 8, 128, 1024, 10, 100, 0), (8, 8, 128, 1024, 10, 256, 0), (16, 16, 64, 1024, 12, 70, 0)])
def test_short_windows_with_more_tiles_than_workgroups_run_at_once(shape):
    """Short windows without global tokens run the forward (and, at head_dim 128, the dK/dV) kernel on the persistent grid
    once a die has more tiles than workgroups in flight: 640 query / key tiles at head_dim 128 (80 per die against 64 / 32
    resident), 1536 query tiles at head_dim 64 (192 per die),
    so workgroups walk several tiles, the last round is partial, and every tile must still be computed exactly once."""
    print(f"case sparse persistent {shape}", flush=True)
    _bhtd("bf16", shape)


@pytest.mark.parametrize("d", [128, 96, 32])  # 96 and 32: zero-padded to the kernels' tilings by the conversion pass
def test_columns_with_mfma_arithmetic_and_fused_rotation(d):
    hq, hkv, t, packs, window, global_tokens = 4, 2, 200, 2, 48, 6
    print(f"case sparse columns bf16 + rope d{d}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=321, dtype="bf16", col0=4, pad=4)
    cos, sin = oracle_lib.rope_tables(d, t)

    def rotate(x, heads, inverse=False):
        y = x.copy()
        for p in range(packs):
            lo = 4 + p * t
            y[:, lo:lo + t] = oracle_lib.rope_rotate(x[:, lo:lo + t], heads, d, cos, sin, inverse=inverse)
        return y
    want = gpu_util.oracle(rotate(q, hq), rotate(k, hkv), v, g, hq, hkv, d, t, packs, col0=4, window=window,
                           global_tokens=global_tokens)
    want["dq"] = np.where(np.isnan(want["dq"]), np.nan, rotate(np.nan_to_num(want["dq"]), hq, inverse=True))
    want["dk"] = np.where(np.isnan(want["dk"]), np.nan, rotate(np.nan_to_num(want["dk"]), hkv, inverse=True))
    rope = (torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda())
    got, sentinel = _columns_fp32(q, k, v, g, hq, hkv, d, t, packs, window, global_tokens, col0=4, compute="bf16", rope=rope)
    for key in ("out", "dq", "dk", "dv"):
        outside = np.isnan(want[key])
        assert np.all(got[key][outside] == sentinel), f"{key}: wrote outside the pack window"
        gpu_util.assert_close_lowp(np.where(outside, np.nan, got[key]), want[key], key, d)


@pytest.mark.parametrize("dtype,d", [("bf16", 128), ("fp16", 64)])
def test_wide_window_is_the_causal_result_bit_for_bit(dtype, d):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    torch.manual_seed(3)
    tdt = gpu_util.TORCH_DTYPE[dtype]
    q, k, v, g = (torch.randn(2, h, 500, d, device="cuda").to(tdt) for h in (4, 2, 2, 4))
    out, lse = flash_attention_forward(q, k, v)
    grads = flash_attention_backward(q, k, v, out, lse, g)
    for window, global_tokens in [(500, 0), (0, 30), (9999, 7)]:
        out2, lse2 = flash_attention_forward(q, k, v, window_size=window, global_token_count=global_tokens)
        grads2 = flash_attention_backward(q, k, v, out2, lse2, g, window_size=window, global_token_count=global_tokens)
        torch.cuda.synchronize()
        assert torch.equal(out, out2) and torch.equal(lse, lse2)
        for a, b in zip(grads, grads2):
            assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,d,t,window,global_tokens", [("bf16", 128, 4096, 512, 64), ("fp16", 64, 8192, 1000, 0),
                                                            ("bf16", 64, 2048, 96, 200)])
def test_reach_of_one_key_at_long_sequences(dtype, d, t, window, global_tokens):
    """Changing K, V of one key changes O, LSE and dQ of exactly the queries that see it (bitwise elsewhere): an
    indexing mistake in the tile lists or mask edges shows at any size."""
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    print(f"case sparse reach {dtype} d{d} T{t} W{window} G{global_tokens}", flush=True)
    torch.manual_seed(17)
    tdt = gpu_util.TORCH_DTYPE[dtype]
    q, k, v, g = (torch.randn(1, h, t, d, device="cuda").to(tdt) for h in (2, 1, 1, 2))
    kw = dict(window_size=window, global_token_count=global_tokens)
    out, lse = flash_attention_forward(q, k, v, **kw)
    dq, dk, dv = flash_attention_backward(q, k, v, out, lse, g, **kw)
    keys = [0, max(global_tokens - 1, 0), global_tokens, t // 2 + 37, t - window - 1, t - 1]
    for key in keys:
        k2, v2 = k.clone(), v.clone()
        k2[:, :, key] = -k2[:, :, key]
        v2[:, :, key] = v2[:, :, key] * 0.5 + 1.0
        out2, lse2 = flash_attention_forward(q, k2, v2, **kw)
        dq2, _, _ = flash_attention_backward(q, k2, v2, out2, lse2, g, **kw)
        torch.cuda.synchronize()
        reach = torch.zeros(t, dtype=torch.bool, device="cuda")
        reach[key:(t if key < global_tokens else min(t, key + window))] = True
        changed = (out != out2).any(dim=3).any(dim=1).any(dim=0)
        assert not (changed & ~reach).any(), f"key {key}: O changed outside the reach"
        # inside the reach the change is a fraction of a percent of the row: a rare row may round to the same 16-bit values
        assert changed[reach].float().mean().item() > 0.97, f"key {key}: O did not change inside the reach"
        assert not ((lse != lse2).any(dim=1).any(dim=0) & ~reach).any(), f"key {key}: LSE changed outside the reach"
        assert not ((dq != dq2).any(dim=3).any(dim=1).any(dim=0) & ~reach).any(), f"key {key}: dQ changed outside the reach"
    # every row of P still sums to one
    vone = torch.full_like(v, 0.5)
    oone, _ = flash_attention_forward(q, k, vone, **kw)
    assert torch.max(torch.abs(oone.float() - 0.5)).item() <= 0.5 * 8e-3
    for x in (out, lse, dq, dk, dv):
        assert torch.isfinite(x.float()).all()


def test_sparse_argument_errors():
    from sentinel_amd import HipFlashAttention
    q = torch.zeros(2 * 16, 32, device="cuda")
    with pytest.raises(ValueError, match="causal must be set"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 2, 16, 0.25, False, 0, 32, 1, window_size=4)
    with pytest.raises(ValueError, match="globalTokenCount must be >= 0"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 2, 16, 0.25, True, 0, 32, 1, window_size=4,
                                             global_token_count=-1)
