"""Helpers for the GPU parity tests: device tensors in both layouts, oracle runs on dtype-rounded inputs."""
import numpy as np
import torch

import brute
import oracle_lib

TORCH_DTYPE = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}


def make_inputs(hq, hkv, d, t, packs, seed, dtype="fp32", sigma_qk=1.0, sigma_v=1.0, col0=0, pad=0):
    """Column-layout fp32 numpy inputs whose values are exactly representable in `dtype`."""
    rng = np.random.default_rng(seed)
    stride = col0 + packs * t + pad

    def draw(heads, sigma):
        x = (sigma * rng.standard_normal((heads * d, stride))).astype(np.float32)
        return torch.from_numpy(x).to(TORCH_DTYPE[dtype]).to(torch.float32).numpy()

    return draw(hq, sigma_qk), draw(hkv, sigma_qk), draw(hkv, sigma_v), draw(hq, 1.0)


def columns_to_device_bhtd(x, heads, d, t, packs, col0, dtype):
    return torch.from_numpy(brute.ref_to_bhtd(x, heads, d, t, packs, col0)).to(TORCH_DTYPE[dtype]).cuda().contiguous()


def bhtd_to_columns(y, like, col0):
    """device [B,H,T,d] -> numpy column layout with NaN outside the window (shape of `like`)."""
    return brute.bhtd_to_ref(y.detach().float().cpu().numpy(), stride=like.shape[1], col0=col0)


def bht_to_columns(y, heads, stride, col0):
    return brute.bht_to_ref(y.detach().float().cpu().numpy(), stride=stride, col0=col0)


def oracle(q, k, v, g, hq, hkv, d, t, packs, col0=0, causal=True, scale=None, window=0, global_tokens=0):
    return oracle_lib.oracle_attention(q, k, v, g, q_heads=hq, kv_heads=hkv, head_dim=d, seq_len=t, pack_count=packs,
                                       col_start=col0, causal=causal, scale=scale, pack_parallel=True, window=window,
                                       global_tokens=global_tokens)


def assert_close_fp32(got, want, name, tol=1e-4):
    """north-star fp32 bar: max-abs / rel 1e-4  (|got - want| <= tol * max(1, |want|))"""
    mask = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), ~mask), f"{name}: window mismatch"
    err = np.abs(got[mask].astype(np.float64) - want[mask].astype(np.float64))
    bound = tol * np.maximum(1.0, np.abs(want[mask].astype(np.float64)))
    worst = float(np.max(err / bound)) if err.size else 0.0
    assert worst <= 1.0, f"{name}: error {float(err.max()):.3e} exceeds {tol} (ratio {worst:.2f})"


def assert_close_lowp(got, want, name, tol=2e-2, floor=1e-5):
    """north-star bf16 / fp16 bar: 2e-2 relative, taken norm-wise: max|got - want| <= tol * max|want| (+ floor).

    The absolute floor only matters where the exact answer is identically zero (a single token has dQ = dK = 0)."""
    mask = ~np.isnan(want)
    assert np.isfinite(got[mask]).all(), f"{name}: non-finite values"
    err = brute.max_abs(got[mask], want[mask])
    scale = float(np.max(np.abs(want[mask])))
    assert err <= tol * scale + floor, f"{name}: error {err:.3e} exceeds {tol} * {scale:.3e}"
    return err / max(scale, 1e-30)
