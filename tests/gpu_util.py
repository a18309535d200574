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


# Worst measured margins of the 16-bit bar, filled by assert_close_lowp and printed by conftest.py at the end of a
# run: tensor kind -> [worst row error / max|row| among rows that are not small, largest row_floor coefficient a row
# needed on top of tol * max|row|, name of the case that set it].
MARGINS = {}
CASE_MARGINS = []  # (name, worst row error / max|row|, row_floor coefficient needed) of every case, in order

# D = rowsum(dO o O) enters dQ and dK only (dS = P o (dP - D)); O and dV never see it.  1.25 x the largest
# coefficient any row of any committed case needs (conftest.py prints it per run).
DELTA_ROW_FLOOR = 1.0e-2


def tensor_kind(name):
    """'out', 'dq', 'dk' or 'dv': the last word of a case's name."""
    kind = name.split()[-1]
    assert kind in ("out", "dq", "dk", "dv"), f"{name}: cannot tell which tensor this is"
    return kind


def assert_close_lowp(got, want, name, head_dim, tol=2e-2, row_floor=None, floor=1e-5, neighbourhood=32):
    """north-star bf16 / fp16 bar: 2e-2 relative, taken per token.

    `got` / `want` are column-layout matrices [(head * head_dim + dim), column] (NaN in `want` = outside the window);
    the last word of `name` says which tensor it is.  Every (head, token) row of head_dim values is judged on its own:
        O, dV:   max|got_row - want_row| <= tol * max|want_row| + floor
        dQ, dK:  max|got_row - want_row| <= tol * max|want_row| + row_floor * max|want rows of any head within
                                                                               +-neighbourhood tokens| + floor
    so a mistake confined to late tokens, whose rows are far smaller than the tensor's largest, cannot hide behind
    the first few tokens.  The row_floor term exists for dQ and dK only (DELTA_ROW_FLOOR unless given): a 16-bit
    backward forms D = rowsum(dO o O) from the 16-bit O it is given, which leaves an error in dS = P o (dP - D)
    proportional to |O| |dO|, i.e. to what the neighbouring rows are made of, not to the row itself; single rows that
    are far smaller than their neighbours by cancellation (the second query's dQ is dS (K1 - K0) with
    dS = P0 P1 (dP1 - dP0)) cannot meet a purely relative bar.  O and dV do not pass through D and get no such term.
    `floor` is absolute and only matters where the exact answer is identically zero (a single token's dQ and dK).
    The norm-wise bar of the whole tensor (max|err| <= tol * max|want|) is kept as a second check.
    Returns the worst row's error relative to max|want_row| among rows that are not small (diagnostic); the same
    figure and the row_floor coefficient the worst row needed go to MARGINS."""
    from scipy.ndimage import maximum_filter1d
    kind = tensor_kind(name)
    if row_floor is None:
        row_floor = DELTA_ROW_FLOOR if kind in ("dq", "dk") else 0.0
    assert got.shape == want.shape and want.ndim == 2 and want.shape[0] % head_dim == 0, f"{name}: shape"
    mask = ~np.isnan(want)
    assert np.isfinite(got[mask]).all(), f"{name}: non-finite values"
    heads = want.shape[0] // head_dim
    w = np.where(mask, want, 0.0).astype(np.float64).reshape(heads, head_dim, -1)
    e = np.where(mask, got.astype(np.float64) - np.where(mask, want, 0.0), 0.0).reshape(heads, head_dim, -1)
    row_err = np.abs(e).max(axis=1)   # [heads, columns]
    row_ref = np.abs(w).max(axis=1)
    scale = float(row_ref.max()) if row_ref.size else 0.0
    local = row_ref
    if row_ref.size:  # heads are statistically alike: the neighbourhood's magnitude is taken over all of them
        local = np.broadcast_to(maximum_filter1d(row_ref.max(axis=0), size=2 * neighbourhood + 1, mode="constant"), row_ref.shape)
    big = row_ref > 0.25 * local
    worst_rel = float((row_err[big] / row_ref[big]).max(initial=0.0)) if big.any() else 0.0
    needed = float(((row_err - tol * row_ref - floor) / np.maximum(local, 1e-30)).max(initial=0.0)) if row_ref.size else 0.0
    CASE_MARGINS.append((name, worst_rel, max(needed, 0.0)))
    seen = MARGINS.setdefault(kind, [0.0, 0.0, "", ""])
    if worst_rel > seen[0]:
        seen[0], seen[2] = worst_rel, name
    if needed > seen[1]:
        seen[1], seen[3] = needed, name
    bar = tol * row_ref + row_floor * local + floor
    ratio = row_err / bar
    worst = np.unravel_index(int(np.argmax(ratio)), ratio.shape) if ratio.size else (0, 0)
    assert ratio.size == 0 or ratio[worst] <= 1.0, (
        f"{name}: head {worst[0]} column {worst[1]}: error {row_err[worst]:.3e} exceeds {tol} * {row_ref[worst]:.3e} "
        f"+ {row_floor} * {local[worst]:.3e} (tensor max {scale:.3e})")
    assert float(row_err.max(initial=0.0)) <= tol * scale + floor, f"{name}: error {row_err.max():.3e} exceeds {tol} * {scale:.3e}"
    return worst_rel
