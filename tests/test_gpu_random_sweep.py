"""Seeded random sweep of the MFMA forward + backward through the C ABI against the oracle: head dims, dtypes, grouped
heads, ragged lengths around the 64 / 128 tile edges, packs, the sparse mask and non-causal attention in combinations the
hand-picked cases of the other files do not list.  Bars as everywhere: 2e-2 relative for 16-bit results, LSE 2e-3."""
import numpy as np
import pytest
import torch

import gpu_util
from sentinel_amd import flash_attention_backward, flash_attention_forward

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 31, 63, 64, 65, 127, 128, 129, 191, 200, 255, 256, 257, 300, 383, 385, 511, 513, 640, 700]


def draw_case(rng):
    d = int(rng.choice([64, 128]))
    dtype = str(rng.choice(["bf16", "fp16"]))
    hkv = int(rng.choice([1, 2, 3]))
    hq = hkv * int(rng.choice([1, 2, 4]))
    t = int(rng.choice(LENGTHS))
    packs = int(rng.choice([1, 2, 5]))
    mode = int(rng.integers(0, 3))
    causal, window, global_tokens = True, 0, 0
    if mode == 1 and t > 4:
        window = int(rng.integers(1, t))
        global_tokens = int(rng.choice([0, 0, 1, 5, 64, 70, 130]))
    if mode == 2:
        causal = bool(rng.integers(0, 2))
    return d, dtype, hq, hkv, t, packs, causal, window, global_tokens, int(rng.integers(0, 1 << 30))


@pytest.mark.parametrize("sweep_seed", [11, 12, 13, 14])
def test_random_shapes_match_the_oracle(sweep_seed):
    rng = np.random.default_rng(sweep_seed)
    for _ in range(10):
        d, dtype, hq, hkv, t, packs, causal, window, global_tokens, seed = draw_case(rng)
        tag = f"d{d} {dtype} hq{hq} hkv{hkv} t{t} packs{packs} causal{causal} window{window} global{global_tokens} seed{seed}"
        print(tag, flush=True)
        q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=seed, dtype=dtype)
        want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, causal=causal, window=window, global_tokens=global_tokens)
        qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, dtype)
                          for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
        kw = dict(causal=causal)
        if window:
            kw.update(window_size=window, global_token_count=global_tokens)
        out, lse = flash_attention_forward(qd, kd, vd, **kw)
        dq, dk, dv = flash_attention_backward(qd, kd, vd, out, lse, gd, **kw)
        torch.cuda.synchronize()
        gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(out, q, 0), want["out"], tag + " out", d)
        gpu_util.assert_close_fp32(gpu_util.bht_to_columns(lse, hq, q.shape[1], 0), want["lse"], tag + " lse", tol=2e-3)
        for name, got, like in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
            gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(got, like, 0), want[name], tag + " " + name, d)
