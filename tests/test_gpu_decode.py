"""Single-query attention against the K/V cache (the generation step) through the C ABI.

The reference checks this path by comparing prefill + decode of the last token with the last column of the full
forward (CudaCausalSelfAttention::runKvCacheSmokeDemo); the same relation is the oracle here: for short caches the
attention oracle's forward is run on the whole sequence and its last column must come back, for long caches
(where the O(T^2) oracle is too slow) a float64 evaluation of softmax(scale q K) V is the check.
"""
import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu


def _case(hq, hkv, d, length, capacity, seed):
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((hkv * d, capacity)).astype(np.float32)
    v = rng.standard_normal((hkv * d, capacity)).astype(np.float32)
    k[:, length:] = np.nan  # positions past the used prefix must never be read into the result
    v[:, length:] = np.nan
    q = rng.standard_normal((hq * d, 1)).astype(np.float32)
    return q, k, v


def _float64(q, k, v, hq, hkv, d, length):
    group = hq // hkv
    out = np.empty((hq * d, 1))
    for h in range(hq):
        kh = k[(h // group) * d:(h // group + 1) * d, :length].astype(np.float64)
        vh = v[(h // group) * d:(h // group + 1) * d, :length].astype(np.float64)
        s = (q[h * d:(h + 1) * d, 0].astype(np.float64) @ kh) / np.sqrt(d)
        p = np.exp(s - s.max())
        out[h * d:(h + 1) * d, 0] = vh @ (p / p.sum())
    return out


@pytest.mark.parametrize("shape", [(4, 4, 16, 48, 64), (8, 2, 8, 16, 16), (2, 2, 64, 1, 8), (4, 1, 128, 300, 512),
                                   (12, 12, 64, 1025, 2048), (8, 8, 32, 77, 77)])
def test_decode_matches_last_column_of_the_full_forward(shape):
    from sentinel_amd import decode_attention
    hq, hkv, d, length, capacity = shape
    print(f"case decode {shape}", flush=True)
    q, k, v = _case(hq, hkv, d, length, capacity, seed=sum(shape))
    # full-sequence oracle: any queries before the last, the last column is the decode result
    rng = np.random.default_rng(1)
    qfull = rng.standard_normal((hq * d, length)).astype(np.float32)
    qfull[:, -1] = q[:, 0]
    want = gpu_util.oracle(qfull, np.ascontiguousarray(k[:, :length]), np.ascontiguousarray(v[:, :length]), None, hq, hkv, d,
                           length, 1)["out"][:, -1:]
    got = decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), length, hq, d,
                           kv_head_count=hkv)
    torch.cuda.synchronize()
    gpu_util.assert_close_fp32(got.cpu().numpy(), want, "decode out")


@pytest.mark.parametrize("shape", [(4, 4, 16, 48, 64, 8, 2), (8, 2, 8, 300, 512, 100, 0), (2, 2, 64, 1025, 2048, 64, 130),
                                   (4, 1, 128, 700, 700, 1, 0), (2, 2, 32, 9000, 9004, 300, 260), (2, 1, 64, 10000, 10240, 5000, 7000),
                                   (2, 2, 16, 50, 64, 50, 3), (2, 2, 16, 50, 64, 0, 9)])
def test_decode_with_sparse_mask_matches_last_column_of_the_full_forward(shape):
    from sentinel_amd import decode_attention
    hq, hkv, d, length, capacity, window, global_tokens = shape
    print(f"case decode sparse {shape}", flush=True)
    q, k, v = _case(hq, hkv, d, length, capacity, seed=sum(shape))
    # the oracle's last column only needs the last query: the other queries are zeros (their columns are not compared)
    if length <= 1100:
        qfull = np.zeros((hq * d, length), dtype=np.float32)
        qfull[:, -1] = q[:, 0]
        want = gpu_util.oracle(qfull, np.ascontiguousarray(k[:, :length]), np.ascontiguousarray(v[:, :length]), None, hq, hkv, d,
                               length, 1, window=window, global_tokens=global_tokens)["out"][:, -1:]
    else:  # long caches: float64 softmax over the visible positions
        pos = np.arange(length)
        visible = (pos < global_tokens) | (pos >= length - window) if 0 < window < length else np.ones(length, dtype=bool)
        want = _float64(q, k[:, :length][:, visible], v[:, :length][:, visible], hq, hkv, d, int(visible.sum()))
    got = decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), length, hq, d,
                           kv_head_count=hkv, window_size=window, global_token_count=global_tokens)
    torch.cuda.synchronize()
    gpu_util.assert_close_fp32(got.cpu().numpy(), want, "decode out")


@pytest.mark.parametrize("shape", [(16, 16, 64, 16384, 16384), (32, 8, 128, 4096, 4100), (32, 4, 128, 5000, 8192),
                                   (8, 4, 64, 9001, 9004), (4, 4, 32, 8195, 8197), (8, 1, 128, 10000, 10240)])
def test_decode_long_cache_against_float64(shape):
    from sentinel_amd import decode_attention
    hq, hkv, d, length, capacity = shape
    print(f"case decode long {shape}", flush=True)
    q, k, v = _case(hq, hkv, d, length, capacity, seed=sum(shape) + 5)
    want = _float64(q, k, v, hq, hkv, d, length)
    got = decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), length, hq, d,
                           kv_head_count=hkv)
    torch.cuda.synchronize()
    gpu_util.assert_close_fp32(got.cpu().numpy(), want.astype(np.float32), "decode out")


def test_decode_argument_errors():
    from sentinel_amd import decode_attention
    q = torch.zeros(64, 1, device="cuda")
    cache = torch.zeros(64, 32, device="cuda")
    with pytest.raises(ValueError, match="cache length exceeds its capacity"):
        decode_attention(q, cache, cache, 33, 4, 16)
    with pytest.raises(ValueError, match="cache is empty"):
        decode_attention(q, cache, cache, 0, 4, 16)
    with pytest.raises(ValueError, match="globalTokenCount must be >= 0"):
        decode_attention(q, cache, cache, 20, 4, 16, window_size=4, global_token_count=-1)
    decode_attention(q, cache, cache, 20, 4, 16, window_size=32)  # a window that covers the cache is the full mask
    with pytest.raises(ValueError, match="key/value rows mismatch"):
        decode_attention(q, cache, cache, 20, 4, 16, kv_head_count=2)
    with pytest.raises(ValueError, match="must be 1, 2, 4 or 8"):
        decode_attention(torch.zeros(48, 1, device="cuda"), torch.zeros(16, 32, device="cuda"), torch.zeros(16, 32, device="cuda"),
                         20, 3, 16, kv_head_count=1)
