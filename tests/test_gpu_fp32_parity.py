"""fp32 path on the GPU against the reference's own outputs (golden fixtures) and the oracle, through the C ABI."""
import glob
import os

import numpy as np
import pytest
import torch

import gpu_util
import oracle_lib

pytestmark = pytest.mark.gpu

CASES = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))
               if not p.endswith("_kat.npz"))


def _dev(x):
    return torch.from_numpy(np.nan_to_num(x, nan=0.0)).cuda()


@pytest.mark.parametrize("name", CASES)
def test_columns_layout_matches_reference_fixtures(golden_dir, name):
    from sentinel_amd import HipFlashAttention
    print(f"case {name}", flush=True)
    fx = np.load(os.path.join(golden_dir, name + ".npz"))
    hq, hkv, d, t, packs, col0, stride = (int(x) for x in fx["geometry"])
    q, k, v, g = (_dev(fx[key]) for key in ("q", "k", "v", "d_out"))
    sentinel = 777.0  # columns outside the window must stay untouched
    out = torch.full_like(q, sentinel)
    lse = torch.full((hq, stride), sentinel, device="cuda")
    scale = 1.0 / np.sqrt(np.float32(d))
    out, lse = HipFlashAttention.forward_multi_head(q, k, v, out, lse, hq, d, scale, True, col0, t, packs, kv_head_count=hkv)
    dq, dk, dv = (torch.full_like(x, sentinel) for x in (q, k, v))
    dq, dk, dv, delta = HipFlashAttention.backward_multi_head(q, k, v, out, lse, g, dq, dk, dv, None, hq, d, scale, True,
                                                              col0, t, packs, kv_head_count=hkv)
    torch.cuda.synchronize()
    for key, got in (("out", out), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
        got = got.cpu().numpy()
        want = fx[key]
        outside = np.isnan(want)
        assert np.all(got[outside] == sentinel), f"{key}: wrote outside the pack window"
        got = np.where(outside, np.nan, got)
        gpu_util.assert_close_fp32(got, want, f"{name}:{key}")
    want_delta = oracle_lib.oracle_delta(fx["out"], fx["d_out"], q_heads=hq, head_dim=d, seq_len=t, pack_count=packs, col_start=col0)
    want_delta = want_delta[:, col0:col0 + packs * t]
    gpu_util.assert_close_fp32(delta.cpu().numpy(), want_delta, f"{name}:delta")


@pytest.mark.parametrize("shape", [(4, 4, 16, 48, 4), (3, 1, 24, 77, 2), (2, 2, 128, 130, 1), (4, 2, 64, 200, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_bhtd_layout_fp32_matches_oracle(shape, causal):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    hq, hkv, d, t, packs = shape
    print(f"case {shape} causal={causal}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape))
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, causal=causal)
    qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, "fp32") for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
    out, lse = flash_attention_forward(qd, kd, vd, causal=causal)
    dq, dk, dv = flash_attention_backward(qd, kd, vd, out, lse, gd, causal=causal)
    torch.cuda.synchronize()
    gpu_util.assert_close_fp32(gpu_util.bhtd_to_columns(out, q, 0), want["out"], "out")
    gpu_util.assert_close_fp32(gpu_util.bht_to_columns(lse, hq, q.shape[1], 0), want["lse"], "lse")
    gpu_util.assert_close_fp32(gpu_util.bhtd_to_columns(dq, q, 0), want["dq"], "dq")
    gpu_util.assert_close_fp32(gpu_util.bhtd_to_columns(dk, k, 0), want["dk"], "dk")
    gpu_util.assert_close_fp32(gpu_util.bhtd_to_columns(dv, v, 0), want["dv"], "dv")


def test_argument_errors_match_reference_exception_types():
    # std::invalid_argument -> ValueError, std::runtime_error -> RuntimeError (CudaFlashAttention.cu:1458-1471, :1533-1552)
    from sentinel_amd import HipFlashAttention
    q = torch.zeros((64, 192), device="cuda")
    kw = dict(out=None, log_sum_exp=None)
    with pytest.raises(ValueError, match="invalid head geometry"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 0, 16, 0.25)
    with pytest.raises(ValueError, match="query rows mismatch"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 3, 16, 0.25)
    with pytest.raises(ValueError, match="headDim exceeds maxHeadDimension"):
        HipFlashAttention.forward_multi_head(torch.zeros((256, 8), device="cuda"), torch.zeros((256, 8), device="cuda"),
                                             torch.zeros((256, 8), device="cuda"), None, None, 1, 256, 0.25)
    with pytest.raises(ValueError, match="invalid column window"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 16, 0.25, True, 100, 100, 1)
    with pytest.raises(ValueError, match="pack window exceeds columns"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 16, 0.25, True, 0, 48, 5)
    with pytest.raises(ValueError, match="sequenceLength mismatch"):
        HipFlashAttention.forward_multi_head(q, torch.zeros((64, 96), device="cuda"), q, None, None, 4, 16, 0.25)
    out, lse = HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 16, 0.25, True, 0, 48, 4)
    with pytest.raises(ValueError, match="logSumExp shape mismatch"):
        HipFlashAttention.backward_multi_head(q, q, q, out, lse[:2], q, None, None, None, None, 4, 16, 0.25, True, 0, 48, 4)
    # column_count <= 0 means "to the end of the matrix" (resolveColumnWindow)
    out2, lse2 = HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 16, 0.25, True, 0, 0, 1)
    assert out2.shape == q.shape and torch.isfinite(out2).all()
