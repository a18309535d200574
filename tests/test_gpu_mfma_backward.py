"""bf16 / fp16 MFMA backward against the fp32 CPU oracle fed the same dtype-rounded inputs (C ABI, [B,H,T,d])."""
import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu

# (q_heads, kv_heads, head_dim, seq_len, packs)
SHAPES = [
    (2, 2, 64, 128, 1),
    (2, 2, 128, 64, 2),
    (4, 1, 128, 300, 2),    # four query heads share one K/V head, ragged tail
    (3, 3, 64, 513, 1),
    (4, 2, 128, 1024, 1),
    (1, 1, 64, 1, 1),
    (2, 1, 64, 129, 1),
    (1, 1, 128, 33, 3),
]


def _run(dtype, shape, causal, sigma_qk=1.0, seed_extra=0):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    hq, hkv, d, t, packs = shape
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape) + 7 + seed_extra, dtype=dtype, sigma_qk=sigma_qk)
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, causal=causal)
    qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, dtype)
                      for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
    out, lse = flash_attention_forward(qd, kd, vd, causal=causal)
    # poison the outputs: every element must be overwritten (the CUDA path needs pre-zeroed dK / dV, this one must not)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (qd, kd, vd))
    flash_attention_backward(qd, kd, vd, out, lse, gd, causal=causal, dq=dq, dk=dk, dv=dv)
    torch.cuda.synchronize()
    errs = {}
    for name, got, like in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        errs[name] = gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(got, like, 0), want[name], name, d)
    return errs


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("causal", [True, False])
def test_backward_matches_oracle(dtype, shape, causal):
    if not causal and shape[3] > 600:
        pytest.skip("non-causal covered by the smaller shapes")
    print(f"case {dtype} {shape} causal={causal}", flush=True)
    _run(dtype, shape, causal)


def test_backward_sharp_softmax_fp16():
    print("case sharp fp16", flush=True)
    _run("fp16", (2, 2, 64, 384, 1), True, sigma_qk=3.0)


def test_backward_is_deterministic():
    """No atomics anywhere: two runs give identical bits."""
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    torch.manual_seed(5)
    q = torch.randn(2, 4, 700, 128, device="cuda").bfloat16()
    k = torch.randn(2, 2, 700, 128, device="cuda").bfloat16()
    v = torch.randn(2, 2, 700, 128, device="cuda").bfloat16()
    g = torch.randn(2, 4, 700, 128, device="cuda").bfloat16()
    out, lse = flash_attention_forward(q, k, v)
    a = flash_attention_backward(q, k, v, out, lse, g)
    b = flash_attention_backward(q, k, v, out, lse, g)
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        assert torch.equal(x, y)
