"""The one-pass backward variant (SENTINEL_HIP_BACKWARD_STORED_SCORES: the dK / dV kernel writes dS out, dQ is formed
from it) against the fp32 CPU oracle and against the default two-pass backward, through the C ABI in both layouts."""
import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu

# (q_heads, kv_heads, head_dim, seq_len, packs): tile edges of the 128-key tiles, 64-query stages and 256-query tiles
SHAPES = [
    (2, 2, 128, 64, 2),
    (4, 1, 128, 300, 2),
    (2, 2, 128, 257, 1),
    (1, 1, 128, 1, 1),
    (1, 1, 128, 129, 3),
    (4, 2, 128, 1024, 1),
    (2, 1, 128, 1300, 1),
]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_stored_scores_backward_matches_oracle_and_default(dtype, shape):
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    hq, hkv, d, t, packs = shape
    print(f"case {dtype} {shape}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape) + 3, dtype=dtype)
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs)
    qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, dtype) for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
    out, lse = flash_attention_forward(qd, kd, vd)
    ref = flash_attention_backward(qd, kd, vd, out, lse, gd)
    dq, dk, dv = (torch.full_like(x, float("nan")) for x in (qd, kd, vd))  # every element must be overwritten
    flash_attention_backward(qd, kd, vd, out, lse, gd, dq=dq, dk=dk, dv=dv, stored_scores=True)
    torch.cuda.synchronize()
    for name, got, like in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        gpu_util.assert_close_lowp(gpu_util.bhtd_to_columns(got, like, 0), want[name], name, d)
    # against the default: D = rowsum(dO o O) is summed in another order, and dQ sums the 16-bit dS in another order
    for got, base in zip((dq, dk, dv), ref):
        err = (got.float() - base.float()).abs().max().item()
        assert err <= 1e-2 * base.float().abs().max().item() + 1e-5


def test_flag_changes_nothing_where_it_does_not_apply():
    from sentinel_amd import flash_attention_backward, flash_attention_forward
    torch.manual_seed(3)
    for d, kw in ((64, {}), (128, dict(causal=False)), (128, dict(window_size=70, global_token_count=3))):
        q = torch.randn(1, 2, 200, d, device="cuda").bfloat16()
        k, v, g = torch.randn_like(q), torch.randn_like(q), torch.randn_like(q)
        out, lse = flash_attention_forward(q, k, v, **kw)
        a = flash_attention_backward(q, k, v, out, lse, g, **kw)
        b = flash_attention_backward(q, k, v, out, lse, g, stored_scores=True, **kw)
        torch.cuda.synchronize()
        for x, y in zip(a, b):
            assert torch.equal(x, y)


def test_workspace_contract_and_column_layout():
    import sentinel_amd
    from sentinel_amd import HipFlashAttention
    from sentinel_amd.flash_attention import BACKWARD_STORED_SCORES
    lib = sentinel_amd.load_library()
    hq, hkv, d, t, packs = 4, 2, 128, 320, 2
    # [B,H,T,d]: the workspace is the stored scores alone; 128-key tiles x 64-query stages of 16 KiB from the diagonal on
    need = lib.sentinel_hip_flash_workspace_bytes(1, -1, 1 | BACKWARD_STORED_SCORES, hq, hkv, d, t, packs, 1)
    stages, tiles = (t + 63) // 64, (t + 127) // 128
    assert need == packs * hq * (tiles * stages - tiles * (tiles - 1)) * 16384
    assert lib.sentinel_hip_flash_workspace_bytes(1, -1, 1 | BACKWARD_STORED_SCORES, hq, hkv, 64, t, packs, 1) == 0
    assert lib.sentinel_hip_flash_workspace_bytes(1, -1, 1 | BACKWARD_STORED_SCORES, hq, hkv, d, t, packs, 0) == 0
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=41, dtype="bf16")
    qd, kd, vd, gd = (gpu_util.columns_to_device_bhtd(x, h, d, t, packs, 0, "bf16") for x, h in ((q, hq), (k, hkv), (v, hkv), (g, hq)))
    out, lse = sentinel_amd.flash_attention_forward(qd, kd, vd)
    small = torch.empty(need - 256, dtype=torch.uint8, device="cuda")
    got = sentinel_amd.flash_attention_backward(qd, kd, vd, out, lse, gd, stored_scores=True, workspace=small)  # replaced by one that fits
    torch.cuda.synchronize()
    assert all(torch.isfinite(x.float()).all() for x in got)
    # the drop-in layout: fp32 column matrices, bf16 arithmetic
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs)
    qc, kc, vc, gc = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    scale = 1.0 / np.sqrt(np.float32(d))
    o, l = HipFlashAttention.forward_multi_head(qc, kc, vc, None, None, hq, d, scale, True, 0, t, packs, kv_head_count=hkv, compute="bf16")
    dq, dk, dv, _ = HipFlashAttention.backward_multi_head(qc, kc, vc, o, l, gc, None, None, None, None, hq, d, scale, True, 0, t,
                                                          packs, kv_head_count=hkv, compute="bf16", stored_scores=True)
    torch.cuda.synchronize()
    for name, got_c in (("dq", dq), ("dk", dk), ("dv", dv)):
        gpu_util.assert_close_lowp(got_c.cpu().numpy(), want[name], name, d)
