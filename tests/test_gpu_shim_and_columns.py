"""The drop-in faces of the library on the GPU: the C++ shims (HipFlashAttention.hpp, HipCausalSelfAttention.hpp) and MFMA arithmetic on
Sentinel's own fp32 column layout (the adapter path), both through the C ABI."""
import os
import subprocess

import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_shim_parity_and_exceptions():
    exe = os.path.join(HERE, "cpp", "test_shim")
    assert os.path.exists(exe), "tests/cpp/test_shim is not built: python -c 'import __graft_entry__ as g; g.build()'"
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "shim ok" in proc.stdout


def test_cpp_attention_layer_parity_and_exceptions():
    """HipCausalSelfAttention (projections + RoPE + flash attention + output projection, forward and backward) against
    the oracle's layer; fp32 at 1e-4, MFMA arithmetic at 2e-2."""
    exe = os.path.join(HERE, "cpp", "test_layer")
    assert os.path.exists(exe), "tests/cpp/test_layer is not built: python -c 'import __graft_entry__ as g; g.build()'"
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "layer ok" in proc.stdout


def test_cpp_layer_bench_runs():
    """tests/cpp/bench_layer (what bench.py's layer_path starts): a short run of every configuration, its JSON parses and
    the mixed-precision timing really took the 16-bit products (the program checks that itself and fails otherwise)."""
    import json
    exe = os.path.join(HERE, "cpp", "bench_layer")
    assert os.path.exists(exe), "tests/cpp/bench_layer is not built: python -c 'import __graft_entry__ as g; g.build()'"
    proc = subprocess.run([exe, "512", "2", "1"], capture_output=True, text=True, timeout=110)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    line = json.loads(proc.stdout.strip().splitlines()[-1])
    assert [s["seq_len"] for s in line["shapes"]] == [128, 256, 1024]
    for shape in line["shapes"]:
        for mode in ("flash", "dense", "flash_mixed_projections"):
            assert shape[mode]["attention_fwd_ms"] > 0 and shape[mode]["attention_bwd_ms"] > 0
            assert shape["tokens_per_s_" + mode] > 0
    one = subprocess.run([exe, "512", "2", "1", "flash", "256"], capture_output=True, text=True, timeout=110)
    assert one.returncode == 0, one.stdout + one.stderr
    only = json.loads(one.stdout.strip().splitlines()[-1])["shapes"]
    assert len(only) == 1 and only[0]["seq_len"] == 256 and "dense" not in only[0] and "flash" in only[0]


@pytest.mark.parametrize("compute", ["bf16", "fp16"])
# (q heads, kv heads, head_dim, T, packs, first column, columns behind the window); head dims the kernels have no tiling of
# their own for (32, 80, 96, 16, 24, 120, 72) are zero-padded to 64 / 128 by the conversion pass
@pytest.mark.parametrize("shape", [(12, 12, 64, 128, 1, 0, 0), (8, 2, 128, 200, 2, 4, 4), (2, 2, 64, 70, 3, 3, 1),
                                   (4, 2, 32, 150, 2, 0, 0), (8, 8, 96, 130, 1, 2, 3), (4, 1, 80, 257, 1, 0, 0),
                                   (3, 3, 16, 48, 4, 0, 0), (2, 2, 24, 65, 2, 1, 0), (2, 1, 120, 100, 1, 0, 5), (2, 2, 72, 33, 2, 3, 0)])
def test_columns_layout_with_mfma_arithmetic(compute, shape):
    from sentinel_amd import HipFlashAttention
    hq, hkv, d, t, packs, col0, pad = shape
    print(f"case {compute} {shape}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape), dtype=compute, col0=col0, pad=pad)
    want = gpu_util.oracle(q, k, v, g, hq, hkv, d, t, packs, col0=col0)
    qd, kd, vd, gd = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    sentinel = 777.0
    out = torch.full_like(qd, sentinel)
    lse = torch.full((hq, q.shape[1]), sentinel, device="cuda")
    scale = 1.0 / np.sqrt(np.float32(d))
    out, lse = HipFlashAttention.forward_multi_head(qd, kd, vd, out, lse, hq, d, scale, True, col0, t, packs,
                                                    kv_head_count=hkv, compute=compute)
    dq, dk, dv = (torch.full_like(x, sentinel) for x in (qd, kd, vd))
    dq, dk, dv, _ = HipFlashAttention.backward_multi_head(qd, kd, vd, out, lse, gd, dq, dk, dv, None, hq, d, scale, True,
                                                          col0, t, packs, kv_head_count=hkv, compute=compute)
    torch.cuda.synchronize()
    for key, got in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        got = got.cpu().numpy()
        outside = np.isnan(want[key])
        assert np.all(got[outside] == sentinel), f"{key}: wrote outside the pack window"
        # the backward consumes `out` rounded to 16 bit a second time (fp32 -> 16 bit adapter), still within the bar
        gpu_util.assert_close_lowp(np.where(outside, np.nan, got), want[key], key, d)
    got = lse.cpu().numpy()
    outside = np.isnan(want["lse"])
    assert np.all(got[outside] == sentinel)
    gpu_util.assert_close_fp32(np.where(outside, np.nan, got), want["lse"], "lse", tol=1e-3)


def test_unsupported_head_dim_is_reported_not_faked():
    from sentinel_amd import HipFlashAttention
    q = torch.zeros((4 * 44, 64), device="cuda")
    with pytest.raises(ValueError, match="head_dim that is a multiple of 8"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 44, 0.1, compute="bf16")
    # the exact fp32 kernels take any head_dim <= 128
    out, lse = HipFlashAttention.forward_multi_head(q + 0.01, q, q, None, None, 4, 44, 0.1)
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("variant", ["plain", "rope", "sparse_rope"])
def test_backward_reuses_the_forward_workspace(variant):
    """SENTINEL_HIP_WORKSPACE_KEEP / _REUSE: the forward call leaves its 16-bit operands in the caller's workspace and
    the backward call converts d_out only.  Same kernels on the same 16-bit operands: gradients identical to the plain
    pair of calls, bit for bit, even when the fp32 q / k / v / out handed to the backward call are garbage."""
    import oracle_lib
    import sentinel_amd
    from sentinel_amd import HipFlashAttention
    hq, hkv, d, t, packs, col0, pad = 8, 2, 128, 200, 2, 4, 4
    print(f"case workspace reuse {variant}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=77, dtype="bf16", col0=col0, pad=pad)
    qd, kd, vd, gd = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    scale = 1.0 / np.sqrt(np.float32(d))
    args = (hq, d, scale, True, col0, t, packs)
    kw = dict(kv_head_count=hkv, compute="bf16")
    if "rope" in variant:
        cos, sin = oracle_lib.rope_tables(d, t)
        kw["rope"] = (torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda())
    if "sparse" in variant:
        kw.update(window_size=60, global_token_count=3)
    out0, lse0 = HipFlashAttention.forward_multi_head(qd, kd, vd, None, None, *args, **kw)
    dq0, dk0, dv0, _ = HipFlashAttention.backward_multi_head(qd, kd, vd, out0, lse0, gd, None, None, None, None, *args, **kw)

    lib = sentinel_amd.load_library()
    need = lib.sentinel_hip_flash_workspace_bytes(0, 1, 0, hq, hkv, d, t, packs, 1)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out1, lse1 = HipFlashAttention.forward_multi_head(qd, kd, vd, None, None, *args, workspace=ws, keep_for_backward=True, **kw)
    junk_q, junk_k, junk_v, junk_o = (torch.full_like(x, float("nan")) for x in (qd, kd, vd, out1))
    dq1, dk1, dv1, _ = HipFlashAttention.backward_multi_head(junk_q, junk_k, junk_v, junk_o, lse1, gd, None, None, None, None,
                                                             *args, workspace=ws, reuse_forward_workspace=True, **kw)
    torch.cuda.synchronize()
    inside = torch.zeros(qd.shape[1], dtype=torch.bool, device="cuda")
    inside[col0:col0 + packs * t] = True
    for name, a, b in (("out", out0, out1), ("lse", lse0, lse1), ("dq", dq0, dq1), ("dk", dk0, dk1), ("dv", dv0, dv1)):
        assert torch.equal(a[:, inside], b[:, inside]), f"{name} differs with the kept workspace"
    # a workspace that is too small for the backward is refused, not silently replaced
    with pytest.raises(ValueError, match="keep_for_backward needs"):
        HipFlashAttention.forward_multi_head(qd, kd, vd, None, None, *args, workspace=ws[:need // 2], keep_for_backward=True, **kw)
