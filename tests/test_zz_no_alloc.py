"""The decode entry point that allocates nothing (sentinel_hip_decode_attention_static: partial results in a device
array that belongs to the library) against sentinel_hip_decode_attention with a caller-provided workspace, through the
C ABI: same kernels, so the results must agree bit for bit (the bar of the fp32 path is 1e-4), on two calls in a row
of which the second is smaller, so stale records of the first call lie behind the ones the second call uses."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util

pytestmark = pytest.mark.gpu

STATIC_BYTES = 4 << 20


def _case(lib, hq, hkv, d, length, capacity, seed, window=0, global_tokens=0):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    q = torch.randn(hq * d, 1, device="cuda", generator=gen)
    k = torch.randn(hkv * d, capacity, device="cuda", generator=gen)
    v = torch.randn(hkv * d, capacity, device="cuda", generator=gen)
    scale = 1.0 / float(np.sqrt(d))
    need = lib.sentinel_hip_decode_workspace_bytes(hq, d, length)
    assert need <= STATIC_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.full((hq * d, 1), float("nan"), device="cuda")
    got = torch.full((hq * d, 1), float("nan"), device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.sentinel_hip_decode_attention(p(q), p(k), p(v), p(want), hq, hkv, d, capacity, length, scale, window,
                                           global_tokens, p(ws), need, stream)
    assert rc == 0, lib.sentinel_hip_last_error()
    rc = lib.sentinel_hip_decode_attention_static(p(q), p(k), p(v), p(got), hq, hkv, d, capacity, length, scale, window,
                                                  global_tokens, stream)
    assert rc == 0, lib.sentinel_hip_last_error()
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    gpu_util.assert_close_fp32(got.cpu().numpy(), want.cpu().numpy(), f"decode static L{length}")
    assert torch.equal(got, want), "same kernels on the same inputs: expected identical bits"
    return q, k, v, got


def test_static_scratch_decode_matches_workspace_decode():
    import sentinel_amd
    lib = sentinel_amd.load_library()
    print("case decode static: L12000 GQA then L700 MHA", flush=True)
    # first a long cache (chunks of 256 positions, grouped heads), then a short one (chunks of 64) whose records
    # occupy the front of the area the first call filled
    q, k, v, got = _case(lib, 16, 4, 128, 12000, 12288, seed=1)
    _case(lib, 8, 8, 64, 700, 1024, seed=2)
    # and under the layer's sparse mask, where only some chunks are launched
    _case(lib, 8, 2, 128, 5000, 5000, seed=3, window=600, global_tokens=70)
    # against the oracle as well: the last column of the full causal forward
    hq, hkv, d, length = 4, 2, 64, 333
    qc, kc, vc, _ = gpu_util.make_inputs(hq, hkv, d, length, 1, seed=17)
    want = gpu_util.oracle(qc, kc, vc, None, hq, hkv, d, length, 1)["out"][:, -1:]
    qd = torch.from_numpy(np.ascontiguousarray(qc[:, -1:])).cuda()
    kd, vd = torch.from_numpy(kc).cuda(), torch.from_numpy(vc).cuda()
    out = torch.empty(hq * d, 1, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.sentinel_hip_decode_attention_static(p(qd), p(kd), p(vd), p(out), hq, hkv, d, length, length,
                                                  1.0 / float(np.sqrt(d)), 0, 0,
                                                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.sentinel_hip_last_error()
    torch.cuda.synchronize()
    gpu_util.assert_close_fp32(out.cpu().numpy(), want, "decode static vs oracle")


def test_static_scratch_decode_rejects_what_does_not_fit():
    import sentinel_amd
    lib = sentinel_amd.load_library()
    hq, d, length = 32, 128, 131072
    assert lib.sentinel_hip_decode_workspace_bytes(hq, d, length) > STATIC_BYTES
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    rc = lib.sentinel_hip_decode_attention_static(one, one, one, one, hq, 8, d, length, length, 0.1, 0, 0, None)
    assert rc == 1 and b"built-in area holds" in lib.sentinel_hip_last_error()
