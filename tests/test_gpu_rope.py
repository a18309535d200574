"""Rotary embedding on the device (C ABI through the Python mirror) against the pinned oracle.

* the in-place fp32 rotation is bit-identical to the oracle (and so to the reference's RotaryEmbedding);
* the fused entry points (unrotated Q, K in; dQ, dK rotated back out) match
  oracle rope -> oracle attention -> oracle inverse rope at the 16-bit bar;
* the fused call agrees bit for bit with the unfused sequence (rotate, attend, rotate back) on the device;
* argument errors carry the reference's exception types and message stems.
"""
import numpy as np
import pytest
import torch

import gpu_util
import oracle_lib

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(3, 16, 40, 0, 0), (2, 64, 130, 0, 0), (4, 128, 300, 7, 0), (2, 32, 96, 0, 32),
                                   (1, 8, 1, 3, 0)])
@pytest.mark.parametrize("inverse", [False, True])
def test_rope_rotate_is_bit_identical_to_the_oracle(shape, inverse):
    from sentinel_amd import HipOps
    heads, d, cols, offset, segment = shape
    print(f"case rope {shape} inverse={inverse}", flush=True)
    rng = np.random.default_rng(sum(shape) + 3)
    x = rng.standard_normal((heads * d, cols)).astype(np.float32)
    cos, sin = oracle_lib.rope_tables(d, cols + offset + 5)
    want = oracle_lib.rope_rotate(x, heads, d, cos, sin, position_offset=offset, segment_length=segment, inverse=inverse)
    xd = torch.from_numpy(x).cuda()
    HipOps.rotary_rotate_in_place(xd, heads, d, d // 2, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), offset,
                                  segment, inverse=inverse)
    torch.cuda.synchronize()
    assert np.array_equal(xd.cpu().numpy(), want)


@pytest.mark.parametrize("compute", ["bf16", "fp16"])
# (q heads, kv heads, head_dim, T, packs, first column, columns behind the window, position offset, spare table rows);
# the gradients and O are written by the attention kernels themselves, 32 tokens per store: sequence lengths around and
# off the multiples of 32, windows that start and end inside a matrix, and tables that end exactly at the last position
@pytest.mark.parametrize("shape", [(4, 4, 64, 128, 1, 0, 0, 0, 3), (8, 2, 128, 200, 2, 4, 4, 0, 3), (2, 1, 64, 70, 3, 3, 1, 11, 3),
                                   (2, 1, 128, 33, 2, 5, 3, 2, 0), (4, 2, 64, 257, 1, 1, 0, 0, 0), (3, 3, 128, 31, 3, 0, 2, 9, 0),
                                   (2, 2, 64, 1, 2, 2, 1, 0, 0),
                                   # head dims padded to the kernels' tilings: the tables keep head_dim / 2 entries per position
                                   (4, 2, 32, 150, 2, 0, 0, 0, 3), (4, 4, 96, 130, 1, 2, 3, 5, 0), (2, 1, 80, 70, 2, 0, 1, 0, 0),
                                   (2, 2, 16, 48, 3, 1, 0, 2, 1)])
def test_fused_rope_attention_matches_oracle(compute, shape):
    from sentinel_amd import HipFlashAttention
    hq, hkv, d, t, packs, col0, pad, offset, spare = shape
    print(f"case fused rope {compute} {shape}", flush=True)
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=sum(shape) + 1, dtype=compute, col0=col0, pad=pad)
    cos, sin = oracle_lib.rope_tables(d, t + offset + spare)
    # the oracle rotates every pack like a sequence of its own: with an offset, segment by segment
    def rotate(x, heads, inverse=False):
        y = x.copy()
        for p in range(packs):
            lo = col0 + p * t
            y[:, lo:lo + t] = oracle_lib.rope_rotate(x[:, lo:lo + t], heads, d, cos, sin, position_offset=offset,
                                                     inverse=inverse)
        return y
    want = gpu_util.oracle(rotate(q, hq), rotate(k, hkv), v, g, hq, hkv, d, t, packs, col0=col0)
    want["dq"] = np.where(np.isnan(want["dq"]), np.nan, rotate(np.nan_to_num(want["dq"]), hq, inverse=True))
    want["dk"] = np.where(np.isnan(want["dk"]), np.nan, rotate(np.nan_to_num(want["dk"]), hkv, inverse=True))

    qd, kd, vd, gd = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    rope = (torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda(), offset)
    sentinel = 555.0
    out = torch.full_like(qd, sentinel)
    lse = torch.full((hq, q.shape[1]), sentinel, device="cuda")
    scale = 1.0 / np.sqrt(np.float32(d))
    out, lse = HipFlashAttention.forward_multi_head(qd, kd, vd, out, lse, hq, d, scale, True, col0, t, packs,
                                                    kv_head_count=hkv, compute=compute, rope=rope)
    dq, dk, dv = (torch.full_like(x, sentinel) for x in (qd, kd, vd))
    dq, dk, dv, _ = HipFlashAttention.backward_multi_head(qd, kd, vd, out, lse, gd, dq, dk, dv, None, hq, d, scale, True,
                                                          col0, t, packs, kv_head_count=hkv, compute=compute, rope=rope)
    torch.cuda.synchronize()
    assert torch.equal(qd.cpu(), torch.from_numpy(q)) and torch.equal(kd.cpu(), torch.from_numpy(k)), "inputs were modified"
    for key, got in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        got = got.cpu().numpy()
        outside = np.isnan(want[key])
        assert np.all(got[outside] == sentinel), f"{key}: wrote outside the pack window"
        gpu_util.assert_close_lowp(np.where(outside, np.nan, got), want[key], key, d)
    got = lse.cpu().numpy()
    outside = np.isnan(want["lse"])
    # the rotated Q, K are rounded to 16 bit before the scores are formed: LSE carries that rounding
    assert np.nanmax(np.abs(np.where(outside, np.nan, got) - want["lse"])) <= 2e-2 * max(1.0, np.nanmax(np.abs(want["lse"])))


def test_fused_equals_rotate_then_attend_on_the_device():
    from sentinel_amd import HipFlashAttention, HipOps
    hq, hkv, d, t, packs = 4, 2, 128, 160, 2
    q, k, v, g = gpu_util.make_inputs(hq, hkv, d, t, packs, seed=99, dtype="bf16")
    cos, sin = oracle_lib.rope_tables(d, t)
    cosd, sind = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    qd, kd, vd, gd = (torch.from_numpy(x).cuda() for x in (q, k, v, g))
    scale = 1.0 / np.sqrt(np.float32(d))
    args = (hq, d, scale, True, 0, t, packs)
    fo, fl = HipFlashAttention.forward_multi_head(qd, kd, vd, None, None, *args, kv_head_count=hkv, compute="bf16",
                                                  rope=(cosd, sind))
    fdq, fdk, fdv, _ = HipFlashAttention.backward_multi_head(qd, kd, vd, fo, fl, gd, None, None, None, None, *args,
                                                             kv_head_count=hkv, compute="bf16", rope=(cosd, sind))
    # the reference's sequence: rotate Q, K in place (segments of t), attend, rotate the gradients back
    qr, kr = qd.clone(), kd.clone()
    HipOps.rotary_rotate_in_place(qr, hq, d, d // 2, cosd, sind, 0, t)
    HipOps.rotary_rotate_in_place(kr, hkv, d, d // 2, cosd, sind, 0, t)
    uo, ul = HipFlashAttention.forward_multi_head(qr, kr, vd, None, None, *args, kv_head_count=hkv, compute="bf16")
    udq, udk, udv, _ = HipFlashAttention.backward_multi_head(qr, kr, vd, uo, ul, gd, None, None, None, None, *args,
                                                             kv_head_count=hkv, compute="bf16")
    HipOps.rotary_rotate_inverse_in_place(udq, hq, d, d // 2, cosd, sind, 0, t)
    HipOps.rotary_rotate_inverse_in_place(udk, hkv, d, d // 2, cosd, sind, 0, t)
    torch.cuda.synchronize()
    # forward: both paths round the same fp32 rotated values to bf16 -> identical
    assert torch.equal(fo, uo) and torch.equal(fl, ul) and torch.equal(fdv, udv)
    # dQ, dK: the fused path rotates the 16-bit gradient back in fp32, the sequence rotates its fp32 copy: same values
    assert torch.equal(fdq, udq) and torch.equal(fdk, udk)


def test_rope_argument_errors():
    from sentinel_amd import HipFlashAttention, HipOps
    d, heads, cols = 16, 2, 12
    x = torch.zeros(heads * d, cols, device="cuda")
    cos = torch.ones(10, d // 2, device="cuda")
    sin = torch.zeros(10, d // 2, device="cuda")
    with pytest.raises(ValueError, match="position exceeds RoPE table"):
        HipOps.rotary_rotate_in_place(x, heads, d, d // 2, cos, sin)
    with pytest.raises(ValueError, match="segmentLength exceeds RoPE table"):
        HipOps.rotary_rotate_in_place(x, heads, d, d // 2, cos, sin, 0, 11)
    with pytest.raises(ValueError, match="negative positionOffset"):
        HipOps.rotary_rotate_in_place(x[:, :4].contiguous(), heads, d, d // 2, cos, sin, -1)
    with pytest.raises(ValueError, match="embedding dim mismatch"):
        HipOps.rotary_rotate_in_place(x, heads + 1, d, d // 2, cos, sin)
    with pytest.raises(ValueError, match="invalid rope dims"):
        HipOps.rotary_rotate_in_place(x, heads, d, 0, cos, sin)
    HipOps.rotary_rotate_in_place(x, heads, d, d // 2, cos, sin, 0, 6)  # 12 columns in segments of 6: fine
    # fused call where there is no conversion pass to ride on: reported, not faked
    q = torch.zeros(4 * 64, 64, device="cuda")
    cos64 = torch.ones(64, 32, device="cuda")
    with pytest.raises(ValueError, match="rotate other tensors with sentinel_hip_rope_rotate"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 64, 0.125, True, 0, 64, 1, compute="fp32",
                                             rope=(cos64, torch.zeros_like(cos64)))
    with pytest.raises(ValueError, match="position exceeds RoPE table"):
        HipFlashAttention.forward_multi_head(q, q, q, None, None, 4, 64, 0.125, True, 0, 64, 1, compute="bf16",
                                             rope=(cos64, torch.zeros_like(cos64), 1))
