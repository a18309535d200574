"""sentinel_hip_cast_to_16bit (the operand cast of the layer's mixed-precision GEMMs, CudaAmp::castFloatBufferToHalf)
through the C ABI: bit-exact against the IEEE round-to-nearest-even conversion (numpy's / torch's) for both 16-bit
types, on sizes around the eight-value groups of the wide path, on misaligned buffers and on the values where rounding
matters (ties, subnormals, overflow to infinity, infinities, NaN)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _special_values():
    ties = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8,  # halfway cases
                     65504.0, 65519.99, 65520.0, 7e4, -7e4, 3.3e38, -3.3e38,  # fp16's edge, fp32's edge
                     6e-8, 2.98e-8, 2.99e-8, 1e-40, -1e-40, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)
    return ties


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("count", [1, 7, 8, 9, 255, 2048, 2049, 100003, 768 * 4096 + 5])
def test_cast_matches_round_to_nearest_even(dtype, count):
    from sentinel_amd import HipAmp
    print(f"case cast {dtype} count {count}", flush=True)
    rng = np.random.default_rng(count)
    host = (rng.standard_normal(count) * np.exp(rng.uniform(-12, 12, count))).astype(np.float32)
    special = _special_values()
    host[:min(count, special.size)] = special[:min(count, special.size)]
    source = torch.from_numpy(host).cuda()
    got = HipAmp.cast_to_half(source, dtype)
    torch.cuda.synchronize()
    want = torch.from_numpy(host).to(dtype)  # the CPU's IEEE conversion
    assert got.dtype == dtype and got.shape == source.shape
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cast_of_misaligned_buffers_and_nan(dtype):
    """Buffers that are not 16-byte aligned take the one-value-per-thread path; NaN stays NaN."""
    from sentinel_amd import HipAmp
    import sentinel_amd
    count = 1001
    host = np.random.default_rng(5).standard_normal(count + 3).astype(np.float32)
    host[17] = np.nan
    whole = torch.from_numpy(host).cuda()
    source = whole[3:]  # 12 bytes into the allocation
    out_whole = torch.full((count + 1,), 7.0, dtype=dtype, device="cuda")
    out = out_whole[1:]  # 2 bytes into the allocation
    lib = sentinel_amd.load_library()
    import ctypes
    code = lib.sentinel_hip_cast_to_16bit(ctypes.c_void_p(source.data_ptr()), ctypes.c_void_p(out.data_ptr()), count,
                                          {torch.bfloat16: 1, torch.float16: 2}[dtype], None)
    assert code == 0, lib.sentinel_hip_last_error()
    torch.cuda.synchronize()
    want = torch.from_numpy(host[3:]).to(dtype)
    got = out.cpu()
    assert float(out_whole[0]) == 7.0  # nothing written in front of the destination
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan) and int(nan.sum()) == 1
    assert torch.equal(got[~nan].view(torch.int16), want[~nan].view(torch.int16))


def test_cast_argument_errors():
    from sentinel_amd import HipAmp
    x = torch.zeros(16, device="cuda")
    with pytest.raises(ValueError, match="dtype must be"):
        HipAmp.cast_to_half(x, torch.float32)
    with pytest.raises(ValueError, match="contiguous fp32"):
        HipAmp.cast_to_half(x.to(torch.float16))
    with pytest.raises(ValueError, match="destination"):
        HipAmp.cast_to_half(x, torch.float16, out=torch.zeros(8, dtype=torch.float16, device="cuda"))
    empty = HipAmp.cast_to_half(torch.zeros(0, device="cuda"))
    assert empty.numel() == 0
