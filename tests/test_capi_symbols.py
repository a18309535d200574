"""CPU-only checks of the boundary: the built library exports every symbol the header declares, argument
validation returns the documented codes without touching a GPU, and the Python mirror refuses to run without it."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sentinel_hip_attn.h")


def _declared():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"SENTINEL_HIP_API\s+[\w\s\*]+?\b(sentinel_hip_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    import sentinel_amd
    if not os.path.exists(sentinel_amd.library_path()):
        from sentinel_amd.build import build_library
        build_library()
    return sentinel_amd.load_library()


def test_every_declared_symbol_is_exported(lib):
    names = _declared()
    assert len(names) >= 9, names
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"


def test_codes_and_messages_without_a_gpu(lib):
    assert lib.sentinel_hip_flash_max_head_dim() == 128
    assert lib.sentinel_hip_strerror(0) == b"ok"
    fwd = lib.sentinel_hip_flash_fwd
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first

    def call(**kw):
        a = dict(io=0, comp=-1, layout=0, hq=4, hkv=4, d=16, stride=192, col0=0, t=48, packs=4, scale=0.25)
        a.update(kw)
        return fwd(one, one, one, one, one, a["io"], a["comp"], a["layout"], a["hq"], a["hkv"], a["d"], a["stride"], a["col0"],
                   a["t"], a["packs"], a["scale"], 1, None, 0, None)

    assert fwd(None, one, one, one, one, 0, -1, 0, 4, 4, 16, 192, 0, 48, 4, 0.25, 1, None, 0, None) == 1
    assert b"empty input" in lib.sentinel_hip_last_error()
    assert call(hq=0) == 1 and b"invalid head geometry" in lib.sentinel_hip_last_error()
    assert call(hq=3, hkv=2) == 1 and b"divisible by kvHeadCount" in lib.sentinel_hip_last_error()
    assert call(d=256) == 1 and b"headDim exceeds maxHeadDimension" in lib.sentinel_hip_last_error()
    assert call(col0=190) == 1 and b"invalid column window" in lib.sentinel_hip_last_error()
    assert call(packs=5) == 1 and b"pack window exceeds columns" in lib.sentinel_hip_last_error()
    assert call(scale=0.0) == 1 and b"scale must be positive" in lib.sentinel_hip_last_error()
    # MFMA arithmetic pads head dims to 64 / 128 in the conversion pass of fp32 column tensors: multiples of 8 only,
    # and 16-bit [B,H,T,d] tensors (no conversion pass) need a head dim the kernels are tiled for
    assert call(comp=1, d=12, stride=192) == 2 and b"multiple of 8" in lib.sentinel_hip_last_error()
    assert call(io=1, layout=1, d=16) == 2 and b"head_dim 64 and 128" in lib.sentinel_hip_last_error()
    assert call(io=1, layout=0, d=64) == 2                                        # 16-bit needs [B,H,T,d]
    # a valid call without a device is a runtime error, not a silent fallback
    if not lib.sentinel_hip_device_available():
        assert call() == 3 and b"no HIP device" in lib.sentinel_hip_last_error()


def test_sparse_rope_and_decode_validation_without_a_gpu(lib):
    """The newer entry points validate before touching the device, with the reference's message stems."""
    one = ctypes.c_void_p(16)
    i, f = ctypes.c_int, ctypes.c_float
    sparse = lib.sentinel_hip_flash_fwd_sparse

    def call(window=4, global_tokens=0, causal=1, cos=None, sin=None, positions=0):
        return sparse(one, one, one, one, one, cos, sin, positions, 0, window, global_tokens, 0, -1, 0, 4, 4, 16, 192, 0, 48, 4,
                      0.25, causal, None, 0, None)

    assert call(global_tokens=-1) == 1 and b"globalTokenCount must be >= 0" in lib.sentinel_hip_last_error()
    assert call(causal=0) == 1 and b"causal must be set" in lib.sentinel_hip_last_error()
    assert call(cos=one) == 1 and b"empty tables" in lib.sentinel_hip_last_error()            # one table without the other
    assert call(cos=one, sin=one, positions=10) == 1 and b"position exceeds RoPE table" in lib.sentinel_hip_last_error()
    if not lib.sentinel_hip_device_available():
        assert call() == 3 and b"no HIP device" in lib.sentinel_hip_last_error()
        assert call(window=0, causal=0) == 3  # no window: the causal flag is free again

    # seq_len <= 0 means "the rest of the window" in the column layout: the tables are checked against the resolved
    # length (here 256 columns against 4 table rows), not against the raw argument
    rope_fwd = lib.sentinel_hip_flash_fwd_rope
    ws = ctypes.c_void_p(256)
    for seq_len in (256, 0):
        assert rope_fwd(one, one, one, one, one, one, one, 4, 0, 0, 1, 0, 2, 2, 64, 256, 0, seq_len, 1, 0.125, 1, ws, 1 << 30,
                        None) == 1, seq_len
        assert b"position exceeds RoPE table" in lib.sentinel_hip_last_error()
    rope_bwd = lib.sentinel_hip_flash_bwd_rope
    assert rope_bwd(one, one, one, one, one, one, one, one, one, one, one, one, 4, 0, 0, 1, 0, 2, 2, 64, 256, 0, 0, 1, 0.125,
                    1, ws, 1 << 30, None) == 1
    assert b"position exceeds RoPE table" in lib.sentinel_hip_last_error()
    assert sparse(one, one, one, one, one, one, one, 4, 0, 8, 0, 0, 1, 0, 2, 2, 64, 256, 0, 0, 1, 0.125, 1, ws, 1 << 30,
                  None) == 1 and b"position exceeds RoPE table" in lib.sentinel_hip_last_error()
    # limits of the 32-bit addressing inside one head and of the conversion grid
    fwd = lib.sentinel_hip_flash_fwd
    assert fwd(one, one, one, one, one, 1, -1, 1, 1, 1, 128, 0, 0, 1 << 24, 1, 0.1, 1, None, 0, None) == 1
    assert b"exceeds 2 GiB" in lib.sentinel_hip_last_error()
    assert fwd(one, one, one, one, one, 0, 1, 0, 70000, 70000, 64, 8, 0, 8, 1, 0.1, 1, ws, 1 << 40, None) == 1
    assert b"65535" in lib.sentinel_hip_last_error()

    rotate = lib.sentinel_hip_rope_rotate
    assert rotate(one, 2, 15, 12, 0, 12, 0, 0, one, one, 32, 0, None) == 1 and b"invalid rope dims" in lib.sentinel_hip_last_error()
    assert rotate(one, 2, 16, 12, 0, 12, 0, 0, one, one, 10, 0, None) == 1 and b"position exceeds RoPE table" in lib.sentinel_hip_last_error()
    assert rotate(one, 2, 16, 12, 4, 12, 0, 0, one, one, 32, 0, None) == 1 and b"column window outside the matrix" in lib.sentinel_hip_last_error()

    decode = lib.sentinel_hip_decode_attention

    def dec(hq=4, hkv=4, d=16, stride=64, length=20, scale=0.25, window=0, global_tokens=0, ws=one, ws_bytes=1 << 20):
        return decode(one, one, one, one, hq, hkv, d, stride, length, scale, window, global_tokens, ws, ws_bytes, None)

    assert dec(length=0) == 1 and b"cache is empty" in lib.sentinel_hip_last_error()
    assert dec(length=65) == 1 and b"cache length exceeds its capacity" in lib.sentinel_hip_last_error()
    assert dec(hq=6, hkv=4) == 1 and b"divisible by kvHeadCount" in lib.sentinel_hip_last_error()
    assert dec(hq=12, hkv=4) == 2 and b"must be 1, 2, 4 or 8" in lib.sentinel_hip_last_error()
    assert dec(d=12) == 2 and b"multiple of 8" in lib.sentinel_hip_last_error()
    assert dec(global_tokens=-1) == 1 and b"globalTokenCount must be >= 0" in lib.sentinel_hip_last_error()
    assert dec(ws_bytes=8) == 1 and b"workspace" in lib.sentinel_hip_last_error()
    need = lib.sentinel_hip_decode_workspace_bytes
    assert need(4, 16, 20) == 512                             # one chunk of 64 positions, 4 heads, d + 2 floats: 288 B, rounded to 256
    assert need(32, 128, 32768) == 128 * 32 * 130 * 4         # chunks of 256 positions past 8192 (a multiple of 256 already)
    assert need(4, 16, 0) == 0


def test_workspace_sizes(lib):
    ws = lib.sentinel_hip_flash_workspace_bytes
    assert ws(0, -1, 0, 4, 4, 16, 48, 4, 1) == 0          # fp32 arithmetic needs none
    assert ws(1, -1, 1, 32, 8, 128, 4096, 4, 1) == 0      # native 16-bit layout needs none
    nq, nkv = 4 * 32 * 4096 * 128 * 2, 4 * 8 * 4096 * 128 * 2
    assert ws(0, 1, 0, 32, 8, 128, 4096, 4, 0) == 2 * nq + 2 * nkv
    assert ws(0, 1, 0, 32, 8, 128, 4096, 4, 1) == 4 * nq + 4 * nkv


def test_python_mirror_has_no_fallback(monkeypatch):
    import sentinel_amd.flash_attention as fa
    monkeypatch.setattr(fa, "_lib", None)
    monkeypatch.setattr(fa, "_LIB_PATH", "/nonexistent/libsentinel_hip_attn.so")
    with pytest.raises(ImportError, match="no fallback"):
        fa.load_library()
