"""ctypes access to the CPU oracle (oracle/) and, where built, the compiled reference (oracle/_ref).

Test infrastructure only: the shipped package never imports this module.
All tensors are float32 numpy arrays in Sentinel's device layout,
``[(head * head_dim + dim), column]`` with ``stride`` columns per row.
"""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libsentinel_attention_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libsentinel_ref_attention.so")

_fp = ctypes.POINTER(ctypes.c_float)


def _ptr(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def build_oracle(force=False):
    """Compile the oracle with the committed Makefile when it is missing (CPU only, about 3 s)."""
    if force or not os.path.exists(ORACLE_SO):
        subprocess.run(["make", "-C", ORACLE_DIR, "oracle"], check=True, capture_output=True)
    return ORACLE_SO


_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        lib = ctypes.CDLL(build_oracle())
        lib.sentinel_oracle_attention.argtypes = [_fp] * 9 + [ctypes.c_int] * 7 + [ctypes.c_float, ctypes.c_int, ctypes.c_int]
        lib.sentinel_oracle_attention.restype = ctypes.c_int
        lib.sentinel_oracle_attention_sparse.argtypes = lib.sentinel_oracle_attention.argtypes + [ctypes.c_int, ctypes.c_int]
        lib.sentinel_oracle_layer_sparse.argtypes = [_fp] * 12 + [ctypes.c_int] * 5 + [ctypes.c_float] + [ctypes.c_int] * 3
        lib.sentinel_oracle_delta.argtypes = [_fp] * 3 + [ctypes.c_int] * 6
        lib.sentinel_oracle_gemm.argtypes = [_fp, ctypes.c_int, ctypes.c_int, _fp, ctypes.c_int, ctypes.c_int, _fp, ctypes.c_int, ctypes.c_int]
        lib.sentinel_oracle_softmax_columns.argtypes = [_fp, _fp, ctypes.c_int, ctypes.c_int]
        lib.sentinel_oracle_max_threads.restype = ctypes.c_int
        lib.sentinel_oracle_rope_tables.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, _fp, _fp]
        lib.sentinel_oracle_rope_rotate.argtypes = [_fp] + [ctypes.c_int] * 7 + [_fp, _fp, ctypes.c_int, ctypes.c_int]
        lib.sentinel_oracle_layer.argtypes = [_fp] * 12 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int]
        _oracle = lib
    return _oracle


def reference():
    """The reference's own compiled CPU path, or None when oracle/_ref was not built."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        lib = ctypes.CDLL(REF_SO)
        lib.sentinel_ref_attention.argtypes = [_fp] * 9 + [ctypes.c_int] * 8
        lib.sentinel_ref_attention_sparse.argtypes = [_fp] * 9 + [ctypes.c_int] * 10
        lib.sentinel_ref_gemm.argtypes = [_fp, ctypes.c_int, ctypes.c_int, _fp, ctypes.c_int, ctypes.c_int, _fp, ctypes.c_int, ctypes.c_int]
        lib.sentinel_ref_softmax_columns.argtypes = [_fp, _fp, ctypes.c_int, ctypes.c_int]
        lib.sentinel_ref_rope_tables.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, _fp, _fp]
        lib.sentinel_ref_rope_rotate.argtypes = [_fp] + [ctypes.c_int] * 4 + [ctypes.c_float, ctypes.c_int]
        lib.sentinel_ref_layer.argtypes = [_fp] * 12 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int]
        _ref = lib
    return _ref


def _alloc_like(x, fill=np.nan):
    return np.full_like(x, fill)


def oracle_attention(q, k, v, d_out=None, *, q_heads, kv_heads, head_dim, seq_len, pack_count=1, col_start=0,
                     scale=None, causal=True, pack_parallel=False, lib="oracle", per_head=False, window=0, global_tokens=0,
                     prefer_sparse=False):
    """Run forward (+ backward when d_out is given). Returns dict(out, lse[, dq, dk, dv]).

    window / global_tokens: Sentinel's sparse mask on top of the causal one (0, 0 = full causal). With lib="ref",
    prefer_sparse picks the reference's sparse-compute path instead of its dense masked path.

    Untouched columns (outside the pack window) come back as NaN so tests can check they were left alone.
    """
    stride = q.shape[1]
    assert q.shape[0] == q_heads * head_dim and k.shape == v.shape == (kv_heads * head_dim, stride)
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(head_dim))
    out = _alloc_like(q)
    lse = np.full((q_heads, stride), np.nan, dtype=np.float32)
    dq = dk = dv = None
    if d_out is not None:
        dq, dk, dv = _alloc_like(q), _alloc_like(k), _alloc_like(v)
    if lib == "oracle":
        rc = oracle().sentinel_oracle_attention_sparse(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(d_out),
                                                        _ptr(dq), _ptr(dk), _ptr(dv), q_heads, kv_heads, head_dim, stride,
                                                        col_start, seq_len, pack_count, float(scale), int(causal),
                                                        int(pack_parallel), int(window), int(global_tokens))
    elif window > 0 or global_tokens > 0:
        assert causal and abs(float(scale) - 1.0 / np.sqrt(head_dim)) < 1e-7
        rc = reference().sentinel_ref_attention_sparse(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(d_out),
                                                        _ptr(dq), _ptr(dk), _ptr(dv), q_heads, kv_heads, head_dim, stride,
                                                        col_start, seq_len, pack_count, int(window), int(global_tokens),
                                                        int(prefer_sparse))
    else:
        assert causal and abs(float(scale) - 1.0 / np.sqrt(head_dim)) < 1e-7
        rc = reference().sentinel_ref_attention(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(d_out), _ptr(dq),
                                                 _ptr(dk), _ptr(dv), q_heads, kv_heads, head_dim, stride, col_start,
                                                 seq_len, pack_count, int(per_head))
    if rc != 0:
        raise ValueError(f"{lib} attention returned {rc}")
    res = {"out": out, "lse": lse}
    if d_out is not None:
        res.update(dq=dq, dk=dk, dv=dv)
    return res


def oracle_delta(out, d_out, *, q_heads, head_dim, seq_len, pack_count=1, col_start=0):
    stride = out.shape[1]
    delta = np.full((q_heads, stride), np.nan, dtype=np.float32)
    rc = oracle().sentinel_oracle_delta(_ptr(out), _ptr(d_out), _ptr(delta), q_heads, head_dim, stride, col_start, seq_len, pack_count)
    if rc != 0:
        raise ValueError(f"oracle delta returned {rc}")
    return delta


def gemm(a, b, trans_a=False, trans_b=False, lib="oracle"):
    m = a.shape[1] if trans_a else a.shape[0]
    n = b.shape[0] if trans_b else b.shape[1]
    c = np.empty((m, n), dtype=np.float32)
    fn = oracle().sentinel_oracle_gemm if lib == "oracle" else reference().sentinel_ref_gemm
    rc = fn(_ptr(a), a.shape[0], a.shape[1], _ptr(b), b.shape[0], b.shape[1], _ptr(c), int(trans_a), int(trans_b))
    if rc != 0:
        raise ValueError(f"{lib} gemm returned {rc}")
    return c


def softmax_columns(x, lib="oracle"):
    y = np.empty_like(x)
    fn = oracle().sentinel_oracle_softmax_columns if lib == "oracle" else reference().sentinel_ref_softmax_columns
    rc = fn(_ptr(x), _ptr(y), x.shape[0], x.shape[1])
    if rc != 0:
        raise ValueError(f"{lib} softmax returned {rc}")
    return y


def rope_tables(head_dim, positions, base=10000.0, lib="oracle"):
    """cos / sin tables [positions, head_dim // 2] as RotaryEmbedding builds them."""
    cos = np.empty((positions, head_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    fn = oracle().sentinel_oracle_rope_tables if lib == "oracle" else reference().sentinel_ref_rope_tables
    if fn(head_dim, positions, float(base), _ptr(cos), _ptr(sin)) != 0:
        raise ValueError("rope tables: invalid arguments")
    return cos, sin


def rope_rotate(x, heads, head_dim, cos, sin, *, col_start=0, columns=None, position_offset=0, segment_length=0,
                inverse=False):
    """Oracle RoPE on a copy of x ([(head*d + dim), stride] fp32); returns the rotated copy."""
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    columns = y.shape[1] - col_start if columns is None else columns
    rc = oracle().sentinel_oracle_rope_rotate(_ptr(y), heads, head_dim, y.shape[1], col_start, columns, position_offset,
                                              segment_length, _ptr(cos), _ptr(sin), cos.shape[0], int(inverse))
    if rc != 0:
        raise ValueError("rope rotate: invalid arguments")
    return y


def ref_rope_rotate(x, heads, head_dim, positions, base=10000.0, inverse=False):
    """The compiled reference's RotaryEmbedding::rotate(Inverse)InPlace on a copy of x (column = position)."""
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    rc = reference().sentinel_ref_rope_rotate(_ptr(y), heads, head_dim, y.shape[1], positions, float(base), int(inverse))
    if rc != 0:
        raise ValueError("reference rope rotate: invalid arguments")
    return y


def layer(x, wq, wk, wv, wo, d_y=None, *, q_heads, kv_heads, head_dim, rope_base=10000.0, rope_positions=None,
          lib="oracle", window=0, global_tokens=0):
    """The attention layer (projections, RoPE, causal attention, output projection) on one sequence x [E, T].

    Returns dict(y[, d_x, d_wq, d_wk, d_wv, d_wo])."""
    e, t = x.shape
    rope_positions = t if rope_positions is None else rope_positions
    y = np.empty((e, t), dtype=np.float32)
    grads = [None] * 5
    if d_y is not None:
        grads = [np.empty_like(x), np.empty_like(wq), np.empty_like(wk), np.empty_like(wv), np.empty_like(wo)]
    if lib == "oracle":
        rc = oracle().sentinel_oracle_layer_sparse(_ptr(x), _ptr(wq), _ptr(wk), _ptr(wv), _ptr(wo), _ptr(d_y), _ptr(y),
                                                    *[_ptr(a) for a in grads], e, q_heads, kv_heads, head_dim, t,
                                                    float(rope_base), rope_positions, int(window), int(global_tokens))
    else:
        assert window == 0 and global_tokens == 0
        rc = reference().sentinel_ref_layer(_ptr(x), _ptr(wq), _ptr(wk), _ptr(wv), _ptr(wo), _ptr(d_y), _ptr(y),
                                            *[_ptr(a) for a in grads], e, q_heads, kv_heads, head_dim, t, float(rope_base),
                                            rope_positions)
    if rc != 0:
        raise ValueError(f"{lib} layer returned {rc}")
    res = {"y": y}
    if d_y is not None:
        res.update(d_x=grads[0], d_wq=grads[1], d_wk=grads[2], d_wv=grads[3], d_wo=grads[4])
    return res
