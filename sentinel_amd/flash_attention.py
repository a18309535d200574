"""Host-side mirror of Sentinel's ``CudaFlashAttention`` over the HIP C ABI.

``HipFlashAttention`` keeps the names, argument order and error behaviour of
``class CudaFlashAttention`` (sentinel/NeuralNet/Cuda/CudaFlashAttention.hpp:12-41): matrices are
``(head_count * head_dimension) x columns`` fp32 device tensors, the column window / pack arguments mean
the same, shape errors raise ``ValueError`` (std::invalid_argument there) and device / launch errors raise
``RuntimeError``.  torch is used only to own device memory and to name the stream; all arithmetic runs in
``libsentinel_hip_attn.so`` and nothing here falls back to another implementation: a missing library is an
error.

``flash_attention_forward`` / ``flash_attention_backward`` are the native entry points on contiguous
``[B, H, T, d]`` bf16 / fp16 (or fp32) tensors.
"""
import ctypes
import math
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# SENTINEL_HIP_ATTN_LIB points at another build of the same library (e.g. an experimental kernel variant)
_LIB_PATH = os.environ.get("SENTINEL_HIP_ATTN_LIB") or os.path.join(_HERE, "lib", "libsentinel_hip_attn.so")

OK, INVALID_ARGUMENT, UNSUPPORTED, RUNTIME = 0, 1, 2, 3
F32, BF16, F16 = 0, 1, 2
COMPUTE_AUTO = -1
LAYOUT_COLUMNS, LAYOUT_BHTD = 0, 1
WORKSPACE_KEEP, WORKSPACE_REUSE = 0x100, 0x200  # OR-ed into the layout argument

_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_COMPUTE_CODE = {None: COMPUTE_AUTO, "auto": COMPUTE_AUTO, "fp32": F32, "bf16": BF16, "fp16": F16,
                 torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}

_lib = None


def library_path():
    return _LIB_PATH


def load_library():
    """Load the built HIP library; raises if it has not been built (python -m sentinel_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(f"{_LIB_PATH} is missing: build it with `python -m sentinel_amd.build` "
                          "(there is no fallback implementation)")
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i, f, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    lib.sentinel_hip_flash_fwd.argtypes = [vp] * 5 + [i] * 10 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_fwd.restype = i
    lib.sentinel_hip_flash_bwd.argtypes = [vp] * 10 + [i] * 10 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_bwd.restype = i
    lib.sentinel_hip_flash_fwd_rope.argtypes = [vp] * 7 + [i] * 12 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_fwd_rope.restype = i
    lib.sentinel_hip_flash_bwd_rope.argtypes = [vp] * 12 + [i] * 12 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_bwd_rope.restype = i
    lib.sentinel_hip_flash_fwd_sparse.argtypes = [vp] * 7 + [i] * 14 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_fwd_sparse.restype = i
    lib.sentinel_hip_flash_bwd_sparse.argtypes = [vp] * 12 + [i] * 14 + [f, i, vp, sz, vp]
    lib.sentinel_hip_flash_bwd_sparse.restype = i
    lib.sentinel_hip_rope_rotate.argtypes = [vp] + [i] * 7 + [vp, vp, i, i, vp]
    lib.sentinel_hip_rope_rotate.restype = i
    lib.sentinel_hip_cast_to_16bit.argtypes = [vp, vp, sz, i, vp]
    lib.sentinel_hip_cast_to_16bit.restype = i
    ll = ctypes.c_longlong
    lib.sentinel_hip_dense_softmax_fwd.argtypes = [vp, i, ll] + [i] * 6 + [f, vp]
    lib.sentinel_hip_dense_softmax_fwd.restype = i
    lib.sentinel_hip_dense_softmax_bwd.argtypes = [vp, ll, vp, ll] + [i] * 7 + [f, vp]
    lib.sentinel_hip_dense_softmax_bwd.restype = i
    lib.sentinel_hip_decode_workspace_bytes.argtypes = [i] * 3
    lib.sentinel_hip_decode_workspace_bytes.restype = sz
    lib.sentinel_hip_decode_attention.argtypes = [vp] * 4 + [i] * 5 + [f, i, i, vp, sz, vp]
    lib.sentinel_hip_decode_attention.restype = i
    lib.sentinel_hip_decode_attention_static.argtypes = [vp] * 4 + [i] * 5 + [f, i, i, vp]
    lib.sentinel_hip_decode_attention_static.restype = i
    lib.sentinel_hip_flash_workspace_bytes.argtypes = [i] * 9
    lib.sentinel_hip_flash_workspace_bytes.restype = sz
    lib.sentinel_hip_flash_max_head_dim.restype = i
    lib.sentinel_hip_device_available.restype = i
    lib.sentinel_hip_strerror.argtypes = [i]
    lib.sentinel_hip_strerror.restype = ctypes.c_char_p
    lib.sentinel_hip_last_error.restype = ctypes.c_char_p
    lib.sentinel_hip_flash_set_timing.argtypes = [i]
    lib.sentinel_hip_flash_set_timing.restype = i
    lib.sentinel_hip_flash_collect_timings.argtypes = [ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(f),
                                                       ctypes.POINTER(i), i]
    lib.sentinel_hip_flash_collect_timings.restype = i
    _lib = lib
    return lib


def set_kernel_timing(enabled):
    """Bracket every kernel launch with hipEvents (diagnostics; not for captured graphs). Returns the old setting."""
    return bool(load_library().sentinel_hip_flash_set_timing(int(bool(enabled))))


def collect_kernel_timings(capacity=32):
    """{kernel name: (total milliseconds, launches)} since the previous collect; waits for the recorded events."""
    lib = load_library()
    names = (ctypes.c_char_p * capacity)()
    total = (ctypes.c_float * capacity)()
    launches = (ctypes.c_int * capacity)()
    count = lib.sentinel_hip_flash_collect_timings(names, total, launches, capacity)
    return {names[j].decode(): (float(total[j]), int(launches[j])) for j in range(count)}


def _check(code):
    if code == OK:
        return
    lib = load_library()
    detail = lib.sentinel_hip_last_error().decode() or lib.sentinel_hip_strerror(code).decode()
    if code in (INVALID_ARGUMENT, UNSUPPORTED):
        raise ValueError(detail)
    raise RuntimeError(detail)


def _stream_handle(stream):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _ensure_size(t, rows, cols, like):
    """CudaMatrix::ensureSize for an optional output tensor: a tensor of another shape is replaced, one of the right
    shape must be a contiguous fp32 matrix on the inputs' device (its raw pointer crosses the C ABI)."""
    if t is None or tuple(t.shape) != (rows, cols):
        return torch.empty((rows, cols), dtype=torch.float32, device=like.device)
    _require(t, (rows, cols), torch.float32, like.device, "output matrix")
    return t


def _require(t, shape, dtype, device, what):
    """Every tensor whose pointer is handed to the library is checked here: the C ABI sees addresses only."""
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{what}: expected a tensor")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{what}: shape {tuple(t.shape)} where {tuple(shape)} is expected")
    if t.dtype != dtype:
        raise ValueError(f"{what}: dtype {t.dtype} where {dtype} is expected")
    if not t.is_contiguous():
        raise ValueError(f"{what}: must be contiguous")
    if t.device != device:
        raise ValueError(f"{what}: on {t.device}, the inputs are on {device}")


def _on_stream(stream, *temporaries):
    """Temporaries come from torch's caching allocator, which hands a freed block to later work on the CURRENT stream;
    when the kernels run on another stream, tell the allocator so."""
    if stream is None:
        return
    for t in temporaries:
        if t is not None and stream != torch.cuda.current_stream(t.device):
            t.record_stream(stream)


def _workspace(lib, io, compute, layout, hq, hkv, d, t, packs, backward, device, workspace):
    need = lib.sentinel_hip_flash_workspace_bytes(io, compute, layout, hq, hkv, d, t, packs, int(backward))
    if need == 0:
        return None, 0, None
    if workspace is not None:
        if not workspace.is_contiguous() or workspace.device != device:
            raise ValueError("workspace must be a contiguous tensor on the inputs' device")
        if workspace.numel() * workspace.element_size() >= need:
            return workspace, workspace.numel() * workspace.element_size(), None
    own = torch.empty(need, dtype=torch.uint8, device=device)
    return own, need, own


def _rope_args(rope, head_dimension):
    cos, sin = rope[0], rope[1]
    offset = int(rope[2]) if len(rope) > 2 else 0
    for t in (cos, sin):
        if t is None or t.dim() != 2 or t.dtype != torch.float32 or not t.is_contiguous() or not t.is_cuda:
            raise ValueError("rope tables must be contiguous fp32 device matrices [positions, head_dim / 2]")
    if cos.shape != sin.shape or cos.shape[1] * 2 != head_dimension:
        raise ValueError("rope tables must be [positions, head_dim / 2]")
    return cos, sin, offset


class HipOps:
    """The rotary-embedding entry points of Sentinel's CudaOps on MI355X (Cuda/CudaOps.hpp:155-159) and the masked
    column softmax of the layer's dense attention path (Cuda/CudaOps.hpp:144-153)."""

    @staticmethod
    def _score_batch(scores, what):
        if not isinstance(scores, torch.Tensor) or scores.dim() not in (2, 3) or scores.numel() == 0:
            raise ValueError(f"{what} expects a [keys, queries] matrix or a [batch, keys, queries] stack")
        _require(scores, None, torch.float32, scores.device, what)
        if not scores.is_cuda:
            raise ValueError(f"{what} must be on the GPU")
        batch = 1 if scores.dim() == 2 else int(scores.shape[0])
        return batch, int(scores.shape[-2]), int(scores.shape[-1])

    @staticmethod
    def masked_softmax_in_place(scores, scale, window_size=0, global_token_count=0, query_position_start=0,
                                segment_length=0, *, stream=None):
        """CudaOps::scaleInPlace + applySparseAttentionMaskInPlace + softmaxInto over keys x queries score matrices
        (rows are keys), in place, for a whole stack at once."""
        batch, keys, queries = HipOps._score_batch(scores, "HipOps::maskedSoftmaxInPlace scores")
        _check(load_library().sentinel_hip_dense_softmax_fwd(_ptr(scores), batch, keys * queries, keys, queries,
                                                             int(query_position_start), int(window_size),
                                                             int(global_token_count), int(segment_length), float(scale),
                                                             _stream_handle(stream)))
        return scores

    @staticmethod
    def masked_softmax_backward_in_place(probabilities, probability_gradient, scale, window_size=0, global_token_count=0,
                                         query_position_start=0, segment_length=0, *, stream=None):
        """CudaOps::softmaxBackwardInto + zeroForbiddenScoreGradientsInPlace + scaleInPlace: the score gradient is
        written over probability_gradient."""
        batch, keys, queries = HipOps._score_batch(probabilities, "HipOps::maskedSoftmaxBackwardInPlace probabilities")
        _require(probability_gradient, probabilities.shape, torch.float32, probabilities.device,
                 "HipOps::maskedSoftmaxBackwardInPlace gradient")
        _check(load_library().sentinel_hip_dense_softmax_bwd(_ptr(probabilities), keys * queries, _ptr(probability_gradient),
                                                             keys * queries, batch, keys, queries, int(query_position_start),
                                                             int(window_size), int(global_token_count), int(segment_length),
                                                             float(scale), _stream_handle(stream)))
        return probability_gradient

    @staticmethod
    def rotary_rotate_in_place(tensor, head_count, head_dimension, pair_count, cos_table, sin_table, position_offset=0,
                               segment_length=0, *, inverse=False, stream=None):
        """CudaOps::rotaryRotateInPlace: rotates the fp32 matrix [(head*d + dim), columns] in place."""
        name = "HipOps::rotaryRotateInverseInPlace" if inverse else "HipOps::rotaryRotateInPlace"
        if tensor is None or tensor.numel() == 0:
            raise ValueError(f"{name} empty tensor")
        if head_count <= 0 or head_dimension <= 0 or pair_count <= 0 or pair_count * 2 != head_dimension:
            raise ValueError(f"{name} invalid rope dims")
        if tensor.dim() != 2 or tensor.dtype != torch.float32 or not tensor.is_contiguous():
            raise ValueError(f"{name} expects a contiguous fp32 matrix")
        if tensor.shape[0] != head_count * head_dimension:
            raise ValueError(f"{name} embedding dim mismatch")
        if cos_table is None or sin_table is None or cos_table.numel() == 0 or sin_table.numel() == 0:
            raise ValueError(f"{name} empty tables")
        cos, sin, _ = _rope_args((cos_table, sin_table), head_dimension)
        cols = int(tensor.shape[1])
        _check(load_library().sentinel_hip_rope_rotate(_ptr(tensor), head_count, head_dimension, cols, 0, cols,
                                                       int(position_offset), int(segment_length), _ptr(cos), _ptr(sin),
                                                       int(cos.shape[0]), int(bool(inverse)), _stream_handle(stream)))
        return tensor

    @staticmethod
    def rotary_rotate_inverse_in_place(tensor, head_count, head_dimension, pair_count, cos_table, sin_table,
                                       position_offset=0, segment_length=0, *, stream=None):
        """CudaOps::rotaryRotateInverseInPlace."""
        return HipOps.rotary_rotate_in_place(tensor, head_count, head_dimension, pair_count, cos_table, sin_table,
                                             position_offset, segment_length, inverse=True, stream=stream)


class HipAmp:
    """The operand cast of the layer's mixed-precision projection GEMMs (class CudaAmp, Cuda/CudaAmp.hpp:54-190)."""

    @staticmethod
    def cast_to_half(source, dtype=torch.float16, out=None, *, stream=None):
        """CudaAmp::castFloatBufferToHalf (Cuda/CudaAmp.cu:523-527): `source` (contiguous fp32) rounded to nearest even
        into a float16 (the reference's type) or bfloat16 tensor of the same shape."""
        name = "HipAmp::castToHalf"
        if source is None or source.dtype != torch.float32 or not source.is_contiguous() or not source.is_cuda:
            raise ValueError(f"{name} expects a contiguous fp32 device tensor")
        if dtype not in (torch.float16, torch.bfloat16):
            raise ValueError(f"{name} dtype must be torch.float16 or torch.bfloat16")
        if out is None:
            out = torch.empty(source.shape, dtype=dtype, device=source.device)
        _require(out, source.shape, dtype, source.device, f"{name} destination")
        _check(load_library().sentinel_hip_cast_to_16bit(_ptr(source), _ptr(out), source.numel(), _DTYPE_CODE[dtype],
                                                         _stream_handle(stream)))
        return out


class HipFlashAttention:
    """Static interface of Sentinel's CudaFlashAttention on MI355X."""

    query_tile_size = 128
    key_tile_size = 64
    max_head_dimension = 128

    @staticmethod
    def forward_multi_head(query, key, value, out, log_sum_exp, head_count, head_dimension, scale, causal=True,
                           column_start=0, column_count=0, pack_count=1, *, kv_head_count=None, compute=None,
                           workspace=None, stream=None, rope=None, window_size=0, global_token_count=0,
                           keep_for_backward=False):
        """CudaFlashAttention::forwardMultiHead. Returns (out, log_sum_exp) (re-allocated if their shape was wrong).

        keep_for_backward (16-bit arithmetic only): `workspace` must be a tensor sized for the backward call; the
        converted operands stay in it, and backward_multi_head(..., workspace=the same tensor,
        reuse_forward_workspace=True) converts d_out only (as the CUDA layer keeps flashLogSumExp between the calls).

        window_size / global_token_count: the attention layer's sparse mask (CausalSelfAttention::allowsKey), which
        the CUDA layer can only run on its dense path.

        rope = (cos_table, sin_table[, position_offset]): query and key are given unrotated and rotated on the way in
        (the two rotaryRotateInPlace calls of CudaCausalSelfAttention.cu:206-207 fused into this call)."""
        lib = load_library()
        HipFlashAttention._validate(query, key, value, head_count, head_dimension, kv_head_count, "forwardMultiHead")
        kv_heads = head_count if kv_head_count in (None, 0) else kv_head_count
        rows, cols = query.shape
        out = _ensure_size(out, rows, cols, query)
        log_sum_exp = _ensure_size(log_sum_exp, head_count, cols, query)
        comp = _COMPUTE_CODE[compute]
        seq = column_count if column_count > 0 else cols - column_start
        ws, ws_bytes, ws_own = _workspace(lib, F32, comp, LAYOUT_COLUMNS, head_count, kv_heads, head_dimension, max(seq, 1),
                                          max(pack_count, 1), bool(keep_for_backward), query.device, workspace)
        if keep_for_backward and ws_own is not None:
            raise ValueError("HipFlashAttention::forwardMultiHead keep_for_backward needs a caller-owned workspace of "
                             f"at least {ws_bytes} bytes")
        _on_stream(stream, ws_own)
        tail = (F32, comp, LAYOUT_COLUMNS | (WORKSPACE_KEEP if keep_for_backward else 0), head_count, kv_heads, head_dimension, cols, column_start, column_count,
                pack_count, float(scale), int(bool(causal)), _ptr(ws), ws_bytes, _stream_handle(stream))
        if window_size > 0 or global_token_count != 0:
            cos, sin, offset = _rope_args(rope, head_dimension) if rope is not None else (None, None, 0)
            _check(lib.sentinel_hip_flash_fwd_sparse(_ptr(query), _ptr(key), _ptr(value), _ptr(out), _ptr(log_sum_exp),
                                                     _ptr(cos), _ptr(sin), int(cos.shape[0]) if cos is not None else 0,
                                                     offset, int(window_size), int(global_token_count), *tail))
        elif rope is None:
            _check(lib.sentinel_hip_flash_fwd(_ptr(query), _ptr(key), _ptr(value), _ptr(out), _ptr(log_sum_exp), *tail))
        else:
            cos, sin, offset = _rope_args(rope, head_dimension)
            _check(lib.sentinel_hip_flash_fwd_rope(_ptr(query), _ptr(key), _ptr(value), _ptr(out), _ptr(log_sum_exp),
                                                   _ptr(cos), _ptr(sin), int(cos.shape[0]), offset, *tail))
        return out, log_sum_exp

    @staticmethod
    def forward(query, key, value, out, log_sum_exp, scale, causal=True, **kw):
        """CudaFlashAttention::forward: single head, head_dimension = rows."""
        return HipFlashAttention.forward_multi_head(query, key, value, out, log_sum_exp, 1, int(query.shape[0]), scale,
                                                    causal, 0, int(query.shape[1]), 1, **kw)

    @staticmethod
    def backward_multi_head(query, key, value, out, log_sum_exp, out_gradient, query_gradient, key_gradient,
                            value_gradient, delta_workspace, head_count, head_dimension, scale, causal=True,
                            column_start=0, column_count=0, pack_count=1, *, kv_head_count=None, compute=None,
                            workspace=None, stream=None, rope=None, window_size=0, global_token_count=0,
                            reuse_forward_workspace=False):
        """CudaFlashAttention::backwardMultiHead. Returns (dQ, dK, dV, delta).

        reuse_forward_workspace: `workspace` is the tensor a forward_multi_head(..., keep_for_backward=True) call with
        the same tensors and arguments filled; query / key / value / out are then not converted again.

        rope as in forward_multi_head: query / key unrotated, dQ / dK come back rotated back
        (rotaryRotateInverseInPlace of CudaCausalSelfAttention.cu:508-509 fused into this call)."""
        lib = load_library()
        HipFlashAttention._validate(query, key, value, head_count, head_dimension, kv_head_count, "backwardMultiHead")
        kv_heads = head_count if kv_head_count in (None, 0) else kv_head_count
        rows, cols = query.shape
        if tuple(out.shape) != (rows, cols):
            raise ValueError("HipFlashAttention::backwardMultiHead out shape mismatch")
        if tuple(out_gradient.shape) != (rows, cols):
            raise ValueError("HipFlashAttention::backwardMultiHead outGradient shape mismatch")
        if tuple(log_sum_exp.shape) != (head_count, cols):
            raise ValueError("HipFlashAttention::backwardMultiHead logSumExp shape mismatch")
        for t, what in ((out, "out"), (out_gradient, "outGradient"), (log_sum_exp, "logSumExp")):
            _require(t, None, torch.float32, query.device, "HipFlashAttention::backwardMultiHead " + what)
        seq = column_count if column_count > 0 else cols - column_start
        packs = max(pack_count, 1)
        query_gradient = _ensure_size(query_gradient, rows, cols, query)
        key_gradient = _ensure_size(key_gradient, key.shape[0], cols, query)
        value_gradient = _ensure_size(value_gradient, value.shape[0], cols, query)
        delta_workspace = _ensure_size(delta_workspace, head_count, packs * max(seq, 1), query)
        comp = _COMPUTE_CODE[compute]
        ws, ws_bytes, ws_own = _workspace(lib, F32, comp, LAYOUT_COLUMNS, head_count, kv_heads, head_dimension,
                                          max(seq, 1), packs, True, query.device, workspace)
        if reuse_forward_workspace and ws_own is not None:
            raise ValueError("HipFlashAttention::backwardMultiHead reuse_forward_workspace needs the forward call's workspace")
        _on_stream(stream, ws_own)
        head = (_ptr(query), _ptr(key), _ptr(value), _ptr(out), _ptr(log_sum_exp), _ptr(out_gradient), _ptr(query_gradient),
                _ptr(key_gradient), _ptr(value_gradient), _ptr(delta_workspace))
        tail = (F32, comp, LAYOUT_COLUMNS | (WORKSPACE_REUSE if reuse_forward_workspace else 0), head_count, kv_heads,
                head_dimension, cols, column_start, column_count,
                pack_count, float(scale), int(bool(causal)), _ptr(ws), ws_bytes, _stream_handle(stream))
        if window_size > 0 or global_token_count != 0:
            cos, sin, offset = _rope_args(rope, head_dimension) if rope is not None else (None, None, 0)
            _check(lib.sentinel_hip_flash_bwd_sparse(*head, _ptr(cos), _ptr(sin), int(cos.shape[0]) if cos is not None else 0,
                                                     offset, int(window_size), int(global_token_count), *tail))
        elif rope is None:
            _check(lib.sentinel_hip_flash_bwd(*head, *tail))
        else:
            cos, sin, offset = _rope_args(rope, head_dimension)
            _check(lib.sentinel_hip_flash_bwd_rope(*head, _ptr(cos), _ptr(sin), int(cos.shape[0]), offset, *tail))
        return query_gradient, key_gradient, value_gradient, delta_workspace

    @staticmethod
    def backward(query, key, value, out, log_sum_exp, out_gradient, query_gradient, key_gradient, value_gradient, scale,
                 causal=True, **kw):
        """CudaFlashAttention::backward: single head."""
        return HipFlashAttention.backward_multi_head(query, key, value, out, log_sum_exp, out_gradient, query_gradient,
                                                     key_gradient, value_gradient, None, 1, int(query.shape[0]), scale,
                                                     causal, 0, int(query.shape[1]), 1, **kw)[:3]

    @staticmethod
    def _validate(query, key, value, head_count, head_dimension, kv_head_count, op):
        # validateMultiHeadShape (CudaFlashAttention.cu:1458-1471), with the K/V rows rule widened to grouped heads
        name = f"HipFlashAttention::{op}"
        for t in (query, key, value):
            if t is None or t.dim() != 2 or t.numel() == 0:
                raise ValueError(f"{name} empty input")
            if t.dtype != torch.float32 or not t.is_contiguous():
                raise ValueError(f"{name} expects contiguous fp32 matrices")
        if head_count <= 0 or head_dimension <= 0:
            raise ValueError(f"{name} invalid head geometry")
        if head_dimension > HipFlashAttention.max_head_dimension:
            raise ValueError(f"{name} headDim exceeds maxHeadDimension")
        kv_heads = head_count if kv_head_count in (None, 0) else kv_head_count
        if kv_heads <= 0 or head_count % kv_heads != 0:
            raise ValueError(f"{name} headCount must be divisible by kvHeadCount")
        if query.shape[0] != head_count * head_dimension:
            raise ValueError(f"{name} query rows mismatch headCount*headDim")
        if key.shape[0] != kv_heads * head_dimension or value.shape[0] != key.shape[0]:
            raise ValueError(f"{name} key/value rows mismatch")
        if query.shape[1] != key.shape[1] or query.shape[1] != value.shape[1]:
            raise ValueError(f"{name} sequenceLength mismatch")
        if not load_library().sentinel_hip_device_available():
            raise RuntimeError(f"{name} no HIP device")


def decode_attention(query, key_cache, value_cache, length, head_count, head_dimension, *, kv_head_count=None, scale=None,
                     window_size=0, global_token_count=0, out=None, workspace=None, stream=None):
    """Attention of the newest token against the first `length` positions of the K/V cache
    (CudaCausalSelfAttention::attendCachedQuery without the output projection).

    query: fp32 [head_count*head_dimension, 1]; caches: fp32 [kv_heads*head_dimension, capacity]. Returns out [rows, 1]."""
    lib = load_library()
    kv_heads = head_count if kv_head_count in (None, 0) else kv_head_count
    for t in (query, key_cache, value_cache):
        if t is None or t.dim() != 2 or t.numel() == 0:
            raise ValueError("decode_attention empty input")
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("decode_attention expects contiguous fp32 matrices")
    if query.shape != (head_count * head_dimension, 1):
        raise ValueError("decode_attention expects a single token column")
    if key_cache.shape[0] != kv_heads * head_dimension or value_cache.shape != key_cache.shape:
        raise ValueError("decode_attention key/value rows mismatch")
    scale = 1.0 / math.sqrt(head_dimension) if scale is None else float(scale)
    out = _ensure_size(out, head_count * head_dimension, 1, query)
    need = lib.sentinel_hip_decode_workspace_bytes(head_count, head_dimension, max(int(length), 1))
    if workspace is not None and (not workspace.is_contiguous() or workspace.device != query.device):
        raise ValueError("decode_attention workspace must be a contiguous tensor on the inputs' device")
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=query.device)
        _on_stream(stream, workspace)
    _check(lib.sentinel_hip_decode_attention(_ptr(query), _ptr(key_cache), _ptr(value_cache), _ptr(out), head_count, kv_heads,
                                             head_dimension, int(key_cache.shape[1]), int(length), scale, int(window_size),
                                             int(global_token_count), _ptr(workspace),
                                             workspace.numel() * workspace.element_size(), _stream_handle(stream)))
    return out


def _bhtd_geometry(q, k, v):
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape:
        raise ValueError("flash_attention expects [B, H, T, d] tensors")
    b, hq, t, d = q.shape
    if k.shape[0] != b or k.shape[2] != t or k.shape[3] != d:
        raise ValueError("flash_attention q / k shape mismatch")
    for x in (q, k, v):
        if not x.is_contiguous() or x.dtype != q.dtype:
            raise ValueError("flash_attention expects contiguous tensors of one dtype")
    if q.dtype not in _DTYPE_CODE:
        raise ValueError(f"flash_attention unsupported dtype {q.dtype}")
    return b, hq, k.shape[1], t, d


def flash_attention_forward(q, k, v, scale=None, causal=True, out=None, lse=None, stream=None, window_size=0,
                            global_token_count=0):
    """Native forward on [B,H,T,d] tensors (k, v may have fewer heads). Returns (out, lse[B,H,T] fp32)."""
    lib = load_library()
    b, hq, hkv, t, d = _bhtd_geometry(q, k, v)
    scale = 1.0 / math.sqrt(d) if scale is None else float(scale)
    out = torch.empty_like(q) if out is None else out
    lse = torch.empty((b, hq, t), dtype=torch.float32, device=q.device) if lse is None else lse
    _require(out, q.shape, q.dtype, q.device, "flash_attention_forward out")
    _require(lse, (b, hq, t), torch.float32, q.device, "flash_attention_forward lse")
    code = _DTYPE_CODE[q.dtype]
    if window_size > 0 or global_token_count != 0:
        _check(lib.sentinel_hip_flash_fwd_sparse(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), None, None, 0, 0,
                                                 int(window_size), int(global_token_count), code, COMPUTE_AUTO, LAYOUT_BHTD,
                                                 hq, hkv, d, 0, 0, t, b, scale, int(bool(causal)), None, 0,
                                                 _stream_handle(stream)))
        return out, lse
    _check(lib.sentinel_hip_flash_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), code, COMPUTE_AUTO, LAYOUT_BHTD, hq,
                                      hkv, d, 0, 0, t, b, scale, int(bool(causal)), None, 0, _stream_handle(stream)))
    return out, lse


def flash_attention_backward(q, k, v, out, lse, d_out, scale=None, causal=True, dq=None, dk=None, dv=None, delta=None,
                             stream=None, window_size=0, global_token_count=0):
    """Native backward on [B,H,T,d] tensors. Returns (dq, dk, dv)."""
    lib = load_library()
    b, hq, hkv, t, d = _bhtd_geometry(q, k, v)
    scale = 1.0 / math.sqrt(d) if scale is None else float(scale)
    dq = torch.empty_like(q) if dq is None else dq
    dk = torch.empty_like(k) if dk is None else dk
    dv = torch.empty_like(v) if dv is None else dv
    own_delta = delta is None
    delta = torch.empty((hq, b * t), dtype=torch.float32, device=q.device) if own_delta else delta
    for x, like, what in ((out, q, "out"), (d_out, q, "d_out"), (dq, q, "dq"), (dk, k, "dk"), (dv, v, "dv")):
        _require(x, like.shape, q.dtype, q.device, "flash_attention_backward " + what)
    _require(lse, (b, hq, t), torch.float32, q.device, "flash_attention_backward lse")
    _require(delta, None, torch.float32, q.device, "flash_attention_backward delta")
    if delta.numel() < hq * b * t:
        raise ValueError(f"flash_attention_backward delta: {delta.numel()} floats where {hq * b * t} are needed")
    if own_delta:
        _on_stream(stream, delta)
    code = _DTYPE_CODE[q.dtype]
    head = (_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(d_out), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(delta))
    tail = (code, COMPUTE_AUTO, LAYOUT_BHTD, hq, hkv, d, 0, 0, t, b, scale, int(bool(causal)), None, 0, _stream_handle(stream))
    if window_size > 0 or global_token_count != 0:
        _check(lib.sentinel_hip_flash_bwd_sparse(*head, None, None, 0, 0, int(window_size), int(global_token_count), *tail))
    else:
        _check(lib.sentinel_hip_flash_bwd(*head, *tail))
    return dq, dk, dv
