"""GPU parity of the dense attention path's fused softmax entry points (sentinel_hip_dense_softmax_fwd / _bwd) against
a float64 restatement of the reference's separate steps: scale, mask with -1e9 (CudaOps::applySparseAttentionMaskInPlace,
Cuda/CudaOps.cu:249-286), softmax down the key rows (:288-309), softmax backward, zero forbidden, scale (:311-344).
The layer that uses them is checked against the oracle layer in tests/cpp/test_layer.cpp."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _allowed(keys, queries, start, window, global_tokens, segment):
    k = np.arange(keys)[:, None]
    q = np.arange(queries)[None, :]
    if segment > 0:
        same = (k // segment) == (q // segment)
        kp, qp = k % segment, q % segment
    else:
        same = np.ones((keys, queries), bool)
        kp, qp = k, q + start
    seen = (kp < global_tokens) | (window <= 0) | (kp >= qp - window + 1)
    return same & (kp <= qp) & seen


CASES = [
    # batch, keys, queries, start, window, global, segment, scale
    (1, 48, 48, 0, 0, 0, 0, 0.25),
    (5, 70, 70, 0, 17, 3, 0, 0.125),
    (3, 96, 96, 0, 0, 0, 32, 0.3),        # three packs in one matrix: block-diagonal mask
    (2, 96, 96, 0, 7, 2, 48, 0.3),
    (4, 300, 1, 299, 0, 0, 0, 0.09),      # one query against a cache (queryPositionStart)
    (2, 130, 65, 65, 40, 5, 0, 0.2),
    (1, 1, 1, 0, 0, 0, 0, 1.0),
    (7, 257, 257, 0, 64, 0, 0, 0.088),
]


@pytest.mark.parametrize("case", CASES)
def test_masked_softmax_and_backward_match_float64(case):
    import torch
    from sentinel_amd import HipOps
    batch, keys, queries, start, window, global_tokens, segment, scale = case
    rng = np.random.default_rng(keys * 131 + queries)
    s = rng.standard_normal((batch, keys, queries)).astype(np.float32) * 3
    dp = rng.standard_normal((batch, keys, queries)).astype(np.float32)
    allowed = _allowed(keys, queries, start, window, global_tokens, segment)
    masked = np.where(allowed, s.astype(np.float64) * np.float64(np.float32(scale)), -1.0e9)
    e = np.exp(masked - masked.max(axis=1, keepdims=True))
    p = e / e.sum(axis=1, keepdims=True)
    ds = np.where(allowed, p * (dp - (dp * p).sum(axis=1, keepdims=True)), 0.0) * np.float64(np.float32(scale))

    sd = torch.from_numpy(s).cuda()
    got_p = HipOps.masked_softmax_in_place(sd, scale, window, global_tokens, start, segment)
    assert got_p.data_ptr() == sd.data_ptr()
    torch.cuda.synchronize()
    got = got_p.cpu().numpy()
    assert np.abs(got - p).max() <= 2e-6
    assert (got[:, ~allowed] == 0).all()          # forbidden pairs underflow to exactly zero, as with the -1e9 fill
    np.testing.assert_allclose(got.sum(axis=1), 1.0, atol=2e-6)

    gd = torch.from_numpy(dp).cuda()
    HipOps.masked_softmax_backward_in_place(got_p, gd, scale, window, global_tokens, start, segment)
    torch.cuda.synchronize()
    got_ds = gd.cpu().numpy()
    assert np.abs(got_ds - ds).max() <= 1e-5 * max(1.0, np.abs(ds).max())
    assert (got_ds[:, ~allowed] == 0).all()


def test_two_dimensional_matrix_and_argument_errors():
    import torch
    from sentinel_amd import HipOps
    s = torch.randn(33, 33, device="cuda")
    want = torch.softmax(torch.where(torch.tril(torch.ones(33, 33, device="cuda")).T.bool(), s * 0.5, torch.tensor(-1e9, device="cuda")), dim=0)
    got = HipOps.masked_softmax_in_place(s.clone(), 0.5)
    assert torch.allclose(got, want, atol=2e-6)
    with pytest.raises(ValueError):
        HipOps.masked_softmax_in_place(s.double(), 0.5)
    with pytest.raises(ValueError):
        HipOps.masked_softmax_in_place(s.t(), 0.5)
    with pytest.raises(ValueError):
        HipOps.masked_softmax_in_place(s, 0.5, global_token_count=-1)
    with pytest.raises(ValueError):
        HipOps.masked_softmax_backward_in_place(s, s[:5], 0.5)
