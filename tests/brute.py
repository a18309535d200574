"""Independent float64 references for causal (grouped-query) attention.

`attention_autograd` builds the forward from torch primitives in float64 and lets autograd produce the
gradients, so it shares no formula with the oracle or the kernels.  Layout helpers convert between
Sentinel's device layout ``[(head*d + dim), stride]`` and ``[B, H, T, d]``.
"""
import numpy as np
import torch


def ref_to_bhtd(x, heads, d, t, packs=1, col0=0):
    """[(h*d+c), stride] -> [B, H, T, d]"""
    w = x[:, col0:col0 + packs * t].reshape(heads, d, packs, t)
    return np.ascontiguousarray(w.transpose(2, 0, 3, 1))


def bhtd_to_ref(y, stride=None, col0=0, fill=np.nan):
    b, h, t, d = y.shape
    stride = stride or (col0 + b * t)
    out = np.full((h * d, stride), fill, dtype=y.dtype)
    out[:, col0:col0 + b * t] = y.transpose(1, 3, 0, 2).reshape(h * d, b * t)
    return out


def bht_to_ref(y, stride=None, col0=0, fill=np.nan):
    b, h, t = y.shape
    stride = stride or (col0 + b * t)
    out = np.full((h, stride), fill, dtype=y.dtype)
    out[:, col0:col0 + b * t] = y.transpose(1, 0, 2).reshape(h, b * t)
    return out


def ref_to_bht(x, heads, t, packs=1, col0=0):
    return np.ascontiguousarray(x[:, col0:col0 + packs * t].reshape(heads, packs, t).transpose(1, 0, 2))


def attention_autograd(q, k, v, g=None, scale=None, causal=True, dtype=torch.float64):
    """q, g: [B,Hq,T,d]; k, v: [B,Hkv,T,d] (numpy or torch). Returns dict of numpy float64 arrays in [B,H,T,(d)]."""
    q, k, v = (torch.as_tensor(np.asarray(x)).to(dtype).clone().requires_grad_(True) for x in (q, k, v))
    b, hq, t, d = q.shape
    group = hq // k.shape[1]
    scale = (1.0 / np.sqrt(d)) if scale is None else float(scale)
    kx = k.repeat_interleave(group, dim=1)
    vx = v.repeat_interleave(group, dim=1)
    s = torch.matmul(q, kx.transpose(-1, -2)) * scale
    if causal:
        mask = torch.ones(t, t, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    out = torch.matmul(torch.softmax(s, dim=-1), vx)
    res = {"out": out.detach().numpy(), "lse": lse.detach().numpy()}
    if g is not None:
        g = torch.as_tensor(np.asarray(g)).to(dtype)
        (out * g).sum().backward()
        res.update(dq=q.grad.numpy(), dk=k.grad.numpy(), dv=v.grad.numpy())
        res["delta"] = (out.detach() * g).sum(-1).numpy()
    return res


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64))))


def rel_max(a, ref):
    """max |a - ref| / max |ref|  (the norm-wise relative error used for the bf16 / fp16 tolerance)"""
    ref = np.asarray(ref, dtype=np.float64)
    return max_abs(a, ref) / max(float(np.max(np.abs(ref))), 1e-30)
