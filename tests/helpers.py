"""Shared test plumbing: seeded inputs, device buffers (torch is only the allocator) and the
tolerance rules of the parity bar."""
from __future__ import annotations

import numpy as np

FP_ATOL = 2e-3   # floating point outputs after LayerNorm / attention: |a-b| <= atol + rtol*|b|
FP_RTOL = 1e-2
INT8_LSB = 1     # requantised INT8 outputs


def rng(seed):
    return np.random.default_rng(seed)


def assert_fp_close(got, ref, atol=FP_ATOL, rtol=FP_RTOL, what=""):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values in result"
    err = np.abs(got - ref)
    bad = err > atol + rtol * np.abs(ref)
    assert not bad.any(), f"{what}: {bad.sum()} / {bad.size} outside tolerance, max abs err {err.max():.3e}"


def assert_int8_close(got, ref, lsb=INT8_LSB, what="", max_frac_off=None):
    got = np.asarray(got, np.int32)
    ref = np.asarray(ref, np.int32)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    diff = np.abs(got - ref)
    assert diff.max(initial=0) <= lsb, f"{what}: max INT8 difference {diff.max()} > {lsb} LSB"
    if max_frac_off is not None:
        frac = float((diff != 0).mean()) if diff.size else 0.0
        assert frac <= max_frac_off, f"{what}: {frac:.4f} of values differ (allowed {max_frac_off})"


# ---- device buffers ---------------------------------------------------------------------------

def dev(a):
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def dev_empty(shape, dtype, fill=None):
    import torch
    t = {np.float32: torch.float32, np.float16: torch.float16, np.int8: torch.int8, np.int32: torch.int32,
         np.uint32: torch.int32, np.uint8: torch.uint8}[dtype]
    x = torch.empty(shape, dtype=t, device="cuda")
    if fill is not None:
        x.fill_(fill)
    return x


def host(t, dtype=None):
    a = t.detach().cpu().numpy()
    if dtype is not None and a.dtype != dtype:
        a = a.view(dtype)
    return a


def ptr(t):
    return 0 if t is None else t.data_ptr()


def stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def sync():
    import torch
    torch.cuda.synchronize()


# ---- closed forms (numpy float64), independent of the oracle ----------------------------------

def layer_norm_f64(v, gamma, beta, eps):
    v = np.asarray(v, np.float64)
    mu = v.mean(-1, keepdims=True)
    var = v.var(-1, keepdims=True)
    return (v - mu) / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)


def attention_f64(q, k, v, scale):
    """q [nq,d], k,v [nk,d] -> [nq,d] in float64."""
    s = (np.asarray(q, np.float64) @ np.asarray(k, np.float64).T) * scale
    s -= s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return p @ np.asarray(v, np.float64)


def quantize_amax(x):
    """Per-tensor symmetric INT8 with scale amax/127
    (tools/pytorch-quantization/pytorch_quantization/tensor_quant.py:535-549)."""
    amax = float(np.abs(x).max())
    scale = amax / 127.0
    q = np.clip(np.rint(x / scale), -127, 127).astype(np.int8)
    return q, np.float32(scale)


def f32_bits(x):
    return int(np.float32(x).view(np.uint32))


def half2_bits(x):
    h = int(np.float16(x).view(np.uint16))
    return h | (h << 16)
