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


# ---- INT8 fused attention on cu_seqlens: the strict decomposition used wherever that kernel is checked ----

def int8_attention_parity(qkv, cu, N, s1, ss, s2, interleaved, S=None, expect=None, D=64):
    """Runs the shipped INT8 var-seqlen kernel and the instantiation that dumps its intermediates on qkv
    ([T, 3*N*D] int8, channel order [N][3][D]) and checks, against the oracle:
    both give the same bytes (and `expect`, [T, N*D], if given); first-GEMM accumulators bit-exact; quantised
    probabilities within 1 with at most max(2, 1e-5 n) off; the second GEMM and the requantisation exact from the
    kernel's own probabilities; rows whose probabilities all agree equal the oracle's bit for bit.
    Returns the kernel's output [T, N*D]."""
    import ctypes as C

    import oracle
    from tensorrt_amd import capi
    api = capi.api()
    cu = np.asarray(cu, np.int32)
    lens = np.diff(cu)
    B, T = len(lens), int(cu[-1])
    S = int(S or max(int(lens.max()), 1))
    ref, a1, p8, _ = oracle.mha_fused_i8_packed(qkv, cu, N, D, s1, ss, s2, want_ints=True)
    if interleaved:
        x = qkv.reshape(T, N, 3, D).transpose(0, 2, 1, 3).reshape(T, 3 * N * D)
        d_qkv = dev(oracle.interleave(x))
    else:
        d_qkv = dev(qkv)
    d_dbg = dev_empty((T * N * D,), np.int8, fill=0x55)
    d_out = dev_empty((T * N * D,), np.int8, fill=0x55)
    d_cu = dev(cu)
    d_a1 = dev_empty((B, N, S, S), np.int32, fill=0)
    d_p8 = dev_empty((B, N, S, S), np.int8, fill=0)
    p = capi.FmhaParams()
    p.qkv_ptr, p.o_ptr, p.cu_seqlens = ptr(d_qkv), ptr(d_dbg), ptr(d_cu)
    p.b, p.h, p.s, p.d = B, N, S, D
    p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = f32_bits(s1), f32_bits(ss), f32_bits(s2)
    p.interleaved, p.use_int8_scale_max = int(interleaved), 1
    p.qkv_stride_in_bytes = T if interleaved else 3 * N * D
    p.o_stride_in_bytes = T if interleaved else N * D
    api.check(api.fused_mha_run_debug(stream(), 2, C.byref(p), ptr(d_a1), ptr(d_p8)))
    p.o_ptr = ptr(d_out)
    api.check(api.fused_mha_run(stream(), 2, C.byref(p)))
    sync()
    got = host(d_out)
    # the shipped instantiation must give the same bytes as the checked one, fill pattern of unowned rows included
    assert np.array_equal(got, host(d_dbg)), "shipped INT8 kernel differs from the instantiation that dumps intermediates"
    got = oracle.deinterleave(got, T, N * D) if interleaved else got.reshape(T, N * D)
    if expect is not None:
        assert np.array_equal(got, np.asarray(expect).reshape(T, N * D)), "kernel output differs from the tensor under test"
    g_a1, g_p8 = host(d_a1), host(d_p8)
    ref3, got3 = ref.reshape(T, N, D), got.reshape(T, N, D)
    n_p8 = n_off = 0
    for b in range(B):
        L = int(lens[b])
        if L == 0:
            continue
        lo, hi = int(cu[b]), int(cu[b + 1])
        assert np.array_equal(g_a1[b, :, :L, :L], a1[b, :, :L, :L]), "first-GEMM accumulators must be bit-exact"
        dp = g_p8[b, :, :L, :L].astype(np.int32) - p8[b, :, :L, :L]
        assert np.abs(dp).max() <= 1, "quantised probabilities differ by more than 1 LSB"
        n_p8 += dp.size
        n_off += int((dp != 0).sum())
        # exact second GEMM from the kernel's own p8
        v = qkv[lo:hi].reshape(L, N, 3, D)[:, :, 2, :].astype(np.int64)               # [L,N,D]
        acc2 = np.einsum("nqk,knd->qnd", g_p8[b, :, :L, :L].astype(np.int64), v)        # [L,N,D]
        want = np.clip(np.rint(acc2.astype(np.float32) * np.float32(s2)), -128, 127).astype(np.int8)
        assert np.array_equal(got3[lo:hi], want), "second GEMM / requantisation must be exact"
        # (query, head) rows whose probabilities agree with the oracle agree with it bit for bit; a probability
        # that rounds the other way (exp differs in the last ulp) moves 64 outputs by up to |v| * scale_bmm2,
        # which the exact check above already covers.
        same = (dp == 0).all(axis=2).T                                                  # [L(q), N]
        assert np.array_equal(got3[lo:hi][same], ref3[lo:hi][same])
    assert n_off <= max(2, 1e-5 * n_p8), f"{n_off} of {n_p8} probabilities differ from the oracle"
    return got
