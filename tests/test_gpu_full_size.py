"""The benchmark configurations at their full sizes, checked through properties that do not need the
oracle on the whole problem: every (sequence, head) of an attention call is independent of the others, so a
sample of sequences is compared with the oracle run on those sequences alone, and the whole output must
follow a permutation of the sequences bit for bit; SkipLayerNorm rows are independent, the C oracle covers all
of them.  Inputs as the configurations state (seeded): attention FP16 B=32, S in {128, 384}, 12 heads, lengths
uniform in [S/2, S]; INT8 layer B=64, S=384, 16 heads, lengths uniform in [192, 384]."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, assert_int8_close, attention_f64, dev, dev_empty, f32_bits, half2_bits, host,
                     int8_attention_parity, ptr, quantize_amax, rng, stream, sync)

pytestmark = pytest.mark.gpu
D = 64


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


def cu_of(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def gather_sequences(x, cu, order):
    return np.concatenate([x[cu[b]:cu[b + 1]] for b in order], axis=0)


def sample_of(lens, r):
    """shortest, longest and two more sequences"""
    picks = {int(np.argmin(lens)), int(np.argmax(lens))}
    while len(picks) < 4:
        picks.add(int(r.integers(0, len(lens))))
    return sorted(picks)


@pytest.mark.parametrize("S", [128, 384])
def test_fp16_attention_at_benchmark_size(api, S):
    from tensorrt_amd import capi
    r = rng(1)
    B, N = 32, 12
    lens = r.integers(S // 2, S + 1, B)
    cu = cu_of(lens)
    T = int(cu[-1])
    qkv = (r.standard_normal((T, 3 * N * D)) / 8).astype(np.float16)

    def run(x, cu_):
        d_qkv, d_cu = dev(x), dev(cu_)
        out = dev_empty((x.shape[0], N * D), np.float16, fill=0)
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = ptr(d_qkv), ptr(out), ptr(d_cu)
        p.b, p.h, p.s, p.d = len(cu_) - 1, N, S, D
        p.qkv_stride_in_bytes, p.o_stride_in_bytes = 2 * 3 * N * D, 2 * N * D
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
        sync()
        return host(out)

    full = run(qkv, cu)
    assert np.isfinite(full).all()
    for b in sample_of(lens, r):
        lo, hi = cu[b], cu[b + 1]
        ref = oracle.mha_fused_f16_packed(qkv[lo:hi], cu_of(lens[b:b + 1]), N, D)
        assert_fp_close(full[lo:hi], ref, what=f"sequence {b} vs oracle")
        x = qkv[lo:hi].astype(np.float64).reshape(hi - lo, N, 3, D)
        o = attention_f64(x[:, 5, 0], x[:, 5, 1], x[:, 5, 2], 0.125)
        assert_fp_close(full[lo:hi, 5 * D:6 * D], o, what=f"sequence {b}, head 5 vs float64")
    order = r.permutation(B)
    moved = run(gather_sequences(qkv, cu, order), cu_of(lens[order]))
    assert np.array_equal(moved.view(np.uint16), gather_sequences(full, cu, order).view(np.uint16))


@pytest.mark.parametrize("dt", [np.float16, np.float32])
@pytest.mark.parametrize("S", [128, 384])
def test_unfused_attention_at_benchmark_size(api, dt, S):
    """The fixed-length [S, B, N, 3, d] layout of the benchmark shape through the unfused path (the route FP32 and
    head sizes the fused kernels lack take): sampled batches against the oracle on those batches alone and one head
    against binary64, and the whole output must follow a permutation of the batches bit for bit."""
    r = rng(3)
    B, N = 32, 12
    lens = r.integers(S // 2, S + 1, B).astype(np.int32)
    qkv = (r.standard_normal((S, B, 3 * N * D)) / 8).astype(dt)
    type_id = 0 if dt == np.float32 else 1
    ws = dev_empty((api.unfused_mha_workspace_size(type_id, S, B, N),), np.uint8)

    def run(x, lens_):
        d_x, d_len = dev(x), dev(lens_)
        out = dev_empty((S, B, N * D), dt, fill=0)
        api.check(api.unfused_mha(stream(), type_id, S, B, N, D, ptr(d_x), ptr(d_len), ptr(out), ptr(ws)))
        sync()
        return host(out)

    full = run(qkv, lens)
    assert np.isfinite(full).all()
    tol = dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}
    for b in sample_of(lens, r):
        ref = oracle.mha_unfused_fixed(qkv[:, b:b + 1], S, 1, N, D, lens[b:b + 1])
        assert_fp_close(full[:, b:b + 1], ref, what=f"batch {b} vs oracle", **tol)
        x = qkv[:, b].astype(np.float64).reshape(S, N, 3, D)
        L = int(lens[b])
        o = attention_f64(x[:, 5, 0], x[:L, 5, 1], x[:L, 5, 2], 0.125)
        assert_fp_close(full[:, b, 5 * D:6 * D], o, what=f"batch {b}, head 5 vs float64",
                        **(dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}))
    order = r.permutation(B)
    moved = run(np.ascontiguousarray(qkv[:, order]), lens[order])
    u = np.uint32 if dt == np.float32 else np.uint16
    assert np.array_equal(moved.view(u), np.ascontiguousarray(full[:, order]).view(u))


def int8_layer_inputs(r, B=64, S=384, N=16):
    lens = r.integers(S // 2, S + 1, B)
    cu = cu_of(lens)
    T = int(cu[-1])
    qkv, s_q = quantize_amax(r.standard_normal((T, 3 * N * D)))
    return lens, cu, T, qkv, s_q


def to_interleaved_qkv(qkv, N):
    """[T, 3*N*D] with channel order [N][3][D] -> channel order [3][N][D] -> [C/32][T][32]"""
    T = qkv.shape[0]
    return oracle.interleave(qkv.reshape(T, N, 3, D).transpose(0, 2, 1, 3).reshape(T, 3 * N * D))


def test_int8_attention_at_benchmark_size(api):
    from tensorrt_amd import capi
    r = rng(1)
    B, S, N = 64, 384, 16
    lens, cu, T, qkv, s_q = int8_layer_inputs(r, B, S, N)
    dq_probs = np.float32(1 / 127)
    s_ctx = np.float32(1.25 * s_q)   # the context is a convex combination of V rows: |ctx| <= amax(V)
    s1 = np.float32(s_q * s_q * np.float32(1 / np.sqrt(np.float32(D))))
    ss = np.float32(1 / dq_probs)
    s2 = np.float32(dq_probs * s_q / s_ctx)

    def run(x, cu_):
        t = x.shape[0]
        d_qkv, d_cu = dev(to_interleaved_qkv(x, N)), dev(cu_)
        out = dev_empty((t * N * D,), np.int8, fill=0x55)
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = ptr(d_qkv), ptr(out), ptr(d_cu)
        p.b, p.h, p.s, p.d = len(cu_) - 1, N, S, D
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = f32_bits(s1), f32_bits(ss), f32_bits(s2)
        p.interleaved, p.use_int8_scale_max = 1, 1
        p.qkv_stride_in_bytes = p.o_stride_in_bytes = t
        api.check(api.fused_mha_run(stream(), 2, C.byref(p)))
        sync()
        return oracle.deinterleave(host(out), t, N * D)

    full = run(qkv, cu)
    # every row was written: a row of the fill pattern would have all 1024 values equal to 0x55
    assert not (full == 0x55).all(axis=1).any()
    # sampled sequences, run alone: the same bytes as in the batch, first accumulators and second product exact,
    # probabilities within one step (<= 1e-5 of them off), rows with agreeing probabilities bit-exact
    for b in sample_of(lens, r):
        lo, hi = cu[b], cu[b + 1]
        int8_attention_parity(qkv[lo:hi], cu_of(lens[b:b + 1]), N, s1, ss, s2, interleaved=True, S=S, expect=full[lo:hi])
    order = r.permutation(B)
    moved = run(gather_sequences(qkv, cu, order), cu_of(lens[order]))
    assert np.array_equal(moved, gather_sequences(full, cu, order))


def test_int8_skip_layer_norm_at_benchmark_size(api):
    r = rng(1)
    ld = 1024
    lens = r.integers(192, 385, 64)
    total = int(lens.sum())
    x, dq_in = quantize_amax(r.standard_normal((total, ld)))
    s, dq_skip = quantize_amax(r.standard_normal((total, ld)))
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.1 * r.standard_normal(ld)).astype(np.float16)
    q_scale = np.float32(127.0 / 4.5)

    def run(a, b):
        a_il, b_il = oracle.interleave(a), oracle.interleave(b)
        out = dev_empty((ld * a.shape[0],), np.int8, fill=0)
        dx, ds, db, dg = dev(a_il), dev(b_il), dev(beta), dev(gamma)
        api.check(api.skipln_interleaved_large_hface(stream(), ld, a.shape[0], ptr(dx), ptr(ds), ptr(db), ptr(dg),
                                                     ptr(out), dq_in, dq_skip, q_scale))
        sync()
        return host(out), a_il, b_il

    got, x_il, s_il = run(x, s)
    st, ref, _ = oracle.skipln_interleaved(0, x_il, s_il, beta, gamma, ld, total, dq_in, dq_skip, q_scale, force=1)
    assert st == 0
    # within one step everywhere; the statistics are accumulated in another order than the oracle's, which moves
    # well under 1 % of the values across a rounding boundary
    assert_int8_close(got, ref, what="all rows vs oracle", max_frac_off=0.01)
    order = r.permutation(total)
    moved, _, _ = run(x[order], s[order])
    assert np.array_equal(oracle.deinterleave(moved, total, ld), oracle.deinterleave(got, total, ld)[order])


@pytest.mark.parametrize("K,N,gelu", [(1024, 4096, True), (4096, 1024, False), (1024, 3072, False)])
def test_int8_linear_at_benchmark_size(K, N, gelu):
    """The encoder's linear layers at 33289 tokens: every output row depends on its own input row only, so the
    oracle is run on a sample of rows (the first and last ones, rows either side of every 256-token tile edge of one
    region, and random ones) and must match there; a second launch on a row permutation must give the permuted
    output everywhere."""
    import torch
    from tensorrt_amd import capi
    r = rng(5)
    T = 33289
    a = np.clip(np.rint(r.standard_normal((T, K)) * 30), -127, 127).astype(np.int8)
    w = np.clip(np.rint(r.standard_normal((N, K)) * 30), -127, 127).astype(np.int8)
    alpha = (r.uniform(0.5, 1.5, N) * (3.0 / (30 * 30 * np.sqrt(K)))).astype(np.float32)
    beta = (0.3 * r.standard_normal(N)).astype(np.float32)
    if not gelu:
        alpha, beta = alpha * np.float32(30), beta * np.float32(30)   # outputs spread over the INT8 range
    api = capi.api()
    dw = dev(oracle.interleave(w).reshape(K // 32, N, 32))
    dal, dbe = dev(alpha), dev(beta)

    def run(x):
        da = dev(oracle.interleave(x).reshape(K // 32, T, 32))
        out = dev_empty((N // 32, T, 32), np.int8, fill=0)
        p = capi.Int8LinearParams()
        p.a, p.w, p.alpha, p.beta, p.out = da.data_ptr(), dw.data_ptr(), dal.data_ptr(), dbe.data_ptr(), out.data_ptr()
        p.T, p.K, p.N = T, K, N
        p.a_interleaved = p.w_interleaved = p.out_interleaved = 1
        p.epilogue, p.out_scale = (capi.LINEAR_GELU if gelu else capi.LINEAR_AFFINE), 30.0
        api.check(api.int8_linear(torch.cuda.current_stream().cuda_stream, C.byref(p)))
        torch.cuda.synchronize()
        return oracle.deinterleave(host(out).ravel(), T, N)

    got = run(a)
    edges = np.concatenate([np.arange(e - 2, e + 2) for e in range(256, 256 * 12, 256)])
    rows = np.unique(np.concatenate([np.arange(4), np.arange(T - 4, T), edges, np.arange(32768 - 3, 32768 + 3),
                                     r.integers(0, T, 1200)]))
    ref = oracle.int8_linear(a[rows], w, alpha, beta, oracle.LINEAR_GELU if gelu else oracle.LINEAR_AFFINE,
                             out_scale=30.0)
    assert np.abs(ref.astype(np.int32)).max() > 60
    assert_int8_close(got[rows], ref, what="sampled rows vs oracle", max_frac_off=2e-3)
    order = r.permutation(T)
    assert np.array_equal(run(a[order]), got[order])
