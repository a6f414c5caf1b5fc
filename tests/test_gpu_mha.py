"""GPU parity of the fused attention kernels (through the C ABI).

INT8: first-GEMM accumulators bit-exact against the oracle; quantised probabilities +-1; the
second GEMM is checked exactly by recomputing sum(p8*V) from the kernel's own p8 in numpy and
requantising; final INT8 output +-1 LSB against the oracle.
FP16: |a-b| <= 2e-3 + 1e-2*|b| against the oracle and against the float64 closed form."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, attention_f64, dev, dev_empty, f32_bits, half2_bits, host, int8_attention_parity,
                     ptr, quantize_amax, rng, stream, sync)

pytestmark = pytest.mark.gpu
D = 64


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


def _params(capi, **kw):
    p = capi.FmhaParams()
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def _cu(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def _ctx_scale(qkv_q, s_q, cu, N):
    """amax of the float attention of the dequantised tensor / 127 (how a calibrator sets it)."""
    x = qkv_q.astype(np.float64) * float(s_q)
    T = x.shape[0]
    x = x.reshape(T, N, 3, D)
    amax = 0.0
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi > lo:
            for n in range(min(N, 2)):
                o = attention_f64(x[lo:hi, n, 0], x[lo:hi, n, 1], x[lo:hi, n, 2], 1 / 8)
                amax = max(amax, np.abs(o).max())
    return np.float32(max(amax, 1e-3) / 127)


INT8_PACKED = [
    # B, N, S (max), lens rule
    (3, 2, 128, "rand"), (2, 16, 384, "c4"), (5, 3, 64, "rand"), (4, 2, 192, "rand"), (3, 2, 256, "full"),
    (2, 2, 512, "rand"), (6, 1, 96, "edge"),
    # unit counts either side of where the launcher stops sharing a (sequence, head) unit between workgroups (896),
    # a count that takes three workgroups per unit, and one whose ids do not fill whole spans of 8 x parts
    (55, 16, 128, "rand"), (56, 16, 128, "rand"), (17, 16, 256, "c4"), (13, 3, 384, "rand"),
]


def _lens(r, B, S, rule):
    if rule == "c4":
        return r.integers(S // 2, S + 1, B)
    if rule == "full":
        return np.full(B, S)
    if rule == "edge":
        base = [1, 0, 15, 16, 17, 64, 65, S]
        return np.array([min(v, S) for v in base][:B])
    return r.integers(1, S + 1, B)


@pytest.mark.parametrize("B,N,S,rule", INT8_PACKED)
@pytest.mark.parametrize("interleaved", [False, True])
def test_fmha_int8_packed(api, B, N, S, rule, interleaved):
    from tensorrt_amd import capi
    r = rng(21)
    lens = _lens(r, B, S, rule)
    cu = _cu(lens)
    T = int(cu[-1])
    qkv_f = r.standard_normal((T, 3 * N * D))
    qkv, s_q = quantize_amax(qkv_f)
    dq_probs = np.float32(1 / 127)
    s_ctx = _ctx_scale(qkv, s_q, cu, N)
    s1 = np.float32(s_q * s_q * np.float32(1 / np.sqrt(np.float32(D))))
    ss = np.float32(1 / dq_probs)
    s2 = np.float32(dq_probs * s_q / s_ctx)
    got = int8_attention_parity(qkv, cu, N, s1, ss, s2, interleaved, S=S)
    # rows of the output that belong to no sequence do not exist in the packed layouts: every row was written
    assert got.shape == (T, N * D)


@pytest.mark.parametrize("S,B,N", [(128, 3, 2), (384, 2, 3), (64, 4, 1), (96, 2, 2)])
@pytest.mark.parametrize("dtype", ["int8", "fp16"])
def test_fmha_fixed_packed_mask(api, S, B, N, dtype):
    """v1 kernels: fixed [S,B,N,3,d] layout, key mask given in the packed XMMA format; every
    query row 0..S-1 is computed."""
    from tensorrt_amd import capi
    r = rng(22)
    lens = r.integers(1, S + 1, B)
    lens[0] = S
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    wm, wn = (2, 2) if S <= 128 else (1, 8)
    packed, over = oracle.convert_mask(mask, wm, wn)
    assert over == 0
    d_mask = dev(packed)
    stride_mask = packed.shape[1] * 4
    if dtype == "int8":
        qkv, s_q = quantize_amax(r.standard_normal((S, B, N, 3, D)))
        s1 = np.float32(s_q * s_q * np.float32(0.125))
        ss, s2 = np.float32(127), np.float32(1 / 127 * s_q / 0.02)
        ref, a1, p8, _ = oracle.mha_fused_i8_fixed(qkv, S, B, N, D, lens, s1, ss, s2, want_ints=True)
        d_qkv, d_out = dev(qkv), dev_empty((S, B, N * D), np.int8, fill=0x55)
        d_dbg = dev_empty((S, B, N * D), np.int8, fill=0x55)
        d_a1 = dev_empty((B, N, S, S), np.int32, fill=0)
        d_p8 = dev_empty((B, N, S, S), np.int8, fill=0)
        p = _params(capi, qkv_ptr=ptr(d_qkv), packed_mask_ptr=ptr(d_mask), o_ptr=ptr(d_out), b=B, h=N, s=S, d=D,
                    qkv_stride_in_bytes=3 * B * N * D, o_stride_in_bytes=B * N * D,
                    packed_mask_stride_in_bytes=stride_mask, scale_bmm1=f32_bits(s1), scale_softmax=f32_bits(ss),
                    scale_bmm2=f32_bits(s2))
        api.check(api.fused_mha_run(stream(), 2, C.byref(p)))
        p.o_ptr = ptr(d_dbg)
        api.check(api.fused_mha_run_debug(stream(), 2, C.byref(p), ptr(d_a1), ptr(d_p8)))
        sync()
        got = host(d_out)
        assert np.array_equal(got, host(d_dbg)), "shipped kernel differs from the instantiation that dumps intermediates"
        g_a1, g_p8 = host(d_a1), host(d_p8)
        n_p8 = n_off = 0
        for b in range(B):
            L = int(lens[b])
            assert np.array_equal(g_a1[b, :, :, :L], a1[b, :, :, :L]), "first-GEMM accumulators must be bit-exact"
            dp = g_p8[b, :, :, :L].astype(np.int32) - p8[b, :, :, :L]
            assert np.abs(dp).max() <= 1
            n_p8 += dp.size
            n_off += int((dp != 0).sum())
            v = qkv[:L, b, :, 2, :].astype(np.int64)                                       # [L,N,D]
            acc2 = np.einsum("nqk,knd->qnd", g_p8[b, :, :, :L].astype(np.int64), v)        # [S,N,D]
            want = np.clip(np.rint(acc2.astype(np.float32) * s2), -128, 127).astype(np.int8)
            assert np.array_equal(got[:, b].reshape(S, N, D), want), "second GEMM / requantisation must be exact"
            same = (dp == 0).all(axis=2).T                                                  # [S(q), N]
            assert np.array_equal(got[:, b].reshape(S, N, D)[same], ref[:, b].reshape(S, N, D)[same])
        assert n_off <= max(2, 1e-5 * n_p8), f"{n_off} of {n_p8} probabilities differ from the oracle"
    else:
        qkv = (r.standard_normal((S, B, N, 3, D)) / 8).astype(np.float16)
        ref = oracle.mha_fused_f16_fixed(qkv, S, B, N, D, lens)
        d_qkv, d_out = dev(qkv), dev_empty((S, B, N * D), np.float16, fill=0)
        p = _params(capi, qkv_ptr=ptr(d_qkv), packed_mask_ptr=ptr(d_mask), o_ptr=ptr(d_out), b=B, h=N, s=S, d=D,
                    qkv_stride_in_bytes=2 * 3 * B * N * D, o_stride_in_bytes=2 * B * N * D,
                    packed_mask_stride_in_bytes=stride_mask, scale_bmm1=half2_bits(0.125),
                    scale_softmax=half2_bits(1.0), scale_bmm2=half2_bits(1.0))
        api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
        sync()
        got = host(d_out)
        assert_fp_close(got, ref, what="fixed FP16 vs oracle")
        x = qkv.astype(np.float64)
        for b in range(B):
            L = int(lens[b])
            for n in range(N):
                o = attention_f64(x[:, b, n, 0], x[:L, b, n, 1], x[:L, b, n, 2], 0.125)
                assert_fp_close(got[:, b, n * D:(n + 1) * D], o, what="fixed FP16 vs float64")


def test_fmha_fixed_nonprefix_mask(api):
    """The packed format carries one bit per key: a mask with holes is honoured key by key."""
    from tensorrt_amd import capi
    r = rng(23)
    S, B, N = 128, 2, 2
    mask = r.integers(0, 2, (S, B)).astype(np.int32)
    mask[0, :] = 1
    packed, _ = oracle.convert_mask(mask, 2, 2)
    qkv = (r.standard_normal((S, B, N, 3, D)) / 8).astype(np.float16)
    d_qkv, d_mask, d_out = dev(qkv), dev(packed), dev_empty((S, B, N * D), np.float16, fill=0)
    p = _params(capi, qkv_ptr=ptr(d_qkv), packed_mask_ptr=ptr(d_mask), o_ptr=ptr(d_out), b=B, h=N, s=S, d=D,
                qkv_stride_in_bytes=2 * 3 * B * N * D, o_stride_in_bytes=2 * B * N * D,
                packed_mask_stride_in_bytes=packed.shape[1] * 4, scale_bmm1=half2_bits(0.125))
    api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
    sync()
    got = host(d_out)
    x = qkv.astype(np.float64)
    for b in range(B):
        keep = mask[:, b] == 1
        for n in range(N):
            o = attention_f64(x[:, b, n, 0], x[keep, b, n, 1], x[keep, b, n, 2], 0.125)
            assert_fp_close(got[:, b, n * D:(n + 1) * D], o, what="non-prefix mask")


@pytest.mark.parametrize("B,N,S,rule", [(4, 12, 128, "c4"), (3, 12, 384, "c4"), (8, 2, 96, "edge"), (2, 16, 512, "rand"),
                                        (3, 3, 192, "rand"), (2, 2, 256, "full"),
                                        # either side of the unit count below which units are shared (160)
                                        (13, 12, 192, "rand"), (14, 12, 192, "rand")])
def test_fmha_fp16_packed(api, B, N, S, rule):
    from tensorrt_amd import capi
    r = rng(24)
    lens = _lens(r, B, S, rule)
    cu = _cu(lens)
    T = int(cu[-1])
    qkv = (r.standard_normal((T, 3 * N * D)) / 8).astype(np.float16)
    ref = oracle.mha_fused_f16_packed(qkv, cu, N, D)
    d_qkv, d_cu = dev(qkv), dev(cu)
    d_out = dev_empty((T, N * D), np.float16, fill=0)
    p = _params(capi, qkv_ptr=ptr(d_qkv), o_ptr=ptr(d_out), b=B, h=N, s=S, d=D, qkv_stride_in_bytes=2 * 3 * N * D,
                o_stride_in_bytes=2 * N * D, scale_bmm1=half2_bits(0.125), scale_softmax=half2_bits(1.0),
                scale_bmm2=half2_bits(1.0), cu_seqlens=ptr(d_cu))
    api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
    sync()
    got = host(d_out)
    assert_fp_close(got, ref, what="FP16 packed vs oracle")
    # the instantiation that dumps the first GEMM must give the same bits as the shipped one
    d_dbg = dev_empty((T, N * D), np.float16, fill=0)
    d_a1 = dev_empty((B, N, S, S), np.int32, fill=0)
    p.o_ptr = ptr(d_dbg)
    api.check(api.fused_mha_run_debug(stream(), 1, C.byref(p), ptr(d_a1), 0))
    sync()
    assert np.array_equal(host(d_dbg).view(np.uint16), got.view(np.uint16))
    s_gpu = host(d_a1).view(np.float32)
    x32 = qkv.astype(np.float32).reshape(T, N, 3, D)
    for b in range(B):
        lo, hi = cu[b], cu[b + 1]
        if hi > lo:
            s_ref = np.einsum("qnd,knd->nqk", x32[lo:hi, :, 0].astype(np.float64), x32[lo:hi, :, 1].astype(np.float64))
            assert np.abs(s_gpu[b, :, :hi - lo, :hi - lo] - s_ref).max() <= 1e-4, "first GEMM (binary32 accumulation)"
    x = qkv.astype(np.float64).reshape(T, N, 3, D)
    for b in range(B):
        lo, hi = cu[b], cu[b + 1]
        for n in range(0, N, max(1, N // 3)):
            if hi > lo:
                o = attention_f64(x[lo:hi, n, 0], x[lo:hi, n, 1], x[lo:hi, n, 2], 0.125)
                assert_fp_close(got[lo:hi, n * D:(n + 1) * D], o, what="FP16 packed vs float64")


def test_fmha_packing_invariance_and_special_cases(api):
    """Per-sequence results do not depend on what else is packed beside them; a length-1
    sequence returns V; identical keys give the plain average of V."""
    from tensorrt_amd import capi
    r = rng(25)
    N, S = 2, 128
    lens = np.array([37, 1, 128, 64])
    cu = _cu(lens)
    T = int(cu[-1])
    qkv = (r.standard_normal((T, N, 3, D)) / 8).astype(np.float16)
    lo, hi = cu[3], cu[4]
    qkv[lo:hi, :, 1, :] = qkv[lo, :, 1, :]  # sequence 3: all keys equal

    def run(x, cu_):
        d_qkv, d_cu = dev(x), dev(cu_)
        out = dev_empty((x.shape[0], N * D), np.float16, fill=0)
        p = _params(capi, qkv_ptr=ptr(d_qkv), o_ptr=ptr(out), b=len(cu_) - 1, h=N, s=S, d=D,
                    qkv_stride_in_bytes=2 * 3 * N * D, o_stride_in_bytes=2 * N * D, scale_bmm1=half2_bits(0.125),
                    cu_seqlens=ptr(d_cu))
        api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
        sync()
        return host(out)

    full = run(qkv, cu)
    for b in range(4):
        alone = run(qkv[cu[b]:cu[b + 1]].copy(), _cu(lens[b:b + 1]))
        assert np.array_equal(alone.view(np.uint16), full[cu[b]:cu[b + 1]].view(np.uint16))
    # length 1: softmax over one key is 1 -> output = V
    assert np.array_equal(full[cu[1]].view(np.uint16), qkv[cu[1], :, 2, :].reshape(-1).view(np.uint16))
    # equal keys: uniform average of V
    avg = qkv[lo:hi, :, 2, :].astype(np.float64).mean(0).reshape(-1)
    assert_fp_close(full[lo:hi], np.broadcast_to(avg, (hi - lo, N * D)), what="uniform attention")


def test_fmha_more_sequences_than_the_ranking_holds(api):
    """Launches of more than 1024 sequences are served in natural order (the longest-first table has 1024 entries);
    INT8 through the strict decomposition, FP16 against the oracle, and the ranked and unranked orders must agree."""
    from tensorrt_amd import capi
    r = rng(27)
    B, N, S = 1100, 1, 64
    lens = r.integers(0, S + 1, B)
    cu = _cu(lens)
    T = int(cu[-1])
    qkv, s_q = quantize_amax(r.standard_normal((T, 3 * N * D)))
    s1 = np.float32(s_q * s_q * np.float32(0.125))
    got = int8_attention_parity(qkv, cu, N, s1, np.float32(127), np.float32(s_q / (127 * 0.02)), False, S=S)
    # the first 1000 sequences alone take the ranked path (1000 x 1 workgroups are more than one round): same bytes
    head = int8_attention_parity(qkv[:cu[1000]].copy(), cu[:1001].copy(), N, s1, np.float32(127),
                                 np.float32(s_q / (127 * 0.02)), False, S=S)
    assert np.array_equal(head, got[:cu[1000]])
    x = (r.standard_normal((T, 3 * N * D)) / 8).astype(np.float16)
    d_x, d_cu = dev(x), dev(cu)
    out = dev_empty((T, N * D), np.float16, fill=0)
    p = _params(capi, qkv_ptr=ptr(d_x), o_ptr=ptr(out), b=B, h=N, s=S, d=D, qkv_stride_in_bytes=2 * 3 * N * D,
                o_stride_in_bytes=2 * N * D, scale_bmm1=half2_bits(0.125), cu_seqlens=ptr(d_cu))
    api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
    sync()
    assert_fp_close(host(out), oracle.mha_fused_f16_packed(x, cu, N, D), what="FP16, 1100 sequences")


def test_fmha_argument_errors(api):
    from tensorrt_amd import capi
    p = _params(capi, qkv_ptr=16, o_ptr=16, b=1, h=1, s=128, d=32, qkv_stride_in_bytes=96, o_stride_in_bytes=32)
    assert api.fused_mha_run(None, 2, C.byref(p)) != 0 and "head size" in api.last_error_str()
    p.d = 64
    p.s = 513
    assert api.fused_mha_run(None, 2, C.byref(p)) != 0 and "512" in api.last_error_str()
    p.s = 128
    assert api.fused_mha_run(None, 0, C.byref(p)) != 0          # FP32 has no fused kernel
    assert api.fused_mha_run(None, 2, C.byref(p)) != 0          # scales are zero / strides too small
    assert api.fused_mha_is_valid(2, 64, 384) == 1 and api.fused_mha_is_valid(1, 64, 512) == 1
    assert api.fused_mha_is_valid(0, 64, 128) == 0 and api.fused_mha_is_valid(1, 32, 128) == 0
    assert api.fused_mha_is_valid(1, 64, 1024) == 0
