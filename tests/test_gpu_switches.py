"""Every tuning switch of the library (README, "Tuning switches") selects a kernel variant other than the default one.
Each setting is put through the parity checks of the kernel it changes, in this process, through the test hook that
stands in for the environment variable of the same name (include/trtamd_test_hooks.h): the variants must give what
the default choice gives, to the same bar against the oracle."""
import contextlib
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, assert_int8_close, attention_f64, dev, dev_empty, half2_bits, host,
                     int8_attention_parity, ptr, quantize_amax, rng, stream, sync)
from tensorrt_amd import capi
from test_gpu_linear import interleave, problem, run_gpu

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def tuning(name, value):
    api = capi.api()
    api.check(api.test_set_tuning(name.encode(), value))
    try:
        yield
    finally:
        api.check(api.test_reset_tuning(name.encode()))


def test_unknown_switch_is_refused():
    api = capi.api()
    assert api.test_set_tuning(b"TRTAMD_NO_SUCH_SWITCH", 1) == 2
    assert "unknown tuning switch" in api.last_error_str()
    assert api.test_reset_tuning(b"TRTAMD_NO_SUCH_SWITCH") == 2


LINEAR_SETTINGS = [("TRTAMD_LINEAR_DIRECT", 0), ("TRTAMD_LINEAR_PERSISTENT", 0), ("TRTAMD_LINEAR_PARTIAL_ROUND", 0),
                   ("TRTAMD_LINEAR_PARTIAL_ROUND", 100)]


def test_remainder_pieces_against_remainder_tiles():
    """More than half a round of large tiles (so that they run, as a partial round) and 60 tokens behind them: by
    default those go in 64 x 64 pieces whose wavefronts split k, with TRTAMD_LINEAR_PIECES=0 in 128 x 128 tiles; both
    must give the oracle's accumulator-exact results and the same bytes."""
    T, K, N = 133 * 256 + 60, 256, 512
    a, w, alpha, beta = problem(93, T, K, N)
    ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE, out_interleaved=True)
    pieces = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=True, out_il=True, w_il=True)
    with tuning("TRTAMD_LINEAR_PIECES", 0):
        tiles = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=True, out_il=True, w_il=True)
    assert_int8_close(pieces, ref, what="pieces", max_frac_off=1e-3)
    assert np.array_equal(pieces, tiles)
    q = float(np.float32(127.0 / 4.0))
    al, be = (alpha * 0.06).astype(np.float32), (beta * 0.02).astype(np.float32)
    ref = oracle.int8_linear(a, w, al, be, oracle.LINEAR_GELU, out_scale=q, out_interleaved=True)
    pieces = run_gpu(a, w, al, be, capi.LINEAR_GELU, out_scale=q, a_il=True, out_il=True, w_il=True)
    with tuning("TRTAMD_LINEAR_PIECES", 0):
        tiles = run_gpu(a, w, al, be, capi.LINEAR_GELU, out_scale=q, a_il=True, out_il=True, w_il=True)
    assert_int8_close(pieces, ref, what="pieces, GELU", max_frac_off=2e-3)
    assert np.array_equal(pieces, tiles)


@pytest.mark.parametrize("name,value", LINEAR_SETTINGS)
@pytest.mark.parametrize("il", [True, False])
def test_linear_variants(name, value, il):
    """Shapes the direct-to-LDS kernel takes by default (N a multiple of 256, K of 256, a ragged token count with
    whole 256-token tiles and a remainder): accumulators bit-exact, affine and GELU outputs to the oracle's bar and
    equal to the default choice's bytes."""
    T, K, N = 777, 1024, 512
    a, w, alpha, beta = problem(91, T, K, N, full_range=True)
    with tuning(name, value):
        raw = run_gpu(a, w, None, None, capi.LINEAR_RAW_INT32, a_il=il, w_il=il)
    assert np.array_equal(raw, oracle.int8_linear(a, w, epilogue=oracle.LINEAR_RAW_INT32))
    a, w, alpha, beta = problem(92, T, K, N)
    for epi, oepi, frac in ((capi.LINEAR_AFFINE, oracle.LINEAR_AFFINE, 1e-3), (capi.LINEAR_GELU, oracle.LINEAR_GELU, 2e-3)):
        # GELU: pre-activations of a few units either side of zero, as in test_gpu_linear.test_gelu_int8
        scale = 1.0 if epi == capi.LINEAR_AFFINE else float(np.float32(127.0 / 4.0))
        al = alpha if epi == capi.LINEAR_AFFINE else (alpha * 0.06).astype(np.float32)
        be = beta if epi == capi.LINEAR_AFFINE else (beta * 0.02).astype(np.float32)
        default = run_gpu(a, w, al, be, epi, out_scale=scale, a_il=il, out_il=il, w_il=il)
        with tuning(name, value):
            got = run_gpu(a, w, al, be, epi, out_scale=scale, a_il=il, out_il=il, w_il=il)
        ref = oracle.int8_linear(a, w, al, be, oepi, out_scale=scale, out_interleaved=il)
        assert_int8_close(got, ref, what=f"{name}={value} epilogue {epi}", max_frac_off=frac)
        assert np.array_equal(got, default), f"{name}={value}: bytes differ from the default kernel choice"


FMHA_SETTINGS = [("TRTAMD_FMHA_GENERIC", 1), ("TRTAMD_FMHA_QSPLIT", 1), ("TRTAMD_FMHA_QSPLIT", 2),
                 ("TRTAMD_FMHA_QSPLIT", 3), ("TRTAMD_FMHA_QSPLIT", 4), ("TRTAMD_FMHA_RANKED", 0),
                 ("TRTAMD_FMHA_RANKED", 1)]


@pytest.mark.parametrize("name,value", FMHA_SETTINGS)
@pytest.mark.parametrize("interleaved", [False, True])
def test_int8_attention_variants(name, value, interleaved):
    r = rng(1200 + value)
    B, N, S = 5, 3, 384
    lens = np.array([384, 1, 200, 65, 129])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    qkv, s_q = quantize_amax(r.standard_normal((T, 3 * N * 64)).astype(np.float32))
    s1, ss, s2 = np.float32(s_q * s_q * 0.125), np.float32(127.0), np.float32(s_q / 127.0 / 0.02)
    default = int8_attention_parity(qkv, cu, N, s1, ss, s2, interleaved, S=S)
    with tuning(name, value):
        int8_attention_parity(qkv, cu, N, s1, ss, s2, interleaved, S=S, expect=default)


@pytest.mark.parametrize("name,value", FMHA_SETTINGS)
def test_fp16_attention_variants(name, value):
    api = capi.api()
    r = rng(1300 + value)
    B, N, S = 4, 3, 384
    lens = np.array([384, 7, 250, 130])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    qkv = (r.standard_normal((T, N, 3, 64)) * 0.7).astype(np.float16)
    d_qkv, d_cu = dev(qkv), dev(cu)

    def run():
        out = dev_empty((T, N * 64), np.float16, fill=0)
        p = capi.FmhaParams()
        p.qkv_ptr, p.o_ptr, p.cu_seqlens = ptr(d_qkv), ptr(out), ptr(d_cu)
        p.qkv_stride_in_bytes, p.o_stride_in_bytes = 2 * 3 * N * 64, 2 * N * 64
        p.b, p.h, p.s, p.d = B, N, S, 64
        p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = half2_bits(0.125), half2_bits(1.0), half2_bits(1.0)
        api.check(api.fused_mha_run(stream(), 1, C.byref(p)))
        sync()
        return host(out)

    default = run()
    with tuning(name, value):
        got = run()
    for b in range(B):
        lo, hi = int(cu[b]), int(cu[b + 1])
        for n in range(N):
            want = attention_f64(qkv[lo:hi, n, 0], qkv[lo:hi, n, 1], qkv[lo:hi, n, 2], 0.125)
            assert_fp_close(got[lo:hi, n * 64:(n + 1) * 64], want, what=f"{name}={value} sequence {b} head {n}")
    # the specialised and the general kernel sum in different orders; the other switches only move work around
    if name == "TRTAMD_FMHA_GENERIC":
        assert_fp_close(got, default, atol=1e-3, rtol=2e-3, what="general kernel vs prefix kernel")
    else:
        assert np.array_equal(got.view(np.uint16), default.view(np.uint16)), f"{name}={value}: bits differ from the default"
