"""INT8 linear layer on the GPU against the CPU oracle, through the C-ABI.

Bar: INT32 accumulators bit-exact; requantised INT8 within 1 LSB (the affine epilogue is a single
fmaf on both sides, the GPU's with 128 folded into the addend because it forms the byte unsigned, so
the two agree except for results within a rounding error of a tie; the GELU epilogue evaluates erf
through a polynomial on the GPU and in binary64 in the oracle); FP16 output within the
floating-point tolerance.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, assert_int8_close, dev, dev_empty, host, rng
from tensorrt_amd import capi

pytestmark = pytest.mark.gpu


def interleave(x):
    """[T, C] -> [C/32, T, 32]"""
    T, Cc = x.shape
    return np.ascontiguousarray(x.reshape(T, Cc // 32, 32).transpose(1, 0, 2))


def run_gpu(a, w, alpha, beta, epilogue, out_scale=1.0, a_il=False, out_il=False, w_il=False):
    import torch
    api = capi.api()
    N, K = w.shape
    T = a.shape[0]
    da = dev(interleave(a) if a_il else a)
    dw = dev(interleave(w) if w_il else w)
    dal = dev(alpha) if alpha is not None else None
    dbe = dev(beta) if beta is not None else None
    if epilogue == capi.LINEAR_RAW_INT32:
        out = dev_empty((T, N), np.int32, fill=-7)
    elif epilogue == capi.LINEAR_AFFINE_FP16:
        out = dev_empty((T, N), np.float16, fill=-7)
    else:
        out = dev_empty((N // 32, T, 32) if out_il else (T, N), np.int8, fill=-7)
    p = capi.Int8LinearParams()
    p.a, p.w, p.out = da.data_ptr(), dw.data_ptr(), out.data_ptr()
    p.alpha = dal.data_ptr() if dal is not None else None
    p.beta = dbe.data_ptr() if dbe is not None else None
    p.T, p.K, p.N = T, K, N
    p.a_interleaved, p.out_interleaved, p.epilogue, p.out_scale = int(a_il), int(out_il), epilogue, out_scale
    p.w_interleaved = int(w_il)
    api.check(api.int8_linear(torch.cuda.current_stream().cuda_stream, C.byref(p)))
    torch.cuda.synchronize()
    return host(out)


def problem(seed, T, K, N, full_range=False):
    r = rng(seed)
    if full_range:
        a = r.integers(-128, 128, (T, K)).astype(np.int8)
        w = r.integers(-128, 128, (N, K)).astype(np.int8)
    else:
        a = np.clip(np.rint(r.standard_normal((T, K)) * 30), -127, 127).astype(np.int8)
        w = np.clip(np.rint(r.standard_normal((N, K)) * 30), -127, 127).astype(np.int8)
    # scales that put the affine result in the INT8 range with some saturation
    sd = 30.0 * 30.0 * np.sqrt(K) * (4.0 if full_range else 1.0)
    alpha = (r.uniform(0.5, 1.5, N) * 50.0 / sd).astype(np.float32)
    beta = r.uniform(-20, 20, N).astype(np.float32)
    return a, w, alpha, beta


SHAPES = [(1, 64, 32), (17, 64, 32), (300, 128, 96), (256, 1024, 256), (1000, 256, 544), (519, 1024, 1024),
          (2100, 192, 3072)]


@pytest.mark.parametrize("T,K,N", SHAPES)
@pytest.mark.parametrize("a_il,w_il", [(False, False), (True, True), (True, False), (False, True)])
def test_accumulators_bit_exact(T, K, N, a_il, w_il):
    a, w, _, _ = problem(11 + T, T, K, N, full_range=True)
    # the extreme corner: -128 * -128 summed over K
    a[0, :] = -128
    w[0, :] = -128
    got = run_gpu(a, w, None, None, capi.LINEAR_RAW_INT32, a_il=a_il, w_il=w_il)
    ref = oracle.int8_linear(a, w, epilogue=oracle.LINEAR_RAW_INT32)
    assert np.array_equal(got, ref)
    assert got[0, 0] == 16384 * K


@pytest.mark.parametrize("T,K,N", SHAPES)
@pytest.mark.parametrize("a_il,out_il", [(False, False), (True, True), (False, True), (True, False)])
def test_affine_int8(T, K, N, a_il, out_il):
    a, w, alpha, beta = problem(23 + T, T, K, N)
    got = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=a_il, out_il=out_il, w_il=a_il)
    ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE, out_interleaved=out_il)
    assert (np.abs(ref.astype(int)) == 127).any() or (ref == -128).any(), "inputs should exercise saturation"
    assert_int8_close(got, ref, what="affine", max_frac_off=1e-3)


@pytest.mark.parametrize("il", [False, True])
@pytest.mark.parametrize("T,K,N", [(255, 64, 32), (512, 256, 256)])
def test_requantisation_ties_and_saturation_are_exact(T, K, N, il):
    """Accumulators -127..127 times scales that are multiples of 1/2: every product is exact in binary32,
    half of them lie on a tie (round to even) and the large scales run into both ends of the INT8 range, so
    the expected bytes follow from integer arithmetic alone."""
    a = np.zeros((T, K), np.int8)
    a[:, 0] = (np.arange(T) % 255 - 127).astype(np.int8)
    w = np.zeros((N, K), np.int8)
    w[:, 0] = 1
    alpha = (0.5 * (1 + np.arange(N) % 7)).astype(np.float32)     # 0.5 .. 3.5
    beta = (0.5 * (np.arange(N) % 5) - 1.0).astype(np.float32)    # -1 .. 1 in halves
    got = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=il, out_il=il, w_il=il)
    y = a[:, :1].astype(np.float64) * alpha[None, :].astype(np.float64) + beta[None, :].astype(np.float64)
    want = np.clip(np.rint(y), -128, 127).astype(np.int8)          # numpy's rint rounds ties to even
    assert (np.abs(y - np.floor(y)) == 0.5).any() and (want == 127).any() and (want == -128).any()
    if il:
        want = interleave(want)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("T,K,N", [(17, 64, 32), (519, 1024, 1024), (700, 1024, 4096)])
@pytest.mark.parametrize("il", [False, True])
def test_gelu_int8(T, K, N, il):
    a, w, alpha, beta = problem(37 + T, T, K, N)
    alpha = (alpha * 0.06).astype(np.float32)   # pre-activations of a few units either side of zero
    beta = (beta * 0.02).astype(np.float32)
    q = np.float32(127.0 / 4.0)
    got = run_gpu(a, w, alpha, beta, capi.LINEAR_GELU, out_scale=float(q), a_il=il, out_il=il, w_il=il)
    ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_GELU, out_scale=float(q), out_interleaved=il)
    assert ref.max() > 60 and ref.min() < 0
    assert_int8_close(got, ref, what="gelu", max_frac_off=2e-3)


@pytest.mark.parametrize("T,K,N", [(33, 64, 64), (519, 1024, 1024)])
def test_affine_fp16(T, K, N):
    a, w, alpha, beta = problem(41 + T, T, K, N)
    got = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE_FP16, a_il=True, w_il=True)
    ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE_FP16)
    assert_fp_close(got, ref, what="fp16 output")


@pytest.mark.parametrize("T,K,N", [(8229, 128, 3072), (16500, 64, 1024), (70000, 64, 256), (9600, 128, 1024),
                                   (28165, 128, 1024), (9600, 256, 1024), (28165, 512, 1024), (20000, 1024, 512), (70000, 256, 1024)])
def test_large_problems_mix_both_tile_sizes(T, K, N):
    """Enough 256 x 256 tiles for whole rounds of the chip, plus a remainder in 128 x 128 tiles.  The last two
    sizes leave more than half a round of large tiles, which then runs as a partial round (one with no whole
    round before it, one where the persistent workgroups get unequal tile counts)."""
    a, w, alpha, beta = problem(51 + T, T, K, N, full_range=True)
    got = run_gpu(a, w, None, None, capi.LINEAR_RAW_INT32, a_il=True, w_il=True)
    ref = oracle.int8_linear(a, w, epilogue=oracle.LINEAR_RAW_INT32)
    assert np.array_equal(got, ref)
    got8 = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=True, w_il=True, out_il=True)
    ref8 = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE, out_interleaved=True)
    assert_int8_close(got8, ref8, what="affine", max_frac_off=1e-3)
    got_lin = run_gpu(a, w, alpha, beta, capi.LINEAR_GELU, out_scale=0.5)
    ref_lin = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_GELU, out_scale=0.5)
    assert_int8_close(got_lin, ref_lin, what="gelu, linear layouts", max_frac_off=2e-3)
    got_il = run_gpu(a, w, alpha, beta, capi.LINEAR_GELU, out_scale=0.5, a_il=True, w_il=True, out_il=True)
    ref_il = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_GELU, out_scale=0.5, out_interleaved=True)
    assert_int8_close(got_il, ref_il, what="gelu, interleaved layouts", max_frac_off=2e-3)
    got_mixed = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=True, w_il=True, out_il=False)
    ref_mixed = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE)
    assert_int8_close(got_mixed, ref_mixed, what="affine, interleaved operands, linear output", max_frac_off=1e-3)


def _random_cases(n, seed):
    r = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        T = int(r.choice([int(r.integers(1, 300)), int(r.integers(300, 3000)), int(r.integers(8000, 12000))]))
        K = 64 * int(r.integers(1, 17))
        N = 32 * int(r.integers(1, 33))
        il = bool(r.integers(0, 2))
        out_il = bool(r.integers(0, 2))
        epi = int(r.integers(0, 3))   # affine, gelu, fp16 output
        cases.append((T, K, N, il, out_il, epi))
    return cases


@pytest.mark.parametrize("T,K,N,il,out_il,epi", _random_cases(20, 20240611))
def test_random_shapes_layouts_and_epilogues(T, K, N, il, out_il, epi):
    """Seeded random draws over the token count (a few rows to several rounds of tiles), K, N, operand and output
    layouts and epilogues: whatever tile plan and kernel variant a shape selects must agree with the oracle."""
    a, w, alpha, beta = problem(1000 + T + K + N, T, K, N)
    if epi == 0:
        got = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE, a_il=il, w_il=il, out_il=out_il)
        ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE, out_interleaved=out_il)
        assert_int8_close(got, ref, what="affine", max_frac_off=1e-3)
    elif epi == 1:
        alpha = (alpha * 0.06).astype(np.float32)
        beta = (beta * 0.02).astype(np.float32)
        got = run_gpu(a, w, alpha, beta, capi.LINEAR_GELU, out_scale=31.75, a_il=il, w_il=il, out_il=out_il)
        ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_GELU, out_scale=31.75, out_interleaved=out_il)
        assert_int8_close(got, ref, what="gelu", max_frac_off=2e-3)
    else:
        got = run_gpu(a, w, alpha, beta, capi.LINEAR_AFFINE_FP16, a_il=il, w_il=il)
        ref = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_AFFINE_FP16)
        assert_fp_close(got, ref, what="fp16 output")


def test_output_untouched_beyond_the_problem():
    """Rows beyond T and the bytes of neighbouring allocations are never written."""
    import torch
    api = capi.api()
    T, K, N = 130, 128, 96
    a, w, alpha, beta = problem(5, T, K, N)
    da, dw, dal, dbe = dev(a), dev(w), dev(alpha), dev(beta)
    out = dev_empty((T + 64, N), np.int8, fill=55)
    p = capi.Int8LinearParams()
    p.a, p.w, p.alpha, p.beta, p.out = da.data_ptr(), dw.data_ptr(), dal.data_ptr(), dbe.data_ptr(), out.data_ptr()
    p.T, p.K, p.N, p.epilogue = T, K, N, capi.LINEAR_AFFINE
    api.check(api.int8_linear(torch.cuda.current_stream().cuda_stream, C.byref(p)))
    torch.cuda.synchronize()
    got = host(out)
    assert (got[T:] == 55).all()
    assert_int8_close(got[:T], oracle.int8_linear(a, w, alpha, beta), what="affine")


def test_bad_arguments_are_refused():
    api = capi.api()
    p = capi.Int8LinearParams()
    assert api.int8_linear(None, C.byref(p)) != 0
    a, w, alpha, beta = problem(1, 16, 64, 32)
    da, dw, dal, dbe = dev(a), dev(w), dev(alpha), dev(beta)
    out = dev_empty((16, 32), np.int8)
    p.a, p.w, p.alpha, p.beta, p.out = da.data_ptr(), dw.data_ptr(), dal.data_ptr(), dbe.data_ptr(), out.data_ptr()
    for T, K, N in [(16, 48, 32), (16, 64, 40), (-1, 64, 32)]:
        p.T, p.K, p.N = T, K, N
        assert api.int8_linear(None, C.byref(p)) != 0
        assert "int8_linear" in api.last_error_str()
    p.T, p.K, p.N, p.epilogue, p.out_interleaved = 16, 64, 32, capi.LINEAR_RAW_INT32, 1
    assert api.int8_linear(None, C.byref(p)) != 0


# ---- FP16 operands ---------------------------------------------------------------------------------

def run_fp16(a, w, alpha, beta, gelu):
    import torch
    api = capi.api()
    T, K = a.shape
    N = w.shape[0]
    da, dw, dal, dbe = dev(a), dev(w), dev(alpha), dev(beta)
    out = dev_empty((T, N), np.float16, fill=-7)
    p = capi.Fp16LinearParams()
    p.a, p.w, p.alpha, p.beta, p.out = da.data_ptr(), dw.data_ptr(), dal.data_ptr(), dbe.data_ptr(), out.data_ptr()
    p.T, p.K, p.N, p.epilogue = T, K, N, capi.LINEAR_GELU if gelu else capi.LINEAR_AFFINE
    api.check(api.fp16_linear(torch.cuda.current_stream().cuda_stream, C.byref(p)))
    torch.cuda.synchronize()
    return host(out)


@pytest.mark.parametrize("T,K,N", [(1, 32, 32), (77, 96, 64), (300, 768, 768), (519, 1024, 3072), (9000, 128, 1024),
                                   (16500, 128, 1024), (20000, 512, 512)])
@pytest.mark.parametrize("gelu", [False, True])
def test_fp16_linear(T, K, N, gelu):
    r = rng(61 + T)
    a = (r.standard_normal((T, K)) * 0.5).astype(np.float16)
    w = (r.standard_normal((N, K)) * (1.0 / np.sqrt(K))).astype(np.float16)
    alpha = r.uniform(0.5, 1.5, N).astype(np.float32)
    beta = (0.5 * r.standard_normal(N)).astype(np.float32)
    got = run_fp16(a, w, alpha, beta, gelu)
    ref = oracle.fp16_linear(a, w, alpha, beta, gelu)
    assert_fp_close(got, ref, what="fp16 linear")
    # and against binary64, so that the oracle's accumulation order is not what is being matched
    y = (a.astype(np.float64) @ w.astype(np.float64).T) * alpha[None, :] + beta[None, :]
    if gelu:
        from scipy.special import erf
        y = 0.5 * y * (1 + erf(y / np.sqrt(2)))
    assert_fp_close(got, y, what="fp16 linear vs binary64")


def test_fp16_linear_identity_is_exact_and_bad_arguments_are_refused():
    api = capi.api()
    a = (rng(3).standard_normal((50, 64))).astype(np.float16)
    got = run_fp16(a, np.eye(64, dtype=np.float16), np.ones(64, np.float32), np.zeros(64, np.float32), False)
    assert np.array_equal(got, a)
    p = capi.Fp16LinearParams()
    assert api.fp16_linear(None, C.byref(p)) != 0
    d = dev(a)
    p.a = p.w = p.alpha = p.beta = p.out = d.data_ptr()
    p.T, p.K, p.N = 50, 48, 64
    assert api.fp16_linear(None, C.byref(p)) != 0 and "fp16_linear" in api.last_error_str()
