"""GPU parity of the SkipLayerNorm kernels (through the C ABI) against the CPU oracle and the
float64 closed form.  Tolerances: floating point |a-b| <= 2e-3 + 1e-2*|b|; INT8 +-1 LSB."""
import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, assert_int8_close, dev, dev_empty, host, layer_norm_f64, ptr, rng, stream, sync)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


def _ln_params(r, ld, dt):
    gamma = r.uniform(0.5, 1.5, ld).astype(dt)
    beta = (r.standard_normal(ld) * 0.1).astype(dt)
    bias = (r.standard_normal(ld) * 0.02).astype(dt)
    return gamma, beta, bias


def _eps(dt, ld):
    if ld in (768, 1024):
        return 2.0 ** -23 if dt == np.float32 else 2.0 ** -10
    return 0.0


# rows x ld: the reference's named configs (fp32 ld=128, fp16 ld=768 with bias), the benchmark
# shapes, ragged/odd sizes that take the generic kernel, and row counts that do not fill a wave.
FP_CASES = [
    (np.float32, 1024, 768, True), (np.float32, 7, 128, True), (np.float32, 33, 1024, False),
    (np.float16, 4096, 768, True), (np.float16, 5, 768, False), (np.float16, 130, 1024, True),
    (np.float16, 9, 100, True), (np.float32, 9, 20, False), (np.float32, 3, 30, True), (np.float16, 17, 2048, True),
    (np.float32, 17, 2048, False), (np.float16, 11, 4096, False), (np.float32, 2, 5000, True), (np.float16, 1, 8, False),
]


@pytest.mark.parametrize("dt,rows,ld,has_bias", FP_CASES)
def test_skipln_fp(api, dt, rows, ld, has_bias):
    r = rng(1)
    x = r.standard_normal((rows, ld)).astype(dt)
    skip = r.standard_normal((rows, ld)).astype(dt)
    gamma, beta, bias = _ln_params(r, ld, dt)
    if not has_bias:
        bias = None
    d_out = dev_empty((rows, ld), dt, fill=0)
    d = [dev(a) if a is not None else None for a in (x, skip, beta, gamma, bias)]
    fn = api.skip_layer_norm_fp32 if dt == np.float32 else api.skip_layer_norm_fp16
    api.check(fn(stream(), ld, rows * ld, ptr(d[0]), ptr(d[1]), ptr(d[2]), ptr(d[3]), ptr(d_out), ptr(d[4])))
    sync()
    got = host(d_out)
    # the residual sum is formed in T, as the reference does
    v = x + skip
    if has_bias:
        v = v + bias
    closed = layer_norm_f64(v.astype(np.float64), gamma, beta, _eps(dt, ld))
    assert_fp_close(got, closed, what="vs float64 closed form")
    ref = oracle.skipln(x, skip, beta, gamma, bias)
    assert_fp_close(got, ref, what="vs oracle")


def test_skipln_fp_errors(api):
    assert api.skip_layer_norm_fp32(None, 768, 100, 0, 0, 0, 0, 0, 0) != 0   # n % ld != 0
    assert "multiple" in api.last_error_str()
    assert api.skip_layer_norm_fp16(None, 768, 768, 0, 0, 0, 0, 0, 0) != 0   # null pointers
    assert api.skip_layer_norm_fp16(None, 768, 0, 0, 0, 0, 0, 0, 0) == 0     # empty tensor


def test_skipln_fp_row_permutation(api):
    """Rows are independent: permuting rows permutes outputs bit for bit."""
    r = rng(5)
    rows, ld = 257, 768
    x = r.standard_normal((rows, ld)).astype(np.float16)
    s = r.standard_normal((rows, ld)).astype(np.float16)
    gamma, beta, _ = _ln_params(r, ld, np.float16)
    perm = r.permutation(rows)

    def run(xx, ss):
        o = dev_empty((rows, ld), np.float16)
        dx, ds, db, dg = dev(xx), dev(ss), dev(beta), dev(gamma)
        api.check(api.skip_layer_norm_fp16(stream(), ld, rows * ld, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(o), 0))
        sync()
        return host(o)

    a = run(x, s)
    b = run(x[perm], s[perm])
    assert np.array_equal(a[perm].view(np.uint16), b.view(np.uint16))


def _int8_inputs(r, rows, ld):
    xf = r.standard_normal((rows, ld))
    sf = r.standard_normal((rows, ld)) * 0.7
    amax_x, amax_s = np.abs(xf).max(), np.abs(sf).max()
    x = np.clip(np.rint(xf * 127 / amax_x), -127, 127).astype(np.int8)
    s = np.clip(np.rint(sf * 127 / amax_s), -127, 127).astype(np.int8)
    return x, s, np.float32(amax_x / 127), np.float32(amax_s / 127)


@pytest.mark.parametrize("rows,ld,has_bias", [(64, 768, True), (1030, 1024, True), (3, 1024, False), (513, 768, False)])
def test_skipln_dqq(api, rows, ld, has_bias):
    r = rng(2)
    x, s, dq_in, dq_skip = _int8_inputs(r, rows, ld)
    gamma, beta, bias = _ln_params(r, ld, np.float16)
    if not has_bias:
        bias = None
    q_scale = np.float32(127.0 / 4.5)
    d_out = dev_empty((rows, ld), np.int8, fill=0)
    d = [dev(a) if a is not None else None for a in (x, s, beta, gamma, bias)]
    api.check(api.skip_layer_norm_dqq(stream(), ld, rows * ld, ptr(d[0]), ptr(d[1]), ptr(d[2]), ptr(d[3]), ptr(d_out),
                                      ptr(d[4]), dq_in, dq_skip, q_scale))
    sync()
    got = host(d_out)
    st, ref = oracle.skipln_dqq(x, s, beta, gamma, bias, dq_in, dq_skip, q_scale)
    assert st == 0
    assert_int8_close(got, ref, what="vs oracle")
    v = x.astype(np.float64) * float(dq_in) + s.astype(np.float64) * float(dq_skip)
    if has_bias:
        v = v + bias.astype(np.float64)
    closed = np.clip(np.rint(layer_norm_f64(v, gamma, beta, 2.0 ** -10) * float(q_scale)), -128, 127)
    assert_int8_close(got, closed, what="vs float64 closed form", max_frac_off=0.01)


def test_skipln_dqq_unsupported_ld(api):
    assert api.skip_layer_norm_dqq(None, 512, 512, 0, 0, 0, 0, 0, 0, 1.0, 1.0, 1.0) != 0
    assert "unsupported hidden layer size" in api.last_error_str()
    st, _ = oracle.skipln_dqq(np.zeros((1, 512), np.int8), np.zeros((1, 512), np.int8), np.zeros(512, np.float16),
                              np.zeros(512, np.float16), None, 1.0, 1.0, 1.0)
    assert st != 0


IL_CASES = [
    # variant (0 hface, 1 mtron), large, ld, total
    (0, False, 768, 100), (0, False, 1024, 1), (0, True, 1024, 4096), (0, True, 768, 4100),
    (1, False, 1024, 37), (1, True, 1024, 5000), (1, True, 768, 4097), (1, False, 2048, 19), (1, False, 4096, 9),
    (1, False, 1536, 33), (1, False, 3072, 8),
]


@pytest.mark.parametrize("variant,large,ld,total", IL_CASES)
def test_skipln_interleaved(api, variant, large, ld, total):
    r = rng(3)
    x, s, dq_in, dq_skip = _int8_inputs(r, total, ld)
    gamma, beta, _ = _ln_params(r, ld, np.float16)
    q_scale = np.float32(127.0 / 4.5)
    q_skip = np.float32(127.0 / 6.0)
    x_il, s_il = oracle.interleave(x), oracle.interleave(s)
    d_out = dev_empty((ld * total,), np.int8, fill=0)
    d_pre = dev_empty((ld * total,), np.int8, fill=0) if variant else None
    dx, ds, db, dg = dev(x_il), dev(s_il), dev(beta), dev(gamma)
    size = "large" if large else "small"
    if variant == 0:
        fn = getattr(api, f"skipln_interleaved_{size}_hface")
        api.check(fn(stream(), ld, total, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(d_out), dq_in, dq_skip, q_scale))
    else:
        fn = getattr(api, f"skipln_interleaved_{size}_mtron")
        api.check(fn(stream(), ld, total, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(d_out), ptr(d_pre), dq_in, dq_skip,
                     q_scale, q_skip))
    sync()
    st, ref, ref_pre = oracle.skipln_interleaved(variant, x_il, s_il, beta, gamma, ld, total, dq_in, dq_skip, q_scale,
                                                 q_skip, force=int(large))
    assert st == 0
    assert_int8_close(host(d_out), ref, what="out vs oracle")
    v = x.astype(np.float64) * float(dq_in) + s.astype(np.float64) * float(dq_skip)
    eps = 2.0 ** -23 if large else 2.0 ** -10
    closed = np.clip(np.rint(layer_norm_f64(v, gamma, beta, eps) * float(q_scale)), -128, 127)
    got_lin = oracle.deinterleave(host(d_out), total, ld)
    assert_int8_close(got_lin, closed, what="out vs float64 closed form", max_frac_off=0.01)
    if variant:
        assert_int8_close(host(d_pre), ref_pre, what="preln vs oracle")
        lo = -128 if large else -127
        closed_pre = np.clip(np.rint(v * float(q_skip)), lo, 127)
        assert_int8_close(oracle.deinterleave(host(d_pre), total, ld), closed_pre, what="preln closed form",
                          max_frac_off=0.01)


@pytest.mark.parametrize("variant,large,ld,total", [
    # token counts just above what one round of resident workgroups covers in blocks of 32 tokens (256 CUs x 4, x 2,
    # x 5 workgroups): the launch then is that one round, each workgroup taking one token more (the kernel's tail
    # path), up to 33 tokens per workgroup; one count beyond, one far beyond
    (0, True, 1024, 32769), (0, True, 1024, 33289), (0, True, 1024, 33792), (0, True, 1024, 33793),
    (1, True, 1024, 16385), (1, True, 1024, 16896), (1, False, 1024, 16700), (0, True, 768, 40999),
    (1, False, 2048, 16500), (1, False, 4096, 8300), (0, False, 768, 33000), (1, False, 1536, 16600),
    (1, False, 3072, 8200), (1, True, 1024, 24577),
])
def test_skipln_interleaved_one_round_with_tail(api, variant, large, ld, total):
    test_skipln_interleaved(api, variant, large, ld, total)


def test_skipln_interleaved_tail_launch_replays_from_a_graph(api):
    """The one-round launch (its workgroup count comes from an occupancy query, its extra tokens travel through LDS)
    recorded in a graph: every replay gives the eager bytes."""
    import torch
    ld, total = 1024, 33001
    r = rng(31)
    x, s, dq_in, dq_skip = _int8_inputs(r, total, ld)
    gamma, beta, _ = _ln_params(r, ld, np.float16)
    q_scale = np.float32(127.0 / 4.5)
    dx, ds, db, dg = dev(oracle.interleave(x)), dev(oracle.interleave(s)), dev(beta), dev(gamma)
    eager, replayed = dev_empty((ld * total,), np.int8, fill=0), dev_empty((ld * total,), np.int8, fill=0)
    api.check(api.skipln_interleaved_large_hface(stream(), ld, total, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(eager),
                                                 dq_in, dq_skip, q_scale))
    sync()
    graph, cap = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=cap):
        api.check(api.skipln_interleaved_large_hface(cap.cuda_stream, ld, total, ptr(dx), ptr(ds), ptr(db), ptr(dg),
                                                     ptr(replayed), dq_in, dq_skip, q_scale))
    for _ in range(3):
        replayed.zero_()
        sync()
        graph.replay()
        sync()
        assert np.array_equal(host(replayed), host(eager))


def test_skipln_interleaved_saturation(api):
    """preln: the small kernel clips to -127, the large one saturates to -128."""
    ld, total = 1024, 8
    x = np.full((total, ld), -127, np.int8)
    s = np.full((total, ld), -127, np.int8)
    x[:, ::2] = 100  # keep a non-zero variance
    gamma = np.ones(ld, np.float16)
    beta = np.zeros(ld, np.float16)
    dx, ds, db, dg = dev(oracle.interleave(x)), dev(oracle.interleave(s)), dev(beta), dev(gamma)
    for large, lo in ((False, -127), (True, -128)):
        out = dev_empty((ld * total,), np.int8)
        pre = dev_empty((ld * total,), np.int8)
        fn = api.skipln_interleaved_large_mtron if large else api.skipln_interleaved_small_mtron
        api.check(fn(stream(), ld, total, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(out), ptr(pre), 1.0, 1.0, 1.0, 1.0))
        sync()
        p = oracle.deinterleave(host(pre), total, ld)
        assert p[:, 1::2].min() == lo and p[:, 1::2].max() == lo   # -254 saturates/clips
        assert (p[:, ::2] == -27).all()


def test_skipln_interleaved_unsupported(api):
    assert api.skipln_interleaved_large_hface(None, 2048, 8, 0, 0, 0, 0, 0, 1.0, 1.0, 1.0) != 0
    assert api.skipln_interleaved_small_hface(None, 2048, 8, 0, 0, 0, 0, 0, 1.0, 1.0, 1.0) != 0
    assert api.skipln_interleaved_large_mtron(None, 2048, 8, 0, 0, 0, 0, 0, 0, 1.0, 1.0, 1.0, 1.0) != 0
    assert api.skipln_interleaved_small_hface(None, 1024, 0, 0, 0, 0, 0, 0, 1.0, 1.0, 1.0) == 0


def test_linear_vs_interleaved_same_values(api):
    """The same tensor through the linear INT8 kernel and through the interleaved one (small
    variant: same epsilon) gives the same bytes after re-layout, up to 1 LSB."""
    r = rng(4)
    rows, ld = 200, 1024
    x, s, dq_in, dq_skip = _int8_inputs(r, rows, ld)
    gamma, beta, _ = _ln_params(r, ld, np.float16)
    q = np.float32(127 / 4.0)
    o1 = dev_empty((rows, ld), np.int8)
    dx, ds, db, dg = dev(x), dev(s), dev(beta), dev(gamma)
    api.check(api.skip_layer_norm_dqq(stream(), ld, rows * ld, ptr(dx), ptr(ds), ptr(db), ptr(dg), ptr(o1), 0, dq_in,
                                      dq_skip, q))
    o2 = dev_empty((rows * ld,), np.int8)
    dxi, dsi = dev(oracle.interleave(x)), dev(oracle.interleave(s))
    api.check(api.skipln_interleaved_small_hface(stream(), ld, rows, ptr(dxi), ptr(dsi), ptr(db), ptr(dg), ptr(o2),
                                                 dq_in, dq_skip, q))
    sync()
    assert_int8_close(host(o1), oracle.deinterleave(host(o2), rows, ld), what="linear vs interleaved")
