"""GPU parity of the unfused attention path (head sizes <= 128: one launch that keeps a query's scores in registers
for S <= 512 and walks the keys twice beyond; larger head sizes: the strided batched GEMMs around the scaled/masked
softmax) and of zeroPadding2d, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, attention_f64, dev, dev_empty, host, ptr, rng, stream, sync
from tensorrt_amd import capi

STATUS_BAD_PARAM, STATUS_NOT_SUPPORTED = 2, 3

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("S,masked", [(16, True), (128, True), (384, False), (100, True), (1000, True), (33, False),
                                      (1024, True), (1536, False), (2048, True), (2056, True)])
def test_scaled_softmax(api, dt, S, masked):
    r = rng(200 + S)
    B, N = 3, 2
    x = (3 * r.standard_normal((B, N, S, S))).astype(dt)
    lens = np.array([S, 1, max(1, S // 3)], np.int32) if masked else None
    out = dev_empty((B, N, S, S), dt, fill=1)
    fn = api.scaled_softmax_fp32 if dt == np.float32 else api.scaled_softmax_fp16
    d_len = dev(lens) if masked else None
    d_x = dev(x)    # held until the result is back: a temporary's memory may be handed out again
    api.check(fn(stream(), S, B, N, 0.125, ptr(d_len), ptr(d_x), ptr(out)))
    sync()
    got = host(out)
    ref = oracle.scaled_softmax(x, 0.125, lens)
    assert_fp_close(got, ref, atol=1e-5 if dt == np.float32 else 1e-3, rtol=1e-4 if dt == np.float32 else 2e-3,
                    what="softmax")
    if masked:
        for b in range(B):
            assert not got[b][..., lens[b]:].any()      # masked positions are exactly zero


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("S,B,N,d,masked", [(128, 2, 12, 64, True), (20, 3, 2, 32, True), (77, 1, 3, 48, False),
                                            (384, 1, 2, 64, True), (5, 2, 1, 8, False), (130, 2, 2, 128, True),
                                            # the last sizes of the one-launch kernel and the first beyond them
                                            (512, 1, 2, 64, True), (513, 1, 2, 64, True), (60, 2, 2, 129, True),
                                            (250, 2, 3, 20, True), (1, 3, 2, 64, False), (65, 1, 1, 100, True),
                                            # two passes over the keys: ragged last stage, every stage whole, head sizes
                                            # that are not multiples of the vector width, no mask
                                            (1024, 1, 2, 64, True), (1024, 2, 1, 64, False), (700, 2, 2, 72, True),
                                            (1500, 1, 1, 128, True), (600, 1, 2, 33, True)])
def test_unfused_mha(api, dt, S, B, N, d, masked):
    r = rng(210 + S + d)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = r.integers(1, S + 1, B).astype(np.int32) if masked else None
    type_id = 0 if dt == np.float32 else 1
    ws_bytes = api.unfused_mha_workspace_size(type_id, S, B, N)
    ws = dev_empty((ws_bytes,), np.uint8)
    out = dev_empty((S, B, N * d), dt, fill=0)
    d_len = dev(lens) if masked else None
    d_qkv = dev(qkv)
    api.check(api.unfused_mha(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(out), ptr(ws)))
    sync()
    got = host(out)
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens)
    tol = dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}
    assert_fp_close(got, ref, what="vs oracle", **tol)
    # and against float64 attention for one (sequence, head)
    t = qkv.reshape(S, B, N, 3, d)
    L = int(lens[0]) if masked else S
    closed = attention_f64(t[:, 0, 0, 0], t[:L, 0, 0, 1], t[:L, 0, 0, 2], 1 / np.sqrt(d))
    assert_fp_close(got.reshape(S, B, N, d)[:, 0, 0], closed, what="vs float64",
                    **(dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else dict(atol=4e-3, rtol=1e-2)))


def _run_unfused(api, dt, S, B, N, d, qkv, lens):
    type_id = 0 if dt == np.float32 else 1
    ws = dev_empty((api.unfused_mha_workspace_size(type_id, S, B, N),), np.uint8)
    out = dev_empty((S, B, N * d), dt, fill=1)
    d_len = dev(lens) if lens is not None else None
    d_qkv = dev(qkv)
    api.check(api.unfused_mha(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(out), ptr(ws)))
    sync()
    return host(out)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("S,B,N,d", [(384, 3, 4, 64), (200, 2, 2, 128), (97, 2, 3, 40), (512, 1, 2, 32),
                                     (640, 2, 2, 64), (1000, 1, 2, 128), (777, 2, 1, 40), (513, 1, 1, 8)])
def test_one_launch_against_the_three_kernels(api, dt, S, B, N, d):
    """Both routes round scores and probabilities to the storage type at the same places; what is left between them
    is the order of the binary32 sums."""
    r = rng(800 + S + d)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    lens[0] = S
    api.check(api.test_set_tuning(b"TRTAMD_UNFUSED_SPLIT", 1))
    try:
        split = _run_unfused(api, dt, S, B, N, d, qkv, lens)
    finally:
        api.check(api.test_reset_tuning(b"TRTAMD_UNFUSED_SPLIT"))
    one = _run_unfused(api, dt, S, B, N, d, qkv, lens)
    tol = dict(atol=2e-6, rtol=2e-5) if dt == np.float32 else dict(atol=1e-3, rtol=2e-3)
    assert_fp_close(one, split, what="one launch vs three kernels", **tol)
    assert_fp_close(one, oracle.mha_unfused_fixed(qkv, S, B, N, d, lens), what="vs oracle",
                    **(dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}))


def _run_routed(api, route, dt, S, B, N, d, qkv, lens):
    ws = dev_empty((api.unfused_mha_workspace_size(0 if dt == np.float32 else 1, S, B, N),), np.uint8)
    out = dev_empty((S, B, N * d), dt, fill=0)
    d_qkv, d_len = dev(qkv), dev(lens)    # held until the result is back
    st = api.unfused_mha_routed(stream(), route, 0 if dt == np.float32 else 1, S, B, N, d, ptr(d_qkv), ptr(d_len),
                                ptr(out), ptr(ws))
    sync()
    return st, host(out)


@pytest.mark.parametrize("dt,S,B,N,d", [(np.float16, 300, 3, 4, 64), (np.float32, 640, 2, 2, 128),
                                        (np.float16, 1030, 2, 3, 80), (np.float32, 77, 5, 2, 24)])
def test_routes_and_their_tuning(api, dt, S, B, N, d):
    """The route can be named; both give the oracle's result, "by shape" is the default entry point, and the tuning
    call times both and returns the faster."""
    r = rng(870 + S)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens)
    tol = dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}
    got = {}
    for route in (capi.UNFUSED_ROUTE_ONE_LAUNCH, capi.UNFUSED_ROUTE_THREE_LAUNCHES, capi.UNFUSED_ROUTE_BY_SHAPE):
        st, got[route] = _run_routed(api, route, dt, S, B, N, d, qkv, lens)
        assert st == 0, api.last_error_str()
        assert_fp_close(got[route], ref, what=f"route {route} vs oracle", **tol)
    assert np.array_equal(got[capi.UNFUSED_ROUTE_BY_SHAPE], _run_unfused(api, dt, S, B, N, d, qkv, lens))
    assert np.array_equal(got[capi.UNFUSED_ROUTE_BY_SHAPE], got[capi.UNFUSED_ROUTE_ONE_LAUNCH]), "head sizes <= 128"
    route, us = C.c_int32(-5), (C.c_float * 2)(0, 0)
    api.check(api.unfused_mha_tune(0 if dt == np.float32 else 1, S, B, N, d, C.byref(route), us))
    assert us[0] > 0 and us[1] > 0
    assert route.value == (capi.UNFUSED_ROUTE_THREE_LAUNCHES if us[1] < us[0] else capi.UNFUSED_ROUTE_ONE_LAUNCH)


def test_routes_that_do_not_exist(api):
    S, B, N, d = 40, 2, 2, 136
    r = rng(880)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(np.float16)
    lens = np.array([40, 9], np.int32)
    st, _ = _run_routed(api, capi.UNFUSED_ROUTE_ONE_LAUNCH, np.float16, S, B, N, d, qkv, lens)
    assert st == STATUS_NOT_SUPPORTED and "head size" in api.last_error_str()
    st, _ = _run_routed(api, 7, np.float16, S, B, N, d, qkv, lens)
    assert st == STATUS_BAD_PARAM and "route" in api.last_error_str()
    st, got = _run_routed(api, capi.UNFUSED_ROUTE_THREE_LAUNCHES, np.float16, S, B, N, d, qkv, lens)
    assert st == 0
    assert_fp_close(got, oracle.mha_unfused_fixed(qkv, S, B, N, d, lens), what="three launches, head size 136")
    # above 128 there is one route and nothing to time
    route, us = C.c_int32(-5), (C.c_float * 2)(0, 0)
    api.check(api.unfused_mha_tune(1, S, B, N, d, C.byref(route), us))
    assert route.value == capi.UNFUSED_ROUTE_THREE_LAUNCHES and us[0] == -1 and us[1] == -1
    assert api.unfused_mha_tune(2, S, B, N, 64, C.byref(route), None) == STATUS_NOT_SUPPORTED
    assert route.value == capi.UNFUSED_ROUTE_BY_SHAPE
    assert api.unfused_mha_tune(1, 0, B, N, 64, C.byref(route), None) == STATUS_BAD_PARAM
    assert api.unfused_mha_tune(1, S, B, N, 64, None, None) == STATUS_BAD_PARAM


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("S", [70, 600])
def test_unfused_mha_batch_without_valid_keys(api, dt, S):
    """A batch whose mask leaves no key gets exact zeros (every probability is 0), its neighbours are untouched by
    that; a length beyond S means all of S."""
    B, N, d = 3, 2, 64
    r = rng(840 + S)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = np.array([0, S + 5, S // 2], np.int32)
    got = _run_unfused(api, dt, S, B, N, d, qkv, lens)
    assert not got[:, 0].any()
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, np.array([0, S, S // 2], np.int32))
    assert_fp_close(got, ref, what="vs oracle", **(dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}))


def test_unfused_mha_unaligned_operands(api):
    """Operands that start 2 bytes off a 16-byte boundary take the element-wise loads and stores."""
    S, B, N, d = 90, 2, 2, 64
    r = rng(860)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(np.float16)
    lens = np.array([90, 31], np.int32)
    raw_in = dev_empty((qkv.size + 8,), np.float16, fill=0)
    raw_in[1:1 + qkv.size].copy_(dev(qkv).reshape(-1))
    raw_out = dev_empty((S * B * N * d + 8,), np.float16, fill=0)
    ws = dev_empty((api.unfused_mha_workspace_size(1, S, B, N),), np.uint8)
    d_len = dev(lens)
    api.check(api.unfused_mha(stream(), 1, S, B, N, d, ptr(raw_in) + 2, ptr(d_len), ptr(raw_out) + 2, ptr(ws)))
    sync()
    got = host(raw_out)
    assert got[0] == 0 and not got[1 + S * B * N * d:].any()
    assert_fp_close(got[1:1 + S * B * N * d].reshape(S, B, N * d), oracle.mha_unfused_fixed(qkv, S, B, N, d, lens),
                    what="vs oracle")


def test_unfused_mha_rejects_int8(api):
    assert api.unfused_mha(None, 2, 16, 1, 1, 64, 0, 0, 0, 0) != 0
    assert "data type" in api.last_error_str()


@pytest.mark.parametrize("spitch,dpitch,height", [(64, 128, 1000), (80, 128, 7), (32, 64, 333), (128, 64, 50),
                                                  (64, 64, 9), (2, 64, 5)])
def test_zero_padding_2d(api, spitch, dpitch, height):
    r = rng(220 + spitch)
    src = r.integers(0, 256, height * spitch).astype(np.uint8)
    dst = dev_empty((height * dpitch,), np.uint8, fill=0xAB)
    d_src = dev(src)
    api.check(api.zero_padding_2d(ptr(d_src), spitch, ptr(dst), dpitch, height, stream()))
    sync()
    assert np.array_equal(host(dst), oracle.zero_padding_2d(src, spitch, dpitch, height))


def test_zero_padding_round_trip_at_attention_size(api):
    """Pad [T,N,3,32] to head size 64 and strip it again: identity."""
    T, N = 2048, 16
    src = rng(221).integers(0, 256, T * N * 3 * 32 * 2).astype(np.uint8)   # binary16 elements
    rows = T * N * 3
    mid = dev_empty((rows * 128,), np.uint8)
    back = dev_empty((rows * 64,), np.uint8)
    d_src = dev(src)
    api.check(api.zero_padding_2d(ptr(d_src), 64, ptr(mid), 128, rows, stream()))
    api.check(api.zero_padding_2d(ptr(mid), 128, ptr(back), 64, rows, stream()))
    sync()
    assert np.array_equal(host(back), src)
    assert not host(mid).reshape(rows, 128)[:, 64:].any()
