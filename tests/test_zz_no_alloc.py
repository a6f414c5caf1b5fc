"""trtamd_unfused_mha_static: the unfused attention with the library's own score-matrix array instead of a caller
workspace, for callers that cannot allocate.  Its output must equal trtamd_unfused_mha's bit for bit (same kernels),
which in turn is held to the floating-point bar against the oracle here; two calls in a row, the second on a
smaller input, share the array.  Head sizes beyond 128 are the ones whose score matrices go through the array; the
others run in a one-launch kernel that stores no score."""
import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, dev, dev_empty, host, ptr, rng, stream, sync

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


def _both(api, dt, S, B, N, d, seed):
    r = rng(seed)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    type_id = 0 if dt == np.float32 else 1
    d_qkv, d_len = dev(qkv), dev(lens)
    ws = dev_empty((api.unfused_mha_workspace_size(type_id, S, B, N),), np.uint8, fill=0)
    want = dev_empty((S, B, N * d), dt, fill=0)
    got = dev_empty((S, B, N * d), dt, fill=0)
    api.check(api.unfused_mha(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(want), ptr(ws)))
    api.check(api.unfused_mha_static(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(got)))
    sync()
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens)
    tol = dict(atol=2e-5, rtol=1e-4) if dt == np.float32 else {}
    assert_fp_close(host(want), ref, what="workspace entry point vs oracle", **tol)
    u = np.uint32 if dt == np.float32 else np.uint16
    assert np.array_equal(host(got).view(u), host(want).view(u)), "static-scratch entry point differs"


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_two_calls_in_a_row_second_smaller(api, dt):
    _both(api, dt, 320, 2, 3, 136, seed=301)    # fills 2 * 320*320 * 6 scores of the array
    _both(api, dt, 100, 1, 2, 144, seed=302)    # a smaller problem over what the first call left behind
    _both(api, dt, 320, 2, 3, 136, seed=303)    # and a larger one again
    _both(api, dt, 640, 2, 3, 64, seed=304)     # a shape of the one-launch kernels in between


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_two_calls_in_a_row_in_registers(api, dt):
    _both(api, dt, 200, 3, 4, 64, seed=311)     # no score matrix: nothing of the array is touched
    _both(api, dt, 77, 2, 3, 32, seed=312)
    _both(api, dt, 200, 3, 4, 64, seed=313)


def test_shapes_that_stay_in_registers_have_no_limit(api):
    """Head sizes up to 128 need no score matrix: accepted although the reference's workspace for it would be
    three times the array."""
    S, B, N, d = 384, 16, 12, 64
    assert api.unfused_mha_workspace_size(1, S, B, N) > api.unfused_mha_static_capacity()
    _both(api, np.float16, S, B, N, d, seed=321)


def test_sizes_beyond_the_array_are_refused(api):
    cap = api.unfused_mha_static_capacity()
    assert cap == 32 << 20
    S, B, N = 1024, 2, 4                        # 2 * 4 * 1024^2 * 8 = 64 MiB of FP32 scores
    assert api.unfused_mha_workspace_size(0, S, B, N) > cap
    x = dev_empty((16,), np.float32, fill=0)
    # head size 136: a shape whose scores go through the array (refused before anything is launched)
    st = api.unfused_mha_static(stream(), 0, S, B, N, 136, ptr(x), 0, ptr(x))
    assert st == 3 and "static scratch" in api.last_error_str() and "workspace" in api.last_error_str()
    # exactly at the capacity is accepted: 2 * 2 * 512^2 * 32 = 32 MiB of FP16 scores
    assert api.unfused_mha_workspace_size(1, 512, 2, 16) == cap
    assert api.unfused_mha_static(stream(), 5, 16, 1, 1, 8, ptr(x), 0, ptr(x)) == 3      # INT8 etc.: as the other entry
    assert api.unfused_mha_static(stream(), 0, 0, 1, 1, 8, ptr(x), 0, ptr(x)) == 2


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_captured_in_a_graph_and_no_device_memory_taken(api, dt):
    """The entry point under stream capture (the array's address looked up beforehand): every replay, with eager work
    between the replays, gives the eager result, and the calls leave the amount of free device memory as it was."""
    import torch
    S, B, N, d = 320, 2, 3, 136                 # scores go through the array
    r = rng(331)
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = np.array([S, 150], np.int32)
    type_id = 0 if dt == np.float32 else 1
    d_qkv, d_len = dev(qkv), dev(lens)
    eager = dev_empty((S, B, N * d), dt, fill=0)
    got = dev_empty((S, B, N * d), dt, fill=0)
    api.check(api.unfused_mha_static_prepare())
    api.check(api.unfused_mha_static(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(eager)))
    sync()
    # no allocation by anyone between the two readings: only calls of the entry point
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        api.check(api.unfused_mha_static(stream(), type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(got)))
    sync()
    assert torch.cuda.mem_get_info()[0] == free_before, "the calls changed the amount of free device memory"
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            api.check(api.unfused_mha_static(side.cuda_stream, type_id, S, B, N, d, ptr(d_qkv), ptr(d_len), ptr(got)))
    u = np.uint32 if dt == np.float32 else np.uint16
    for replay in range(3):
        got.zero_()
        # eager work of the same entry point on another problem between the replays: it overwrites the array
        _both(api, dt, 100, 1, 2, 144, seed=340 + replay)
        graph.replay()
        sync()
        assert np.array_equal(host(got).view(u), host(eager).view(u)), f"replay {replay} differs from the eager call"
    del graph
