"""Layout / quantisation reformats on the GPU against the CPU oracle, through the C-ABI.
Pure byte permutations and the quantiser are bit-exact (the division and the rounding are IEEE on
both sides); the dequantiser is one binary32 product rounded to binary16, also exact."""
import numpy as np
import pytest

import oracle
from helpers import dev, dev_empty, host, rng
from tensorrt_amd import capi

pytestmark = pytest.mark.gpu

SHAPES = [(1, 32), (31, 64), (32, 256), (100, 288), (1000, 1024), (777, 3072), (4099, 4096)]


def stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def sync():
    import torch
    torch.cuda.synchronize()


@pytest.mark.parametrize("T,C", SHAPES)
def test_int8_layout_round_trip(T, C):
    api = capi.api()
    x = rng(T + C).integers(-128, 128, (T, C)).astype(np.int8)
    dx = dev(x)
    il = dev_empty((C // 32, T, 32), np.int8, fill=77)
    api.check(api.int8_linear_to_interleaved(stream(), T, C, dx.data_ptr(), il.data_ptr()))
    sync()
    assert np.array_equal(host(il).ravel(), oracle.interleave(x))
    back = dev_empty((T, C), np.int8, fill=77)
    api.check(api.int8_interleaved_to_linear(stream(), T, C, il.data_ptr(), back.data_ptr()))
    sync()
    assert np.array_equal(host(back), x)


@pytest.mark.parametrize("T,C", SHAPES)
def test_quantize_and_dequantize(T, C):
    api = capi.api()
    r = rng(3 * T + C)
    x = (r.standard_normal((T, C)) * 2).astype(np.float16)
    x.ravel()[:6] = [0.5, 1.5, -2.5, 300.0, -300.0, 0.0]
    for scale in (1.0, 0.0421):
        dx = dev(x)
        q = dev_empty((C // 32, T, 32), np.int8, fill=77)
        api.check(api.quantize_fp16_to_interleaved(stream(), T, C, dx.data_ptr(), scale, q.data_ptr()))
        sync()
        want = oracle.quantize_f16_interleave(x, scale)
        assert np.array_equal(host(q), want)
        y = dev_empty((T, C), np.float16, fill=-7)
        api.check(api.dequantize_interleaved_to_fp16(stream(), T, C, q.data_ptr(), scale, y.data_ptr()))
        sync()
        assert np.array_equal(host(y), oracle.dequantize_deinterleave_f16(want, scale))


def test_reformat_refuses_bad_arguments():
    api = capi.api()
    x = dev(np.zeros((4, 64), np.int8))
    y = dev_empty((2, 4, 32), np.int8)
    assert api.int8_linear_to_interleaved(None, 4, 48, x.data_ptr(), y.data_ptr()) != 0
    assert "multiple of 32" in api.last_error_str()
    assert api.int8_linear_to_interleaved(None, 4, 64, None, y.data_ptr()) != 0
    assert api.quantize_fp16_to_interleaved(None, 4, 64, x.data_ptr(), 0.0, y.data_ptr()) != 0
    assert api.int8_linear_to_interleaved(None, 0, 64, x.data_ptr(), y.data_ptr()) == 0
