"""GPU parity of the embedding + LayerNorm, mask index and packed mask kernels."""
import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, dev, dev_empty, host, layer_norm_f64, ptr, rng, stream, sync

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from tensorrt_amd import capi
    return capi.api()


def _tables(r, vocab, npos, ld, dt):
    word = (r.standard_normal((vocab, ld)) * 0.02).astype(dt)
    pos = (r.standard_normal((npos, ld)) * 0.02).astype(dt)
    tok = (r.standard_normal((2, ld)) * 0.02).astype(dt)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float32)
    beta = (r.standard_normal(ld) * 0.1).astype(np.float32)
    return word, pos, tok, gamma, beta


def _closed(word, pos, tok, ids, segs, positions, gamma, beta, dt):
    """(word + tok) + pos in T, LayerNorm without epsilon in float64, gamma/beta rounded to T."""
    v = (word[ids] + tok[segs]) + pos[positions]
    g = gamma.astype(dt).astype(np.float64)
    b = beta.astype(dt).astype(np.float64)
    return v, layer_norm_f64(v.astype(np.float64), g, b, 0.0)


# the reference's named config (fp32, vocab 100, 20 positions, E=128), BERT-base fp16, odd sizes
@pytest.mark.parametrize("dt,S,B,ld,vocab", [(np.float32, 20, 3, 128, 100), (np.float16, 128, 32, 768, 30522),
                                              (np.float16, 7, 5, 1024, 1000), (np.float32, 5, 2, 36, 50),
                                              (np.float16, 4, 3, 2048, 64)])
def test_embln_fixed(api, dt, S, B, ld, vocab):
    r = rng(11)
    word, pos, tok, gamma, beta = _tables(r, vocab, max(S, 8), ld, dt)
    ids = r.integers(0, vocab, (S, B)).astype(np.int32)
    segs = r.integers(0, 2, (S, B)).astype(np.int32)
    out = dev_empty((S * B, ld), dt, fill=0)
    d = [dev(a) for a in (ids, segs, beta, gamma, word, pos, tok)]
    fn = api.emb_layer_norm_fp32 if dt == np.float32 else api.emb_layer_norm_fp16
    api.check(fn(stream(), ld, B, S, *(ptr(t) for t in d), vocab, 2, ptr(out)))
    sync()
    got = host(out)
    positions = np.repeat(np.arange(S), B)
    _, closed = _closed(word, pos, tok, ids.ravel(), segs.ravel(), positions, gamma, beta, dt)
    tol = dict(atol=1e-5, rtol=1e-5) if dt == np.float32 else {}
    assert_fp_close(got, closed, what="vs closed form", **tol)
    ref, _, valid = oracle.embln(0, ids, segs, None, beta, gamma, word, pos, tok, S, B)
    assert valid.all()
    assert_fp_close(got, ref, what="vs oracle")


@pytest.mark.parametrize("dt,mode", [(np.float16, 1), (np.float16, 2), (np.float32, 1), (np.float32, 2)])
def test_embln_varseqlen(api, dt, mode):
    r = rng(12)
    B, S, ld, vocab = 9, 48, 768, 500
    lens = r.integers(1, S + 1, B)
    lens[3] = 0  # an empty sequence
    lens[5] = S
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    word, pos, tok, gamma, beta = _tables(r, vocab, S, ld, dt)
    ids = r.integers(0, vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    out = dev_empty((T, ld), dt, fill=0)
    skip = dev_empty((T, ld), dt, fill=0) if mode == 2 else None
    d = [dev(a) for a in (ids, segs, cu, beta, gamma, word, pos, tok)]
    suffix = "fp32" if dt == np.float32 else "fp16"
    if mode == 1:
        fn = getattr(api, f"emb_layer_norm_hface_{suffix}")
        api.check(fn(stream(), ld, B, S, *(ptr(t) for t in d), vocab, 2, ptr(out)))
    else:
        fn = getattr(api, f"emb_layer_norm_mtron_{suffix}")
        api.check(fn(stream(), ld, B, S, *(ptr(t) for t in d), vocab, 2, ptr(out), ptr(skip)))
    sync()
    positions = np.concatenate([np.arange(n) for n in lens]).astype(np.int64)
    v, closed = _closed(word, pos, tok, ids, segs, positions, gamma, beta, dt)
    tol = dict(atol=1e-5, rtol=1e-5) if dt == np.float32 else {}
    assert_fp_close(host(out), closed, what="vs closed form", **tol)
    ref, ref_skip, valid = oracle.embln(mode, ids, segs, cu, beta, gamma, word, pos, tok, S, B)
    assert valid.all()
    assert_fp_close(host(out), ref, what="vs oracle")
    if mode == 2:
        # the gather is exact: the pre-LayerNorm sum matches bit for bit
        bits = np.uint16 if dt == np.float16 else np.uint32
        assert np.array_equal(host(skip).view(bits), v.view(bits))
        assert np.array_equal(host(skip).view(bits), ref_skip.view(bits))


def test_embln_out_of_range_ids(api):
    """Out-of-range ids: the reference leaves the row undefined; this library writes beta and
    touches nothing outside the row."""
    r = rng(13)
    S, B, ld, vocab = 4, 2, 768, 10
    word, pos, tok, gamma, beta = _tables(r, vocab, S, ld, np.float16)
    ids = r.integers(0, vocab, (S, B)).astype(np.int32)
    segs = np.zeros((S, B), np.int32)
    ids[1, 1] = vocab
    ids[2, 0] = -1
    segs[3, 1] = 2
    out = dev_empty((S * B, ld), np.float16, fill=0)
    d = [dev(a) for a in (ids, segs, beta, gamma, word, pos, tok)]
    api.check(api.emb_layer_norm_fp16(stream(), ld, B, S, *(ptr(t) for t in d), vocab, 2, ptr(out)))
    sync()
    got = host(out)
    _, _, valid = oracle.embln(0, ids, segs, None, beta, gamma, word, pos, tok, S, B)
    bad = np.flatnonzero(valid == 0)
    assert set(bad) == {1 * B + 1, 2 * B + 0, 3 * B + 1}
    for row in bad:
        assert np.array_equal(got[row], beta.astype(np.float16))
    assert np.isfinite(got).all()


@pytest.mark.parametrize("S,B", [(8, 3), (32, 4), (128, 32), (384, 7), (200, 5), (1, 1)])
def test_mask_idx(api, S, B):
    r = rng(14)
    lens = r.integers(0, S + 1, B)
    lens[0] = S
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    if S > 4:
        mask[S - 1, B - 1] = 1  # a non-prefix mask: first zero still wins
    out = dev_empty((B,), np.int32, fill=-1)
    dm = dev(mask)
    api.check(api.compute_mask_idx(stream(), S, B, ptr(dm), ptr(out)))
    sync()
    assert np.array_equal(host(out), oracle.mask_idx(mask))


@pytest.mark.parametrize("S,wm,wn", [(64, 2, 2), (96, 2, 2), (128, 2, 2), (384, 1, 8), (192, 1, 4), (256, 1, 4),
                                     (512, 1, 8)])
def test_convert_mask(api, S, wm, wn):
    r = rng(15)
    B = 6
    lens = r.integers(1, S + 1, B)
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    mask[:, 1] = r.integers(0, 2, S)  # arbitrary (non-prefix) mask
    mask[:, 2] = 7 * mask[:, 2]       # only the value 1 counts as valid
    ref, over = oracle.convert_mask(mask, wm, wn)
    assert over == 0
    out = dev_empty(ref.shape, np.uint32, fill=0)
    dm = dev(mask)
    api.check(api.convert_mask(S, B, wm, wn, 1, ptr(dm), ptr(out), stream()))
    sync()
    assert np.array_equal(host(out, np.uint32), ref)
