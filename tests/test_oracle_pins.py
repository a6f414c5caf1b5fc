"""Pins the CPU oracle.

The reference ships no golden vectors for these plugins, so every oracle routine is checked here
against something the mathematics fixes independently of the oracle's own code: float64 closed
forms written with numpy, brute-force index loops, exact integer matrix products, invariants
(scale / permutation), and special cases with a known answer.  Each check is chosen so that a
plausible slip (swapped gamma/beta, dropped bias, wrong stride, transposed operand, off-by-one
mask) fails it.
"""
import numpy as np
import pytest

import oracle
from helpers import attention_f64, layer_norm_f64, rng

# oracle-vs-float64 agreement: binary32 paths are tight, binary16 paths carry half rounding
F32_TOL = dict(atol=2e-5, rtol=2e-5)
F16_TOL = dict(atol=3e-2, rtol=3e-2)


def close(a, b, atol, rtol):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    err = np.abs(a - b)
    assert (err <= atol + rtol * np.abs(b)).all(), f"max err {err.max():.3e}"


# ---- conversions ---------------------------------------------------------------------------------

def test_binary16_rounding_matches_ieee():
    r = rng(1)
    x = np.concatenate([
        r.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** r.integers(-9, 5, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 5.9604645e-8, 2.9802322e-8, 2.98023e-8,
                  6.1035156e-5, 6.0975552e-5, 1.0009765625, 1.00048828125, 1.00146484375], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = oracle.f32_to_f16(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_float_to_int8_rounding():
    v = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 300.0, -127.5, -128.5, -300.0, np.nan, 3.4999, 3.5001],
                 np.float32)
    # round-half-even, saturate to [-128, 127], NaN -> 0
    assert oracle.float4_to_char4(v).tolist() == [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, -128, 0, 3, 4]
    # quantize(): round-half-even of q*x clipped to [-127, 127]
    assert oracle.quantize(v, 1.0).tolist() == [0, 2, 2, 0, -2, -2, 126, 127, 127, -127, -127, -127, 0, 3, 4]
    x = rng(2).standard_normal(5000).astype(np.float32) * 3
    q = np.float32(17.3)
    want = np.clip(np.rint(q * x), -127, 127).astype(np.int8)
    assert np.array_equal(oracle.quantize(x, q), want)


def test_interleave_is_the_chw32_permutation():
    t, c = 7, 96
    x = rng(3).integers(-128, 128, (t, c)).astype(np.int8)
    il = oracle.interleave(x)
    brute = np.empty(t * c, np.int8)
    for tok in range(t):
        for ch in range(c):
            brute[(ch // 32) * t * 32 + tok * 32 + ch % 32] = x[tok, ch]
    assert np.array_equal(il, brute)
    assert np.array_equal(oracle.deinterleave(il, t, c), x)
    # same thing as a reshape/transpose
    assert np.array_equal(il.reshape(c // 32, t, 32), x.reshape(t, c // 32, 32).transpose(1, 0, 2))


def test_zero_padding_2d():
    rows, sp, dp = 13, 40, 64
    src = rng(4).integers(0, 256, rows * sp).astype(np.uint8)
    out = oracle.zero_padding_2d(src, sp, dp, rows).reshape(rows, dp)
    assert np.array_equal(out[:, :sp], src.reshape(rows, sp))
    assert not out[:, sp:].any()
    back = oracle.zero_padding_2d(out.ravel(), dp, sp, rows)
    assert np.array_equal(back, src)


# ---- SkipLayerNorm -------------------------------------------------------------------------------

@pytest.mark.parametrize("ld", [8, 32, 128, 320, 768, 1024])
@pytest.mark.parametrize("has_bias", [False, True])
def test_skipln_f32_closed_form(ld, has_bias):
    r = rng(10 + ld)
    rows = 5
    x = r.standard_normal((rows, ld)).astype(np.float32)
    skip = r.standard_normal((rows, ld)).astype(np.float32) + 0.5
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float32)
    beta = r.standard_normal(ld).astype(np.float32)
    bias = r.standard_normal(ld).astype(np.float32) if has_bias else None
    got = oracle.skipln(x, skip, beta, gamma, bias)
    v = x.astype(np.float64) + skip + (bias if has_bias else 0.0)
    eps = np.finfo(np.float32).eps if ld in (768, 1024) else 0.0
    close(got, layer_norm_f64(v, gamma, beta, eps), **F32_TOL)


def test_skipln_known_answers_and_invariants():
    ld = 64
    # one row with a hand-computable answer: v = (+1,-1,+1,...) has mean 0, variance 1
    v = np.tile(np.array([1.0, -1.0], np.float32), ld // 2)[None]
    gamma = np.arange(1, ld + 1, dtype=np.float32)
    beta = np.full(ld, 0.25, np.float32)
    got = oracle.skipln(v, np.zeros_like(v), beta, gamma)
    assert np.allclose(got, gamma * v + beta, atol=1e-5)
    # power-of-two input scaling leaves LayerNorm unchanged (exact in binary arithmetic, no epsilon)
    r = rng(11)
    x = r.standard_normal((3, ld)).astype(np.float32)
    s = r.standard_normal((3, ld)).astype(np.float32)
    a = oracle.skipln(x, s, beta, gamma)
    b = oracle.skipln(4 * x, 4 * s, beta, gamma)
    assert np.array_equal(a, b)
    # bias enters exactly like a second residual
    bias = r.standard_normal(ld).astype(np.float32)
    a = oracle.skipln(x, np.zeros_like(x), beta, gamma, bias)
    b = oracle.skipln(x, np.broadcast_to(bias, x.shape).copy(), beta, gamma)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("ld", [32, 256, 768, 1024])
def test_skipln_f16_closed_form(ld):
    r = rng(20 + ld)
    rows = 4
    x = r.standard_normal((rows, ld)).astype(np.float16)
    skip = r.standard_normal((rows, ld)).astype(np.float16)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = r.standard_normal(ld).astype(np.float16)
    bias = (0.1 * r.standard_normal(ld)).astype(np.float16)
    got = oracle.skipln(x, skip, beta, gamma, bias)
    v = (x.astype(np.float16) + skip).astype(np.float16).astype(np.float64) + bias
    eps = 2.0 ** -10 if ld in (768, 1024) else 0.0
    close(got, layer_norm_f64(v, gamma, beta, eps), **F16_TOL)


def test_skipln_dqq_rejects_other_hidden_sizes():
    z = np.zeros((1, 128), np.int8)
    h = np.zeros(128, np.float16)
    st, _ = oracle.skipln_dqq(z, z, h, h, None, 1.0, 1.0, 1.0)
    assert st != 0  # only hidden sizes 768 and 1024 exist in the reference


@pytest.mark.parametrize("ld", [768, 1024])
def test_skipln_dqq_closed_form(ld):
    r = rng(30 + ld)
    rows = 6
    x = r.integers(-127, 128, (rows, ld)).astype(np.int8)
    skip = r.integers(-127, 128, (rows, ld)).astype(np.int8)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.5 * r.standard_normal(ld)).astype(np.float16)
    bias = (0.1 * r.standard_normal(ld)).astype(np.float16)
    dq_in, dq_skip, q = 4.0 / 127, 2.0 / 127, 127 / 4.0
    st, got = oracle.skipln_dqq(x, skip, beta, gamma, bias, dq_in, dq_skip, q)
    assert st == 0
    v = x.astype(np.float64) * dq_in + skip.astype(np.float64) * dq_skip + bias.astype(np.float64)
    want = np.clip(np.rint(layer_norm_f64(v, gamma, beta, 2.0 ** -10) * q), -128, 127)
    diff = np.abs(got.astype(np.int32) - want)
    # binary16 statistics against float64: a few LSB at |y*q| ~ 100, most values exact or off by one
    assert diff.max() <= 3 and (diff <= 1).mean() > 0.97


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("ld,total,force", [(768, 40, -1), (1024, 24, -1), (1024, 24, 1), (768, 16, 1)])
def test_skipln_interleaved_closed_form(variant, ld, total, force):
    r = rng(40 + ld + total + variant)
    x = r.integers(-127, 128, (total, ld)).astype(np.int8)
    skip = r.integers(-127, 128, (total, ld)).astype(np.int8)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.5 * r.standard_normal(ld)).astype(np.float16)
    dq_in, dq_skip, q, q_skip = 3.0 / 127, 2.5 / 127, 127 / 3.5, 127 / 6.0
    st, out, pre = oracle.skipln_interleaved(variant, oracle.interleave(x), oracle.interleave(skip), beta, gamma, ld,
                                             total, dq_in, dq_skip, q, q_skip, force=force)
    assert st == 0
    got = oracle.deinterleave(out, total, ld).astype(np.int32)
    v = x.astype(np.float64) * dq_in + skip.astype(np.float64) * dq_skip
    # binary16 statistics (small kernel 2^-10 epsilon, large kernel FLT_EPSILON) against float64:
    # never more than one step apart, and a few percent of values sit close enough to a tie to flip
    eps = 2.0 ** -10 if (force != 1 and total < 4096) else 0.0
    want = np.clip(np.rint(layer_norm_f64(v, gamma, beta, eps) * q), -128, 127)
    diff = np.abs(got - want)
    assert diff.max() <= 1 and (diff == 0).mean() > 0.95
    if variant == 1:
        # the Megatron variant also emits the quantised residual sum
        pre_tc = oracle.deinterleave(pre, total, ld).astype(np.int32)
        want_pre = np.clip(np.rint(v * q_skip), -127, 127)
        dpre = np.abs(pre_tc - want_pre)
        assert dpre.max() <= 1 and (dpre == 0).mean() > 0.93  # residual sum passes through binary16
    else:
        assert pre is None


# ---- EmbLayerNorm, maskIdx, packed mask -------------------------------------------------------------

def _emb_tables(r, ld, vocab, types, npos, dt):
    word = r.standard_normal((vocab, ld)).astype(dt)
    pos = r.standard_normal((npos, ld)).astype(dt)
    tok = r.standard_normal((types, ld)).astype(dt)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float32)
    beta = r.standard_normal(ld).astype(np.float32)
    return word, pos, tok, gamma, beta


@pytest.mark.parametrize("dt,tol", [(np.float32, F32_TOL), (np.float16, F16_TOL)])
def test_embln_fixed_closed_form(dt, tol):
    r = rng(50)
    S, B, ld = 12, 3, 128
    word, pos, tok, gamma, beta = _emb_tables(r, ld, 50, 2, S, dt)
    ids = r.integers(0, 50, (S, B)).astype(np.int32)
    segs = r.integers(0, 2, (S, B)).astype(np.int32)
    out, skip, valid = oracle.embln(0, ids, segs, None, beta, gamma, word, pos, tok, S, B)
    assert skip is None and valid.all()
    emb = (word[ids].astype(np.float64) + tok[segs].astype(np.float64)
           + pos[np.arange(S)][:, None, :].astype(np.float64))
    want = layer_norm_f64(emb, gamma, beta, 0.0).reshape(S * B, ld)
    close(out, want, **tol)


@pytest.mark.parametrize("mode", [1, 2])
def test_embln_varseqlen_closed_form(mode):
    r = rng(51 + mode)
    ld, B = 256, 4
    lens = np.array([5, 1, 9, 3])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    S = 16
    word, pos, tok, gamma, beta = _emb_tables(r, ld, 40, 2, S, np.float32)
    ids = r.integers(0, 40, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    out, skip, valid = oracle.embln(mode, ids, segs, cu, beta, gamma, word, pos, tok, S, B)
    posidx = np.concatenate([np.arange(n) for n in lens])  # position restarts at every sequence
    emb = word[ids].astype(np.float64) + tok[segs] + pos[posidx]
    close(out, layer_norm_f64(emb, gamma, beta, 0.0), **F32_TOL)
    if mode == 2:
        close(skip, emb, atol=1e-6, rtol=1e-6)  # Megatron: the un-normalised sum is the skip output
    else:
        assert skip is None


def test_mask_idx_brute_force():
    r = rng(60)
    S, B = 37, 9
    lens = r.integers(0, S + 1, B)
    lens[0], lens[1] = 0, S
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    assert oracle.mask_idx(mask).tolist() == lens.tolist()
    # the first zero decides, later ones do not matter
    mask[20:, 2] = 1
    mask[7, 2] = 0
    assert oracle.mask_idx(mask)[2] == min(7, lens[2])


@pytest.mark.parametrize("S,wm,wn", [(128, 2, 2), (384, 1, 8), (64, 2, 2), (96, 2, 2)])
def test_packed_mask_is_a_bijection_onto_the_score_tile(S, wm, wn):
    """Decode the packed words with the m16n8 accumulator-fragment layout (row = lane/4 (+8),
    col = 2*(lane%4) (+1), second n8 block at +8) and check that the S x S score matrix of every
    sequence is covered exactly once by a column-prefix pattern."""
    r = rng(61 + S)
    B = 3
    lens = np.array([S, 1, int(r.integers(2, S))])
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    packed, over = oracle.convert_mask(mask, wm, wn)
    xm, xn, threads = oracle.packed_mask_geometry(S, wm, wn)
    assert packed.shape == (B, xm * threads)
    if S % (16 * wn) == 0:
        assert over == 0
    row_off = [0, 0, 8, 8, 0, 0, 8, 8]
    col_off = [0, 1, 0, 1, 8, 9, 8, 9]
    for b in range(B):
        hits = np.zeros((xm * 16 * wm, xn * 16 * wn), np.int32)
        vals = np.zeros_like(hits)
        words = packed[b].reshape(xm, threads)
        for mi in range(xm):
            for t in range(threads):
                warp, lane = divmod(t, 32)
                warp_m, warp_n = warp % wm, warp // wm
                for ni in range(xn):
                    for bit in range(8):
                        row = (mi * wm + warp_m) * 16 + lane // 4 + row_off[bit]
                        col = (ni * wn + warp_n) * 16 + 2 * (lane % 4) + col_off[bit]
                        hits[row, col] += 1
                        vals[row, col] = (int(words[mi, t]) >> (8 * ni + bit)) & 1
        assert (hits == 1).all()
        want = np.broadcast_to(np.arange(hits.shape[1])[None, :] < lens[b], hits.shape)
        assert np.array_equal(vals.astype(bool), want)
        assert sum(bin(int(w)).count("1") for w in packed[b]) == hits.shape[0] * lens[b]


# ---- softmax and attention ---------------------------------------------------------------------------

@pytest.mark.parametrize("dt,tol", [(np.float32, F32_TOL), (np.float16, dict(atol=1e-3, rtol=2e-3))])
def test_scaled_softmax_closed_form(dt, tol):
    r = rng(70)
    B, N, S = 3, 2, 40
    x = (4 * r.standard_normal((B, N, S, S))).astype(dt)
    w = 0.125
    lens = np.array([S, 17, 1], np.int32)
    got = oracle.scaled_softmax(x, w, lens).astype(np.float64)
    for b in range(B):
        z = x[b].astype(np.float64)[..., :lens[b]] * w
        z -= z.max(-1, keepdims=True)
        p = np.exp(z)
        p /= p.sum(-1, keepdims=True)
        close(got[b][..., :lens[b]], p, **tol)
        assert not got[b][..., lens[b]:].any()
    # without a mask every position takes part
    full = oracle.scaled_softmax(x, w).astype(np.float64)
    assert np.allclose(full.sum(-1), 1.0, atol=5e-3)


def _split_fixed(qkv, S, B, N, d):
    t = qkv.reshape(S, B, N, 3, d)
    return t[:, :, :, 0], t[:, :, :, 1], t[:, :, :, 2]


@pytest.mark.parametrize("dt,tol", [(np.float32, F32_TOL), (np.float16, dict(atol=4e-3, rtol=1e-2))])
def test_unfused_attention_closed_form(dt, tol):
    r = rng(80)
    S, B, N, d = 24, 3, 2, 32
    qkv = r.standard_normal((S, B, 3 * N * d)).astype(dt)
    lens = np.array([S, 10, 1], np.int32)
    got = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens).reshape(S, B, N, d)
    q, k, v = _split_fixed(qkv, S, B, N, d)
    for b in range(B):
        for n in range(N):
            want = attention_f64(q[:, b, n], k[:lens[b], b, n], v[:lens[b], b, n], 1 / np.sqrt(d))
            close(got[:, b, n], want, **tol)
    # an all-valid mask equals no mask
    a = oracle.mha_unfused_fixed(qkv, S, B, N, d, np.full(B, S, np.int32))
    assert np.array_equal(a, oracle.mha_unfused_fixed(qkv, S, B, N, d, None))


def test_fused_f16_attention_closed_form():
    r = rng(81)
    N, d = 2, 64
    lens = np.array([9, 33, 1, 20])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    qkv = r.standard_normal((T, 3 * N * d)).astype(np.float16)
    got = oracle.mha_fused_f16_packed(qkv, cu, N, d).reshape(T, N, d)
    t = qkv.reshape(T, N, 3, d)
    for b in range(len(lens)):
        sl = slice(cu[b], cu[b + 1])
        for n in range(N):
            want = attention_f64(t[sl, n, 0], t[sl, n, 1], t[sl, n, 2], 1 / np.sqrt(d))
            close(got[sl, n], want, atol=4e-3, rtol=1e-2)
    # fixed layout with a key-prefix mask: same numbers for the valid keys, all S query rows written
    S, B = 16, 2
    qf = r.standard_normal((S, B, 3 * N * d)).astype(np.float16)
    lk = np.array([16, 5])
    gf = oracle.mha_fused_f16_fixed(qf, S, B, N, d, lk).reshape(S, B, N, d)
    q, k, v = _split_fixed(qf, S, B, N, d)
    for b in range(B):
        want = attention_f64(q[:, b, 1], k[:lk[b], b, 1], v[:lk[b], b, 1], 1 / np.sqrt(d))
        close(gf[:, b, 1], want, atol=4e-3, rtol=1e-2)


def test_fused_int8_attention_integer_chain():
    """acc1 and acc2 are exact integer matrix products; p8 and the output follow the float64
    softmax within one rounding step."""
    r = rng(82)
    N, d = 2, 64
    lens = np.array([17, 40, 1])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    qkv = r.integers(-127, 128, (T, 3 * N * d)).astype(np.int8)
    sq, sctx, dqp = 0.02, 0.015, 1 / 127.0
    s1, ssm, s2 = np.float32(sq * sq / 8), np.float32(1 / dqp), np.float32(dqp * sq / sctx)
    out, a1, p8, a2 = oracle.mha_fused_i8_packed(qkv, cu, N, d, s1, ssm, s2, want_ints=True)
    t = qkv.reshape(T, N, 3, d).astype(np.int64)
    a2 = a2.reshape(T, N, d)
    out = out.reshape(T, N, d)
    for b, ln in enumerate(lens):
        sl = slice(cu[b], cu[b + 1])
        for n in range(N):
            q, k, v = t[sl, n, 0], t[sl, n, 1], t[sl, n, 2]
            acc1 = q @ k.T
            assert np.array_equal(a1[b, n, :ln, :ln], acc1)                      # exact
            s = acc1.astype(np.float64) * float(s1)
            s -= s.max(-1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(-1, keepdims=True)
            want_p8 = np.clip(np.rint(p * float(ssm)), -128, 127)
            got_p8 = p8[b, n, :ln, :ln].astype(np.int64)
            assert np.abs(got_p8 - want_p8).max() <= 1
            assert (got_p8 == want_p8).mean() > 0.999
            acc2 = got_p8 @ v
            assert np.array_equal(a2[sl, n], acc2)                               # exact given p8
            want_out = np.clip(np.rint(acc2.astype(np.float64) * float(s2)), -128, 127)
            assert np.abs(out[sl, n].astype(np.int64) - want_out).max() <= 1
            # and end to end against float attention on the dequantised tensors
            ref = attention_f64(q * sq, k * sq, v * sq, 1 / 8.0) / sctx
            err = np.abs(out[sl, n] - np.clip(ref, -128, 127))
            assert err.max() <= 6 and err.mean() < 1  # INT8 probabilities cost a few output steps


def test_fused_int8_fixed_and_packed_agree():
    r = rng(83)
    S, B, N, d = 32, 2, 2, 64
    qkv = r.integers(-127, 128, (S, B, 3 * N * d)).astype(np.int8)
    lens = np.array([32, 11])
    sc = (np.float32(1e-4), np.float32(127.0), np.float32(0.01))
    fixed = oracle.mha_fused_i8_fixed(qkv, S, B, N, d, lens, *sc)
    for b in range(B):
        ln = int(lens[b])
        packed = oracle.mha_fused_i8_packed(qkv[:ln, b], np.array([0, ln], np.int32), N, d, *sc)
        assert np.array_equal(fixed[:ln, b], packed)


def test_packed_mask_all_contiguous_lengths():
    """Every prefix length 0..S for the four sequence lengths that have a packed mask: decoding
    (by the fragment layout above, vectorised) gives back `col < len` everywhere."""
    for S, wm, wn in ((64, 2, 2), (96, 2, 2), (128, 2, 2), (384, 1, 8)):
        lens = np.arange(S + 1)
        mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
        packed, over = oracle.convert_mask(mask, wm, wn)
        assert over == 0
        xm, xn, threads = oracle.packed_mask_geometry(S, wm, wn)
        t = np.arange(threads)
        warp_n, lane = (t // 32) // wm, t % 32
        col_off = np.array([0, 1, 0, 1, 8, 9, 8, 9])
        # column of bit (ni, k) of thread t
        col = ((np.arange(xn)[None, :, None] * wn + warp_n[:, None, None]) * 16 + 2 * (lane % 4)[:, None, None]
               + col_off[None, None, :])                                        # [threads, xn, 8]
        shift = (8 * np.arange(xn)[:, None] + np.arange(8)[None, :])[None]       # [1, xn, 8]
        words = packed.reshape(S + 1, xm, threads)
        bits = (words[..., None, None] >> shift[None]) & 1                       # [S+1, xm, threads, xn, 8]
        want = col[None, None] < lens[:, None, None, None, None]
        assert np.array_equal(bits.astype(bool), np.broadcast_to(want, bits.shape))


def test_attention_special_cases():
    r = rng(90)
    N, d = 2, 64
    # a sequence of one token attends only itself: the context is V
    qkv = r.standard_normal((1, 3 * N * d)).astype(np.float16)
    out = oracle.mha_fused_f16_packed(qkv, np.array([0, 1], np.int32), N, d)
    assert np.array_equal(out, qkv.reshape(1, N, 3, d)[:, :, 2].reshape(1, N * d))
    # identical keys give uniform probabilities: the context is the mean of V, for every query
    L = 16
    qkv = r.standard_normal((L, N, 3, d)).astype(np.float32)
    qkv[:, :, 1] = qkv[0, :, 1]
    got = oracle.mha_unfused_fixed(qkv.reshape(L, 1, 3 * N * d), L, 1, N, d).reshape(L, N, d)
    close(got, np.broadcast_to(qkv[:, :, 2].mean(0), (L, N, d)), atol=1e-5, rtol=1e-5)
    # INT8, one token: p8 = 127 exactly, context = sat(rne(127 * v * scale_bmm2))
    q8 = r.integers(-127, 128, (1, 3 * N * d)).astype(np.int8)
    s2 = np.float32(0.006)
    o8, a1, p8, a2 = oracle.mha_fused_i8_packed(q8, np.array([0, 1], np.int32), N, d, np.float32(1e-4),
                                                np.float32(127.0), s2, want_ints=True)
    v = q8.reshape(1, N, 3, d)[:, :, 2].astype(np.int64)
    assert (p8[:, :, 0, 0] == 127).all()
    assert np.array_equal(a2.reshape(1, N, d), 127 * v)
    assert np.array_equal(o8.reshape(1, N, d), np.clip(np.rint((127 * v).astype(np.float32) * s2), -128, 127))
    # packing invariance: a sequence computes the same alone or inside a batch
    lens = np.array([5, 12, 7])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = r.integers(-127, 128, (int(cu[-1]), 3 * N * d)).astype(np.int8)
    sc = (np.float32(2e-4), np.float32(127.0), np.float32(0.01))
    whole = oracle.mha_fused_i8_packed(x, cu, N, d, *sc)
    for b in range(3):
        alone = oracle.mha_fused_i8_packed(x[cu[b]:cu[b + 1]], np.array([0, lens[b]], np.int32), N, d, *sc)
        assert np.array_equal(whole[cu[b]:cu[b + 1]], alone)


def test_int8_layernorm_all_byte_pairs():
    """Every (input, skip) byte pair appears in one hidden vector: the dequantised sum the oracle
    normalises is exactly dqIn*a + dqSkip*b for all 65536 pairs (checked through the Megatron
    variant's pre-LayerNorm output, quantised with scale 1)."""
    a = np.arange(-128, 128, dtype=np.int16)
    pairs = np.stack(np.meshgrid(a, a, indexing="ij"), -1).reshape(-1, 2).astype(np.int8)   # 65536 pairs
    ld = 1024
    total = pairs.shape[0] // ld                                                           # 64 tokens
    x = pairs[:, 0].reshape(total, ld)
    s = pairs[:, 1].reshape(total, ld)
    gamma = np.ones(ld, np.float16)
    beta = np.zeros(ld, np.float16)
    for force, lo in ((0, -127), (1, -128)):
        st, _, pre = oracle.skipln_interleaved(1, oracle.interleave(x), oracle.interleave(s), beta, gamma, ld, total,
                                               0.5, 0.25, 1.0, 1.0, force=force)
        assert st == 0
        want = np.clip(np.rint(0.5 * x.astype(np.float64) + 0.25 * s.astype(np.float64)), lo, 127)
        # .5 ties: 0.5*a + 0.25*b is exact in binary16/32, so round-half-even decides identically
        assert np.array_equal(oracle.deinterleave(pre, total, ld), want.astype(np.int8))


# ---- INT8 linear layer ---------------------------------------------------------------------------

def _interleave(x):
    T, Cc = x.shape
    return np.ascontiguousarray(x.reshape(T, Cc // 32, 32).transpose(1, 0, 2))


def test_int8_linear_accumulators_against_int64_matmul():
    r = rng(3)
    T, K, N = 37, 192, 96
    a = r.integers(-128, 128, (T, K)).astype(np.int8)
    w = r.integers(-128, 128, (N, K)).astype(np.int8)
    want = a.astype(np.int64) @ w.astype(np.int64).T        # a transposed operand or a dropped row fails here
    got = oracle.int8_linear(a, w, epilogue=oracle.LINEAR_RAW_INT32)
    assert np.array_equal(got.astype(np.int64), want)
    # the interleaved activation layout is only a permutation of the same bytes
    got_il = oracle.int8_linear(_interleave(a), w, epilogue=oracle.LINEAR_RAW_INT32, a_interleaved=True)
    assert np.array_equal(got_il, got)
    # extreme corner: -128 * -128 * K fits INT32 for every K the layers use
    a[:] = -128
    w[:] = -128
    assert (oracle.int8_linear(a, w, epilogue=oracle.LINEAR_RAW_INT32) == 16384 * K).all()


def test_int8_linear_identity_weights_pass_the_input_through():
    r = rng(4)
    T, K = 20, 64
    a = r.integers(-128, 128, (T, K)).astype(np.int8)
    w = np.eye(K, dtype=np.int8)
    one, zero = np.ones(K, np.float32), np.zeros(K, np.float32)
    assert np.array_equal(oracle.int8_linear(a, w, one, zero), a)
    # output layout: channel n of token t lands at [n/32][t][n%32]
    out_il = oracle.int8_linear(a, w, one, zero, out_interleaved=True)
    assert np.array_equal(out_il, _interleave(a))
    # per-channel scale and offset: channel n is doubled and shifted by n - 32, then saturated
    alpha = np.full(K, 2, np.float32)
    beta = (np.arange(K) - 32).astype(np.float32)
    want = np.clip(2 * a.astype(np.int64) + (np.arange(K) - 32)[None, :], -128, 127)
    assert np.array_equal(oracle.int8_linear(a, w, alpha, beta).astype(np.int64), want)


def test_int8_linear_affine_rounds_half_to_even_after_one_fma():
    # one weight of 1 picks activation k=0; alpha = 0.5 makes every odd activation a tie
    K, N = 64, 32
    a = np.zeros((256, K), np.int8)
    a[:, 0] = np.arange(-128, 128)
    w = np.zeros((N, K), np.int8)
    w[:, 0] = 1
    got = oracle.int8_linear(a, w, np.full(N, 0.5, np.float32), np.zeros(N, np.float32))[:, 0]
    half = np.arange(-128, 128) / 2.0
    want = np.where(np.abs(half - np.trunc(half)) == 0.5, 2 * np.round(half / 2), np.round(half))
    assert np.array_equal(got.astype(np.float64), want)
    # fused multiply-add: acc*alpha + beta is rounded once.  With acc = 3, alpha = fl(1/3) and beta = -1 a
    # separately rounded product is exactly 1 and the result 0; the fused result is 3*fl(1/3) - 1 = 2^-25.
    a1 = np.zeros((1, K), np.int8)
    a1[0, 0] = 3
    al = np.full(N, np.float32(1.0) / np.float32(3.0), np.float32)
    be = np.full(N, -1.0, np.float32)
    out16 = oracle.int8_linear(a1, w, al * np.float32(2 ** 20), be * np.float32(2 ** 20),
                               epilogue=oracle.LINEAR_AFFINE_FP16)
    # both constants scaled by 2^20 so that the result, 2^-5, is a normal binary16 number
    assert float(out16[0, 0]) == 2.0 ** -5


def test_int8_linear_gelu_against_binary64_erf():
    from scipy.special import erf
    K, N = 64, 32
    vals = np.arange(-128, 128)
    a = np.zeros((256, K), np.int8)
    a[:, 0] = vals
    w = np.zeros((N, K), np.int8)
    w[:, 0] = 1
    alpha = np.linspace(0.001, 0.06, N).astype(np.float32)      # pre-activations from -7.7 to 7.6
    beta = np.linspace(-0.5, 0.5, N).astype(np.float32)
    q = 127.0 / 8.0
    got = oracle.int8_linear(a, w, alpha, beta, oracle.LINEAR_GELU, out_scale=q).astype(np.float64)
    y = vals[:, None].astype(np.float64) * alpha[None, :].astype(np.float64) + beta[None, :].astype(np.float64)
    g = 0.5 * y * (1.0 + erf(y / np.sqrt(2.0))) * q
    assert np.abs(got - np.clip(g, -128, 127)).max() <= 0.5 + 1e-4
    # GELU facts: zero maps to zero, large positive is the identity, large negative vanishes
    z = oracle.int8_linear(np.zeros((1, K), np.int8), w, alpha, np.zeros(N, np.float32), oracle.LINEAR_GELU, out_scale=q)
    assert (z == 0).all()
    big = oracle.int8_linear(a[255:256], w, np.full(N, 0.05, np.float32), np.zeros(N, np.float32), oracle.LINEAR_GELU,
                             out_scale=10.0)
    assert (big == round(127 * 0.05 * 10.0)).all()               # gelu(6.35) = 6.35 to 1e-9
    neg = oracle.int8_linear(a[0:1], w, np.full(N, 0.05, np.float32), np.zeros(N, np.float32), oracle.LINEAR_GELU,
                             out_scale=10.0)
    assert (neg == 0).all()


def test_quantize_dequantize_reformat_closed_form():
    r = rng(6)
    T, Cc = 45, 96
    x = (r.standard_normal((T, Cc)) * 3).astype(np.float16)
    x[0, :8] = [0.5, 1.5, 2.5, -0.5, -1.5, 1000, -1000, 0]       # ties go to even, range saturates
    q = oracle.quantize_f16_interleave(x, 1.0)
    assert list(q[0, 0, :8]) == [0, 2, 2, 0, -2, 127, -128, 0]
    scale = np.float32(0.037)
    q = oracle.quantize_f16_interleave(x, float(scale))
    want = np.clip(np.rint((x.astype(np.float32) / scale).astype(np.float32)), -128, 127).astype(np.int8)
    assert np.array_equal(q, _interleave(want))
    back = oracle.dequantize_deinterleave_f16(q, float(scale))
    assert np.array_equal(back, (want.astype(np.float32) * scale).astype(np.float16))
    # quantise(dequantise(q)) is the identity when no value saturates the binary16 mantissa (|q| <= 128)
    assert np.array_equal(oracle.quantize_f16_interleave(back, float(scale)), q)


def test_fp16_linear_against_float64():
    from scipy.special import erf
    r = rng(8)
    T, K, N = 33, 96, 64
    a = (r.standard_normal((T, K)) * 0.5).astype(np.float16)
    w = (r.standard_normal((N, K)) * 0.2).astype(np.float16)
    alpha = r.uniform(0.5, 1.5, N).astype(np.float32)
    beta = r.standard_normal(N).astype(np.float32)
    y = (a.astype(np.float64) @ w.astype(np.float64).T) * alpha[None, :] + beta[None, :]
    got = oracle.fp16_linear(a, w, alpha, beta).astype(np.float64)
    assert np.abs(got - y).max() <= 2e-3 + 1e-3 * np.abs(y).max()
    g = 0.5 * y * (1 + erf(y / np.sqrt(2)))
    got = oracle.fp16_linear(a, w, alpha, beta, gelu=True).astype(np.float64)
    assert np.abs(got - g).max() <= 2e-3 + 1e-3 * np.abs(g).max()
    # identity weights, unit scale, zero offset: the input comes back bit for bit
    eye = np.eye(K, dtype=np.float16)
    assert np.array_equal(oracle.fp16_linear(a, eye, np.ones(K, np.float32), np.zeros(K, np.float32)), a)
