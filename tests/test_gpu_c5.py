"""The headline configuration at its own dimensions: BERT-large (hidden 1024, 16 heads of 64, feed-forward 4096),
B = 128 sequences with lengths uniform in [128, 384] (seed 1: 33289 packed tokens), INT8, 32-interleaved tensors.

The oracle cannot run the whole problem in test time, and does not have to: every (sequence, head) of the attention
and every token row of the other operations is independent of the rest.  So the full-size GPU result is checked
(a) against the oracle on a sample of sequences / token rows, to the bar of the small tests (first accumulators and
second product exact, probabilities within one step, rows with agreeing probabilities bit-exact; INT8 outputs of the
other operations within one step), and (b) everywhere through the permutation property: permuting sequences or rows
of the input permutes the output bit for bit."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, assert_int8_close, dev, dev_empty, f32_bits, host, int8_attention_parity, ptr,
                     quantize_amax, rng, stream, sync)

pytestmark = pytest.mark.gpu
D, N, E, F, S, B = 64, 16, 1024, 4096, 384, 128


def c5_lengths():
    lens = np.random.default_rng(1).integers(128, 385, B)
    assert int(lens.sum()) == 33289
    return lens


def cu_of(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def sample_sequences(lens, r, n=4):
    picks = {int(np.argmin(lens)), int(np.argmax(lens))}
    while len(picks) < n:
        picks.add(int(r.integers(0, len(lens))))
    return sorted(picks)


def gather(x, cu, order):
    return np.concatenate([x[cu[b]:cu[b + 1]] for b in order], axis=0)


def to_interleaved_qkv(qkv):
    t = qkv.shape[0]
    return oracle.interleave(qkv.reshape(t, N, 3, D).transpose(0, 2, 1, 3).reshape(t, 3 * N * D))


def run_attention(qkv, cu, s1, ss, s2):
    from tensorrt_amd import capi
    api = capi.api()
    t = qkv.shape[0]
    d_qkv, d_cu = dev(to_interleaved_qkv(qkv)), dev(cu)
    out = dev_empty((t * N * D,), np.int8, fill=0x55)
    p = capi.FmhaParams()
    p.qkv_ptr, p.o_ptr, p.cu_seqlens = ptr(d_qkv), ptr(out), ptr(d_cu)
    p.b, p.h, p.s, p.d = len(cu) - 1, N, S, D
    p.scale_bmm1, p.scale_softmax, p.scale_bmm2 = f32_bits(s1), f32_bits(ss), f32_bits(s2)
    p.interleaved, p.use_int8_scale_max = 1, 1
    p.qkv_stride_in_bytes = p.o_stride_in_bytes = t
    api.check(api.fused_mha_run(stream(), 2, C.byref(p)))
    sync()
    return oracle.deinterleave(host(out), t, N * D)


def test_attention_at_c5_size():
    r = rng(1)
    lens = c5_lengths()
    cu = cu_of(lens)
    T = int(cu[-1])
    qkv, s_q = quantize_amax(r.standard_normal((T, 3 * N * D)))
    dq_probs = np.float32(1 / 127)
    s_ctx = np.float32(0.5 * s_q)        # below the input scale: a probability off by one step would move outputs by 2
    s1 = np.float32(s_q * s_q * np.float32(1 / np.sqrt(np.float32(D))))
    ss = np.float32(1 / dq_probs)
    s2 = np.float32(dq_probs * s_q / s_ctx)
    full = run_attention(qkv, cu, s1, ss, s2)
    assert not (full == 0x55).all(axis=1).any(), "a token row was not written"
    # sampled sequences, run alone: the strict decomposition against the oracle, and the same bytes as in the batch
    for b in sample_sequences(lens, r):
        lo, hi = cu[b], cu[b + 1]
        int8_attention_parity(qkv[lo:hi], cu_of(lens[b:b + 1]), N, s1, ss, s2, interleaved=True, S=S,
                              expect=full[lo:hi])
    order = r.permutation(B)
    moved = run_attention(gather(qkv, cu, order), cu_of(lens[order]), s1, ss, s2)
    assert np.array_equal(moved, gather(full, cu, order))


def test_skip_layer_norm_at_c5_size():
    from tensorrt_amd import capi
    api = capi.api()
    r = rng(2)
    total = int(c5_lengths().sum())
    x, dq_in = quantize_amax(r.standard_normal((total, E)))
    s, dq_skip = quantize_amax(r.standard_normal((total, E)))
    gamma = r.uniform(0.5, 1.5, E).astype(np.float16)
    beta = (0.1 * r.standard_normal(E)).astype(np.float16)
    q_scale = np.float32(127.0 / 4.5)
    db, dg = dev(beta), dev(gamma)

    def run(a, b):
        out = dev_empty((E * a.shape[0],), np.int8, fill=0)
        dx, ds = dev(oracle.interleave(a)), dev(oracle.interleave(b))
        api.check(api.skipln_interleaved_large_hface(stream(), E, a.shape[0], ptr(dx), ptr(ds), ptr(db), ptr(dg),
                                                     ptr(out), dq_in, dq_skip, q_scale))
        sync()
        return oracle.deinterleave(host(out), a.shape[0], E)

    got = run(x, s)
    rows = np.unique(np.concatenate([np.arange(40), np.arange(total - 40, total), r.integers(0, total, 4000)]))
    st, ref, _ = oracle.skipln_interleaved(0, oracle.interleave(x[rows]), oracle.interleave(s[rows]), beta, gamma, E,
                                           len(rows), dq_in, dq_skip, q_scale, force=1)
    assert st == 0
    assert_int8_close(got[rows], oracle.deinterleave(ref, len(rows), E), what="sampled rows vs oracle", max_frac_off=0.01)
    order = r.permutation(total)
    assert np.array_equal(run(x[order], s[order]), got[order])


@pytest.fixture(scope="module")
def c5_layer():
    """One BERT-large layer of the encoder at the full batch, every activation captured."""
    import torch
    from tensorrt_amd.encoder import EncoderConfig, Int8BertEncoder
    cfg = EncoderConfig(hidden=E, heads=N, ffn=F, layers=1, vocab=3000, max_pos=512, max_seqlen=S, seed=11)
    enc = Int8BertEncoder(cfg)
    r = rng(1)
    lens = c5_lengths()
    cu = cu_of(lens)
    T = int(cu[-1])
    ids = r.integers(0, cfg.vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    enc.calibrate(ids, segs, cu)
    cap = {}
    out = enc.enqueue(ids, segs, cu, capture=cap)
    torch.cuda.synchronize()
    return cfg, enc, ids, segs, cu, lens, cap, out.cpu().numpy()


def test_layer_operations_at_c5_size(c5_layer):
    cfg, enc, ids, segs, cu, lens, cap, _ = c5_layer
    T = int(cu[-1])
    r = rng(3)
    L, sc = enc.layers[0], enc.layers[0]["scales"]
    lin_of = lambda k, c: oracle.deinterleave(np.ascontiguousarray(cap[k]).ravel(), T, c)
    rows = np.unique(np.concatenate([np.arange(8), np.arange(T - 8, T), np.arange(32768 - 4, 32768 + 4),
                                     r.integers(0, T, 600)]))

    def linear(name, src_key, c_in, dst_key, c_out, gelu=False, frac=1e-3):
        lin = L[name]
        ref = oracle.int8_linear(lin_of(src_key, c_in)[rows], lin.w_q, lin.alpha_h, lin.beta_h,
                                 oracle.LINEAR_GELU if gelu else oracle.LINEAR_AFFINE, out_scale=lin.out_scale)
        assert_int8_close(lin_of(dst_key, c_out)[rows], ref, what=name, max_frac_off=frac)

    # embedding (sampled tokens keep their position inside their sequence) and the quantiser (everywhere)
    w = enc.emb_weights
    tabs = {k: w[k].astype(np.float16) for k in ("word", "pos", "tok")}
    for b in sample_sequences(lens, r, 3):
        lo, hi = cu[b], cu[b + 1]
        ref, _, _ = oracle.embln(1, ids[lo:hi], segs[lo:hi], cu_of(lens[b:b + 1]), w["beta"], w["gamma"], tabs["word"],
                                 tabs["pos"], tabs["tok"], cfg.max_seqlen, 1)
        assert_fp_close(cap["emb"][lo:hi], ref, what="embedding")
    assert np.array_equal(cap["l0.x"], oracle.quantize_f16_interleave(cap["emb"], enc.s_emb))

    linear("qkv", "l0.x", E, "l0.qkv", 3 * E)
    # attention: sampled sequences alone reproduce the batch's bytes and pass the strict decomposition
    qkv_lin = lin_of("l0.qkv", 3 * E).reshape(T, 3, N, D).transpose(0, 2, 1, 3).reshape(T, 3 * E)
    ctx = lin_of("l0.ctx", E)
    s_q, s_ctx, dqp = np.float32(sc["qkv"]), np.float32(sc["ctx"]), np.float32(np.float32(1.0) / np.float32(127.0))
    s1 = np.float32(np.float32(s_q * s_q) * (np.float32(1) / np.sqrt(np.float32(D))))
    s2 = np.float32(np.float32(dqp * s_q) / s_ctx)
    for b in sample_sequences(lens, r, 3):
        lo, hi = cu[b], cu[b + 1]
        int8_attention_parity(qkv_lin[lo:hi], cu_of(lens[b:b + 1]), N, s1, np.float32(1) / dqp, s2, interleaved=True, S=S,
                              expect=ctx[lo:hi])
    linear("proj", "l0.ctx", E, "l0.ao", E)

    def skipln(ln, src_key, s_src, skip_key, s_skip, dst, s_out):
        st, ref, _ = oracle.skipln_interleaved(0, oracle.interleave(lin_of(src_key, E)[rows]),
                                               oracle.interleave(lin_of(skip_key, E)[rows]), L[ln + "_beta"],
                                               L[ln + "_gamma"], E, len(rows), np.float32(s_src), np.float32(s_skip),
                                               np.float32(1) / np.float32(s_out), force=1)
        assert st == 0
        assert_int8_close(dst[rows], oracle.deinterleave(ref, len(rows), E), what=ln)

    skipln("ln1", "l0.ao", sc["ao"], "l0.x", sc["x"], lin_of("l0.h", E), sc["h"])
    linear("ffn1", "l0.h", E, "l0.m", F, gelu=True, frac=2e-3)
    linear("ffn2", "l0.m", F, "l0.f", E)
    skipln("ln2", "l0.f", sc["f"], "l0.h", sc["h"], lin_of("x_out", E), sc["out"])


def test_native_runner_at_c5_size(c5_layer):
    """The C++ runner's pass over the full batch gives the bytes of the checked chain."""
    import torch
    cfg, enc, ids, segs, cu, lens, cap, out = c5_layer
    got = enc.enqueue_native(ids, segs, cu)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), out)
    assert np.isfinite(out.astype(np.float32)).all()
    # the same batch as two halves that run at the same time (the benchmark's default): same bytes
    got.fill_(float("nan"))
    got = enc.enqueue_native_concurrent(2)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), out)
