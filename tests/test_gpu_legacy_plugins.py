"""The IPluginV2DynamicExt ("Legacy") versions on the GPU: each is created from its PluginFieldCollection,
configured, serialised, rebuilt with deserializePlugin and enqueued; its output must equal, byte for byte, the
output of the IPluginV3 version it corresponds to (they launch the same kernels), and for one case per operator
also the oracle, so the pairing of legacy and current versions is itself checked."""
import numpy as np
import pytest

import oracle
from helpers import assert_fp_close, assert_int8_close, dev, dev_empty, host, ptr, quantize_amax, rng, stream, sync
from tensorrt_amd.plugin import (DataType, PluginField, PluginFieldType, TensorDesc, TensorFormat, TensorRTPhase,
                                 capture_log, get_plugin_registry, last_log)

pytestmark = pytest.mark.gpu

SKIPLN = "CustomSkipLayerNormPluginDynamic"
EMBLN = "CustomEmbLayerNormPluginDynamic"
QKV = "CustomQKVToContextPluginDynamic"
I32, F32, F16 = PluginFieldType.INT32, PluginFieldType.FLOAT32, PluginFieldType.FLOAT16


def i32(name, v):
    return PluginField(name, np.array([v], np.int32), I32)


def f32(name, v):
    return PluginField(name, np.array([v], np.float32), F32)


@pytest.fixture(scope="module")
def reg():
    capture_log(True)
    last_log()
    return get_plugin_registry()


def both(reg, name, legacy, current, fields, ins, outs):
    """(legacy plugin after a serialise/deserialise round trip, V3 plugin after its own)."""
    lc, cc = reg.get_legacy_creator(name, legacy), reg.get_creator(name, current)
    lp = lc.create_plugin("legacy", fields)
    assert lp is not None, last_log()
    lp.configure_plugin(ins, outs)
    lp = lc.deserialize_plugin("legacy", lp.serialize())
    assert lp is not None, last_log()
    cp = cc.create_plugin("current", fields, TensorRTPhase.BUILD)
    assert cp.configure_plugin(ins, outs) == 0, last_log()
    cp = cc.create_plugin("current", cp.get_fields_to_serialize(), TensorRTPhase.RUNTIME)
    assert cp is not None, last_log()
    return lp, cp


def run_both(lp, cp, ins, outs, inputs, out_shapes, out_dtypes, ws_bytes=0):
    res = []
    for plugin, legacy in ((lp, True), (cp, False)):
        bufs = [dev_empty(s, d, fill=0) for s, d in zip(out_shapes, out_dtypes)]
        ws = dev_empty((max(ws_bytes, 1),), np.uint8)
        if not legacy:
            assert plugin.on_shape_change(ins, outs) == 0, last_log()
        st = plugin.enqueue(ins, outs, [ptr(t) for t in inputs], [ptr(b) for b in bufs], ptr(ws), stream())
        assert st == 0, last_log()
        sync()
        res.append([host(b) for b in bufs])
    for a, b in zip(*res):
        assert np.array_equal(a, b), "legacy and current versions disagree"
    return res[0]


@pytest.mark.parametrize("legacy,current", [("1", "5"), ("2", "6")])
def test_legacy_skipln_fp16(reg, legacy, current):
    r = rng(31)
    S, B, ld = 20, 3, 768
    x, skip = (r.standard_normal((S, B, ld)).astype(np.float16) for _ in range(2))
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float32)
    beta = (0.3 * r.standard_normal(ld)).astype(np.float32)
    bias = (0.1 * r.standard_normal(ld)).astype(np.float32)
    fs = [i32("type_id", 1), PluginField("beta", beta, F32), PluginField("gamma", gamma, F32), PluginField("bias", bias, F32)]
    if legacy == "1":
        fs.append(i32("ld", ld))
    d = TensorDesc([S, B, ld, 1, 1], DataType.HALF)
    lp, cp = both(reg, SKIPLN, legacy, current, fs, [d, d], [d])
    (out,) = run_both(lp, cp, [d, d], [d], [dev(x), dev(skip)], [(S, B, ld)], [np.float16])
    ref = oracle.skipln(x.reshape(-1, ld), skip.reshape(-1, ld), beta.astype(np.float16), gamma.astype(np.float16),
                        bias.astype(np.float16))
    assert_fp_close(out.reshape(-1, ld), ref, what="legacy SkipLN")


@pytest.mark.parametrize("legacy,current", [("3", "7"), ("4", "8")])
def test_legacy_skipln_interleaved(reg, legacy, current):
    r = rng(32)
    ld, total = 1024, 333
    x, dq_in = quantize_amax(r.standard_normal((total, ld)))
    s, dq_skip = quantize_amax(r.standard_normal((total, ld)))
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.3 * r.standard_normal(ld)).astype(np.float16)
    fs = [PluginField("beta", beta, F16), PluginField("gamma", gamma, F16)]
    shape, fmt = [1, ld, total, 1], TensorFormat.CHW32
    out_scale, pre_scale = np.float32(4.5 / 127), np.float32(6.0 / 127)
    ins = [TensorDesc(shape, DataType.INT8, fmt, dq_in), TensorDesc(shape, DataType.INT8, fmt, dq_skip)]
    outs = [TensorDesc(shape, DataType.INT8, fmt, out_scale)]
    mtron = legacy == "4"
    if mtron:
        outs.append(TensorDesc(shape, DataType.INT8, fmt, pre_scale))
    lp, cp = both(reg, SKIPLN, legacy, current, fs, ins, outs)
    x_il, s_il = oracle.interleave(x), oracle.interleave(s)
    res = run_both(lp, cp, ins, outs, [dev(x_il), dev(s_il)], [(ld * total,)] * len(outs), [np.int8] * len(outs))
    st, ref, ref_pre = oracle.skipln_interleaved(int(mtron), x_il, s_il, beta, gamma, ld, total, dq_in, dq_skip,
                                                 np.float32(1) / out_scale, np.float32(1) / pre_scale)
    assert st == 0
    assert_int8_close(res[0], ref, what="legacy interleaved SkipLN")
    if mtron:
        assert_int8_close(res[1], ref_pre, what="legacy interleaved SkipLN preln")


@pytest.mark.parametrize("legacy,current", [("2", "4"), ("3", "5")])
def test_legacy_embln_varseqlen(reg, legacy, current):
    r = rng(33)
    ld, vocab = 384, 300
    lens = np.array([17, 1, 128, 60])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, B = int(cu[-1]), len(lens)
    w = dict(beta=(0.1 * r.standard_normal(ld)).astype(np.float32), gamma=r.uniform(0.5, 1.5, ld).astype(np.float32),
             word=(0.02 * r.standard_normal((vocab, ld))).astype(np.float32),
             tok=(0.02 * r.standard_normal((2, ld))).astype(np.float32),
             pos=(0.02 * r.standard_normal((128, ld))).astype(np.float32))
    fs = [PluginField("bert_embeddings_layernorm_beta", w["beta"], F32),
          PluginField("bert_embeddings_layernorm_gamma", w["gamma"], F32),
          PluginField("bert_embeddings_word_embeddings", w["word"], F32),
          PluginField("bert_embeddings_token_type_embeddings", w["tok"], F32),
          PluginField("bert_embeddings_position_embeddings", w["pos"], F32), i32("output_fp16", 1)]
    ids = r.integers(0, vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    mtron = legacy == "3"
    ins = [TensorDesc([T], DataType.INT32), TensorDesc([T], DataType.INT32), TensorDesc([B + 1], DataType.INT32),
           TensorDesc([128], DataType.INT32)]
    outs = [TensorDesc([T, ld, 1, 1], DataType.HALF),
            TensorDesc([T, ld, 1, 1], DataType.HALF) if mtron else TensorDesc([], DataType.INT32)]
    lp, cp = both(reg, EMBLN, legacy, current, fs, ins, outs)
    shapes = [(T, ld), (T, ld) if mtron else (1,)]
    dtypes = [np.float16, np.float16 if mtron else np.int32]
    res = run_both(lp, cp, ins, outs, [dev(ids), dev(segs), dev(cu), dev(np.zeros(128, np.int32))], shapes, dtypes)
    tabs = {k: w[k].astype(np.float16) for k in ("word", "pos", "tok")}
    ref, ref_skip, _ = oracle.embln(2 if mtron else 1, ids, segs, cu, w["beta"], w["gamma"], tabs["word"], tabs["pos"],
                                    tabs["tok"], 128, B)
    assert_fp_close(res[0], ref, what="legacy EmbLN")
    if mtron:
        assert_fp_close(res[1], ref_skip, what="legacy EmbLN skip")


def test_legacy_embln_fixed_feeds_legacy_qkv(reg):
    """EmbLayerNorm version 1 -> packed mask -> QKV-to-context version 1 (fused FP16), both through the legacy API."""
    r = rng(34)
    S, B, N, d = 128, 3, 4, 64
    ld = N * d
    vocab = 200
    w = dict(beta=(0.1 * r.standard_normal(ld)).astype(np.float32), gamma=r.uniform(0.5, 1.5, ld).astype(np.float32),
             word=(0.02 * r.standard_normal((vocab, ld))).astype(np.float32),
             tok=(0.02 * r.standard_normal((2, ld))).astype(np.float32),
             pos=(0.02 * r.standard_normal((S, ld))).astype(np.float32))
    fs = [PluginField("bert_embeddings_layernorm_beta", w["beta"], F32),
          PluginField("bert_embeddings_layernorm_gamma", w["gamma"], F32),
          PluginField("bert_embeddings_word_embeddings", w["word"], F32),
          PluginField("bert_embeddings_token_type_embeddings", w["tok"], F32),
          PluginField("bert_embeddings_position_embeddings", w["pos"], F32), i32("output_fp16", 1), i32("full_mask", 0),
          i32("mha_type_id", 1)]
    lens = np.array([128, 40, 77])
    ids = r.integers(0, vocab, (S, B)).astype(np.int32)
    segs = r.integers(0, 2, (S, B)).astype(np.int32)
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    e_ins = [TensorDesc([S, B], DataType.INT32)] * 3
    e_outs = [TensorDesc([S, B, ld, 1, 1], DataType.HALF), TensorDesc([B, 512], DataType.INT32)]
    lp, cp = both(reg, EMBLN, "1", "6", fs, e_ins, e_outs)
    emb, packed = run_both(lp, cp, e_ins, e_outs, [dev(ids), dev(segs), dev(mask)], [(S, B, ld), (B, 512)],
                           [np.float16, np.int32])
    tabs = {k: w[k].astype(np.float16) for k in ("word", "pos", "tok")}
    ref, _, _ = oracle.embln(0, ids, segs, None, w["beta"], w["gamma"], tabs["word"], tabs["pos"], tabs["tok"], S, B)
    assert_fp_close(emb.reshape(S * B, ld), ref, what="legacy EmbLN v1")

    qkv = (r.standard_normal((S, B, N, 3, d)) / 8).astype(np.float16)
    qfs = [i32("type_id", 1), i32("hidden_size", ld), i32("num_heads", N), i32("has_mask", 1)]
    q_ins = [TensorDesc([S, B, 3 * ld, 1, 1], DataType.HALF), TensorDesc([B, 512], DataType.INT32)]
    q_outs = [TensorDesc([S, B, ld, 1, 1], DataType.HALF)]
    lq, cq = both(reg, QKV, "1", "4", qfs, q_ins, q_outs)
    (ctx,) = run_both(lq, cq, q_ins, q_outs, [dev(qkv), dev(packed)], [(S, B, ld)], [np.float16])
    want = oracle.mha_fused_f16_fixed(qkv, S, B, N, d, lens)
    valid = np.arange(S)[:, None] < lens[None, :]
    assert_fp_close(ctx[valid], want[valid], what="legacy QKV v1 through the packed mask")


@pytest.mark.parametrize("legacy,current,dt", [("2", "5", DataType.HALF), ("3", "6", DataType.INT8)])
def test_legacy_qkv_varseqlen(reg, legacy, current, dt):
    r = rng(35)
    N, d = 4, 64
    hidden = N * d
    lens = np.array([384, 200, 1, 97])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, B = int(cu[-1]), len(lens)
    qf = r.standard_normal((T, 3 * hidden))
    dummy = dev(np.zeros(384, np.int32))
    if legacy == "2":
        q = (qf / 8).astype(np.float16)
        fs = [i32("type_id", 1), i32("hidden_size", hidden), i32("num_heads", N), i32("has_mask", 1), i32("var_seqlen", 1)]
        ins = [TensorDesc([T, 3 * hidden, 1, 1], dt), TensorDesc([1], DataType.INT32), TensorDesc([B + 1], DataType.INT32),
               TensorDesc([384], DataType.INT32)]
        outs = [TensorDesc([T, hidden, 1, 1], dt)]
        lp, cp = both(reg, QKV, legacy, current, fs, ins, outs)
        (out,) = run_both(lp, cp, ins, outs, [dev(q), dev(np.zeros(1, np.int32)), dev(cu), dummy], [(T, hidden)],
                          [np.float16])
        assert_fp_close(out, oracle.mha_fused_f16_packed(q, cu, N, d), what="legacy QKV v2")
    else:
        q, s_q = quantize_amax(qf)
        s_ctx = s_q
        fs = [i32("hidden_size", hidden), i32("num_heads", N), f32("dq_probs", 1 / 127)]
        fmt = TensorFormat.CHW32
        ins = [TensorDesc([1, 3 * hidden, T, 1], dt, fmt, s_q), TensorDesc([B + 1], DataType.INT32),
               TensorDesc([384], DataType.INT32)]
        outs = [TensorDesc([1, hidden, T, 1], dt, fmt, s_ctx)]
        lp, cp = both(reg, QKV, legacy, current, fs, ins, outs)
        x = q.reshape(T, N, 3, d).transpose(0, 2, 1, 3).reshape(T, 3 * hidden)
        (out,) = run_both(lp, cp, ins, outs, [dev(oracle.interleave(x)), dev(cu), dummy], [(hidden * T,)], [np.int8])
        dqp = np.float32(1 / 127)
        s1 = np.float32(np.float32(s_q * s_q) * (np.float32(1) / np.sqrt(np.float32(d))))
        s2 = np.float32(np.float32(dqp * s_q) / s_ctx)
        ref = oracle.mha_fused_i8_packed(q, cu, N, d, s1, np.float32(1) / dqp, s2)
        assert_int8_close(oracle.deinterleave(out, T, hidden), ref, what="legacy QKV v3", max_frac_off=0.002)


@pytest.mark.parametrize("has_mask", [0, 1])
def test_legacy_qkv_version_2_without_var_seqlen(reg, has_mask):
    """Version 2 with var_seqlen = 0 is the fixed-length operator: qkv and, with has_mask, the mask.  The
    deserialised plugin must know its input count from the stream alone (enqueue does not state it)."""
    r = rng(36 + has_mask)
    S, B, N, d = 40, 3, 2, 32
    hidden = N * d
    qkv = (r.standard_normal((S, B, 3 * hidden)) / 4).astype(np.float32)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    fs = [i32("type_id", 0), i32("hidden_size", hidden), i32("num_heads", N), i32("has_mask", has_mask),
          i32("var_seqlen", 0)]
    ins = [TensorDesc([S, B, 3 * hidden, 1, 1], DataType.FLOAT)]
    inputs = [dev(qkv)]
    if has_mask:
        ins.append(TensorDesc([B], DataType.INT32))
        inputs.append(dev(lens))
    outs = [TensorDesc([S, B, hidden, 1, 1], DataType.FLOAT)]
    lp, cp = both(reg, QKV, "2", "5", fs, ins, outs)
    ws_bytes = cp.get_workspace_size(ins, outs)
    (out,) = run_both(lp, cp, ins, outs, inputs, [(S, B, hidden)], [np.float32], ws_bytes)
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens if has_mask else None)
    assert_fp_close(out, ref, what="legacy QKV v2, fixed length")
