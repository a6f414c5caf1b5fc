"""GPU parity through the plugin objects: every CustomSkipLayerNorm / CustomEmbLayerNorm /
CustomQKVToContext version is created from a PluginFieldCollection, configured, and enqueued on
device buffers exactly as an engine would do, and its outputs are compared with the oracle
(bit-exact for indices and masks, +-1 LSB for requantised INT8, |a-b| <= 2e-3 + 1e-2*|b| for
floating point)."""
import numpy as np
import pytest

import oracle
from helpers import (assert_fp_close, assert_int8_close, dev, dev_empty, host, ptr, quantize_amax, rng, stream, sync)
from tensorrt_amd.plugin import (DataType, PluginField, PluginFieldType, TensorDesc, TensorFormat, TensorRTPhase,
                                 capture_log, get_plugin_registry, last_log)

pytestmark = pytest.mark.gpu

SKIPLN = "CustomSkipLayerNormPluginDynamic"
EMBLN = "CustomEmbLayerNormPluginDynamic"
QKV = "CustomQKVToContextPluginDynamic"
I32, F32, F16 = PluginFieldType.INT32, PluginFieldType.FLOAT32, PluginFieldType.FLOAT16
NPDT = {DataType.FLOAT: np.float32, DataType.HALF: np.float16, DataType.INT8: np.int8}


def i32(name, v):
    return PluginField(name, np.array([v], np.int32), I32)


def f32(name, v):
    return PluginField(name, np.array([v], np.float32), F32)


@pytest.fixture(scope="module")
def reg():
    capture_log(True)
    last_log()
    return get_plugin_registry()


def run(plugin, in_descs, out_descs, inputs, outputs, workspace=None):
    assert plugin.on_shape_change(in_descs, out_descs) == 0, last_log()
    st = plugin.enqueue(in_descs, out_descs, [ptr(t) for t in inputs], [ptr(t) for t in outputs],
                        ptr(workspace), stream())
    assert st == 0, last_log()
    sync()


def through_runtime(creator, plugin):
    """What engine deserialisation does: rebuild the plugin from its serialised fields."""
    p = creator.create_plugin("rt", plugin.get_fields_to_serialize(), TensorRTPhase.RUNTIME)
    assert p is not None, last_log()
    return p


# ---- SkipLayerNorm ---------------------------------------------------------------------------------

@pytest.mark.parametrize("version", ["5", "6"])
@pytest.mark.parametrize("dt,ld,bias", [(DataType.FLOAT, 768, True), (DataType.HALF, 1024, True),
                                        (DataType.HALF, 320, False), (DataType.FLOAT, 32, False)])
def test_skipln_plugin_float(reg, version, dt, ld, bias):
    r = rng(100 + ld)
    npdt = NPDT[dt]
    S, B = 24, 3
    x = r.standard_normal((S, B, ld)).astype(npdt)
    skip = r.standard_normal((S, B, ld)).astype(npdt)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float32)
    beta = (0.3 * r.standard_normal(ld)).astype(np.float32)
    b = (0.1 * r.standard_normal(ld)).astype(np.float32) if bias else None
    fs = [i32("type_id", int(dt)), PluginField("beta", beta, F32), PluginField("gamma", gamma, F32)]
    if version == "5":
        fs.append(i32("ld", ld))
    if bias:
        fs.append(PluginField("bias", b, F32))
    c = reg.get_creator(SKIPLN, version)
    p = through_runtime(c, c.create_plugin("sln", fs))
    d = TensorDesc([S, B, ld, 1, 1], dt)
    out = dev_empty((S, B, ld), npdt, fill=0)
    run(p, [d, d], [d], [dev(x), dev(skip)], [out])
    ref = oracle.skipln(x.reshape(-1, ld), skip.reshape(-1, ld), beta.astype(npdt), gamma.astype(npdt),
                        None if b is None else b.astype(npdt))
    assert_fp_close(host(out).reshape(-1, ld), ref, what=f"SkipLN v{version}")


@pytest.mark.parametrize("version", ["5", "6"])
def test_skipln_plugin_int8(reg, version):
    r = rng(101)
    ld, S, B = 1024, 16, 4
    xf, sf = r.standard_normal((S * B, ld)), r.standard_normal((S * B, ld))
    x, dq_in = quantize_amax(xf)
    s, dq_skip = quantize_amax(sf)
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.3 * r.standard_normal(ld)).astype(np.float16)
    bias = (0.1 * r.standard_normal(ld)).astype(np.float16)
    out_scale = np.float32(4.0 / 127)
    fs = [i32("type_id", 2), PluginField("beta", beta, F16), PluginField("gamma", gamma, F16),
          PluginField("bias", bias, F16)]
    if version == "5":
        fs.append(i32("ld", ld))
    c = reg.get_creator(SKIPLN, version)
    p = c.create_plugin("sln", fs)
    fmt = TensorFormat.CHW32
    shape = [S, B, ld, 1, 1]
    ins = [TensorDesc(shape, DataType.INT8, fmt, dq_in), TensorDesc(shape, DataType.INT8, fmt, dq_skip)]
    outs = [TensorDesc(shape, DataType.INT8, fmt, out_scale)]
    out = dev_empty((S * B, ld), np.int8, fill=0)
    run(p, ins, outs, [dev(x), dev(s)], [out])
    st, ref = oracle.skipln_dqq(x, s, beta, gamma, bias, dq_in, dq_skip, np.float32(1) / out_scale)
    assert st == 0
    assert_int8_close(host(out), ref, what="SkipLN INT8")


@pytest.mark.parametrize("version,total", [("7", 300), ("7", 4200), ("8", 77), ("8", 4100)])
def test_skipln_interleaved_plugin(reg, version, total):
    r = rng(102 + total)
    ld = 1024
    x, dq_in = quantize_amax(r.standard_normal((total, ld)))
    s, dq_skip = quantize_amax(r.standard_normal((total, ld)))
    gamma = r.uniform(0.5, 1.5, ld).astype(np.float16)
    beta = (0.3 * r.standard_normal(ld)).astype(np.float16)
    out_scale, pre_scale = np.float32(4.5 / 127), np.float32(6.0 / 127)
    c = reg.get_creator(SKIPLN, version)
    p = through_runtime(c, c.create_plugin("sln", [PluginField("beta", beta, F16), PluginField("gamma", gamma, F16)]))
    shape = [1, ld, total, 1]
    fmt = TensorFormat.CHW32
    ins = [TensorDesc(shape, DataType.INT8, fmt, dq_in), TensorDesc(shape, DataType.INT8, fmt, dq_skip)]
    outs = [TensorDesc(shape, DataType.INT8, fmt, out_scale)]
    d_out = dev_empty((ld * total,), np.int8, fill=0)
    bufs = [d_out]
    mtron = version == "8"
    if mtron:
        outs.append(TensorDesc(shape, DataType.INT8, fmt, pre_scale))
        bufs.append(dev_empty((ld * total,), np.int8, fill=0))
    x_il, s_il = oracle.interleave(x), oracle.interleave(s)
    run(p, ins, outs, [dev(x_il), dev(s_il)], bufs)
    st, ref, ref_pre = oracle.skipln_interleaved(int(mtron), x_il, s_il, beta, gamma, ld, total, dq_in, dq_skip,
                                                 np.float32(1) / out_scale, np.float32(1) / pre_scale)
    assert st == 0
    assert_int8_close(host(d_out), ref, what="out")
    if mtron:
        assert_int8_close(host(bufs[1]), ref_pre, what="preln")


# ---- EmbLayerNorm ----------------------------------------------------------------------------------

def emb_weights(r, ld, vocab, npos):
    return dict(beta=(0.1 * r.standard_normal(ld)).astype(np.float32),
                gamma=r.uniform(0.5, 1.5, ld).astype(np.float32),
                word=(0.02 * r.standard_normal((vocab, ld))).astype(np.float32),
                tok=(0.02 * r.standard_normal((2, ld))).astype(np.float32),
                pos=(0.02 * r.standard_normal((npos, ld))).astype(np.float32))


def emb_fields(w, fp16, extra=()):
    return [PluginField("bert_embeddings_layernorm_beta", w["beta"], F32),
            PluginField("bert_embeddings_layernorm_gamma", w["gamma"], F32),
            PluginField("bert_embeddings_word_embeddings", w["word"], F32),
            PluginField("bert_embeddings_token_type_embeddings", w["tok"], F32),
            PluginField("bert_embeddings_position_embeddings", w["pos"], F32),
            i32("output_fp16", fp16)] + list(extra)


@pytest.mark.parametrize("S,mha_type,fp16", [(128, 1, 1), (384, 2, 1), (64, 1, 1), (100, 1, 1), (128, 0, 0)])
def test_embln_v6_plugin(reg, S, mha_type, fp16):
    r = rng(110 + S)
    ld, B, vocab = 256, 4, 500
    w = emb_weights(r, ld, vocab, S)
    c = reg.get_creator(EMBLN, "6")
    p = through_runtime(c, c.create_plugin("emb", emb_fields(w, fp16, [i32("mha_type_id", mha_type)])))
    ids = r.integers(0, vocab, (S, B)).astype(np.int32)
    segs = r.integers(0, 2, (S, B)).astype(np.int32)
    lens = r.integers(1, S + 1, B)
    lens[0] = S
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    dt = DataType.HALF if fp16 else DataType.FLOAT
    npdt = NPDT[dt]
    ins = [TensorDesc([S, B], DataType.INT32)] * 3
    shapes = p.get_output_shapes(ins)
    packed = shapes[1][1]
    assert packed == ({64: 512, 96: 512, 128: 512, 384: 6144}.get(S, 1) if mha_type else 1)
    outs = [TensorDesc(shapes[0], dt), TensorDesc(shapes[1], DataType.INT32)]
    emb = dev_empty((S * B, ld), npdt, fill=0)
    mout = dev_empty((B, packed), np.int32, fill=0)
    run(p, ins, outs, [dev(ids), dev(segs), dev(mask)], [emb, mout])
    tabs = {k: w[k].astype(npdt) for k in ("word", "pos", "tok")}
    ref, _, _ = oracle.embln(0, ids, segs, None, w["beta"], w["gamma"], tabs["word"], tabs["pos"], tabs["tok"], S, B)
    assert_fp_close(host(emb), ref, what="embedding")
    if packed == 1:
        assert np.array_equal(host(mout).ravel(), oracle.mask_idx(mask))
    else:
        wm, wn = (1, 8) if S == 384 else (2, 2)
        want, _ = oracle.convert_mask(mask, wm, wn)
        # S = 64 and 96 share the S = 128 tensor size but are packed densely at its start
        got = host(mout).view(np.uint32).ravel()
        assert np.array_equal(got[:want.size], want.ravel())
        assert not got[want.size:].any()


@pytest.mark.parametrize("version", ["4", "5"])
@pytest.mark.parametrize("fp16", [0, 1])
def test_embln_varseqlen_plugin(reg, version, fp16):
    r = rng(111)
    ld, vocab, B = 384, 300, 5
    lens = np.array([17, 1, 128, 60, 33])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    w = emb_weights(r, ld, vocab, 128)
    c = reg.get_creator(EMBLN, version)
    p = through_runtime(c, c.create_plugin("emb", emb_fields(w, fp16)))
    ids = r.integers(0, vocab, T).astype(np.int32)
    segs = r.integers(0, 2, T).astype(np.int32)
    dt = DataType.HALF if fp16 else DataType.FLOAT
    npdt = NPDT[dt]
    ins = [TensorDesc([T], DataType.INT32), TensorDesc([T], DataType.INT32), TensorDesc([B + 1], DataType.INT32),
           TensorDesc([128], DataType.INT32)]
    mtron = version == "5"
    outs = [TensorDesc([T, ld, 1, 1], dt), TensorDesc([T, ld, 1, 1], dt) if mtron else TensorDesc([], DataType.INT32)]
    emb = dev_empty((T, ld), npdt, fill=0)
    skip = dev_empty((T, ld), npdt, fill=0) if mtron else None
    dummy = dev(np.zeros(128, np.int32))
    run(p, ins, outs, [dev(ids), dev(segs), dev(cu), dummy], [emb, skip])
    tabs = {k: w[k].astype(npdt) for k in ("word", "pos", "tok")}
    ref, ref_skip, _ = oracle.embln(2 if mtron else 1, ids, segs, cu, w["beta"], w["gamma"], tabs["word"],
                                    tabs["pos"], tabs["tok"], 128, B)
    assert_fp_close(host(emb), ref, what="embedding")
    if mtron:
        assert_fp_close(host(skip), ref_skip, what="skip")


# ---- QKVToContext ----------------------------------------------------------------------------------

def qkv_fields(type_id, hidden, heads, has_mask, extra=()):
    return [i32("type_id", type_id), i32("hidden_size", hidden), i32("num_heads", heads),
            i32("has_mask", has_mask)] + list(extra)


def int8_scales(qkv_f, widen=1.0):
    """Quantised tensor, its scale, and a context scale as a calibrator would set it: attention
    output is a convex combination of V rows, so amax(V) bounds it (reached by 1-token sequences).
    With s_ctx >= s_q a one-step difference in a single quantised probability moves the output by
    at most 127*dq_probs*s_q/s_ctx <= 1 step."""
    q, s_q = quantize_amax(qkv_f)
    return q, s_q, np.float32(s_q * widen)


def chain(s_q, s_ctx, d, dq_probs=np.float32(1 / 127)):
    """The scale chain of the INT8 runners (mhaRunner.cu:838-850) in binary32."""
    rs = np.float32(1) / np.sqrt(np.float32(d))
    s1 = np.float32(np.float32(s_q * s_q) * rs)
    s2 = np.float32(np.float32(dq_probs * s_q) / s_ctx)
    return s1, np.float32(1) / dq_probs, s2


@pytest.mark.parametrize("S", [128, 384, 64])
def test_qkv_v4_fp16_fused_with_packed_mask(reg, S):
    r = rng(120 + S)
    N, d, B = 4, 64, 3
    hidden = N * d
    qkv = r.standard_normal((S, B, 3 * hidden)).astype(np.float16)
    lens = np.array([S, 1, int(r.integers(2, S))])
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    wm, wn = (1, 8) if S == 384 else (2, 2)
    dense, _ = oracle.convert_mask(mask, wm, wn)
    size = 6144 if S == 384 else 512            # the mask tensor is sized for S = 128; shorter S pack densely
    packed = np.zeros(B * size, np.uint32)
    packed[:dense.size] = dense.ravel()
    packed = packed.reshape(B, size)
    c = reg.get_creator(QKV, "4")
    p = c.create_plugin("qkv", qkv_fields(1, hidden, N, 1))
    ins = [TensorDesc([S, B, 3 * hidden, 1, 1], DataType.HALF), TensorDesc([B, packed.shape[1]], DataType.INT32)]
    outs = [TensorDesc([S, B, hidden, 1, 1], DataType.HALF)]
    assert p.configure_plugin(ins, outs) == 0, last_log()
    assert p.get_workspace_size(ins, outs) == 0
    p = through_runtime(c, p)
    out = dev_empty((S, B, hidden), np.float16, fill=0)
    run(p, ins, outs, [dev(qkv), dev(packed)], [out])
    ref = oracle.mha_fused_f16_fixed(qkv, S, B, N, d, lens)
    got = host(out)
    for b in range(B):
        # rows past the sequence end attend the same keys and are defined; compare them all
        assert_fp_close(got[:, b], ref[:, b], what=f"sequence {b}")


@pytest.mark.parametrize("S", [128, 384])
def test_qkv_v4_int8_fused(reg, S):
    r = rng(121 + S)
    N, d, B = 2, 64, 3
    hidden = N * d
    q, s_q, s_ctx = int8_scales(r.standard_normal((S, B, 3 * hidden)))
    lens = np.array([S, 7, int(r.integers(8, S))])
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    wm, wn = (1, 8) if S == 384 else (2, 2)
    packed, _ = oracle.convert_mask(mask, wm, wn)
    c = reg.get_creator(QKV, "4")
    p = c.create_plugin("qkv", qkv_fields(2, hidden, N, 1))
    fmt = TensorFormat.CHW32
    ins = [TensorDesc([S, B, 3 * hidden, 1, 1], DataType.INT8, fmt, s_q),
           TensorDesc([B, packed.shape[1]], DataType.INT32)]
    outs = [TensorDesc([S, B, hidden, 1, 1], DataType.INT8, fmt, s_ctx)]
    assert p.configure_plugin(ins, outs) == 0, last_log()
    out = dev_empty((S, B, hidden), np.int8, fill=0)
    run(p, ins, outs, [dev(q), dev(packed)], [out])
    ref = oracle.mha_fused_i8_fixed(q, S, B, N, d, lens, *chain(s_q, s_ctx, d))
    assert_int8_close(host(out), ref, what="INT8 fused", max_frac_off=0.002)


@pytest.mark.parametrize("version", ["4", "5"])
@pytest.mark.parametrize("dt,S,has_mask", [(DataType.FLOAT, 48, 1), (DataType.HALF, 100, 1), (DataType.FLOAT, 33, 0)])
def test_qkv_unfused_path(reg, version, dt, S, has_mask):
    r = rng(122 + S)
    N, d, B = 3, 32, 4
    hidden = N * d
    npdt = NPDT[dt]
    qkv = r.standard_normal((S, B, 3 * hidden)).astype(npdt)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    c = reg.get_creator(QKV, version)
    p = c.create_plugin("qkv", qkv_fields(int(dt), hidden, N, has_mask))
    assert p is not None, last_log()
    ins = [TensorDesc([S, B, 3 * hidden, 1, 1], dt)]
    bufs = [dev(qkv)]
    if has_mask:
        ins.append(TensorDesc([B, 1], DataType.INT32) if version == "4" else TensorDesc([B], DataType.INT32))
        bufs.append(dev(lens))
    outs = [TensorDesc([S, B, hidden, 1, 1], dt)]
    assert p.configure_plugin(ins, outs) == 0, last_log()
    ws_bytes = p.get_workspace_size(ins, outs)
    assert ws_bytes == 2 * np.dtype(npdt).itemsize * S * S * B * N
    p = through_runtime(c, p)
    ws = dev_empty((ws_bytes,), np.uint8)
    out = dev_empty((S, B, hidden), npdt, fill=0)
    run(p, ins, outs, bufs, [out], ws)
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens if has_mask else None)
    assert_fp_close(host(out), ref, what="unfused attention")


@pytest.mark.parametrize("version", ["4", "5"])
def test_qkv_unfused_route_is_tuned_at_configure_and_travels_with_the_state(reg, version):
    """configurePlugin on a GPU times the unfused routes for the shape and writes the faster one into the first
    algorithm slot of the serialised runner state; a runtime plugin follows whatever the slot holds (either route, the
    default, a cuBLAS algorithm number written by the reference) to the same result."""
    r = rng(150)
    S, B, N, d = 70, 3, 2, 48
    hidden = N * d
    dt, npdt = DataType.HALF, np.float16
    qkv = r.standard_normal((S, B, 3 * hidden)).astype(npdt)
    lens = r.integers(1, S + 1, B).astype(np.int32)
    c = reg.get_creator(QKV, version)
    p = c.create_plugin("qkv", qkv_fields(int(dt), hidden, N, 1))
    ins = [TensorDesc([S, B, 3 * hidden, 1, 1], dt),
           TensorDesc([B, 1], DataType.INT32) if version == "4" else TensorDesc([B], DataType.INT32)]
    outs = [TensorDesc([S, B, hidden, 1, 1], dt)]
    assert p.configure_plugin(ins, outs) == 0, last_log()
    fields = p.get_fields_to_serialize()
    state = next(f for f in fields if f.name == "runnerStateBuffer")
    words = state.data.view(np.int32)
    assert words.tolist()[1:] == [99, S, B, d]
    assert words[0] in (0, 1), "the route found at configure time"
    ref = oracle.mha_unfused_fixed(qkv, S, B, N, d, lens)
    ws = dev_empty((p.get_workspace_size(ins, outs),), np.uint8)
    for slot in (0, 1, 99, 103):
        forged = [f if f.name != "runnerStateBuffer" else
                  PluginField("runnerStateBuffer", np.array([slot, 99, S, B, d], np.int32).view(np.uint8), f.type)
                  for f in fields]
        rt = c.create_plugin("rt", forged, TensorRTPhase.RUNTIME)
        assert rt is not None, last_log()
        out = dev_empty((S, B, hidden), npdt, fill=0)
        run(rt, ins, outs, [dev(qkv), dev(lens)], [out], ws)
        assert_fp_close(host(out), ref, what=f"unfused attention, slot {slot}")
        kept = next(f for f in rt.get_fields_to_serialize() if f.name == "runnerStateBuffer").data.view(np.int32)
        assert kept.tolist() == [slot, 99, S, B, d], "a runtime plugin keeps the state it was given"


@pytest.mark.parametrize("dt,d", [(DataType.HALF, 64), (DataType.INT8, 64), (DataType.HALF, 32), (DataType.INT8, 32),
                                  (DataType.HALF, 40)])
def test_qkv_v5_varseqlen(reg, dt, d):
    r = rng(123 + d)
    N = 3
    hidden = N * d
    lens = np.array([50, 1, 128, 77])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, B = int(cu[-1]), len(lens)
    qf = r.standard_normal((T, 3 * hidden))
    c = reg.get_creator(QKV, "5")
    p = c.create_plugin("qkv", qkv_fields(int(dt), hidden, N, 1, [i32("var_seqlen", 1)]))
    assert p is not None, last_log()
    if dt == DataType.INT8:
        q, s_q, s_ctx = int8_scales(qf)
        fmt = TensorFormat.CHW32 if (3 * hidden) % 32 == 0 else TensorFormat.CHW4
    else:
        q, s_q, s_ctx, fmt = qf.astype(np.float16), 1.0, 1.0, TensorFormat.LINEAR
    ins = [TensorDesc([T, 3 * hidden, 1, 1], dt, fmt, s_q), TensorDesc([1], DataType.INT32),
           TensorDesc([B + 1], DataType.INT32), TensorDesc([128], DataType.INT32)]
    outs = [TensorDesc([T, hidden, 1, 1], dt, fmt, s_ctx)]
    assert p.configure_plugin(ins, outs) == 0, last_log()
    ws_bytes = p.get_workspace_size(ins, outs)
    assert (ws_bytes == 0) == (d == 64)
    p = through_runtime(c, p)
    ws = dev_empty((max(ws_bytes, 1),), np.uint8)
    out = dev_empty((T, hidden), NPDT[dt], fill=0)
    dummy = dev(np.zeros(128, np.int32))
    run(p, ins, outs, [dev(q), dev(np.zeros(1, np.int32)), dev(cu), dummy], [out], ws)
    # the kernels run at the padded head size (32 or 64): zero columns change nothing but the
    # softmax scale, which is 1/sqrt(padded size)
    pad = 32 if d <= 32 else 64
    qp = np.zeros((T, N, 3, pad), q.dtype)
    qp[..., :d] = q.reshape(T, N, 3, d)
    qp = qp.reshape(T, 3 * N * pad)
    if dt == DataType.INT8:
        ref = oracle.mha_fused_i8_packed(qp, cu, N, pad, *chain(s_q, s_ctx, pad))
        ref = ref.reshape(T, N, pad)[..., :d].reshape(T, hidden)
        assert_int8_close(host(out), ref, what="INT8 varseqlen", max_frac_off=0.002)
    else:
        ref = oracle.mha_fused_f16_packed(qp, cu, N, pad)
        ref = ref.reshape(T, N, pad)[..., :d].reshape(T, hidden)
        assert_fp_close(host(out), ref, what="FP16 varseqlen")


@pytest.mark.parametrize("explicit", [0, 1])
def test_qkv_v6_interleaved(reg, explicit):
    r = rng(124)
    N, d = 4, 64
    hidden = N * d
    lens = np.array([384, 200, 1, 97, 256])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, B = int(cu[-1]), len(lens)
    dq_probs = np.float32(1 / 100) if explicit else np.float32(1 / 127)
    q, s_q, s_ctx = int8_scales(r.standard_normal((T, 3 * hidden)), widen=1.3 if explicit else 1.0)
    fs = [i32("hidden_size", hidden), i32("num_heads", N), f32("dq_probs", dq_probs)]
    if explicit:
        fs += [i32("use_explicit_int8", 1), f32("input_qkv_scale", s_q), f32("output_ctx_scale", s_ctx)]
    c = reg.get_creator(QKV, "6")
    p = through_runtime(c, c.create_plugin("qkv", fs))
    fmt = TensorFormat.CHW32
    # with explicit scales the tensor scales are ignored
    in_scale, out_scale = (123.0, 456.0) if explicit else (s_q, s_ctx)
    ins = [TensorDesc([1, 3 * hidden, T, 1], DataType.INT8, fmt, in_scale), TensorDesc([B + 1], DataType.INT32),
           TensorDesc([384], DataType.INT32)]
    outs = [TensorDesc([1, hidden, T, 1], DataType.INT8, fmt, out_scale)]
    # channel order of the interleaved tensor is [3][N][d]
    x = q.reshape(T, N, 3, d).transpose(0, 2, 1, 3).reshape(T, 3 * hidden)
    out = dev_empty((hidden * T,), np.int8, fill=0)
    dummy = dev(np.zeros(384, np.int32))
    run(p, ins, outs, [dev(oracle.interleave(x)), dev(cu), dummy], [out])
    ref = oracle.mha_fused_i8_packed(q, cu, N, d, *chain(s_q, s_ctx, d, dq_probs))
    assert_int8_close(oracle.deinterleave(host(out), T, hidden), ref, what="INT8 interleaved", max_frac_off=0.002)


def test_embln_feeds_qkv_through_the_packed_mask(reg):
    """Two plugins back to back, as in the encoder: the mask the embedding plugin emits is the one
    the attention plugin consumes."""
    r = rng(125)
    S, B, N, d, vocab = 128, 3, 2, 64, 200
    hidden = N * d
    w = emb_weights(r, hidden, vocab, S)
    ce = reg.get_creator(EMBLN, "6")
    pe = ce.create_plugin("emb", emb_fields(w, 1, [i32("mha_type_id", 1)]))
    lens = np.array([128, 5, 70])
    mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
    ids = r.integers(0, vocab, (S, B)).astype(np.int32)
    segs = np.zeros((S, B), np.int32)
    e_ins = [TensorDesc([S, B], DataType.INT32)] * 3
    e_outs = [TensorDesc([S, B, hidden, 1, 1], DataType.HALF), TensorDesc([B, 512], DataType.INT32)]
    emb = dev_empty((S, B, hidden), np.float16, fill=0)
    pm = dev_empty((B, 512), np.int32, fill=0)
    run(pe, e_ins, e_outs, [dev(ids), dev(segs), dev(mask)], [emb, pm])
    qkv = r.standard_normal((S, B, 3 * hidden)).astype(np.float16)
    cq = reg.get_creator(QKV, "4")
    pq = cq.create_plugin("qkv", qkv_fields(1, hidden, N, 1))
    q_ins = [TensorDesc([S, B, 3 * hidden, 1, 1], DataType.HALF), e_outs[1]]
    q_outs = [TensorDesc([S, B, hidden, 1, 1], DataType.HALF)]
    assert all(pq.supports_format_combination(i, q_ins + q_outs, 2) for i in range(3))
    assert pq.configure_plugin(q_ins, q_outs) == 0
    out = dev_empty((S, B, hidden), np.float16, fill=0)
    run(pq, q_ins, q_outs, [dev(qkv), pm], [out])
    assert_fp_close(host(out), oracle.mha_fused_f16_fixed(qkv, S, B, N, d, lens), what="attention")
