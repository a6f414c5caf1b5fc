"""Host-side behaviour of the IPluginV3 classes: registration, PluginField parsing and its error
messages, output shapes and types, supportsFormatCombination, workspace sizes, clone and the
serialise -> createPlugin(kRUNTIME) round trip.  Nothing here launches a kernel; the expectations
are the reference's (plugin/skipLayerNormPlugin, plugin/embLayerNormPlugin,
plugin/bertQKVToContextPlugin *.cpp)."""
import numpy as np
import pytest

from tensorrt_amd.plugin import (DataType, PluginField, PluginFieldType, TensorDesc, TensorFormat, TensorRTPhase,
                                 capture_log, get_plugin_registry, last_log)

SKIPLN = "CustomSkipLayerNormPluginDynamic"
EMBLN = "CustomEmbLayerNormPluginDynamic"
QKV = "CustomQKVToContextPluginDynamic"

I32 = PluginFieldType.INT32
F32 = PluginFieldType.FLOAT32
F16 = PluginFieldType.FLOAT16


def i32(name, v):
    return PluginField(name, np.array([v], np.int32), I32)


def f32(name, v):
    return PluginField(name, np.array([v], np.float32), F32)


@pytest.fixture(scope="module")
def reg():
    capture_log(True)
    last_log()
    return get_plugin_registry()


def fields_dict(fields):
    return {f.name: f for f in fields}


def roundtrip(creator, plugin, name="rt"):
    """serialise, re-create in the runtime phase, serialise again: same fields, same bytes."""
    a = plugin.get_fields_to_serialize()
    assert a is not None
    again = creator.create_plugin(name, a, TensorRTPhase.RUNTIME)
    assert again is not None, last_log()
    b = again.get_fields_to_serialize()
    assert [f.name for f in a] == [f.name for f in b]
    for x, y in zip(a, b):
        assert x.type == y.type and x.length == y.length, x.name
        if x.data is not None:
            assert x.data.tobytes() == y.data.tobytes(), x.name
    return again


# ---- registry --------------------------------------------------------------------------------------

def test_all_creators_registered(reg):
    want = {(SKIPLN, v) for v in "12345678"} | {(EMBLN, v) for v in "123456"} | {(QKV, v) for v in "123456"}
    assert set(reg.all_creators) == want
    # versions 1..(3|4) are IPluginCreator objects, the later ones IPluginCreatorV3One: each lookup sees its own kind
    assert reg.get_creator(SKIPLN, "1") is None and reg.get_legacy_creator(SKIPLN, "1") is not None
    assert reg.get_legacy_creator(SKIPLN, "5") is None
    assert reg.get_creator(SKIPLN, "5", "other_ns") is None
    assert reg.get_creator("NoSuchPlugin", "1") is None


def test_advertised_field_names(reg):
    names = lambda n, v: [f.name for f in reg.get_creator(n, v).field_names]
    assert names(SKIPLN, "5") == ["type_id", "ld", "beta", "gamma", "bias"]
    assert names(SKIPLN, "6") == ["type_id", "beta", "gamma", "bias"]
    assert names(SKIPLN, "7") == ["beta", "gamma"]
    assert names(SKIPLN, "8") == ["beta", "gamma"]
    emb = ["bert_embeddings_layernorm_beta", "bert_embeddings_layernorm_gamma", "bert_embeddings_word_embeddings",
           "bert_embeddings_token_type_embeddings", "bert_embeddings_position_embeddings", "output_fp16"]
    assert names(EMBLN, "6") == emb + ["full_mask", "mha_type_id"]
    assert set(names(EMBLN, "4")) == set(emb)
    assert set(names(EMBLN, "5")) == set(emb)
    assert names(QKV, "4") == ["type_id", "hidden_size", "num_heads", "has_mask", "dq_probs"]
    assert names(QKV, "5") == ["type_id", "hidden_size", "num_heads", "has_mask", "dq_probs", "var_seqlen",
                               "use_int8_scale_max"]
    assert names(QKV, "6") == ["hidden_size", "num_heads", "dq_probs", "use_int8_scale_max", "use_explicit_int8",
                               "input_qkv_scale", "output_ctx_scale"]


# ---- SkipLayerNorm ---------------------------------------------------------------------------------

def skipln_fields(ld=768, type_id=1, bias=False, with_ld=True, wtype=np.float32):
    r = np.random.default_rng(0)
    ft = F32 if wtype == np.float32 else F16
    fs = [i32("type_id", type_id),
          PluginField("beta", r.standard_normal(ld).astype(wtype), ft),
          PluginField("gamma", r.standard_normal(ld).astype(wtype), ft)]
    if with_ld:
        fs.append(i32("ld", ld))
    if bias:
        fs.append(PluginField("bias", r.standard_normal(ld).astype(wtype), ft))
    return fs


def test_skipln_missing_fields_are_reported(reg):
    c = reg.get_creator(SKIPLN, "5")
    assert c.create_plugin("x", [i32("ld", 768)]) is None
    assert "missing required fields: {beta, gamma, type_id}" in last_log()
    c6 = reg.get_creator(SKIPLN, "6")
    assert c6.create_plugin("x", [i32("type_id", 0)]) is None
    assert "missing required fields: {beta, gamma}" in last_log()
    bad = skipln_fields(type_id=7)
    assert c.create_plugin("x", bad) is None
    assert "Invalid type ID" in last_log()


@pytest.mark.parametrize("version", ["5", "6"])
@pytest.mark.parametrize("type_id", [0, 1, 2])
def test_skipln_linear_host_contract(reg, version, type_id):
    c = reg.get_creator(SKIPLN, version)
    ld = 768
    p = c.create_plugin("sln", skipln_fields(ld, type_id, bias=True, with_ld=version == "5"))
    assert p is not None, last_log()
    assert (p.plugin_name, p.plugin_version, p.plugin_namespace, p.num_outputs) == (SKIPLN, version, "", 1)
    dt = DataType(type_id)
    assert p.get_output_data_types([dt, dt]) == [dt]
    assert p.get_output_shapes([TensorDesc([128, 2, ld, 1, 1])] * 2) == [[128, 2, ld, 1, 1]]
    # INT8 I/O travels as CHW32 (CHW4 below 32 channels); the floating types are linear
    fmt = TensorFormat.CHW32 if type_id == 2 else TensorFormat.LINEAR
    good = [TensorDesc([128, 2, ld, 1, 1], dt, fmt)] * 3
    assert all(p.supports_format_combination(i, good, 2) for i in range(3))
    other_fmt = TensorFormat.LINEAR if type_id == 2 else TensorFormat.CHW32
    wrong = [TensorDesc([128, 2, ld, 1, 1], dt, other_fmt)] * 3
    assert not p.supports_format_combination(0, wrong, 2)
    other = DataType.HALF if dt != DataType.HALF else DataType.FLOAT
    mixed = [good[0], TensorDesc([128, 2, ld, 1, 1], other, fmt), good[0]]
    assert not p.supports_format_combination(1, mixed, 2)
    assert p.get_workspace_size(good[:2], good[2:]) == 0
    ser = fields_dict(p.get_fields_to_serialize())
    assert int(ser["type_id"].data[0]) == type_id
    # parameters are stored in binary16 unless the plugin computes in binary32
    want_t = F32 if type_id == 0 else F16
    assert ser["beta"].type == want_t and ser["gamma"].type == want_t and ser["bias"].type == want_t
    assert ser["beta"].length == ld
    q = p.clone()
    assert q is not None and q.plugin_version == version
    assert fields_dict(q.get_fields_to_serialize())["gamma"].data.tobytes() == ser["gamma"].data.tobytes()
    roundtrip(c, p)


def test_skipln_weight_conversion_is_round_to_nearest_even(reg):
    c = reg.get_creator(SKIPLN, "6")
    vals = np.array([1.0, 1.00048828125, 1.00146484375, -3.3333333, 65504.0, 1e-7, 0.0, 5.9604645e-8] * 4, np.float32)
    p = c.create_plugin("sln", [i32("type_id", 1), PluginField("beta", vals, F32), PluginField("gamma", vals, F32)])
    ser = fields_dict(p.get_fields_to_serialize())
    assert np.array_equal(ser["beta"].data.view(np.uint16), vals.astype(np.float16).view(np.uint16))
    # binary16 in, binary32 plugin: widening is exact
    h = vals.astype(np.float16)
    p = c.create_plugin("sln", [i32("type_id", 0), PluginField("beta", h, F16), PluginField("gamma", h, F16)])
    ser = fields_dict(p.get_fields_to_serialize())
    assert np.array_equal(ser["gamma"].data, h.astype(np.float32))


@pytest.mark.parametrize("version", ["7", "8"])
def test_skipln_interleaved_host_contract(reg, version):
    c = reg.get_creator(SKIPLN, version)
    ld, total = 1024, 300
    r = np.random.default_rng(1)
    fs = [PluginField("beta", r.standard_normal(ld).astype(np.float32), F32),
          PluginField("gamma", r.standard_normal(ld).astype(np.float16), F16)]
    p = c.create_plugin("sln", fs)
    assert p is not None, last_log()
    n_out = 2 if version == "8" else 1
    assert p.num_outputs == n_out
    assert p.get_output_data_types([DataType.INT8] * 2) == [DataType.INT8] * n_out
    shape = [1, ld, total, 1]
    assert p.get_output_shapes([TensorDesc(shape)] * 2) == [shape] * n_out
    il = [TensorDesc(shape, DataType.INT8, TensorFormat.CHW32)] * (2 + n_out)
    assert all(p.supports_format_combination(i, il, 2) for i in range(2 + n_out))
    lin = [TensorDesc(shape, DataType.INT8, TensorFormat.LINEAR)] * (2 + n_out)
    assert not p.supports_format_combination(0, lin, 2)
    half = [TensorDesc(shape, DataType.HALF, TensorFormat.CHW32)] * (2 + n_out)
    assert not p.supports_format_combination(0, half, 2)
    ser = fields_dict(p.get_fields_to_serialize())
    assert set(ser) == {"beta", "gamma"} and ser["beta"].type == F16 and ser["beta"].length == ld
    roundtrip(c, p)
    assert c.create_plugin("x", fs[:1]) is None
    assert "missing required fields: {gamma}" in last_log()


# ---- EmbLayerNorm ----------------------------------------------------------------------------------

def emb_fields(ld=128, vocab=30, types=2, npos=16, fp16=1, extra=()):
    r = np.random.default_rng(2)
    fs = [PluginField("bert_embeddings_layernorm_beta", r.standard_normal(ld).astype(np.float32), F32),
          PluginField("bert_embeddings_layernorm_gamma", r.standard_normal(ld).astype(np.float32), F32),
          PluginField("bert_embeddings_word_embeddings", r.standard_normal(vocab * ld).astype(np.float32), F32),
          PluginField("bert_embeddings_token_type_embeddings", r.standard_normal(types * ld).astype(np.float32), F32),
          PluginField("bert_embeddings_position_embeddings", r.standard_normal(npos * ld).astype(np.float32), F32),
          i32("output_fp16", fp16)]
    return fs + list(extra)


@pytest.mark.parametrize("mha_type,S,packed", [(1, 128, 512), (1, 384, 6144), (2, 64, 512), (1, 96, 512),
                                               (1, 200, 1), (0, 128, 1), (2, 256, 1)])
def test_embln_v6_shapes_and_mask_size(reg, mha_type, S, packed):
    c = reg.get_creator(EMBLN, "6")
    ld, B = 128, 3
    p = c.create_plugin("emb", emb_fields(ld, extra=[i32("mha_type_id", mha_type)]))
    assert p is not None, last_log()
    assert p.num_outputs == 2
    ins = [TensorDesc([S, B], DataType.INT32)] * 3
    assert p.get_output_shapes(ins) == [[S, B, ld, 1, 1], [B, packed]]
    assert p.get_output_data_types([DataType.INT32] * 3) == [DataType.HALF, DataType.INT32]
    io = ins + [TensorDesc([S, B, ld, 1, 1], DataType.HALF), TensorDesc([B, packed], DataType.INT32)]
    assert all(p.supports_format_combination(i, io, 3) for i in range(5))
    bad = list(io)
    bad[3] = TensorDesc([S, B, ld, 1, 1], DataType.FLOAT)
    assert not p.supports_format_combination(3, bad, 3)
    bad = list(io)
    bad[1] = TensorDesc([S, B + 1], DataType.INT32)
    assert not p.supports_format_combination(1, bad, 3)
    assert p.on_shape_change(io[:3], io[3:]) == 0
    wrong_mask = io[:4] + [TensorDesc([B, packed + 7], DataType.INT32)]
    assert p.on_shape_change(wrong_mask[:3], wrong_mask[3:]) != 0
    last_log()


def test_embln_v6_serialisation(reg):
    c = reg.get_creator(EMBLN, "6")
    p = c.create_plugin("emb", emb_fields(64, fp16=1, extra=[i32("mha_type_id", 2), i32("full_mask", 0)]))
    ser = fields_dict(p.get_fields_to_serialize())
    assert int(ser["output_fp16"].data[0]) == 1 and int(ser["mha_type_id"].data[0]) == 2
    assert ser["bert_embeddings_layernorm_beta"].type == F32          # LayerNorm parameters stay binary32
    assert ser["bert_embeddings_word_embeddings"].type == F16         # tables follow the output type
    assert ser["bert_embeddings_word_embeddings"].length == 30 * 64
    roundtrip(c, p)
    assert p.clone().get_output_shapes([TensorDesc([128, 2], DataType.INT32)] * 3)[1] == [2, 512]
    fs = emb_fields(64)
    assert c.create_plugin("emb", fs[1:]) is None
    assert "missing required fields: {bert_embeddings_layernorm_beta}" in last_log()
    # word table that is not a multiple of the hidden size
    fs = emb_fields(64)
    fs[2] = PluginField(fs[2].name, np.zeros(100, np.float32), F32)
    assert c.create_plugin("emb", fs) is None
    last_log()


@pytest.mark.parametrize("version", ["4", "5"])
def test_embln_varseqlen_host_contract(reg, version):
    c = reg.get_creator(EMBLN, version)
    ld, T, B = 128, 37, 4
    p = c.create_plugin("emb", emb_fields(ld, fp16=0))
    assert p is not None, last_log()
    assert p.num_outputs == 2
    ins = [TensorDesc([T], DataType.INT32), TensorDesc([T], DataType.INT32), TensorDesc([B + 1], DataType.INT32),
           TensorDesc([40], DataType.INT32)]
    shapes = p.get_output_shapes(ins)
    assert shapes[0] == [T, ld, 1, 1]
    if version == "4":
        assert p.get_output_data_types([DataType.INT32] * 4) == [DataType.FLOAT, DataType.INT32]
    else:
        assert shapes[1] == [T, ld, 1, 1]                  # Megatron: second output is the skip tensor
        assert p.get_output_data_types([DataType.INT32] * 4) == [DataType.FLOAT, DataType.FLOAT]
    ser = fields_dict(p.get_fields_to_serialize())
    assert int(ser["output_fp16"].data[0]) == 0
    assert ser["bert_embeddings_position_embeddings"].type == F32
    roundtrip(c, p)


# ---- QKVToContext ----------------------------------------------------------------------------------

def qkv_fields(type_id=1, hidden=768, heads=12, has_mask=1, extra=()):
    return [i32("type_id", type_id), i32("hidden_size", hidden), i32("num_heads", heads),
            i32("has_mask", has_mask)] + list(extra)


def test_qkv_v4_field_validation(reg):
    c = reg.get_creator(QKV, "4")
    assert c.create_plugin("q", qkv_fields()[:3]) is None
    assert "missing required fields: {has_mask}" in last_log()
    for bad, msg in ((qkv_fields(type_id=5), "Invalid TypeId"), (qkv_fields(hidden=0), "Invalid hiddenSize"),
                     (qkv_fields(heads=0), "Invalid numHeads"), (qkv_fields(has_mask=2), "Invalid hasMask"),
                     (qkv_fields(extra=[f32("dq_probs", -1.0)]), "Invalid dqProbs")):
        assert c.create_plugin("q", bad) is None
        assert msg in last_log()
    # runtime-only attributes are refused while building
    assert c.create_plugin("q", qkv_fields(extra=[i32("S", 128)])) is None
    last_log()


@pytest.mark.parametrize("type_id,S,fused", [(1, 128, True), (1, 384, True), (1, 64, True), (1, 100, False),
                                             (0, 128, False), (2, 384, True)])
def test_qkv_v4_host_contract(reg, type_id, S, fused):
    c = reg.get_creator(QKV, "4")
    hidden, heads, B = 768, 12, 2
    p = c.create_plugin("q", qkv_fields(type_id, hidden, heads, 1))
    assert p is not None, last_log()
    dt = DataType(type_id)
    fmt = TensorFormat.CHW32 if type_id == 2 else TensorFormat.LINEAR
    packed = {64: 512, 96: 512, 128: 512, 384: 6144}.get(S, 1) if type_id != 0 else 1
    qkv = TensorDesc([S, B, 3 * hidden, 1, 1], dt, fmt, scale=0.05)
    mask = TensorDesc([B, packed], DataType.INT32)
    out = TensorDesc([S, B, hidden, 1, 1], dt, fmt, scale=0.04)
    assert p.get_output_shapes([qkv, mask]) == [[S, B, hidden, 1, 1]]
    assert p.get_output_data_types([dt, DataType.INT32]) == [dt]
    io = [qkv, mask, out]
    assert all(p.supports_format_combination(i, io, 2) for i in range(3)), last_log()
    if packed != 1:
        wrong = [qkv, TensorDesc([B, 1], DataType.INT32), out]
        assert not p.supports_format_combination(1, wrong, 2)
        assert "expects mask pack size" in last_log()
    assert p.configure_plugin([qkv, mask], [out]) == 0, last_log()
    esize = {0: 4, 1: 2, 2: 1}[type_id]
    want_ws = 0 if fused else 2 * esize * S * S * B * heads
    assert p.get_workspace_size([qkv, mask], [out]) == want_ws
    ser = fields_dict(p.get_fields_to_serialize())
    assert int(ser["S"].data[0]) == S and int(ser["B"].data[0]) == B and int(ser["SM"].data[0]) >= 75
    assert int(ser["hasUnfusedDispatcher"].data[0]) == (0 if fused else 1)
    assert ("runnerStateBuffer" in ser) == (not fused)
    if not fused:
        st = ser["runnerStateBuffer"].data.view(np.int32)
        assert st[2:].tolist() == [S, B, hidden // heads]     # two GEMM algorithm ids, then S, B, head size
    if type_id == 2:
        assert abs(float(ser["dq_probs"].data[0]) - 1 / 127) < 1e-9
    rt = roundtrip(c, p)
    assert rt.get_workspace_size([qkv, mask], [out]) == want_ws
    assert rt.on_shape_change([qkv, mask], [out]) == 0
    cl = p.clone()
    assert cl.get_workspace_size([qkv, mask], [out]) == want_ws


def test_qkv_v4_int8_needs_a_fused_sequence_length(reg):
    c = reg.get_creator(QKV, "4")
    p = c.create_plugin("q", qkv_fields(2, 768, 12, 1))
    qkv = TensorDesc([200, 2, 2304, 1, 1], DataType.INT8, TensorFormat.CHW32)
    io = [qkv, TensorDesc([2, 1], DataType.INT32), TensorDesc([200, 2, 768, 1, 1], DataType.INT8, TensorFormat.CHW32)]
    assert not p.supports_format_combination(0, io, 2)
    assert "only support sequence length 128,384" in last_log()
    dyn = [TensorDesc([-1, 2, 2304, 1, 1], DataType.INT8, TensorFormat.CHW32)] + io[1:]
    assert not p.supports_format_combination(0, dyn, 2)
    assert "dynamic shape in sequence dimension" in last_log()


def test_qkv_v4_dynamic_sequence_sizes_workspace_for_the_longest_unfused_length(reg):
    c = reg.get_creator(QKV, "4")
    p = c.create_plugin("q", qkv_fields(1, 768, 12, 1))
    B = 2
    qkv = TensorDesc([-1, B, 2304, 1, 1], DataType.HALF, min=[1, B, 2304, 1, 1], max=[384, B, 2304, 1, 1],
                     opt=[128, B, 2304, 1, 1])
    mask = TensorDesc([B, -1], DataType.INT32, min=[B, 1], max=[B, 6144], opt=[B, 512])
    out = TensorDesc([-1, B, 768, 1, 1], DataType.HALF, min=[1, B, 768, 1, 1], max=[384, B, 768, 1, 1],
                     opt=[128, B, 768, 1, 1])
    assert p.configure_plugin([qkv, mask], [out]) == 0, last_log()
    # 384 is fused, so the largest length that needs scratch is 383
    assert p.get_workspace_size([qkv, mask], [out]) == 2 * 2 * 383 * 383 * B * 12


def test_qkv_v5_host_contract(reg):
    c = reg.get_creator(QKV, "5")
    hidden, heads = 1024, 16
    p = c.create_plugin("q", qkv_fields(2, hidden, heads, 1, extra=[i32("var_seqlen", 1)]))
    assert p is not None, last_log()
    T, B = 1000, 8
    qkv = TensorDesc([T, 3 * hidden, 1, 1], DataType.INT8, TensorFormat.CHW32, scale=0.05)
    ins = [qkv, TensorDesc([1], DataType.INT32), TensorDesc([B + 1], DataType.INT32), TensorDesc([384], DataType.INT32)]
    out = TensorDesc([T, hidden, 1, 1], DataType.INT8, TensorFormat.CHW32, scale=0.04)
    assert p.get_output_shapes(ins) == [[T, hidden, 1, 1]]
    io = ins + [out]
    assert all(p.supports_format_combination(i, io, 4) for i in range(5)), last_log()
    lin = [TensorDesc([T, 3 * hidden, 1, 1], DataType.INT8, TensorFormat.LINEAR)] + io[1:]
    assert not p.supports_format_combination(0, lin, 4)
    assert p.configure_plugin(ins, [out]) == 0
    assert p.get_workspace_size(ins, [out]) == 0            # head size 64: no padding, fused kernels need no scratch
    ser = fields_dict(p.get_fields_to_serialize())
    assert int(ser["var_seqlen"].data[0]) == 1 and int(ser["use_int8_scale_max"].data[0]) == 1
    assert ser["runnerStateBuffer"].data.view(np.int32).tolist() == [256, 1, 64]
    roundtrip(c, p)
    # a smaller head is zero-padded to 64 in scratch: 3 input + 1 output copies of [T, heads, 64]
    p32 = c.create_plugin("q", qkv_fields(1, 512, 16, 1, extra=[i32("var_seqlen", 1)]))
    q32 = TensorDesc([T, 3 * 512, 1, 1], DataType.HALF)
    assert p32.get_workspace_size([q32] + ins[1:], [TensorDesc([T, 512, 1, 1], DataType.HALF)]) \
        == 4 * T * 16 * 64 * 2 + 16
    # INT8 without variable sequence length has no implementation
    assert c.create_plugin("q", qkv_fields(2, hidden, heads, 1)) is None
    last_log()
    # head sizes above 64 are refused for variable sequence length
    assert c.create_plugin("q", qkv_fields(1, 2048, 16, 1, extra=[i32("var_seqlen", 1)])) is None
    last_log()


def test_qkv_v5_fixed_length_uses_the_unfused_runner(reg):
    c = reg.get_creator(QKV, "5")
    hidden, heads, S, B = 256, 4, 48, 3
    p = c.create_plugin("q", qkv_fields(0, hidden, heads, 1))
    qkv = TensorDesc([S, B, 3 * hidden, 1, 1], DataType.FLOAT)
    mask = TensorDesc([B], DataType.INT32)
    out = TensorDesc([S, B, hidden, 1, 1], DataType.FLOAT)
    io = [qkv, mask, out]
    assert all(p.supports_format_combination(i, io, 2) for i in range(3)), last_log()
    assert p.configure_plugin([qkv, mask], [out]) == 0
    assert p.get_workspace_size([qkv, mask], [out]) == 2 * 4 * S * S * B * heads
    ser = fields_dict(p.get_fields_to_serialize())
    assert ser["runnerStateBuffer"].data.view(np.int32)[2:].tolist() == [S, B, hidden // heads]
    rt = roundtrip(c, p)
    assert rt.get_workspace_size([qkv, mask], [out]) == 2 * 4 * S * S * B * heads


def test_qkv_v6_host_contract(reg):
    c = reg.get_creator(QKV, "6")
    assert c.create_plugin("q", [i32("hidden_size", 1024)]) is None
    assert "missing required fields: {num_heads}" in last_log()
    hidden, heads, total, B = 1024, 16, 5000, 16
    p = c.create_plugin("q", [i32("hidden_size", hidden), i32("num_heads", heads), f32("dq_probs", 1 / 100.0),
                              i32("use_explicit_int8", 1), f32("input_qkv_scale", 0.07), f32("output_ctx_scale", 0.03)])
    assert p is not None, last_log()
    ins = [TensorDesc([1, 3 * hidden, total, 1], DataType.INT8, TensorFormat.CHW32),
           TensorDesc([B + 1], DataType.INT32), TensorDesc([384], DataType.INT32)]
    out = TensorDesc([1, hidden, total, 1], DataType.INT8, TensorFormat.CHW32)
    assert p.get_output_shapes(ins) == [[1, hidden, total, 1]]
    assert p.get_output_data_types([DataType.INT8, DataType.INT32, DataType.INT32]) == [DataType.INT8]
    io = ins + [out]
    assert all(p.supports_format_combination(i, io, 3) for i in range(4))
    lin = [TensorDesc([1, 3 * hidden, total, 1], DataType.INT8, TensorFormat.LINEAR)] + io[1:]
    assert not p.supports_format_combination(0, lin, 3)
    assert p.get_workspace_size(ins, [out]) == 0
    ser = fields_dict(p.get_fields_to_serialize())
    assert abs(float(ser["dq_probs"].data[0]) - 0.01) < 1e-9
    assert abs(float(ser["input_qkv_scale"].data[0]) - 0.07) < 1e-8
    assert int(ser["use_explicit_int8"].data[0]) == 1 and int(ser["use_int8_scale_max"].data[0]) == 1
    roundtrip(c, p)
    for bad, msg in (([i32("hidden_size", 0), i32("num_heads", 16)], "Invalid hiddenSize"),
                     ([i32("hidden_size", 1024), i32("num_heads", 16), f32("input_qkv_scale", -1.0)],
                      "Invalid input_qkv_scale")):
        assert c.create_plugin("q", bad) is None
        assert msg in last_log()


def test_enqueue_without_a_gpu_fails_cleanly(reg):
    """On a host with no device the parameters never reach device memory; enqueue reports failure
    instead of touching a null pointer.  (On a GPU box this path is covered by the parity tests.)"""
    import torch
    if torch.cuda.is_available():
        pytest.skip("needs a host without a GPU")
    c = reg.get_creator(SKIPLN, "6")
    p = c.create_plugin("sln", skipln_fields(768, 1, with_ld=False))
    d = TensorDesc([4, 1, 768, 1, 1], DataType.HALF)
    assert p.enqueue([d, d], [d], [0, 0], [0]) != 0
    assert last_log() != ""


# ---- the IPluginV2DynamicExt ("Legacy") versions ------------------------------------------------------

LEGACY = [(SKIPLN, "1", "5"), (SKIPLN, "2", "6"), (SKIPLN, "3", "7"), (SKIPLN, "4", "8"),
          (EMBLN, "1", "6"), (EMBLN, "2", "4"), (EMBLN, "3", "5"),
          (QKV, "1", "4"), (QKV, "2", "5"), (QKV, "3", "6")]


def legacy_fields(name, version):
    r = np.random.default_rng(5)
    if name == SKIPLN:
        ld = 768
        fs = [PluginField("beta", r.standard_normal(ld).astype(np.float32), F32),
              PluginField("gamma", r.standard_normal(ld).astype(np.float32), F32)]
        if version in "12":
            fs += [i32("type_id", 1), PluginField("bias", r.standard_normal(ld).astype(np.float32), F32)]
        if version == "1":
            fs.append(i32("ld", ld))
        return fs
    if name == EMBLN:
        ld = 128
        fs = [PluginField("bert_embeddings_layernorm_beta", r.standard_normal(ld).astype(np.float32), F32),
              PluginField("bert_embeddings_layernorm_gamma", r.standard_normal(ld).astype(np.float32), F32),
              PluginField("bert_embeddings_word_embeddings", r.standard_normal((50, ld)).astype(np.float32), F32),
              PluginField("bert_embeddings_token_type_embeddings", r.standard_normal((2, ld)).astype(np.float32), F32),
              PluginField("bert_embeddings_position_embeddings", r.standard_normal((64, ld)).astype(np.float32), F32),
              i32("output_fp16", 1)]
        if version == "1":
            fs += [i32("full_mask", 0), i32("mha_type_id", 1)]
        return fs
    if version == "3":
        return [i32("hidden_size", 1024), i32("num_heads", 16), f32("dq_probs", 1 / 127)]
    fs = [i32("type_id", 1), i32("hidden_size", 768), i32("num_heads", 12), i32("has_mask", 1)]
    if version == "2":
        fs.append(i32("var_seqlen", 1))
    return fs


@pytest.mark.parametrize("name,legacy,current", LEGACY)
def test_legacy_versions_wrap_the_current_plugins(reg, name, legacy, current):
    """Versions and creator fields of the reference's *Legacy.cpp files; same behaviour as the V3 version."""
    lc = reg.get_legacy_creator(name, legacy)
    cc = reg.get_creator(name, current)
    assert lc is not None and cc is not None
    assert sorted(f.name for f in lc.field_names) == sorted(f.name for f in cc.field_names)
    fs = legacy_fields(name, legacy)
    p = lc.create_plugin("layer", fs)
    assert p is not None, last_log()
    ref = cc.create_plugin("layer", fs, TensorRTPhase.BUILD)
    assert p.plugin_type == name and p.plugin_version == legacy
    assert p.num_outputs == ref.num_outputs
    # IPluginV2DynamicExt::getTensorRTVersion: PluginVersion::kV2_DYNAMICEXT in the top byte, TensorRT 11.1.0 below
    assert p.tensorrt_version == (3 << 24) | 110100
    assert p.initialize() == 0
    p.terminate()
    if name == QKV and legacy != "3":
        # the attention plugins serialise the runner chosen in configurePlugin (S, B), as the reference's do
        if legacy == "1":
            ins = [TensorDesc([128, 2, 3 * 768, 1, 1], DataType.HALF), TensorDesc([2, 512], DataType.INT32)]
            outs = [TensorDesc([128, 2, 768, 1, 1], DataType.HALF)]
        else:
            ins = [TensorDesc([300, 3 * 768, 1, 1], DataType.HALF), TensorDesc([1], DataType.INT32),
                   TensorDesc([5], DataType.INT32), TensorDesc([128], DataType.INT32)]
            outs = [TensorDesc([300, 768, 1, 1], DataType.HALF)]
        p.configure_plugin(ins, outs)

    # serialize -> deserializePlugin -> serialize reproduces the bytes; a clone serialises to the same bytes
    blob = p.serialize()
    assert len(blob) == p.get_serialization_size() > 0
    q = lc.deserialize_plugin("layer", blob)
    assert q is not None, last_log()
    assert q.plugin_version == legacy and q.serialize() == blob
    assert p.clone().serialize() == blob
    # a damaged stream is refused with a message, not a crash
    assert lc.deserialize_plugin("layer", blob[: len(blob) // 2]) is None
    assert "truncated" in last_log()
    assert lc.deserialize_plugin("layer", b"\0" * 64) is None
    last_log()


def test_legacy_streams_have_the_reference_byte_layout(reg):
    """serialize() writes the members of the reference's legacy classes in the order and widths of their own
    serialize() functions (bool 1 byte, int32_t / DataType / float 4, size_t 8, weights raw, no padding).  The
    expected bytes are put together by hand here, one plugin of each family and layout."""
    import struct
    r = np.random.default_rng(11)
    HALF, FLOAT, INT32 = 1, 0, 3
    SM = 80

    # SkipLayerNorm 1 (skipLayerNormPluginLegacy.cpp:381-402): mType, mCfgType, mLd, mHasBias, beta, gamma, bias
    ld = 64
    beta, gamma, bias = (r.standard_normal(ld).astype(np.float32) for _ in range(3))
    lc = reg.get_legacy_creator(SKIPLN, "1")
    p = lc.create_plugin("l", [PluginField("beta", beta, F32), PluginField("gamma", gamma, F32),
                               PluginField("bias", bias, F32), i32("type_id", HALF), i32("ld", ld)])
    want = struct.pack("<iiQB", HALF, HALF, ld, 1) + b"".join(a.astype(np.float16).tobytes() for a in (beta, gamma, bias))
    assert p.serialize() == want
    p = lc.create_plugin("l", [PluginField("beta", beta, F32), PluginField("gamma", gamma, F32), i32("type_id", FLOAT),
                               i32("ld", ld)])
    assert p.serialize() == struct.pack("<iiQB", FLOAT, FLOAT, ld, 0) + beta.tobytes() + gamma.tobytes()
    q = lc.deserialize_plugin("l", want)
    assert q is not None and q.serialize() == want

    # SkipLayerNorm 3 (skipLayerNormInt8InterleavedPluginLegacy.cpp): mLd, beta, gamma in binary16
    p = reg.get_legacy_creator(SKIPLN, "3").create_plugin("l", [PluginField("beta", beta, F32), PluginField("gamma", gamma, F32)])
    assert p.serialize() == struct.pack("<Q", ld) + beta.astype(np.float16).tobytes() + gamma.astype(np.float16).tobytes()

    # EmbLayerNorm 1 (embLayerNormPluginLegacy.cpp): mType, mMhaType, mLd, mS, three vocabulary sizes, mUseFullMask,
    # mSM, beta, gamma (binary32), word, position, token-type tables (mType)
    E, V, P, T = 32, 10, 16, 2
    eb, eg = r.standard_normal(E).astype(np.float32), r.standard_normal(E).astype(np.float32)
    word, pos, tok = (r.standard_normal((n, E)).astype(np.float32) for n in (V, P, T))
    emb = [PluginField("bert_embeddings_layernorm_beta", eb, F32), PluginField("bert_embeddings_layernorm_gamma", eg, F32),
           PluginField("bert_embeddings_word_embeddings", word, F32),
           PluginField("bert_embeddings_token_type_embeddings", tok, F32),
           PluginField("bert_embeddings_position_embeddings", pos, F32), i32("output_fp16", 1)]
    lc = reg.get_legacy_creator(EMBLN, "1")
    p = lc.create_plugin("l", emb + [i32("full_mask", 1), i32("mha_type_id", HALF)])
    tables = b"".join(a.astype(np.float16).tobytes() for a in (word, pos, tok))
    head = lambda S: struct.pack("<iiQQQQQBi", HALF, HALF, E, S, V, P, T, 1, SM)
    assert p.serialize() == head(0) + eb.tobytes() + eg.tobytes() + tables
    ids = TensorDesc([128, 4], DataType.INT32)
    p.configure_plugin([ids, ids, ids], [TensorDesc([128, 4, E, 1, 1], DataType.HALF), TensorDesc([4, 512], DataType.INT32)])
    blob = p.serialize()
    assert blob == head(128) + eb.tobytes() + eg.tobytes() + tables      # configurePlugin sets mS
    q = lc.deserialize_plugin("l", blob)
    assert q is not None and q.serialize() == blob and q.clone().serialize() == blob

    # EmbLayerNorm 2 / 3 (embLayerNormVarSeqlenPluginLegacy.cpp:544-562): mType, mLd, vocabulary sizes, mMaskType
    for version, mask_type in (("2", INT32), ("3", FLOAT)):
        fields = emb[:-1] + [i32("output_fp16", 0)]
        p = reg.get_legacy_creator(EMBLN, version).create_plugin("l", fields)
        want = struct.pack("<iQQQQi", FLOAT, E, V, P, T, mask_type) + eb.tobytes() + eg.tobytes() + word.tobytes() \
            + pos.tobytes() + tok.tobytes()
        assert p.serialize() == want

    # QKV-to-context 1 (qkvToContextPluginLegacy.cpp:399-422): mType, mNumHeads, mHeadSize, mHasImask, mHiddenSize, mSM,
    # mS, mB, mDqProbs, hasUnfusedRunner, then the unfused runner: two GEMM algorithms, S, B, head size
    lc = reg.get_legacy_creator(QKV, "1")
    p = lc.create_plugin("l", [i32("type_id", HALF), i32("hidden_size", 768), i32("num_heads", 12), i32("has_mask", 1)])
    assert p.serialize() == struct.pack("<iiiBiiiifi", HALF, 12, 64, 1, 768, SM, 0, 0, -1.0, 0)
    p.configure_plugin([TensorDesc([128, 2, 3 * 768, 1, 1], DataType.HALF), TensorDesc([2, 512], DataType.INT32)],
                       [TensorDesc([128, 2, 768, 1, 1], DataType.HALF)])
    # S = 128 has a fused kernel: only that runner is set up, and no runner state is written
    assert p.serialize() == struct.pack("<iiiBiiiifi", HALF, 12, 64, 1, 768, SM, 128, 2, -1.0, 0)
    p.configure_plugin([TensorDesc([200, 2, 3 * 768, 1, 1], DataType.HALF), TensorDesc([2, 1], DataType.INT32)],
                       [TensorDesc([200, 2, 768, 1, 1], DataType.HALF)])
    blob = p.serialize()
    assert blob == struct.pack("<iiiBiiiifi", HALF, 12, 64, 1, 768, SM, 200, 2, -1.0, 1) \
        + struct.pack("<iiiii", 99, 99, 200, 2, 64)          # CUBLAS_GEMM_DEFAULT_TENSOR_OP = 99 twice
    q = lc.deserialize_plugin("l", blob)
    assert q is not None and q.serialize() == blob

    # QKV-to-context 2 (:909-925): ..., mDqProbs, mUseVarSeqlen, mHdim, mUseInt8ScaleMax, then the fused runner: S, B,
    # head size
    lc = reg.get_legacy_creator(QKV, "2")
    p = lc.create_plugin("l", [i32("type_id", 2), i32("hidden_size", 1024), i32("num_heads", 16), i32("has_mask", 1),
                               i32("var_seqlen", 1), f32("dq_probs", 0.5)])
    p.configure_plugin([TensorDesc([300, 3 * 1024, 1, 1], DataType.INT8, TensorFormat.CHW32, 0.1), TensorDesc([1], DataType.INT32),
                        TensorDesc([5], DataType.INT32), TensorDesc([128], DataType.INT32)],
                       [TensorDesc([300, 1024, 1, 1], DataType.INT8, TensorFormat.CHW32, 0.1)])
    blob = p.serialize()
    # variable sequence length: mS and mB stay unset, the runner holds the placeholder geometry (256, 1) that
    # configurePlugin gives it (qkvToContextPluginLegacy.cpp, QKVToContextVarSeqlenPluginLegacy::configurePlugin)
    assert blob == struct.pack("<iiiBiiiifBiB", 2, 16, 64, 1, 1024, SM, 0, 0, 0.5, 1, 1, 1) + struct.pack("<iii", 256, 1, 64)
    q = lc.deserialize_plugin("l", blob)
    assert q is not None and q.serialize() == blob

    # QKV-to-context 3 (qkvToContextInt8InterleavedPluginLegacy.cpp): heads, head size, hidden, SM, S, B, dq_probs,
    # use_int8_scale_max, use_explicit_int8, the two explicit scales
    lc = reg.get_legacy_creator(QKV, "3")
    p = lc.create_plugin("l", [i32("hidden_size", 1024), i32("num_heads", 16), f32("dq_probs", 0.25),
                               i32("use_explicit_int8", 1), f32("input_qkv_scale", 0.5), f32("output_ctx_scale", 0.125)])
    blob = p.serialize()
    assert blob == struct.pack("<iiiiiifBBff", 16, 64, 1024, SM, 0, 0, 0.25, 1, 1, 0.5, 0.125)
    q = lc.deserialize_plugin("l", blob)
    assert q is not None and q.serialize() == blob
    for cut in (1, 8, len(blob) - 1):
        assert lc.deserialize_plugin("l", blob[:cut]) is None
        assert "truncated" in last_log()


def test_legacy_skipln_shapes_types_formats(reg):
    lc = reg.get_legacy_creator(SKIPLN, "1")
    p = lc.create_plugin("sln", legacy_fields(SKIPLN, "1"))
    shape = [128, 4, 768, 1, 1]
    half = TensorDesc(shape, DataType.HALF)
    assert p.get_output_dimensions(0, [half, half]) == shape
    assert p.get_output_dimensions(1, [half, half]) is None
    assert p.get_output_data_type(0, [DataType.HALF, DataType.HALF]) == DataType.HALF
    assert p.supports_format_combination(0, [half, half, half], 2)
    assert p.supports_format_combination(2, [half, half, half], 2)
    assert not p.supports_format_combination(1, [half, TensorDesc(shape, DataType.FLOAT), half], 2)
    assert p.get_workspace_size([half, half], [half]) == 0


def test_legacy_enqueue_without_a_gpu_fails_cleanly(reg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lc = reg.get_legacy_creator(SKIPLN, "3")
    p = lc.create_plugin("sln", legacy_fields(SKIPLN, "3"))
    d = TensorDesc([1, 768, 64, 1], DataType.INT8, TensorFormat.CHW32, 0.1)
    assert p.enqueue([d, d], [d], [0, 0], [0]) != 0
