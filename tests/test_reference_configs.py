"""The reference's own plugin descriptions as test cases.

tests/golden/reference_plugin_configs.json is the data of the three *_PluginConfig.yaml files the reference keeps
beside the plugins on this path (written by tests/golden/make_reference_plugin_configs.py): per plugin version the
input/output names, accepted input types, PluginField attributes with types and required-ness, output shape
expressions, tolerances and named configurations.  The host tests check that the creators registered here accept
exactly that description; the GPU tests run every named configuration through the plugin object and compare with
the oracle under the tolerances the description states (the description names golden-output scripts that are not
part of the reference checkout, so expected values come from the oracle)."""
import json
import os

import numpy as np
import pytest

from tensorrt_amd.plugin import (DataType, PluginField, PluginFieldType, TensorDesc, TensorFormat, TensorRTPhase,
                                 capture_log, get_plugin_registry, last_log)

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_plugin_configs.json")) as _fh:
    GOLDEN = json.load(_fh)

SKIPLN = "CustomSkipLayerNormPluginDynamic"
EMBLN = "CustomEmbLayerNormPluginDynamic"
QKV = "CustomQKVToContextPluginDynamic"
FIELD_TYPE = {"int32": PluginFieldType.INT32, "float32": PluginFieldType.FLOAT32}
NP_TYPE = {"int32": np.int32, "float32": np.float32, "float16": np.float16}
DATA_TYPE = {"int32": DataType.INT32, "float32": DataType.FLOAT, "float16": DataType.HALF}

CASES = [(name, version, cfg) for name, body in sorted(GOLDEN.items())
         for version, desc in sorted(body["versions"].items()) for cfg in sorted(desc.get("configs") or {})]
VERSIONS = [(name, version) for name, body in sorted(GOLDEN.items()) for version in sorted(body["versions"])]


@pytest.fixture(scope="module")
def reg():
    capture_log(True)
    last_log()
    return get_plugin_registry()


def shape_of(text):
    return [int(v) for v in str(text).split(",")]


def make_fields(name, version, cfg_name, seed=7):
    """PluginFields of one named configuration: scalars take the stated value, tensors the stated shape with
    seeded values of the kind the plugin expects (gamma around 1, tables around 0)."""
    desc = GOLDEN[name]["versions"][version]
    cfg = desc["configs"][cfg_name]
    r = np.random.default_rng(seed)
    fields, values = [], {}
    for attr in desc["attributes"]:
        opt = cfg["attribute_options"].get(attr)
        if opt is None:
            continue
        kind = desc["attribute_types"][attr]
        if "value" in opt:
            data = np.array([opt["value"]], NP_TYPE[kind])
        else:
            shape = shape_of(opt["shape"])
            if "gamma" in attr:
                data = r.uniform(0.5, 1.5, shape)
            elif "embeddings" in attr and "layernorm" not in attr:
                data = 0.02 * r.standard_normal(shape)
            else:
                data = 0.1 * r.standard_normal(shape)
            data = data.astype(NP_TYPE[kind])
        values[attr] = data
        fields.append(PluginField(attr, data, FIELD_TYPE[kind]))
    return fields, values


def input_shapes(name, version, cfg_name, values):
    """Input shapes that satisfy the description's rank and constraints for this configuration."""
    cfg = GOLDEN[name]["versions"][version]["configs"][cfg_name]
    if name == SKIPLN:
        ld = values["beta"].shape[-1]
        return {"input": [6, 3, ld, 1, 1], "skip": [6, 3, ld, 1, 1]}
    if name == EMBLN:
        S = values["bert_embeddings_position_embeddings"].shape[0]  # token_id_0 == position_embeddings_0
        return {k: [S, 3] for k in ("token_id", "segment_id", "input_mask")}
    hidden = int(values["hidden_size"][0])
    shapes = {"input": [40, 2, 3 * hidden, 1, 1]}
    if "input_mask" in cfg["input_types"]:
        shapes["input_mask"] = [2, 1]
    return shapes


def input_names(desc, conf):
    """The version's inputs that the configuration feeds, then inputs only the configuration names (version 4 of
    the attention plugin lists `input` alone; its `has_mask` configuration adds `input_mask`)."""
    named = [n for n in desc["inputs"] if n in conf["input_types"]]
    return named + [n for n in conf["input_types"] if n not in named]


def evaluate_dims(expr, shapes, values):
    """'input_0, input_1, hidden_size_0, 1, 1': <input>_<i> is a dimension of an input, <attribute>_<i> a
    dimension of a tensor attribute or, for a one-element attribute, its value."""
    dims = []
    for tok in (t.strip() for t in expr.split(",")):
        if tok.lstrip("-").isdigit():
            dims.append(int(tok))
            continue
        base, idx = tok.rsplit("_", 1)
        if base in shapes:
            dims.append(shapes[base][int(idx)])
        elif values[base].size == 1:
            dims.append(int(values[base].ravel()[0]))
        else:
            dims.append(values[base].shape[int(idx)])
    return dims


# ---- host side ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("name,version", VERSIONS)
def test_described_versions_are_registered_with_the_described_attributes(reg, name, version):
    assert GOLDEN[name]["interface"] == "IPluginV3"
    creator = reg.get_creator(name, version)
    assert creator is not None, f"{name} version {version}"
    desc = GOLDEN[name]["versions"][version]
    advertised = [f.name for f in creator.field_names]
    assert set(desc["attributes"]) == set(advertised)
    assert set(desc["attributes_required"]) <= set(advertised)


@pytest.mark.parametrize("name,version,cfg", CASES)
def test_required_attributes_are_required_and_the_others_optional(reg, name, version, cfg):
    desc = GOLDEN[name]["versions"][version]
    fields, _ = make_fields(name, version, cfg)
    creator = reg.get_creator(name, version)
    assert creator.create_plugin("full", fields) is not None, last_log()
    required = set(desc["attributes_required"])
    only_required = [f for f in fields if f.name in required]
    assert creator.create_plugin("required only", only_required) is not None, last_log()
    for missing in sorted(required):
        assert creator.create_plugin("missing", [f for f in fields if f.name != missing]) is None, missing
        assert last_log() != ""


@pytest.mark.parametrize("name,version,cfg", CASES)
def test_described_types_formats_and_output_shapes(reg, name, version, cfg):
    desc = GOLDEN[name]["versions"][version]
    conf = desc["configs"][cfg]
    fields, values = make_fields(name, version, cfg)
    plugin = reg.get_creator(name, version).create_plugin("p", fields)
    assert plugin is not None, last_log()
    shapes = input_shapes(name, version, cfg, values)
    in_names = input_names(desc, conf)
    ins = [TensorDesc(shapes[n], DATA_TYPE[conf["input_types"][n]]) for n in in_names]
    for n in in_names:
        assert len(shapes[n]) == desc["input_dims"].get(n, len(shapes[n]))
    got_shapes = plugin.get_output_shapes(ins)
    got_types = plugin.get_output_data_types([d.type for d in ins])
    outs = []
    for i, out_name in enumerate(desc["outputs"]):
        assert list(got_shapes[i]) == evaluate_dims(desc["output_dims"][out_name], shapes, values), out_name
        outs.append(TensorDesc(got_shapes[i], got_types[i]))
    if "output_types" in conf:
        assert [got_types[i] for i in range(len(outs))] == [DATA_TYPE[conf["output_types"][n]] for n in desc["outputs"]]
    elif name == SKIPLN:
        assert got_types[0] == ins[0].type
    for pos in range(len(ins) + len(outs)):
        assert plugin.supports_format_combination(pos, ins + outs, len(ins)), f"position {pos}: {last_log()}"
    # a linear tensor of another floating type at the first input is not part of the description
    other = DataType.HALF if ins[0].type == DataType.FLOAT else DataType.FLOAT
    if ins[0].type != DataType.INT32:
        bad = [TensorDesc(shapes[in_names[0]], other)] + ins[1:]
        assert not plugin.supports_format_combination(0, bad + outs, len(ins))


# ---- GPU: every named configuration against the oracle, tolerances as described ------------------------

def close(got, ref, atol, rtol, what):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    err = np.abs(got - ref) - (atol + rtol * np.abs(ref))
    assert np.isfinite(got).all(), what
    assert err.max() <= 0, f"{what}: worst excess {err.max():.3e} (atol {atol}, rtol {rtol})"


@pytest.mark.gpu
@pytest.mark.parametrize("name,version,cfg", CASES)
def test_named_configuration_matches_the_oracle(reg, name, version, cfg):
    import oracle
    from helpers import dev, dev_empty, host, ptr, stream, sync

    desc = GOLDEN[name]["versions"][version]
    conf = desc["configs"][cfg]
    fields, values = make_fields(name, version, cfg)
    creator = reg.get_creator(name, version)
    built = creator.create_plugin("p", fields)
    plugin = creator.create_plugin("rt", built.get_fields_to_serialize(), TensorRTPhase.RUNTIME)
    assert plugin is not None, last_log()
    shapes = input_shapes(name, version, cfg, values)
    in_names = input_names(desc, conf)
    ins = [TensorDesc(shapes[n], DATA_TYPE[conf["input_types"][n]]) for n in in_names]
    out_shapes = plugin.get_output_shapes(ins)
    out_types = plugin.get_output_data_types([d.type for d in ins])
    outs = [TensorDesc(s, t) for s, t in zip(out_shapes, out_types)]
    r = np.random.default_rng(11)
    first = conf["input_types"][in_names[0]]
    atol, rtol = float(desc["abs_tol"]), float(desc["rel_tol"])
    if first == "float16" and "fp16_atol" in desc:
        atol, rtol = float(desc["fp16_atol"]), float(desc["fp16_rtol"])

    def run(inputs, outputs, workspace=None):
        assert plugin.configure_plugin(ins, outs) == 0, last_log()
        assert plugin.on_shape_change(ins, outs) == 0, last_log()
        st = plugin.enqueue(ins, outs, [ptr(t) for t in inputs], [ptr(t) for t in outputs], ptr(workspace), stream())
        assert st == 0, last_log()
        sync()

    if name == SKIPLN:
        npdt = NP_TYPE[first]
        ld = shapes["input"][2]
        x = r.standard_normal(shapes["input"][:3]).astype(npdt)
        skip = r.standard_normal(shapes["input"][:3]).astype(npdt)
        out = dev_empty(shapes["input"][:3], npdt, fill=0)
        run([dev(x), dev(skip)], [out])
        as_t = lambda k: values[k].reshape(-1).astype(npdt)
        ref = oracle.skipln(x.reshape(-1, ld), skip.reshape(-1, ld), as_t("beta"), as_t("gamma"), as_t("bias"))
        close(host(out).reshape(-1, ld), ref, atol, rtol, f"SkipLayerNorm v{version} {cfg}")
    elif name == EMBLN:
        S, B = shapes["token_id"]
        vocab, ld = values["bert_embeddings_word_embeddings"].shape
        ids = r.integers(0, vocab, (S, B)).astype(np.int32)
        segs = r.integers(0, 2, (S, B)).astype(np.int32)
        lens = r.integers(1, S + 1, B)
        mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
        npdt = np.float16 if int(values["output_fp16"][0]) else np.float32
        emb = dev_empty((S * B, ld), npdt, fill=0)
        mask_idx = dev_empty(tuple(out_shapes[1]), np.int32, fill=0)
        run([dev(ids), dev(segs), dev(mask)], [emb, mask_idx])
        tab = lambda k: values["bert_embeddings_" + k].astype(npdt)
        ref, _, _ = oracle.embln(0, ids, segs, None, values["bert_embeddings_layernorm_beta"],
                                 values["bert_embeddings_layernorm_gamma"], tab("word_embeddings"),
                                 tab("position_embeddings"), tab("token_type_embeddings"), S, B)
        close(host(emb), ref, atol, rtol, f"EmbLayerNorm v{version} {cfg}")
        assert np.array_equal(host(mask_idx).ravel(), lens)
    else:
        npdt = NP_TYPE[first]
        S, B = shapes["input"][:2]
        hidden, heads = int(values["hidden_size"][0]), int(values["num_heads"][0])
        d = hidden // heads
        qkv = (r.standard_normal((S, B, 3 * hidden)) / 8).astype(npdt)
        bufs = [dev(qkv)]
        lens = None
        if "input_mask" in shapes:
            lens = r.integers(1, S + 1, B).astype(np.int32)
            bufs.append(dev(lens))
        assert plugin.configure_plugin(ins, outs) == 0, last_log()
        ws = dev_empty((max(plugin.get_workspace_size(ins, outs), 1),), np.uint8)
        out = dev_empty((S, B, hidden), npdt, fill=0)
        run(bufs, [out], ws)
        ref = oracle.mha_unfused_fixed(qkv, S, B, heads, d, lens)
        close(host(out), ref, atol, rtol, f"QKVToContext v{version} {cfg}")
