"""The shared library loads without a GPU and exports every symbol the headers declare.
No compute entry point is called here."""
import ctypes
import os
import re

import pytest

import tensorrt_amd
from tensorrt_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def _declared(header, macro):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"^\s*#[^\n]*", "", text, flags=re.M)
    names = re.findall(macro + r"\s+[^;{(]*?\b(\w+)\s*\(", text)
    return sorted(set(names))


@pytest.fixture(scope="module")
def lib():
    return tensorrt_amd.load_library()


def test_kernel_header_symbols_exported(lib):
    names = _declared("trtamd_bert_kernels.h", "TRTAMD_API")
    assert len(names) >= 24
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trtamd_bert_kernels.h but not exported"
    # the ctypes table covers the same set
    assert sorted(capi.HEADER_SYMBOLS) == names


def test_test_hook_header_symbols_exported(lib):
    names = _declared("trtamd_test_hooks.h", "TRTAMD_API")
    assert names == sorted(capi.TEST_HOOK_SYMBOLS)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trtamd_test_hooks.h but not exported"


def test_every_exported_trtamd_symbol_is_declared_in_a_header(lib):
    """Nothing is exported behind the headers' back."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", tensorrt_amd._LIB], capture_output=True, text=True, check=True)
    exported = {l.split()[-1] for l in out.stdout.splitlines() if " T " in l and l.split()[-1].startswith("trtamd_")}
    declared = set()
    for h, macro in (("trtamd_bert_kernels.h", "TRTAMD_API"), ("trtamd_test_hooks.h", "TRTAMD_API"),
                     ("trtamd_encoder_ops.h", "TRTAMD_API"), ("trtamd_encoder_runtime.h", "TRTAMD_API"),
                     ("trtamd_plugin_c.h", "TRTAMD_PLUGIN_API")):
        declared |= set(_declared(h, macro))
    assert exported <= declared, sorted(exported - declared)


def test_encoder_ops_header_symbols_exported(lib):
    names = _declared("trtamd_encoder_ops.h", "TRTAMD_API")
    assert names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trtamd_encoder_ops.h but not exported"
    assert sorted(capi.ENCODER_OPS_SYMBOLS) == names


def test_encoder_runtime_header_symbols_exported(lib):
    names = _declared("trtamd_encoder_runtime.h", "TRTAMD_API")
    assert names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trtamd_encoder_runtime.h but not exported"
    assert sorted(capi.ENCODER_RUNTIME_SYMBOLS) == names


def test_encoder_runtime_rejects_bad_configurations(lib):
    a = capi.api()
    bad = capi.EncoderConfig(hidden=1000, heads=16, ffn=4096, layers=2, vocab=10, max_pos=8, type_vocab=2, max_seqlen=128)
    assert not a.encoder_create(ctypes.byref(bad))
    assert "64 channels" in a.last_error_str()
    ok = capi.EncoderConfig(hidden=128, heads=2, ffn=256, layers=1, vocab=10, max_pos=8, type_vocab=2, max_seqlen=128)
    h = a.encoder_create(ctypes.byref(ok))
    assert h
    # emb fp16 + five hidden-wide INT8 tensors + QKV + FFN intermediate + the two small extras, each 256-byte aligned
    assert a.encoder_workspace_size(h, 100) == 25600 + 5 * 12800 + 38400 + 25600 + 512 + 256
    assert a.encoder_enqueue(h, None, None, None, 1, 100, None, None, None) != 0
    assert "set_embedding" in a.last_error_str()
    assert a.encoder_set_layer(h, 3, ctypes.byref(capi.EncoderLayer())) != 0
    a.encoder_destroy(h)


def test_plugin_c_header_symbols_exported(lib):
    from tensorrt_amd import plugin
    names = _declared("trtamd_plugin_c.h", "TRTAMD_PLUGIN_API")
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trtamd_plugin_c.h but not exported"
    assert sorted(plugin.plugin_c_symbols()) == names


def test_nvinfer_entry_points_exported(lib):
    names = _declared("trtamd_nvinfer_api.h", r'extern\s+"C"\s+TENSORRTAPI')
    assert set(names) == {"getPluginRegistry", "getLogger", "initLibNvInferPlugins", "setLoggerFinder", "getCreators"}
    for n in names:
        assert hasattr(lib, n)


def test_version_and_error_string(lib):
    a = capi.api()
    assert a.version() >= 1
    assert isinstance(a.last_error_str(), str)


def test_fused_kernel_validity_table():
    a = capi.api()
    for dtype in (1, 2):
        for s in (1, 64, 96, 128, 192, 256, 384, 512):
            assert a.fused_mha_is_valid(dtype, 64, s) == 1
        assert a.fused_mha_is_valid(dtype, 64, 513) == 0
        assert a.fused_mha_is_valid(dtype, 32, 128) == 0
        assert a.fused_mha_is_valid(dtype, 128, 128) == 0
    assert a.fused_mha_is_valid(0, 64, 128) == 0  # no fused kernel in binary32


def test_unfused_workspace_formula():
    a = capi.api()
    # two S x S score matrices per (batch, head) in the compute type (mhaRunner.cu:522-525)
    assert a.unfused_mha_workspace_size(0, 128, 2, 12) == 2 * 4 * 128 * 128 * 2 * 12
    assert a.unfused_mha_workspace_size(1, 384, 1, 16) == 2 * 2 * 384 * 384 * 16


def test_missing_library_is_loud(monkeypatch, tmp_path):
    """No fallback: without the built library the package raises."""
    monkeypatch.setattr(tensorrt_amd, "_handle", None)
    monkeypatch.setattr(tensorrt_amd, "_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(tensorrt_amd.LibraryNotBuilt):
        tensorrt_amd.load_library()
