"""Python view of the IPluginV3 classes in libtrtamd_bert_plugins.so.

The names follow TensorRT's Python API (``trt.PluginField``, ``trt.PluginFieldType``,
``trt.get_plugin_registry().get_creator(name, version)``, ``creator.create_plugin(name, fc, phase)``,
python/src/infer/pyPlugin.cpp), so code written against the reference's demo builders
(demo/BERT/builder.py:130-200 builds exactly such field collections) reads the same here.  The calls
go through the flat C functions of include/trtamd_plugin_c.h; device buffers are raw addresses.
"""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass, field
from typing import Iterable, Sequence

import numpy as np

from . import load_library

MAX_DIMS = 8


class DataType(enum.IntEnum):
    FLOAT = 0
    HALF = 1
    INT8 = 2
    INT32 = 3
    BOOL = 4
    UINT8 = 5
    FP8 = 6
    BF16 = 7
    INT64 = 8
    INT4 = 9


class TensorFormat(enum.IntEnum):
    LINEAR = 0
    CHW2 = 1
    HWC8 = 2
    CHW4 = 3
    CHW16 = 4
    CHW32 = 5


class PluginFieldType(enum.IntEnum):
    FLOAT16 = 0
    FLOAT32 = 1
    FLOAT64 = 2
    INT8 = 3
    INT16 = 4
    INT32 = 5
    CHAR = 6
    DIMS = 7
    UNKNOWN = 8
    BF16 = 9
    INT64 = 10


class TensorRTPhase(enum.IntEnum):
    BUILD = 0
    RUNTIME = 1


_NP_OF_FIELD = {
    PluginFieldType.FLOAT16: np.float16, PluginFieldType.FLOAT32: np.float32, PluginFieldType.FLOAT64: np.float64,
    PluginFieldType.INT8: np.int8, PluginFieldType.INT16: np.int16, PluginFieldType.INT32: np.int32,
    PluginFieldType.CHAR: np.uint8, PluginFieldType.UNKNOWN: np.uint8, PluginFieldType.INT64: np.int64,
}


class _CField(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("type", C.c_int32), ("length", C.c_int32)]


class _CDesc(C.Structure):
    _fields_ = [("nb_dims", C.c_int32), ("dims", C.c_int64 * MAX_DIMS), ("min", C.c_int64 * MAX_DIMS),
                ("max", C.c_int64 * MAX_DIMS), ("opt", C.c_int64 * MAX_DIMS), ("type", C.c_int32),
                ("format", C.c_int32), ("scale", C.c_float)]


@dataclass
class PluginField:
    """trt.PluginField: a named array; ``data`` is a numpy array (or scalar) kept alive by the field."""
    name: str
    data: np.ndarray | None
    type: PluginFieldType = PluginFieldType.UNKNOWN

    def __post_init__(self):
        if self.data is not None:
            self.data = np.ascontiguousarray(self.data)

    @property
    def length(self) -> int:
        return 0 if self.data is None else int(self.data.size)


@dataclass
class TensorDesc:
    """PluginTensorDesc / DynamicPluginTensorDesc; min/max/opt default to dims."""
    dims: Sequence[int]
    type: DataType = DataType.FLOAT
    format: TensorFormat = TensorFormat.LINEAR
    scale: float = 1.0
    min: Sequence[int] | None = None
    max: Sequence[int] | None = None
    opt: Sequence[int] | None = None

    def to_c(self) -> _CDesc:
        d = _CDesc()
        d.nb_dims = len(self.dims)
        for dst, src in (("dims", self.dims), ("min", self.min or self.dims), ("max", self.max or self.dims),
                         ("opt", self.opt or self.dims)):
            arr = getattr(d, dst)
            for i, v in enumerate(src):
                arr[i] = int(v)
        d.type = int(self.type)
        d.format = int(self.format)
        d.scale = float(self.scale)
        return d


def _descs(seq: Iterable[TensorDesc]):
    lst = [t.to_c() for t in seq]
    return (_CDesc * max(len(lst), 1))(*lst), len(lst)


_lib = None


def _library():
    global _lib
    if _lib is not None:
        return _lib
    lib = load_library()
    vp, i32 = C.c_void_p, C.c_int32
    pf = C.POINTER(_CField)
    pd = C.POINTER(_CDesc)
    sigs = {
        "trtamd_plugin_get_creator": (vp, [C.c_char_p, C.c_char_p, C.c_char_p]),
        "trtamd_plugin_num_creators": (i32, []),
        "trtamd_plugin_creator_name": (C.c_char_p, [i32]),
        "trtamd_plugin_creator_version": (C.c_char_p, [i32]),
        "trtamd_plugin_creator_field_names": (i32, [vp, C.POINTER(pf)]),
        "trtamd_plugin_create": (vp, [vp, C.c_char_p, pf, i32, i32]),
        "trtamd_plugin_destroy": (None, [vp]),
        "trtamd_plugin_clone": (vp, [vp]),
        "trtamd_plugin_name": (C.c_char_p, [vp]),
        "trtamd_plugin_version": (C.c_char_p, [vp]),
        "trtamd_plugin_namespace": (C.c_char_p, [vp]),
        "trtamd_plugin_nb_outputs": (i32, [vp]),
        "trtamd_plugin_output_types": (i32, [vp, C.POINTER(i32), i32, C.POINTER(i32), i32]),
        "trtamd_plugin_output_shapes": (i32, [vp, pd, i32, pd, i32]),
        "trtamd_plugin_supports_format": (i32, [vp, i32, pd, i32, i32]),
        "trtamd_plugin_configure": (i32, [vp, pd, i32, pd, i32]),
        "trtamd_plugin_workspace_size": (C.c_size_t, [vp, pd, i32, pd, i32]),
        "trtamd_plugin_on_shape_change": (i32, [vp, pd, i32, pd, i32]),
        "trtamd_plugin_enqueue": (i32, [vp, pd, i32, pd, i32, C.POINTER(vp), C.POINTER(vp), vp, vp]),
        "trtamd_plugin_fields_to_serialize": (i32, [vp, C.POINTER(pf)]),
        "trtamd_legacy_get_creator": (vp, [C.c_char_p, C.c_char_p, C.c_char_p]),
        "trtamd_legacy_creator_field_names": (i32, [vp, C.POINTER(pf)]),
        "trtamd_legacy_create": (vp, [vp, C.c_char_p, pf, i32]),
        "trtamd_legacy_deserialize": (vp, [vp, C.c_char_p, C.c_void_p, C.c_size_t]),
        "trtamd_legacy_destroy": (None, [vp]),
        "trtamd_legacy_clone": (vp, [vp]),
        "trtamd_legacy_type": (C.c_char_p, [vp]),
        "trtamd_legacy_version": (C.c_char_p, [vp]),
        "trtamd_legacy_nb_outputs": (i32, [vp]),
        "trtamd_legacy_tensorrt_version": (i32, [vp]),
        "trtamd_legacy_initialize": (i32, [vp]),
        "trtamd_legacy_terminate": (None, [vp]),
        "trtamd_legacy_serialization_size": (C.c_size_t, [vp]),
        "trtamd_legacy_serialize": (None, [vp, C.c_void_p]),
        "trtamd_legacy_output_type": (i32, [vp, i32, C.POINTER(i32), i32]),
        "trtamd_legacy_output_dims": (i32, [vp, i32, pd, i32, pd]),
        "trtamd_legacy_supports_format": (i32, [vp, i32, pd, i32, i32]),
        "trtamd_legacy_configure": (None, [vp, pd, i32, pd, i32]),
        "trtamd_legacy_workspace_size": (C.c_size_t, [vp, pd, i32, pd, i32]),
        "trtamd_legacy_enqueue": (i32, [vp, pd, i32, pd, i32, C.POINTER(vp), C.POINTER(vp), vp, vp]),
        "trtamd_plugin_capture_log": (None, [i32]),
        "trtamd_plugin_last_log": (C.c_char_p, []),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._trtamd_plugin_symbols = list(sigs)
    _lib = lib
    return lib


# Symbols include/trtamd_plugin_c.h declares.
def plugin_c_symbols() -> list[str]:
    return list(_library()._trtamd_plugin_symbols)


def capture_log(enable: bool = True) -> None:
    _library().trtamd_plugin_capture_log(1 if enable else 0)


def last_log() -> str:
    return (_library().trtamd_plugin_last_log() or b"").decode()


def _fields_from_c(ptr, n) -> list[PluginField]:
    out = []
    for i in range(n):
        f = ptr[i]
        ftype = PluginFieldType(f.type)
        data = None
        if f.data and f.length > 0:
            dt = np.dtype(_NP_OF_FIELD[ftype])
            buf = C.string_at(f.data, f.length * dt.itemsize)
            data = np.frombuffer(buf, dtype=dt).copy()
        out.append(PluginField(f.name.decode() if f.name else "", data, ftype))
    return out


class Plugin:
    """An IPluginV3 instance (owns the C++ object)."""

    def __init__(self, handle: int):
        self._h = handle
        self._lib = _library()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.trtamd_plugin_destroy(self._h)
            self._h = None

    # IPluginV3
    def clone(self) -> "Plugin | None":
        h = self._lib.trtamd_plugin_clone(self._h)
        return Plugin(h) if h else None

    # IPluginV3OneCore
    @property
    def plugin_name(self) -> str:
        return self._lib.trtamd_plugin_name(self._h).decode()

    @property
    def plugin_version(self) -> str:
        return self._lib.trtamd_plugin_version(self._h).decode()

    @property
    def plugin_namespace(self) -> str:
        return self._lib.trtamd_plugin_namespace(self._h).decode()

    # IPluginV3OneBuild
    @property
    def num_outputs(self) -> int:
        return self._lib.trtamd_plugin_nb_outputs(self._h)

    def get_output_data_types(self, input_types: Sequence[DataType], nb_outputs: int | None = None):
        nb = self.num_outputs if nb_outputs is None else nb_outputs
        out = (C.c_int32 * max(nb, 1))()
        inp = (C.c_int32 * max(len(input_types), 1))(*[int(t) for t in input_types])
        st = self._lib.trtamd_plugin_output_types(self._h, out, nb, inp, len(input_types))
        if st != 0:
            return None
        return [DataType(out[i]) for i in range(nb)]

    def get_output_shapes(self, inputs: Sequence[TensorDesc], nb_outputs: int | None = None):
        nb = self.num_outputs if nb_outputs is None else nb_outputs
        cin, n = _descs(inputs)
        cout = (_CDesc * max(nb, 1))()
        st = self._lib.trtamd_plugin_output_shapes(self._h, cin, n, cout, nb)
        if st != 0:
            return None
        return [[int(cout[i].dims[k]) for k in range(cout[i].nb_dims)] for i in range(nb)]

    def supports_format_combination(self, pos: int, in_out: Sequence[TensorDesc], num_inputs: int) -> bool:
        c, n = _descs(in_out)
        return bool(self._lib.trtamd_plugin_supports_format(self._h, pos, c, num_inputs, n - num_inputs))

    def configure_plugin(self, inputs: Sequence[TensorDesc], outputs: Sequence[TensorDesc]) -> int:
        ci, ni = _descs(inputs)
        co, no = _descs(outputs)
        return self._lib.trtamd_plugin_configure(self._h, ci, ni, co, no)

    def get_workspace_size(self, inputs: Sequence[TensorDesc], outputs: Sequence[TensorDesc]) -> int:
        ci, ni = _descs(inputs)
        co, no = _descs(outputs)
        return int(self._lib.trtamd_plugin_workspace_size(self._h, ci, ni, co, no))

    # IPluginV3OneRuntime
    def on_shape_change(self, inputs: Sequence[TensorDesc], outputs: Sequence[TensorDesc]) -> int:
        ci, ni = _descs(inputs)
        co, no = _descs(outputs)
        return self._lib.trtamd_plugin_on_shape_change(self._h, ci, ni, co, no)

    def enqueue(self, input_desc: Sequence[TensorDesc], output_desc: Sequence[TensorDesc], inputs: Sequence[int],
                outputs: Sequence[int], workspace: int = 0, stream: int = 0) -> int:
        ci, ni = _descs(input_desc)
        co, no = _descs(output_desc)
        pin = (C.c_void_p * max(len(inputs), 1))(*[C.c_void_p(int(p)) for p in inputs])
        pout = (C.c_void_p * max(len(outputs), 1))(*[C.c_void_p(int(p)) for p in outputs])
        return self._lib.trtamd_plugin_enqueue(self._h, ci, ni, co, no, pin, pout, C.c_void_p(int(workspace)),
                                               C.c_void_p(int(stream)))

    def get_fields_to_serialize(self) -> list[PluginField] | None:
        ptr = C.POINTER(_CField)()
        n = self._lib.trtamd_plugin_fields_to_serialize(self._h, C.byref(ptr))
        if n < 0:
            return None
        return _fields_from_c(ptr, n)


class LegacyPlugin:
    """An IPluginV2DynamicExt instance (one of the reference's "Legacy" plugin versions)."""

    def __init__(self, handle: int):
        self._h = handle
        self._lib = _library()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.trtamd_legacy_destroy(self._h)
            self._h = None

    # IPluginV2
    @property
    def plugin_type(self) -> str:
        return self._lib.trtamd_legacy_type(self._h).decode()

    @property
    def plugin_version(self) -> str:
        return self._lib.trtamd_legacy_version(self._h).decode()

    @property
    def num_outputs(self) -> int:
        return self._lib.trtamd_legacy_nb_outputs(self._h)

    @property
    def tensorrt_version(self) -> int:
        return self._lib.trtamd_legacy_tensorrt_version(self._h)

    def initialize(self) -> int:
        return self._lib.trtamd_legacy_initialize(self._h)

    def terminate(self) -> None:
        self._lib.trtamd_legacy_terminate(self._h)

    def get_serialization_size(self) -> int:
        return int(self._lib.trtamd_legacy_serialization_size(self._h))

    def serialize(self) -> bytes:
        n = self.get_serialization_size()
        buf = C.create_string_buffer(max(n, 1))
        self._lib.trtamd_legacy_serialize(self._h, buf)
        return buf.raw[:n]

    def clone(self) -> "LegacyPlugin | None":
        h = self._lib.trtamd_legacy_clone(self._h)
        return LegacyPlugin(h) if h else None

    # IPluginV2Ext
    def get_output_data_type(self, index: int, input_types: Sequence[DataType]) -> DataType:
        inp = (C.c_int32 * max(len(input_types), 1))(*[int(t) for t in input_types])
        return DataType(self._lib.trtamd_legacy_output_type(self._h, index, inp, len(input_types)))

    # IPluginV2DynamicExt
    def get_output_dimensions(self, index: int, inputs: Sequence[TensorDesc]):
        cin, n = _descs(inputs)
        cout = (_CDesc * 1)()
        if self._lib.trtamd_legacy_output_dims(self._h, index, cin, n, cout) != 0:
            return None
        return [int(cout[0].dims[k]) for k in range(cout[0].nb_dims)]

    def supports_format_combination(self, pos: int, in_out: Sequence[TensorDesc], num_inputs: int) -> bool:
        c, n = _descs(in_out)
        return bool(self._lib.trtamd_legacy_supports_format(self._h, pos, c, num_inputs, n - num_inputs))

    def configure_plugin(self, inputs: Sequence[TensorDesc], outputs: Sequence[TensorDesc]) -> None:
        ci, ni = _descs(inputs)
        co, no = _descs(outputs)
        self._lib.trtamd_legacy_configure(self._h, ci, ni, co, no)

    def get_workspace_size(self, inputs: Sequence[TensorDesc], outputs: Sequence[TensorDesc]) -> int:
        ci, ni = _descs(inputs)
        co, no = _descs(outputs)
        return int(self._lib.trtamd_legacy_workspace_size(self._h, ci, ni, co, no))

    def enqueue(self, input_desc: Sequence[TensorDesc], output_desc: Sequence[TensorDesc], inputs: Sequence[int],
                outputs: Sequence[int], workspace: int = 0, stream: int = 0) -> int:
        ci, ni = _descs(input_desc)
        co, no = _descs(output_desc)
        pin = (C.c_void_p * max(len(inputs), 1))(*[C.c_void_p(int(p)) for p in inputs])
        pout = (C.c_void_p * max(len(outputs), 1))(*[C.c_void_p(int(p)) for p in outputs])
        return self._lib.trtamd_legacy_enqueue(self._h, ci, ni, co, no, pin, pout, C.c_void_p(int(workspace)),
                                               C.c_void_p(int(stream)))


class LegacyPluginCreator:
    """An IPluginCreator (owned by the registry)."""

    def __init__(self, handle: int):
        self._h = handle
        self._lib = _library()

    @property
    def field_names(self) -> list[PluginField]:
        ptr = C.POINTER(_CField)()
        n = self._lib.trtamd_legacy_creator_field_names(self._h, C.byref(ptr))
        return _fields_from_c(ptr, max(n, 0))

    def create_plugin(self, name: str, fc) -> LegacyPlugin | None:
        fields = list(fc)
        arr = (_CField * max(len(fields), 1))()
        keep = []
        for i, f in enumerate(fields):
            nm = f.name.encode()
            keep.append(nm)
            arr[i].name = nm
            arr[i].data = f.data.ctypes.data if f.data is not None else None
            arr[i].type = int(f.type)
            arr[i].length = f.length
        h = self._lib.trtamd_legacy_create(self._h, name.encode(), arr, len(fields))
        return LegacyPlugin(h) if h else None

    def deserialize_plugin(self, name: str, data: bytes) -> LegacyPlugin | None:
        buf = C.create_string_buffer(data, len(data))
        h = self._lib.trtamd_legacy_deserialize(self._h, name.encode(), buf, len(data))
        return LegacyPlugin(h) if h else None


@dataclass
class PluginFieldCollection:
    fields: list[PluginField] = field(default_factory=list)

    def __iter__(self):
        return iter(self.fields)


class PluginCreator:
    """An IPluginCreatorV3One (owned by the registry)."""

    def __init__(self, handle: int):
        self._h = handle
        self._lib = _library()

    @property
    def field_names(self) -> list[PluginField]:
        ptr = C.POINTER(_CField)()
        n = self._lib.trtamd_plugin_creator_field_names(self._h, C.byref(ptr))
        return _fields_from_c(ptr, max(n, 0))

    def create_plugin(self, name: str, fc: PluginFieldCollection | Sequence[PluginField],
                      phase: TensorRTPhase = TensorRTPhase.BUILD) -> Plugin | None:
        fields = list(fc)
        arr = (_CField * max(len(fields), 1))()
        keep = []
        for i, f in enumerate(fields):
            nm = f.name.encode()
            keep.append(nm)
            arr[i].name = nm
            arr[i].data = f.data.ctypes.data if f.data is not None else None
            arr[i].type = int(f.type)
            arr[i].length = f.length
        h = self._lib.trtamd_plugin_create(self._h, name.encode(), arr, len(fields), int(phase))
        return Plugin(h) if h else None


class PluginRegistry:
    """getPluginRegistry()."""

    def __init__(self):
        self._lib = _library()

    def get_creator(self, name: str, version: str, plugin_namespace: str = "") -> PluginCreator | None:
        h = self._lib.trtamd_plugin_get_creator(name.encode(), version.encode(), plugin_namespace.encode())
        return PluginCreator(h) if h else None

    def get_legacy_creator(self, name: str, version: str, plugin_namespace: str = "") -> LegacyPluginCreator | None:
        """The IPluginCreator registered under (name, version), if that version is a legacy one."""
        h = self._lib.trtamd_legacy_get_creator(name.encode(), version.encode(), plugin_namespace.encode())
        return LegacyPluginCreator(h) if h else None

    @property
    def all_creators(self) -> list[tuple[str, str]]:
        n = self._lib.trtamd_plugin_num_creators()
        return [(self._lib.trtamd_plugin_creator_name(i).decode(), self._lib.trtamd_plugin_creator_version(i).decode())
                for i in range(n)]


def get_plugin_registry() -> PluginRegistry:
    return PluginRegistry()
