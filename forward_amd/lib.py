"""ctypes binding of ``libfwdmi.so``: every symbol ``include/fwdmi.h`` declares.

Loading never compiles silently on a GPU box: the library is built ahead of time (``python -m
forward_amd.build`` or ``__graft_entry__.build()``); if the file is absent it is built once here
so a fresh checkout works, and a failure to build or load raises ``ImportError``.
"""
import ctypes as C
import os

# PyTorch-ROCm wheels bundle their own HIP runtime whose SONAME (libamdhip64.so.7) equals the
# system one libfwdmi.so is linked against.  Importing torch first makes the dynamic loader
# resolve libfwdmi.so's dependency to the runtime torch already loaded; the other order puts
# two HIP runtimes into one process, and device pointers / streams from one are garbage to
# the other.
import torch  # noqa: F401  (must precede the CDLL below)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfwdmi.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "fwdmi.h")

OK, ERR_UNSUPPORTED, ERR_BAD_ARG, ERR_HIP, ERR_NOT_CONFIGURED, ERR_TRUNCATED = 0, -1, -2, -3, -4, -5
F32, F16, I8, I32, BOOL, I64 = 0, 1, 2, 3, 4, 10
FIELD_F16, FIELD_F32, FIELD_F64, FIELD_I8, FIELD_I16, FIELD_I32, FIELD_CHAR, FIELD_DIMS, FIELD_UNKNOWN = range(9)
FORMAT_LINEAR = 0
OP_SUM, OP_MEAN, OP_MAX, OP_SQUARE_SUM, OP_GATHER = 0, 1, 2, 3, 999
BAG_XCD_TABLE_AFFINITY = 1
BAG_TABLE_WEIGHTS = 2
BAG_TABLE_AVG_LEN = 4
BAG_INLINE_TABLES = 40        # FWDMI_BAG_INLINE_TABLES


class BagExt(C.Structure):
    _fields_ = [("table_dtype", C.c_int32), ("index_dtype", C.c_int32), ("out_dtype", C.c_int32),
                ("include_last_offset", C.c_int32), ("per_sample_weights", C.c_void_p),
                ("max_indices", C.c_void_p), ("out_row_stride", C.c_int64), ("oob_flag", C.c_void_p),
                ("flags", C.c_int32), ("table_cost", C.c_void_p), ("square_sum_out", C.c_void_p),
                ("table_avg_len", C.c_void_p)]


class EmbExt(C.Structure):
    _fields_ = [("batch_major", C.c_int32), ("eps2", C.c_float), ("skip", C.c_void_p), ("gamma2", C.c_void_p),
                ("beta2", C.c_void_p), ("bias2", C.c_void_p), ("emb_output", C.c_void_p)]


class BagTable(C.Structure):
    _fields_ = [("data", C.c_void_p), ("input", C.c_void_p), ("input_2", C.c_void_p), ("count", C.c_int64),
                ("input_size", C.c_int64), ("data_offset", C.c_int64), ("out_col", C.c_int64),
                ("weights", C.c_void_p)]


class Dims(C.Structure):
    _fields_ = [("nbDims", C.c_int32), ("d", C.c_int32 * 8)]

    @classmethod
    def of(cls, *shape):
        d = cls()
        d.nbDims = len(shape)
        for i, v in enumerate(shape):
            d.d[i] = int(v)
        return d

    def tolist(self):
        return [int(self.d[i]) for i in range(self.nbDims)]


class TensorDesc(C.Structure):
    _fields_ = [("dims", Dims), ("type", C.c_int32), ("format", C.c_int32), ("scale", C.c_float)]

    @classmethod
    def of(cls, shape, dtype, fmt=FORMAT_LINEAR):
        t = cls()
        t.dims = Dims.of(*shape)
        t.type, t.format, t.scale = dtype, fmt, 1.0
        return t


class PluginField(C.Structure):
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("type", C.c_int32), ("length", C.c_int32)]


_vp, _i32, _i64, _sz, _cp = C.c_void_p, C.c_int32, C.c_int64, C.c_size_t, C.c_char_p

# name -> (restype, argtypes); the test-suite checks this table against the header.
SIGNATURES = {
    "fwdmi_version": (_cp, []),
    "fwdmi_last_error": (_cp, []),
    "fwdmi_device_count": (C.c_int, []),
    "fwdmi_embedding_bag": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _i32, _i64, _i32, C.POINTER(BagExt), _vp]),
    "fwdmi_embedding_bag_fixed": (C.c_int, [_vp, _vp, _i64, _i64, _vp, _i64, _i32, _i64, _i32, C.POINTER(BagExt), _vp]),
    "fwdmi_gather": (C.c_int, [_vp, _vp, _i64, _i64, _vp, _i64, _i32, _i64, C.POINTER(BagExt), _vp]),
    "fwdmi_bag_table_cost": (C.c_int, [_vp, _i32, _vp]),
    "fwdmi_bag_device_topology": (C.c_int, [C.POINTER(_i32), C.POINTER(_i32)]),
    "fwdmi_bag_tables_fill": (C.c_int, [_vp, _i32, _vp, _vp]),
    "fwdmi_embedding_bag_multi": (C.c_int, [_vp, _i32, _i64, _vp, _i32, _i32, C.c_double, C.POINTER(BagExt), _vp]),
    "fwdmi_embedding_bag_multi_host": (C.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _i32, C.c_double, C.POINTER(BagExt),
                                                 _vp]),
    "fwdmi_embedding_bag_multi_noalloc": (C.c_int, [_vp, _i32, _i64, _vp, _i32, _i32, C.c_double, C.POINTER(BagExt),
                                                    _vp]),
    "fwdmi_layer_norm": (C.c_int, [_vp, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _i32, C.c_float]),
    "fwdmi_skip_layer_norm": (C.c_int, [_vp, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i32, C.c_float]),
    "fwdmi_emb_layer_norm": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32,
                                       _i32, _vp, _vp, _i32, C.c_float, _vp]),
    "fwdmi_emb_layer_norm_ex": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32,
                                          _i32, _vp, _vp, _i32, C.c_float, _vp, C.POINTER(EmbExt)]),
    "fwdmi_get_plugin_creator": (_vp, [_cp, _cp]),
    "fwdmi_registry_size": (C.c_int, []),
    "fwdmi_registry_at": (_vp, [C.c_int]),
    "fwdmi_creator_name": (_cp, [_vp]),
    "fwdmi_creator_version": (_cp, [_vp]),
    "fwdmi_creator_num_fields": (C.c_int, [_vp]),
    "fwdmi_creator_field_name": (_cp, [_vp, C.c_int]),
    "fwdmi_creator_field_type": (C.c_int, [_vp, C.c_int]),
    "fwdmi_creator_create_plugin": (_vp, [_vp, _cp, C.POINTER(PluginField), C.c_int]),
    "fwdmi_creator_deserialize_plugin": (_vp, [_vp, _cp, _vp, _sz]),
    "fwdmi_plugin_get_nb_outputs": (C.c_int, [_vp]),
    "fwdmi_plugin_get_output_dimensions": (C.c_int, [_vp, C.c_int, C.POINTER(Dims), C.c_int, C.POINTER(Dims)]),
    "fwdmi_plugin_supports_format_combination": (C.c_int, [_vp, C.c_int, C.POINTER(TensorDesc), C.c_int, C.c_int]),
    "fwdmi_plugin_configure": (C.c_int, [_vp, C.POINTER(TensorDesc), C.c_int, C.POINTER(TensorDesc), C.c_int]),
    "fwdmi_plugin_get_workspace_size": (_sz, [_vp, C.POINTER(TensorDesc), C.c_int, C.POINTER(TensorDesc), C.c_int]),
    "fwdmi_plugin_initialize": (C.c_int, [_vp]),
    "fwdmi_plugin_terminate": (None, [_vp]),
    "fwdmi_plugin_enqueue": (C.c_int, [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.POINTER(_vp),
                                       C.POINTER(_vp), _vp, _vp]),
    "fwdmi_plugin_get_serialization_size": (_sz, [_vp]),
    "fwdmi_plugin_serialize": (C.c_int, [_vp, _vp]),
    "fwdmi_plugin_get_type": (_cp, [_vp]),
    "fwdmi_plugin_get_version": (_cp, [_vp]),
    "fwdmi_plugin_set_namespace": (None, [_vp, _cp]),
    "fwdmi_plugin_get_namespace": (_cp, [_vp]),
    "fwdmi_plugin_get_output_data_type": (C.c_int, [_vp, C.c_int, C.POINTER(_i32), C.c_int]),
    "fwdmi_plugin_clone": (_vp, [_vp]),
    "fwdmi_plugin_destroy": (None, [_vp]),
    "fwdmi_plugin_take_oob_flag": (C.c_int, [_vp, _vp]),
    "fwdmi_plan_save": (C.c_int, [_cp, C.POINTER(_vp), C.POINTER(_cp), C.c_int, _cp]),
    "fwdmi_plan_load": (_vp, [_cp]),
    "fwdmi_plan_size": (C.c_int, [_vp]),
    "fwdmi_plan_layer_name": (_cp, [_vp, C.c_int]),
    "fwdmi_plan_take_plugin": (_vp, [_vp, C.c_int]),
    "fwdmi_plan_meta": (_cp, [_vp]),
    "fwdmi_plan_close": (None, [_vp]),
    "fwdmi_meta_new": (_vp, []),
    "fwdmi_meta_load": (_vp, [_cp]),
    "fwdmi_meta_parse": (_vp, [_cp]),
    "fwdmi_plan_meta_data": (_vp, [_vp]),
    "fwdmi_meta_save": (C.c_int, [_vp, _cp]),
    "fwdmi_meta_json": (_cp, [_vp]),
    "fwdmi_meta_infer_mode": (_i32, [_vp]),
    "fwdmi_meta_opt_batch_size": (_i32, [_vp]),
    "fwdmi_meta_max_batch_size": (_i32, [_vp]),
    "fwdmi_meta_torch_module_path": (_cp, [_vp]),
    "fwdmi_meta_unused_input_indices": (_i32, [_vp, C.POINTER(C.POINTER(_i32))]),
    "fwdmi_meta_output_indices": (_i32, [_vp, C.POINTER(C.POINTER(_i32))]),
    "fwdmi_meta_set": (C.c_int, [_vp, _i32, _i32, _i32, C.POINTER(_i32), _i32, C.POINTER(_i32), _i32, _cp]),
    "fwdmi_meta_free": (None, [_vp]),
}


class FwdmiError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("fwdmi status %d: %s" % (code, text))
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        from . import build as _build
        try:
            _build.build(force=False)
        except Exception as e:  # pragma: no cover
            raise ImportError("libfwdmi.so is missing and could not be built: %s" % e)
    try:
        dll = C.CDLL(LIB_PATH)
    except OSError as e:
        raise ImportError("cannot load %s: %s" % (LIB_PATH, e))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(dll, name)  # AttributeError if the library lacks a declared symbol
        fn.restype, fn.argtypes = res, args
    return dll


dll = _load()


def last_error():
    return dll.fwdmi_last_error().decode()


def check(rc):
    if rc != OK:
        raise FwdmiError(rc, last_error())
    return rc
