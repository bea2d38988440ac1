"""Python mirror of the plugin objects exported by ``libfwdmi.so``.

Method names follow the reference's plugin interface (``getOutputDimensions``,
``supportsFormatCombination``, ``configurePlugin``, ``enqueue``, ``serialize`` ... on plugins;
``createPlugin`` / ``deserializePlugin`` / ``getFieldNames`` on creators;
``getPluginCreator(name, version)`` on the registry), so host code and tests read like the
reference's own layer creators.  Creator fields are given as numpy arrays / ints; ``enqueue``
takes device tensors.
"""
import ctypes as C

import numpy as np
import torch

from . import lib

_NP_FIELD = {np.dtype(np.float16): lib.FIELD_F16, np.dtype(np.float32): lib.FIELD_F32,
             np.dtype(np.float64): lib.FIELD_F64, np.dtype(np.int8): lib.FIELD_I8,
             np.dtype(np.int16): lib.FIELD_I16, np.dtype(np.int32): lib.FIELD_I32}
_T2DT = {torch.float32: lib.F32, torch.float16: lib.F16, torch.int32: lib.I32, torch.int64: lib.I64,
         torch.int8: lib.I8, torch.bool: lib.BOOL}
_DT2T = {v: k for k, v in _T2DT.items()}


class PluginFieldData:
    """One creator field: a name plus a numpy array (scalars become 1-element int32 / float32)."""

    def __init__(self, name, value, ftype=None):
        if isinstance(value, (bool, int, np.integer)):
            value = np.array([value], np.int32)
        elif isinstance(value, float):
            value = np.array([value], np.float32)
        self.name = name
        self.array = np.ascontiguousarray(value)
        self.type = _NP_FIELD[self.array.dtype] if ftype is None else ftype

    def c_field(self):
        f = lib.PluginField()
        f.name = self.name.encode()
        f.data = self.array.ctypes.data
        f.type = self.type
        f.length = self.array.size
        return f


def _descs(items):
    arr = (lib.TensorDesc * max(1, len(items)))()
    for i, (shape, dtype) in enumerate(items):
        arr[i] = lib.TensorDesc.of(shape, dtype)
    return arr


def _desc_of(t):
    return (tuple(t.shape), _T2DT[t.dtype])


class Plugin:
    def __init__(self, handle):
        if not handle:
            raise lib.FwdmiError(lib.ERR_BAD_ARG, lib.last_error())
        self._h = C.c_void_p(handle)

    # -- shape / format negotiation ---------------------------------------------------------
    def getNbOutputs(self):
        return lib.dll.fwdmi_plugin_get_nb_outputs(self._h)

    def getOutputDimensions(self, outputIndex, inputs):
        arr = (lib.Dims * max(1, len(inputs)))(*[lib.Dims.of(*s) for s in inputs])
        out = lib.Dims()
        lib.check(lib.dll.fwdmi_plugin_get_output_dimensions(self._h, outputIndex, arr, len(inputs), C.byref(out)))
        return out.tolist()

    def supportsFormatCombination(self, pos, inOut, nbInputs, nbOutputs):
        """``inOut``: list of (shape, dtype[, format])."""
        arr = (lib.TensorDesc * max(1, len(inOut)))()
        for i, it in enumerate(inOut):
            arr[i] = lib.TensorDesc.of(it[0], it[1], it[2] if len(it) > 2 else lib.FORMAT_LINEAR)
        rc = lib.dll.fwdmi_plugin_supports_format_combination(self._h, pos, arr, nbInputs, nbOutputs)
        if rc < 0:
            raise lib.FwdmiError(rc, "supportsFormatCombination: bad arguments")
        return bool(rc)

    def getOutputDataType(self, index, inputTypes):
        arr = (C.c_int32 * max(1, len(inputTypes)))(*inputTypes)
        return lib.dll.fwdmi_plugin_get_output_data_type(self._h, index, arr, len(inputTypes))

    # -- lifecycle ------------------------------------------------------------------------------
    def configurePlugin(self, inputs, outputs):
        """``inputs`` / ``outputs``: lists of (shape, dtype).  Uploads tables to the current device."""
        lib.check(lib.dll.fwdmi_plugin_configure(self._h, _descs(inputs), len(inputs), _descs(outputs), len(outputs)))

    def getWorkspaceSize(self, inputs, outputs):
        return lib.dll.fwdmi_plugin_get_workspace_size(self._h, _descs(inputs), len(inputs), _descs(outputs),
                                                       len(outputs))

    def initialize(self):
        return lib.dll.fwdmi_plugin_initialize(self._h)

    def terminate(self):
        lib.dll.fwdmi_plugin_terminate(self._h)

    def enqueue_raw(self, in_descs, out_descs, in_ptrs, out_ptrs, stream_handle=None, workspace_ptr=None):
        """``enqueue`` on raw device addresses; returns the status instead of raising."""
        ins = (C.c_void_p * max(1, len(in_ptrs)))(*in_ptrs)
        outs = (C.c_void_p * max(1, len(out_ptrs)))(*out_ptrs)
        s = torch.cuda.current_stream().cuda_stream if stream_handle is None else stream_handle
        return lib.dll.fwdmi_plugin_enqueue(self._h, _descs(in_descs), _descs(out_descs), ins, outs,
                                            C.c_void_p(workspace_ptr) if workspace_ptr else None, C.c_void_p(s))

    def enqueue(self, inputs, outputs, stream=None, workspace=None):
        """Device tensors in, device tensors out (written in place); raises on a non-zero status.
        ``workspace``: a device byte tensor of at least ``getWorkspaceSize`` bytes; when the plugin
        asks for one and none is given, one is allocated (and kept) here, as the engine hosting
        the plugin would."""
        for t in list(inputs) + list(outputs):
            if not t.is_cuda or not t.is_contiguous():
                raise RuntimeError("enqueue needs contiguous device tensors")
        s = None if stream is None else stream.cuda_stream
        ind, outd = [_desc_of(t) for t in inputs], [_desc_of(t) for t in outputs]
        if workspace is None:
            need = self.getWorkspaceSize(ind, outd)
            if need:
                if getattr(self, "_ws", None) is None or self._ws.numel() < need:
                    self._ws = torch.empty(need, dtype=torch.uint8, device=inputs[0].device)
                workspace = self._ws
        rc = self.enqueue_raw(ind, outd, [t.data_ptr() for t in inputs], [t.data_ptr() for t in outputs], s,
                              None if workspace is None else workspace.data_ptr())
        return lib.check(rc)

    def __call__(self, *inputs):
        """Convenience: infer output shapes/types, allocate, enqueue, return the outputs."""
        shapes = [tuple(t.shape) for t in inputs]
        outs = []
        for i in range(self.getNbOutputs()):
            dims = self.getOutputDimensions(i, shapes)
            dt = self.getOutputDataType(i, [_T2DT[t.dtype] for t in inputs])
            outs.append(torch.empty(dims, dtype=_DT2T[dt], device=inputs[0].device))
        self.configurePlugin([_desc_of(t) for t in inputs], [_desc_of(t) for t in outs])
        self.enqueue(list(inputs), outs)
        return outs[0] if len(outs) == 1 else tuple(outs)

    # -- identity / persistence -----------------------------------------------------------------
    def getSerializationSize(self):
        return lib.dll.fwdmi_plugin_get_serialization_size(self._h)

    def serialize(self):
        buf = np.zeros(self.getSerializationSize(), np.uint8)
        lib.check(lib.dll.fwdmi_plugin_serialize(self._h, C.c_void_p(buf.ctypes.data)))
        return buf.tobytes()

    def getPluginType(self):
        return lib.dll.fwdmi_plugin_get_type(self._h).decode()

    def getPluginVersion(self):
        return lib.dll.fwdmi_plugin_get_version(self._h).decode()

    def setPluginNamespace(self, ns):
        self._ns = ns.encode()  # the reference borrows the pointer; keep it alive anyway
        lib.dll.fwdmi_plugin_set_namespace(self._h, self._ns)

    def getPluginNamespace(self):
        return lib.dll.fwdmi_plugin_get_namespace(self._h).decode()

    def clone(self):
        return Plugin(lib.dll.fwdmi_plugin_clone(self._h))

    def takeOobFlag(self):
        rc = lib.dll.fwdmi_plugin_take_oob_flag(self._h, C.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc < 0:
            raise lib.FwdmiError(rc, lib.last_error())
        return bool(rc)

    def destroy(self):
        if self._h:
            lib.dll.fwdmi_plugin_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class PluginCreator:
    def __init__(self, handle):
        self._h = C.c_void_p(handle)

    def getPluginName(self):
        return lib.dll.fwdmi_creator_name(self._h).decode()

    def getPluginVersion(self):
        return lib.dll.fwdmi_creator_version(self._h).decode()

    def getFieldNames(self):
        n = lib.dll.fwdmi_creator_num_fields(self._h)
        return [(lib.dll.fwdmi_creator_field_name(self._h, i).decode(), lib.dll.fwdmi_creator_field_type(self._h, i))
                for i in range(n)]

    def createPlugin(self, name, fields):
        """``fields``: list of PluginFieldData (or (name, value) pairs).  Raises FwdmiError on a
        contract violation (where the reference aborts)."""
        fields = [f if isinstance(f, PluginFieldData) else PluginFieldData(*f) for f in fields]
        arr = (lib.PluginField * max(1, len(fields)))(*[f.c_field() for f in fields])
        return Plugin(lib.dll.fwdmi_creator_create_plugin(self._h, name.encode(), arr, len(fields)))

    def deserializePlugin(self, name, data):
        buf = np.frombuffer(bytes(data), np.uint8)
        ptr = C.c_void_p(buf.ctypes.data) if buf.size else C.c_void_p(0)
        return Plugin(lib.dll.fwdmi_creator_deserialize_plugin(self._h, name.encode(), ptr, buf.size))


class PluginRegistry:
    def getPluginCreator(self, name, version):
        h = lib.dll.fwdmi_get_plugin_creator(name.encode(), version.encode())
        return PluginCreator(h) if h else None

    def getPluginCreatorList(self):
        return [PluginCreator(lib.dll.fwdmi_registry_at(i)) for i in range(lib.dll.fwdmi_registry_size())]


def getPluginRegistry():
    return PluginRegistry()


# InferMode of the reference (source/common/fwd_common.h:40-60): the sidecar stores the number.
INFER_MODES = {"float": 0, "float32": 0, "half": 1, "float16": 1, "int8": 2, "int8_calib": 3}


class EngineMetaData:
    """The engine sidecar ``<engine file>.meta``, typed: mirror of the reference's ``EngineMetaData``
    (source/trt_engine/trt_common/trt_meta_data.h:37-90, .cpp:42-97) over the library's reader and
    writer.  ``infer_mode`` is an int (0 float, 1 half, 2 int8, 3 int8_calib), ``opt_batch_size`` /
    ``max_batch_size`` ints, ``unused_input_indices`` a sorted list without repeats (a set in the
    reference), ``output_indices`` a list, ``torch_module_path`` a string."""

    KEYS = ("infer_mode", "max_batch_size", "opt_batch_size", "output_indices", "torch_module_path",
            "unused_input_indices")

    def __init__(self, infer_mode=0, opt_batch_size=-1, max_batch_size=-1, unused_input_indices=(),
                 output_indices=(), torch_module_path=""):
        if isinstance(infer_mode, str):
            infer_mode = INFER_MODES[infer_mode]
        self.infer_mode, self.opt_batch_size, self.max_batch_size = int(infer_mode), int(opt_batch_size), int(max_batch_size)
        self.unused_input_indices = sorted(set(int(v) for v in unused_input_indices))
        self.output_indices = [int(v) for v in output_indices]
        self.torch_module_path = str(torch_module_path)

    def __eq__(self, other):
        return isinstance(other, EngineMetaData) and self.to_dict() == other.to_dict()

    def __repr__(self):
        return "EngineMetaData(%r)" % (self.to_dict(),)

    def to_dict(self):
        return {k: getattr(self, k) for k in self.KEYS}

    @classmethod
    def from_dict(cls, d):
        """From a dict with the sidecar's keys, through the library's own reader: a missing key or
        a value of the wrong type raises FwdmiError, as ``LoadMetaData`` returns false."""
        import json
        return cls._take(lib.dll.fwdmi_meta_parse(json.dumps(d).encode()))

    @classmethod
    def _take(cls, h):
        if not h:
            raise lib.FwdmiError(lib.ERR_BAD_ARG, lib.last_error())
        h = C.c_void_p(h)
        try:
            def ints(fn):
                p = C.POINTER(C.c_int32)()
                n = fn(h, C.byref(p))
                return [int(p[i]) for i in range(n)]
            return cls(lib.dll.fwdmi_meta_infer_mode(h), lib.dll.fwdmi_meta_opt_batch_size(h),
                       lib.dll.fwdmi_meta_max_batch_size(h), ints(lib.dll.fwdmi_meta_unused_input_indices),
                       ints(lib.dll.fwdmi_meta_output_indices), lib.dll.fwdmi_meta_torch_module_path(h).decode())
        finally:
            lib.dll.fwdmi_meta_free(h)

    def _handle(self):
        h = C.c_void_p(lib.dll.fwdmi_meta_new())
        u = (C.c_int32 * max(1, len(self.unused_input_indices)))(*self.unused_input_indices)
        o = (C.c_int32 * max(1, len(self.output_indices)))(*self.output_indices)
        lib.check(lib.dll.fwdmi_meta_set(h, self.infer_mode, self.opt_batch_size, self.max_batch_size, u,
                                         len(self.unused_input_indices), o, len(self.output_indices),
                                         self.torch_module_path.encode()))
        return h

    def to_json(self):
        """The text ``SaveMetaData`` writes (keys in alphabetical order, four-space indentation)."""
        h = self._handle()
        try:
            return lib.dll.fwdmi_meta_json(h).decode()
        finally:
            lib.dll.fwdmi_meta_free(h)

    def SaveMetaData(self, meta_file):
        h = self._handle()
        try:
            lib.check(lib.dll.fwdmi_meta_save(h, meta_file.encode()))
        finally:
            lib.dll.fwdmi_meta_free(h)
        return True

    @classmethod
    def LoadMetaData(cls, meta_file):
        return cls._take(lib.dll.fwdmi_meta_load(meta_file.encode()))


def save_plan(path, layers, meta=None):
    """Writes ``layers`` = [(layer_name, Plugin), ...] to ``path`` and ``meta`` (an EngineMetaData, or
    a dict with the sidecar's keys and types) to ``path + ".meta"``: the plugin part of
    ``TrtForwardEngine::Save``.  A ``meta`` the reference's reader would reject raises FwdmiError
    and nothing is written."""
    import json
    n = len(layers)
    handles = (C.c_void_p * max(1, n))(*[p._h for _, p in layers])
    names = (C.c_char_p * max(1, n))(*[name.encode() for name, _ in layers])
    if isinstance(meta, EngineMetaData):
        meta = meta.to_dict()
    text = None if meta is None else json.dumps(meta).encode()
    lib.check(lib.dll.fwdmi_plan_save(path.encode(), handles, names, n, text))


def load_plan(path):
    """Returns ``([(layer_name, Plugin), ...], EngineMetaData or None)``: the plugin part of
    ``TrtForwardEngine::Load``.  A sidecar that is present but malformed fails the load."""
    h = lib.dll.fwdmi_plan_load(path.encode())
    if not h:
        raise lib.FwdmiError(lib.ERR_TRUNCATED, lib.last_error())
    h = C.c_void_p(h)
    try:
        layers = [(lib.dll.fwdmi_plan_layer_name(h, i).decode(), Plugin(lib.dll.fwdmi_plan_take_plugin(h, i)))
                  for i in range(lib.dll.fwdmi_plan_size(h))]
        m = lib.dll.fwdmi_plan_meta_data(h)
        meta = EngineMetaData._take(m) if m else None
    finally:
        lib.dll.fwdmi_plan_close(h)
    return layers, meta
