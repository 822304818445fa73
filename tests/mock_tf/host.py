"""Python driver of the mock TensorFlow host (tests/mock_tf/mock_tf.cc): loads the plugin the way
TensorFlow does (dlopen + TF_InitKernel), instantiates kernels from node attributes and runs them."""
import collections
import ctypes as C
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
MOCK_LIB = os.path.join(HERE, "libmock_tf.so")
PLUGIN_LIB = os.path.join(ROOT, "intel-extension-for-tensorflow_amd", "lib", "libitex_amd.so")

FLOAT, INT32, QINT8, QUINT8, QINT32, BFLOAT16, HALF = 1, 3, 11, 12, 13, 14, 19
NP_OF = {FLOAT: np.float32, INT32: np.int32, QINT8: np.int8, QUINT8: np.uint8, QINT32: np.int32}
OK, INVALID_ARGUMENT, NOT_FOUND, ABORTED, UNIMPLEMENTED = 0, 3, 5, 10, 12

_ALLOC = C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_int)
_FREE = C.CFUNCTYPE(None, C.c_void_p, C.c_int)

_state = {}


def load(device="XPU", stock_ops=("QuantizeV2", "Dequantize", "QuantizedMatMulWithBias", "QuantizedMatMulWithBiasAndRelu",
                                   "QuantizedMatMulWithBiasAndReluAndRequantize", "QuantizedMatMulWithBiasAndRequantize",
                                   "QuantizedMatMulWithBiasAndDequantize", "RequantizePerChannel",
                                   "RequantizationRangePerChannel", "QuantizedReshape", "MatMul", "Relu", "QuantizedConv2D",
                                   "QuantizedConv2DPerChannel", "QuantizedConv2DWithBias", "QuantizedConv2DWithBiasAndRelu",
                                   "QuantizedConv2DAndRelu", "QuantizedConv2DAndRequantize", "QuantizedConv2DAndReluAndRequantize",
                                   "QuantizedConv2DWithBiasAndRequantize", "QuantizedConv2DWithBiasAndReluAndRequantize",
                                   "QuantizedConv2DWithBiasSumAndReluAndRequantize",
                                   "QuantizedConv2DWithBiasSignedSumAndReluAndRequantize", "QuantizedDepthwiseConv2D",
                                   "QuantizedDepthwiseConv2DWithBias", "QuantizedDepthwiseConv2DWithBiasAndRelu",
                                   "QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize")):
    """Loads the mock host and the plugin once per process; returns the mock's ctypes handle."""
    if "lib" in _state:
        return _state["lib"]
    if not os.path.exists(MOCK_LIB):
        from . import build as _b
        _b.build()
    if not os.path.exists(PLUGIN_LIB):
        raise RuntimeError("plugin library missing: " + PLUGIN_LIB)
    try:
        import torch  # noqa: F401  one HIP runtime per process: PyTorch's must be mapped first
    except ImportError:
        pass
    os.environ.setdefault("ITEX_AMD_DEVICE_TYPE", device)
    lib = C.CDLL(MOCK_LIB, mode=C.RTLD_GLOBAL)
    lib.mock_dump_registry.restype = C.c_char_p
    lib.mock_node_new.restype = C.c_void_p
    lib.mock_node_construction_message.restype = C.c_char_p
    lib.mock_node_compute_message.restype = C.c_char_p
    for name in stock_ops:
        lib.mock_add_stock_op(name.encode())
    rc = lib.mock_load_plugin(PLUGIN_LIB.encode())
    if rc != 0:
        raise RuntimeError("mock_load_plugin failed: %d" % rc)
    _state["lib"] = lib
    _state["device"] = os.environ["ITEX_AMD_DEVICE_TYPE"]
    return lib


def registry():
    return json.loads(load().mock_dump_registry().decode())


def use_torch_allocator(dev):
    """Device allocations of the mock (outputs, temporaries) come from PyTorch on `dev`."""
    import torch
    lib = load()
    live = {}

    def alloc(nbytes, on_host):
        t = torch.empty(max(int(nbytes), 1) + 64, dtype=torch.uint8, device=dev)
        live[t.data_ptr()] = t
        return t.data_ptr()

    def free(ptr, on_host):
        live.pop(ptr, None)

    _state["alloc_cb"] = (_ALLOC(alloc), _FREE(free), live)
    lib.mock_set_allocator(_state["alloc_cb"][0], _state["alloc_cb"][1])


class Node:
    """One graph node: attributes -> kernel instance -> compute calls."""

    def __init__(self, op, attrs, device=None):
        self.lib = load()
        self.h = C.c_void_p(self.lib.mock_node_new(op.encode(), (device or _state["device"]).encode()))
        for k, v in attrs.items():
            kb = k.encode()
            if isinstance(v, bool):
                self.lib.mock_node_attr_bool(self.h, kb, int(v))
            elif isinstance(v, DType):
                self.lib.mock_node_attr_type(self.h, kb, int(v))
            elif isinstance(v, int):
                self.lib.mock_node_attr_int(self.h, kb, C.c_int64(v))
            elif isinstance(v, float):
                self.lib.mock_node_attr_float(self.h, kb, C.c_float(v))
            elif isinstance(v, str):
                self.lib.mock_node_attr_string(self.h, kb, v.encode())
            elif isinstance(v, (list, tuple)) and all(isinstance(x, DType) for x in v):
                arr = (C.c_int * len(v))(*[int(x) for x in v])
                self.lib.mock_node_attr_type_list(self.h, kb, arr, len(v))
            elif isinstance(v, (list, tuple)) and len(v) > 0 and all(isinstance(x, int) for x in v):
                arr = (C.c_int64 * len(v))(*v)
                self.lib.mock_node_attr_int_list(self.h, kb, arr, len(v))
            elif isinstance(v, (list, tuple)):
                arr = (C.c_char_p * len(v))(*[x.encode() for x in v])
                self.lib.mock_node_attr_string_list(self.h, kb, arr, len(v))
            else:
                raise TypeError("attr %s: %r" % (k, v))
        self.code = self.lib.mock_node_instantiate(self.h)
        self.message = self.lib.mock_node_construction_message(self.h).decode()
        self._keep = []

    def run(self, inputs, outputs, stream=0):
        """inputs: list of (dtype, shape, address, on_host[, allow_forward]); outputs: list of (dtype, on_host).
        Returns (code, message, [ (dtype, shape, address, forwarded_from) | None ])."""
        lib = self.lib
        lib.mock_node_clear_io(self.h)
        for spec in inputs:
            dtype, shape, addr, on_host = spec[:4]
            fwd = spec[4] if len(spec) > 4 else False
            dims = (C.c_int64 * max(len(shape), 1))(*shape)
            lib.mock_node_add_input(self.h, int(dtype), dims, len(shape), C.c_void_p(addr), int(on_host), int(fwd))
        for dtype, on_host in outputs:
            lib.mock_node_add_output(self.h, int(dtype), int(on_host))
        lib.mock_node_set_stream(self.h, C.c_void_p(stream))
        code = lib.mock_node_compute(self.h)
        msg = lib.mock_node_compute_message(self.h).decode()
        outs = []
        for i in range(len(outputs)):
            dt, nd, data, fwd = C.c_int(), C.c_int(), C.c_void_p(), C.c_int()
            dims = (C.c_int64 * 8)()
            if lib.mock_node_output(self.h, i, C.byref(dt), dims, C.byref(nd), C.byref(data), C.byref(fwd)) == 0:
                outs.append((dt.value, tuple(dims[d] for d in range(nd.value)), data.value, fwd.value))
            else:
                outs.append(None)
        return code, msg, outs

    def temp_allocs(self):
        return self.lib.mock_node_temp_allocs(self.h)

    def close(self):
        if self.h:
            self.lib.mock_node_delete(self.h)
            self.h = None


class DType(int):
    """Marks an integer attribute value as a TF_DataType."""


_recent_host_arrays = collections.deque(maxlen=512)


def host_array(a):
    """(dtype-agnostic) address of a numpy array.  The last few hundred arrays passed here are kept alive, so that a
    temporary handed over in a call expression cannot be freed (and its memory reused) before the op has read it."""
    _recent_host_arrays.append(a)
    return a.ctypes.data


def read_host(addr, dtype, shape):
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    buf = (C.c_char * (n * np.dtype(NP_OF[dtype]).itemsize)).from_address(addr)
    return np.frombuffer(buf, dtype=NP_OF[dtype]).reshape(shape).copy()


# ------------------------------------------------------------------------------------------------
# the StreamExecutor side of the plugin (SE_InitPlugin), driven like TensorFlow's PluggableDevice code
# ------------------------------------------------------------------------------------------------
class DevicePlugin:
    """Device 0 of the plugin: its allocator, stream, copies and fills, through the function tables
    SE_InitPlugin filled.  load_device() returns the process-wide instance."""

    def __init__(self, lib):
        self.lib = lib
        lib.mock_device_error.restype = C.c_char_p
        lib.mock_device_describe.restype = C.c_char_p
        lib.mock_device_stream.restype = C.c_void_p
        lib.mock_device_alloc.restype = C.c_void_p
        lib.mock_device_alloc.argtypes = [C.c_uint64]
        lib.mock_device_free.argtypes = [C.c_void_p]
        lib.mock_device_host_alloc.restype = C.c_void_p
        lib.mock_device_host_alloc.argtypes = [C.c_uint64]
        lib.mock_device_host_free.argtypes = [C.c_void_p]
        for f in (lib.mock_device_h2d, lib.mock_device_d2h, lib.mock_device_d2d):
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int]
        lib.mock_device_memset.argtypes = [C.c_void_p, C.c_int, C.c_uint32, C.c_uint64]
        lib.mock_device_stats.argtypes = [C.POINTER(C.c_int64)]
        lib.mock_device_stream_event_test.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]

    def error(self):
        return self.lib.mock_device_error().decode()

    def describe(self):
        return json.loads(self.lib.mock_device_describe().decode())

    @property
    def stream(self):
        return self.lib.mock_device_stream() or 0

    def alloc(self, nbytes):
        p = self.lib.mock_device_alloc(int(nbytes))
        if not p:
            raise MemoryError("device allocation of %d bytes failed" % nbytes)
        return p

    def free(self, ptr):
        self.lib.mock_device_free(ptr)

    def upload(self, array, sync=False):
        """Allocates device memory for `array` and copies it there; returns the device address."""
        a = np.ascontiguousarray(array)
        p = self.alloc(max(a.nbytes, 1))
        rc = self.lib.mock_device_h2d(p, a.ctypes.data, a.nbytes, int(sync))
        assert rc == 0, self.error()
        if not sync:
            self.sync()  # `a` may be a temporary
        return p

    def download(self, ptr, dtype, shape, sync=False):
        out = np.empty(shape, dtype)
        rc = self.lib.mock_device_d2h(out.ctypes.data, ptr, out.nbytes, int(sync))
        assert rc == 0, self.error()
        if not sync:
            self.sync()
        return out

    def copy(self, dst, src, nbytes, sync=False):
        assert self.lib.mock_device_d2d(dst, src, int(nbytes), int(sync)) == 0, self.error()

    def memset(self, ptr, kind, pattern, nbytes):
        assert self.lib.mock_device_memset(ptr, kind, pattern, int(nbytes)) == 0, self.error()

    def sync(self, everything=False):
        assert self.lib.mock_device_sync(int(everything)) == 0, self.error()

    def stats(self):
        out = (C.c_int64 * 8)()
        assert self.lib.mock_device_stats(out) == 0
        return dict(zip(("num_allocs", "bytes_in_use", "peak_bytes_in_use", "largest_alloc_size", "bytes_reserved",
                         "largest_free_block_bytes", "device_free", "device_total"), out))

    def use_for_tensors(self):
        """Outputs, temporaries and host-pinned tensors of the mock now come from the plugin's allocators."""
        self.lib.mock_device_use_allocator()


def load_device(ordinal=0):
    """SE_InitPlugin + device / stream executor / stream creation; returns (rc, DevicePlugin).  rc 4 means
    the plugin initialised but reports no device with that ordinal (no GPU in this process)."""
    lib = load()
    if "devplug" not in _state:
        _state["devplug"] = DevicePlugin(lib)
        _state["devplug_rc"] = lib.mock_device_load(PLUGIN_LIB.encode(), ordinal)
    return _state["devplug_rc"], _state["devplug"]
