"""Python driver of the mock TensorFlow host (tests/mock_tf/mock_tf.cc): loads the plugin the way
TensorFlow does (dlopen + TF_InitKernel), instantiates kernels from node attributes and runs them."""
import ctypes as C
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
MOCK_LIB = os.path.join(HERE, "libmock_tf.so")
PLUGIN_LIB = os.path.join(ROOT, "intel-extension-for-tensorflow_amd", "lib", "libitex_amd.so")

FLOAT, INT32, QINT8, QUINT8, QINT32 = 1, 3, 11, 12, 13
NP_OF = {FLOAT: np.float32, INT32: np.int32, QINT8: np.int8, QUINT8: np.uint8, QINT32: np.int32}
OK, INVALID_ARGUMENT, NOT_FOUND, ABORTED, UNIMPLEMENTED = 0, 3, 5, 10, 12

_ALLOC = C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_int)
_FREE = C.CFUNCTYPE(None, C.c_void_p, C.c_int)

_state = {}


def load(device="XPU", stock_ops=("QuantizeV2", "Dequantize", "QuantizedMatMulWithBias", "QuantizedMatMulWithBiasAndRelu",
                                   "QuantizedMatMulWithBiasAndReluAndRequantize", "QuantizedMatMulWithBiasAndRequantize",
                                   "QuantizedMatMulWithBiasAndDequantize", "RequantizePerChannel",
                                   "RequantizationRangePerChannel", "MatMul", "Relu")):
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


def host_array(a):
    """(dtype-agnostic) address of a numpy array that the caller keeps alive."""
    return a.ctypes.data


def read_host(addr, dtype, shape):
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    buf = (C.c_char * (n * np.dtype(NP_OF[dtype]).itemsize)).from_address(addr)
    return np.frombuffer(buf, dtype=NP_OF[dtype]).reshape(shape).copy()
