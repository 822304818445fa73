"""ctypes binding of lib/libitexhip.so (the C ABI declared in include/itexhip.h).

All buffers are raw device addresses (ints) or objects with a `data_ptr()` method (torch tensors);
streams are raw hipStream_t handles (ints, 0 = default stream).  Every call checks the status and
raises ItexHipError with the library's message.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("ITEXHIP_LIB") or os.path.join(_HERE, "lib", "libitexhip.so")  # ITEXHIP_LIB: another build, for A/B timing

OK, INVALID_ARGUMENT, UNIMPLEMENTED, INTERNAL = 0, 3, 12, 13
FLOAT, INT32, QINT8, QUINT8, QINT32, BFLOAT16, HALF = 1, 3, 11, 12, 13, 14, 19
MIN_COMBINED, MIN_FIRST, SCALED, MIN_FIRST_CLASSIC = 0, 1, 2, 3
DYNAMIC_STATE_FLOATS = 1032   # floats of device memory itexhip_quantize_dynamic needs for its state
API_V2, API_V1, API_LEGACY = 0, 1, 2
ACT_NONE, ACT_RELU, ACT_RELU6, ACT_LEAKYRELU, ACT_GELU_APPROX, ACT_GELU_EXACT = 0, 1, 2, 3, 4, 5
ACT_ELU, ACT_SIGMOID, ACT_TANH, ACT_SWISH, ACT_MISH = 6, 7, 8, 9, 10
ELT_RELU, ELT_CLIP, ELT_LINEAR, ELT_GELU_TANH, ELT_GELU_ERF, ELT_SUM = 1, 2, 3, 4, 5, 6
ELT_ELU, ELT_LOGISTIC, ELT_TANH, ELT_SWISH, ELT_MISH = 7, 8, 9, 10, 11

EXPORTS = [
    "itexhip_device_count", "itexhip_device_info", "itexhip_mem_info", "itexhip_malloc", "itexhip_free",
    "itexhip_host_malloc", "itexhip_host_free", "itexhip_stream_create", "itexhip_stream_destroy",
    "itexhip_stream_query", "itexhip_event_create", "itexhip_event_destroy", "itexhip_event_record",
    "itexhip_event_query", "itexhip_event_synchronize", "itexhip_stream_wait_event", "itexhip_device_synchronize",
    "itexhip_memcpy_d2h_async", "itexhip_memset8_async", "itexhip_memset32_async", "itexhip_launch_host_func",
    "itexhip_last_error", "itexhip_build_info", "itexhip_test_force_tile_shape", "itexhip_memcpy_h2d_async", "itexhip_memcpy_d2h", "itexhip_memcpy_d2d_async", "itexhip_stream_synchronize", "itexhip_quantize", "itexhip_quantize_axis",
    "itexhip_dequantize", "itexhip_dequantize_axis", "itexhip_quantize_bf16", "itexhip_quantize_axis_bf16",
    "itexhip_dequantize16", "itexhip_dequantize_axis16", "itexhip_requantize_per_channel",
    "itexhip_requantize", "itexhip_minmax_i32_per_channel", "itexhip_minmax_f32",
    "itexhip_qmatmul_epilogue_desc", "itexhip_qmatmul_prepare", "itexhip_qgemm_packed_bytes",
    "itexhip_qgemm_prepack_b", "itexhip_qgemm", "itexhip_qgemm_tile", "itexhip_qgemv", "itexhip_qmatmul", "itexhip_qmatmul_per_row", "itexhip_qmatmul_device_range", "itexhip_quantize_dynamic", "itexhip_quantize_dynamic_static", "itexhip_quantize_dynamic_rows", "itexhip_qmatmul_unpacked", "itexhip_mfma_probe", "itexhip_read_probe",
    "itexhip_qgemm_naive", "itexhip_qbatch_matmul", "itexhip_transpose", "itexhip_im2col8", "itexhip_pad_nhwc8", "itexhip_scale_vector",
    "itexhip_qconv2d_implicit_ok", "itexhip_qconv2d", "itexhip_qgemm_sum", "itexhip_qconv2d_sum", "itexhip_qdepthwise_conv2d",
]


class ItexHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("itexhip status %d: %s" % (code, msg))
        self.code = code


class Eltwise(C.Structure):
    _fields_ = [("alg", C.c_int), ("alpha", C.c_float), ("beta", C.c_float)]


class Epilogue(C.Structure):
    _fields_ = [("n_scales", C.c_int), ("n_eltwise", C.c_int), ("elt", Eltwise * 3)]


class MatmulParams(C.Structure):
    _fields_ = [("api", C.c_int), ("t_in", C.c_int), ("t_out", C.c_int), ("input_mode", C.c_int),
                ("out_min_first", C.c_int), ("activation", C.c_int), ("has_requantize", C.c_int),
                ("has_dequantize", C.c_int), ("n_fused_ops", C.c_int), ("leakyrelu_alpha", C.c_float),
                ("min_a", C.c_float), ("max_a", C.c_float), ("min_out", C.c_float),
                ("max_out", C.c_float), ("add_position", C.c_int), ("t_bias", C.c_int)]


# One HIP runtime per process: PyTorch ships its own libamdhip64.so.7 and loads it by path.  If this
# library were loaded first, the system runtime would be mapped as well and the second one to
# initialise finds no device.  Importing torch first lets the dynamic loader satisfy this library's
# libamdhip64.so.7 dependency with the copy that is already mapped.
try:
    import torch  # noqa: F401
except ImportError:  # a process without PyTorch uses the system runtime
    pass

if not os.path.exists(LIB_PATH):
    raise ImportError("native library missing: %s (run intel-extension-for-tensorflow_amd/build.py)"
                      % LIB_PATH)
_lib = C.CDLL(LIB_PATH)
_lib.itexhip_last_error.restype = C.c_char_p
_lib.itexhip_build_info.restype = C.c_char_p
_lib.itexhip_qgemm_packed_bytes.restype = C.c_int64
_lib.itexhip_qgemm_packed_bytes.argtypes = [C.c_int64, C.c_int64]


def raw():
    """The ctypes.CDLL handle."""
    return _lib


def _ptr(x):
    if x is None:
        return C.c_void_p(0)
    if hasattr(x, "data_ptr"):
        return C.c_void_p(x.data_ptr())
    return C.c_void_p(int(x))


def _check(st):
    if st != OK:
        raise ItexHipError(st, _lib.itexhip_last_error().decode())


def _i64(v):
    return C.c_int64(int(v))


def build_info():
    return _lib.itexhip_build_info().decode()


def force_tile_shape(matmul=-1, conv=-1):
    """Test hook: forces the tile shape of the MatMul tile kernel / the implicit-GEMM Conv2D for every later call (-1: the
    library chooses)."""
    _lib.itexhip_test_force_tile_shape.restype = None
    _lib.itexhip_test_force_tile_shape(C.c_int(int(matmul)), C.c_int(int(conv)))


def memcpy_d2h(host_array, src, nbytes, stream=0):
    """Device -> host (a numpy array) copy that returns when the bytes have arrived."""
    _check(_lib.itexhip_memcpy_d2h(C.c_void_p(host_array.ctypes.data), _ptr(src), C.c_size_t(int(nbytes)), _ptr(stream)))


def memcpy_d2d_async(dst, src, nbytes, stream=0):
    _check(_lib.itexhip_memcpy_d2d_async(_ptr(dst), _ptr(src), C.c_size_t(int(nbytes)), _ptr(stream)))


def quantize(x, q, n, dst_type, scale, addend=0.0, stream=0):
    _check(_lib.itexhip_quantize(_ptr(x), _ptr(q), _i64(n), dst_type, C.c_float(scale),
                                 C.c_float(addend), _ptr(stream)))


def quantize_axis(x, q, outer, slices, inner, dst_type, scales, addends=None, stream=0):
    _check(_lib.itexhip_quantize_axis(_ptr(x), _ptr(q), _i64(outer), _i64(slices), _i64(inner),
                                      dst_type, _ptr(scales), _ptr(addends), _ptr(stream)))


def quantize_bf16(x, q, n, dst_type, scale, addend=0.0, stream=0):
    _check(_lib.itexhip_quantize_bf16(_ptr(x), _ptr(q), _i64(n), dst_type, C.c_float(scale), C.c_float(addend),
                                      _ptr(stream)))


def quantize_axis_bf16(x, q, outer, slices, inner, dst_type, scales, addends=None, stream=0):
    _check(_lib.itexhip_quantize_axis_bf16(_ptr(x), _ptr(q), _i64(outer), _i64(slices), _i64(inner), dst_type,
                                           _ptr(scales), _ptr(addends), _ptr(stream)))


def dequantize16(q, y, n, src_type, y_type, scale, zero_point=0, stream=0):
    _check(_lib.itexhip_dequantize16(_ptr(q), _ptr(y), _i64(n), src_type, y_type, C.c_float(scale),
                                     C.c_int32(int(zero_point)), _ptr(stream)))


def dequantize_axis16(q, y, outer, slices, inner, src_type, y_type, scales, zero_points=None, stream=0):
    _check(_lib.itexhip_dequantize_axis16(_ptr(q), _ptr(y), _i64(outer), _i64(slices), _i64(inner), src_type, y_type,
                                          _ptr(scales), _ptr(zero_points), _ptr(stream)))


def dequantize(q, y, n, src_type, scale, zero_point=0, stream=0):
    _check(_lib.itexhip_dequantize(_ptr(q), _ptr(y), _i64(n), src_type, C.c_float(scale),
                                   C.c_int32(int(zero_point)), _ptr(stream)))


def dequantize_axis(q, y, outer, slices, inner, src_type, scales, zero_points=None, stream=0):
    _check(_lib.itexhip_dequantize_axis(_ptr(q), _ptr(y), _i64(outer), _i64(slices), _i64(inner),
                                        src_type, _ptr(scales), _ptr(zero_points), _ptr(stream)))


def requantize_per_channel(x, q, rows, depth, dst_type, scales, stream=0):
    _check(_lib.itexhip_requantize_per_channel(_ptr(x), _ptr(q), _i64(rows), _i64(depth), dst_type,
                                               _ptr(scales), _ptr(stream)))


def requantize(x, q, n, dst_type, scale, stream=0):
    _check(_lib.itexhip_requantize(_ptr(x), _ptr(q), _i64(n), dst_type, C.c_float(scale),
                                   _ptr(stream)))


def minmax_i32_per_channel(x, rows, depth, min_out, max_out, stream=0):
    _check(_lib.itexhip_minmax_i32_per_channel(_ptr(x), _i64(rows), _i64(depth), _ptr(min_out),
                                               _ptr(max_out), _ptr(stream)))


def minmax_f32(x, n, minmax_out, stream=0):
    _check(_lib.itexhip_minmax_f32(_ptr(x), _i64(n), _ptr(minmax_out), _ptr(stream)))


def matmul_params(api=API_V2, t_in=QUINT8, t_out=FLOAT, input_mode=MIN_FIRST, out_min_first=False,
                  activation=ACT_NONE, has_requantize=False, has_dequantize=False, n_fused_ops=1,
                  leakyrelu_alpha=0.2, min_a=0.0, max_a=0.0, min_out=0.0, max_out=0.0, add_position=0, t_bias=0):
    return MatmulParams(api, t_in, t_out, input_mode, int(out_min_first), activation,
                        int(has_requantize), int(has_dequantize), n_fused_ops, leakyrelu_alpha,
                        min_a, max_a, min_out, max_out, int(add_position), int(t_bias))


def qmatmul_epilogue_desc(params, nb):
    ep = Epilogue()
    _check(_lib.itexhip_qmatmul_epilogue_desc(C.byref(params), _i64(nb), C.byref(ep)))
    return ep


def qmatmul_prepare(params, min_b, max_b, nb, bias, colsum, N, scales_out, bias_out, stream=0):
    _check(_lib.itexhip_qmatmul_prepare(C.byref(params), _ptr(min_b), _ptr(max_b), _i64(nb),
                                        _ptr(bias), _ptr(colsum), _i64(N), _ptr(scales_out),
                                        _ptr(bias_out), _ptr(stream)))


def qgemm_packed_bytes(K, N):
    return int(_lib.itexhip_qgemm_packed_bytes(int(K), int(N)))


def qgemm_prepack_b(w, transpose_b, K, N, packed, colsum, stream=0):
    _check(_lib.itexhip_qgemm_prepack_b(_ptr(w), int(bool(transpose_b)), _i64(K), _i64(N),
                                        _ptr(packed), _ptr(colsum), _ptr(stream)))


def _gemm_call(fn, a, a_type, b, colsum, M, K, N, scales, bias, ep, out_type, out, stream):
    _check(fn(_ptr(a), a_type, _ptr(b), _ptr(colsum), _i64(M), _i64(K), _i64(N), _ptr(scales),
              _ptr(bias), C.byref(ep), out_type, _ptr(out), _ptr(stream)))


def qgemm(a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream=0):
    _gemm_call(_lib.itexhip_qgemm, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type,
               out, stream)


def qgemm_tile(a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream=0):
    _gemm_call(_lib.itexhip_qgemm_tile, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep,
               out_type, out, stream)


def qgemv(a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type, out, stream=0):
    _gemm_call(_lib.itexhip_qgemv, a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, out_type,
               out, stream)


def qmatmul(p, a, packed_b, colsum, M, K, N, min_b, max_b, nb, bias, out, stream=0, addend=None):
    """The whole op in one launch (parameters derived inside the MatMul kernel)."""
    _check(_lib.itexhip_qmatmul(C.byref(p), _ptr(a), _ptr(packed_b), _ptr(colsum), _i64(M), _i64(K), _i64(N),
                                _ptr(min_b), _ptr(max_b), _i64(nb), _ptr(bias), _ptr(addend), _ptr(out),
                                _ptr(stream)))


def qmatmul_per_row(p, a, packed_b, colsum, M, K, N, row_min_a, row_max_a, min_b, max_b, nb, bias, out, stream=0,
                    addend=None):
    _check(_lib.itexhip_qmatmul_per_row(C.byref(p), _ptr(a), _ptr(packed_b), _ptr(colsum), _i64(M), _i64(K), _i64(N),
                                        _ptr(row_min_a), _ptr(row_max_a), _ptr(min_b), _ptr(max_b), _i64(nb),
                                        _ptr(bias), _ptr(addend), _ptr(out), _ptr(stream)))


def qmatmul_device_range(p, a, packed_b, colsum, M, K, N, range_a, min_b, max_b, nb, bias, out, stream=0, addend=None):
    _check(_lib.itexhip_qmatmul_device_range(C.byref(p), _ptr(a), _ptr(packed_b), _ptr(colsum), _i64(M), _i64(K), _i64(N),
                                             _ptr(range_a), _ptr(min_b), _ptr(max_b), _i64(nb), _ptr(bias),
                                             _ptr(addend), _ptr(out), _ptr(stream)))


def quantize_dynamic(x, q, n, dst_type, mode, ensure_minimum_range, state, stream=0):
    _check(_lib.itexhip_quantize_dynamic(_ptr(x), _ptr(q), _i64(n), int(dst_type), int(mode),
                                         C.c_float(ensure_minimum_range), _ptr(state), _ptr(stream)))


def read_probe(src, nbytes, sink, stream=0):
    _check(_lib.itexhip_read_probe(_ptr(src), C.c_size_t(nbytes), _ptr(sink), _ptr(stream)))


def quantize_dynamic_static(x, q, n, dst_type, mode, ensure_minimum_range, range_out, stream=0):
    _check(_lib.itexhip_quantize_dynamic_static(_ptr(x), _ptr(q), _i64(n), int(dst_type), int(mode),
                                                C.c_float(ensure_minimum_range), _ptr(range_out), _ptr(stream)))


def quantize_dynamic_rows(x, q, rows, cols, dst_type, mode, ensure_minimum_range, row_min_out, row_max_out, stream=0):
    _check(_lib.itexhip_quantize_dynamic_rows(_ptr(x), _ptr(q), _i64(rows), _i64(cols), int(dst_type), int(mode),
                                              C.c_float(ensure_minimum_range), _ptr(row_min_out), _ptr(row_max_out),
                                              _ptr(stream)))


def qmatmul_unpacked(p, a, w, transpose_b, M, K, N, min_b, max_b, nb, bias, out, stream=0, addend=None):
    _check(_lib.itexhip_qmatmul_unpacked(C.byref(p), _ptr(a), _ptr(w), int(bool(transpose_b)), _i64(M), _i64(K), _i64(N),
                                         _ptr(min_b), _ptr(max_b), _i64(nb), _ptr(bias), _ptr(addend), _ptr(out),
                                         _ptr(stream)))


def mfma_probe(workgroups, iters, operands, sink, stream=0):
    _check(_lib.itexhip_mfma_probe(int(workgroups), int(iters), _ptr(operands), _ptr(sink), _ptr(stream)))


def qgemm_naive(a, a_type, w, transpose_b, M, K, N, scales, bias, ep, out_type, out, stream=0):
    _check(_lib.itexhip_qgemm_naive(_ptr(a), a_type, _ptr(w), int(bool(transpose_b)), _i64(M),
                                    _i64(K), _i64(N), _ptr(scales), _ptr(bias), C.byref(ep),
                                    out_type, _ptr(out), _ptr(stream)))


# ---- quantized BatchMatMul -----------------------------------------------------------------------
BIN_MUL, BIN_ADD = 1, 2


class BmmBinary(C.Structure):
    _fields_ = [("alg", C.c_int), ("data", C.c_void_p), ("batch_stride", C.c_int64 * 4), ("stride_m", C.c_int64),
                ("stride_n", C.c_int64)]


class BmmParams(C.Structure):
    _fields_ = [("n_batch_dims", C.c_int), ("batch_dims", C.c_int64 * 4), ("x_batch_stride", C.c_int64 * 4),
                ("y_batch_stride", C.c_int64 * 4), ("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("adj_x", C.c_int), ("adj_y", C.c_int), ("out_type", C.c_int), ("scale", C.c_float),
                ("n_binary", C.c_int), ("binary", BmmBinary * 2)]


def _broadcast_strides(shape, out_shape):
    """Row-major element strides of `shape` (right-aligned against out_shape), 0 where it broadcasts."""
    shape = (1,) * (len(out_shape) - len(shape)) + tuple(shape)
    strides, st = [], 1
    for d, o in zip(reversed(shape), reversed(out_shape)):
        if d != o and d != 1:
            raise ValueError("shape %r does not broadcast to %r" % (shape, out_shape))
        strides.append(0 if d == 1 else st)
        st *= d
    return strides[::-1]


def bmm_params(x_shape, y_shape, adj_x, adj_y, out_type, scale, binary=()):
    """Shapes, broadcast strides and post-ops of one quantized BatchMatMul call.
    binary: sequence of (BIN_MUL | BIN_ADD, device buffer, shape); returns (params, output shape)."""
    xm = tuple(x_shape[-2:][::-1]) if adj_x else tuple(x_shape[-2:])
    ym = tuple(y_shape[-2:][::-1]) if adj_y else tuple(y_shape[-2:])
    if xm[1] != ym[0]:
        raise ValueError("inner dimensions differ")
    xb, yb = tuple(x_shape[:-2]), tuple(y_shape[:-2])
    nb = max(len(xb), len(yb))
    xb, yb = (1,) * (nb - len(xb)) + xb, (1,) * (nb - len(yb)) + yb
    batch = tuple(max(a, b) if 0 not in (a, b) else 0 for a, b in zip(xb, yb))
    if nb > 4:
        raise ValueError("at most 4 batch dimensions")
    p = BmmParams()
    p.n_batch_dims = nb
    p.M, p.K, p.N = xm[0], xm[1], ym[1]
    xs = _broadcast_strides(xb + (1,), batch + (1,))[:-1]
    ys = _broadcast_strides(yb + (1,), batch + (1,))[:-1]
    for d in range(nb):
        p.batch_dims[d] = batch[d]
        p.x_batch_stride[d] = xs[d] * xm[0] * xm[1]
        p.y_batch_stride[d] = ys[d] * ym[0] * ym[1]
    p.adj_x, p.adj_y, p.out_type, p.scale = int(bool(adj_x)), int(bool(adj_y)), out_type, scale
    out_shape = batch + (xm[0], ym[1])
    p.n_binary = len(binary)
    for i, (alg, buf, shape) in enumerate(binary):
        n_el = 1
        for d in shape:
            n_el *= d
        st = [0] * len(out_shape) if n_el == 1 else _broadcast_strides(tuple(shape), out_shape)
        if n_el != 1 and len(shape) != len(out_shape):
            raise ValueError("a binary operand has one element or the output's rank")
        p.binary[i].alg = alg
        p.binary[i].data = _ptr(buf).value
        for d in range(nb):
            p.binary[i].batch_stride[d] = st[d]
        p.binary[i].stride_m, p.binary[i].stride_n = st[nb], st[nb + 1]
    return p, out_shape


def qbatch_matmul(p, x, y, out, stream=0):
    _check(_lib.itexhip_qbatch_matmul(C.byref(p), _ptr(x), _ptr(y), _ptr(out), _ptr(stream)))


def transpose(x, y, elem_size, dims, perm, stream=0):
    rank = len(dims)
    d = (C.c_int64 * max(rank, 1))(*dims)
    pm = (C.c_int32 * max(rank, 1))(*perm)
    _check(_lib.itexhip_transpose(_ptr(x), _ptr(y), int(elem_size), rank, d, pm, _ptr(stream)))


class ConvGeometry(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("batch", "in_h", "in_w", "in_c", "k_h", "k_w", "out_h", "out_w")] + \
               [(n, C.c_int) for n in ("stride_h", "stride_w", "dil_h", "dil_w")] + [("pad_top", C.c_int64), ("pad_left", C.c_int64)]


def im2col8(x, geometry, row_bytes, cols, stream=0):
    _check(_lib.itexhip_im2col8(_ptr(x), C.byref(geometry), _i64(row_bytes), _ptr(cols), _ptr(stream)))


def pad_nhwc8(x, n, h, w, c, lead_h, lead_w, out_h, out_w, out_c, out, stream=0):
    _check(_lib.itexhip_pad_nhwc8(_ptr(x), _i64(n), _i64(h), _i64(w), _i64(c), _i64(lead_h), _i64(lead_w), _i64(out_h),
                                  _i64(out_w), _i64(out_c), _ptr(out), _ptr(stream)))


def qconv2d_implicit_ok(geometry, x, out_channels, out_type, out):
    return bool(_lib.itexhip_qconv2d_implicit_ok(C.byref(geometry), _ptr(x), _i64(out_channels), int(out_type), _ptr(out)))


def qconv2d(x, x_type, geometry, packed_filter, colsum, out_channels, scales, bias, ep, out_type, out, stream=0):
    _check(_lib.itexhip_qconv2d(_ptr(x), int(x_type), C.byref(geometry), _ptr(packed_filter), _ptr(colsum), _i64(out_channels),
                                _ptr(scales), _ptr(bias), C.byref(ep), int(out_type), _ptr(out), _ptr(stream)))


def qconv2d_sum(x, x_type, geometry, packed_filter, colsum, out_channels, scales, bias, ep, addend, addend_type, out_type, out,
                stream=0):
    _check(_lib.itexhip_qconv2d_sum(_ptr(x), int(x_type), C.byref(geometry), _ptr(packed_filter), _ptr(colsum), _i64(out_channels),
                                    _ptr(scales), _ptr(bias), C.byref(ep), _ptr(addend), int(addend_type), int(out_type),
                                    _ptr(out), _ptr(stream)))


def qgemm_sum(a, a_type, packed_b, colsum, M, K, N, scales, bias, ep, addend, addend_type, out_type, out, stream=0):
    _check(_lib.itexhip_qgemm_sum(_ptr(a), int(a_type), _ptr(packed_b), _ptr(colsum), _i64(M), _i64(K), _i64(N), _ptr(scales),
                                  _ptr(bias), C.byref(ep), _ptr(addend), int(addend_type), int(out_type), _ptr(out), _ptr(stream)))


def qdepthwise_conv2d(x, x_type, geometry, multiplier, filt, scales, bias, ep, out_type, out, stream=0):
    _check(_lib.itexhip_qdepthwise_conv2d(_ptr(x), int(x_type), C.byref(geometry), _i64(multiplier), _ptr(filt), _ptr(scales),
                                          _ptr(bias), C.byref(ep), int(out_type), _ptr(out), _ptr(stream)))


def scale_vector(bias, bias_type, factors, n_factors, n, out, stream=0):
    _check(_lib.itexhip_scale_vector(_ptr(bias), int(bias_type), _ptr(factors), _i64(n_factors), _i64(n), _ptr(out), _ptr(stream)))
