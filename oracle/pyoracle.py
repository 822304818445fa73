"""ctypes binding of the CPU oracle (oracle/libitex_oracle.so).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
of bench.py, always as the checker or the timed CPU baseline, never by the shipped library.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libitex_oracle.so")

FLOAT, INT32, QINT8, QUINT8, QINT32, BFLOAT16, HALF = 1, 3, 11, 12, 13, 14, 19
MIN_COMBINED, MIN_FIRST, SCALED = 0, 1, 2
API_V2, API_V1, API_LEGACY = 0, 1, 2
ACT_NONE, ACT_RELU, ACT_RELU6, ACT_LEAKYRELU, ACT_GELU_APPROX, ACT_GELU_EXACT = 0, 1, 2, 3, 4, 5
ACT_ELU, ACT_SIGMOID, ACT_TANH, ACT_SWISH, ACT_MISH = 6, 7, 8, 9, 10
OK, INVALID_ARGUMENT, UNIMPLEMENTED = 0, 3, 12

NP_OF = {QINT8: np.int8, QUINT8: np.uint8, QINT32: np.int32, FLOAT: np.float32, BFLOAT16: np.uint16, HALF: np.uint16}


def build():
    """Compile the oracle with its Makefile (gcc, contraction off)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libitex_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


class Eltwise(C.Structure):
    _fields_ = [("alg", C.c_int), ("alpha", C.c_float), ("beta", C.c_float)]


class MatmulAttrs(C.Structure):
    _fields_ = [("api", C.c_int), ("t_in", C.c_int), ("t_out", C.c_int), ("input_mode", C.c_int),
                ("out_min_first", C.c_int), ("activation", C.c_int), ("has_requantize", C.c_int),
                ("has_dequantize", C.c_int), ("n_fused_ops", C.c_int),
                ("leakyrelu_alpha", C.c_float), ("add_position", C.c_int), ("t_bias", C.c_int)]


class EpilogueDesc(C.Structure):
    _fields_ = [("n_scales", C.c_int), ("n_eltwise", C.c_int), ("elt", Eltwise * 3)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_legacy_min_first_scale.restype = C.c_float
        _lib.orc_legacy_min_first_scale.argtypes = [C.c_int, C.c_float, C.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(v):
    return np.ascontiguousarray(np.atleast_1d(np.asarray(v, dtype=np.float32)))


def adjust_input_range(mn, mx, ensure_minimum_range=0.01):
    a, b = C.c_float(), C.c_float()
    st = lib().orc_adjust_input_range(C.c_float(mn), C.c_float(mx), C.c_float(ensure_minimum_range),
                                      C.byref(a), C.byref(b))
    return st, np.float32(a.value), np.float32(b.value)


def scale_zeropoint_align(T, mode, dequantize, mn, mx):
    mn, mx = _f32(mn).copy(), _f32(mx).copy()
    n = mn.size
    sc = np.zeros(n, np.float32)
    zp = np.zeros(n, np.int32)
    st = lib().orc_scale_zeropoint_align(T, mode, int(dequantize), _p(mn), _p(mx), n, _p(sc), _p(zp))
    return st, mn, mx, sc, zp


def legacy_min_first_scale(T, mn, mx):
    return np.float32(lib().orc_legacy_min_first_scale(T, C.c_float(mn), C.c_float(mx)))


def _split(shape, axis):
    shape = tuple(int(s) for s in shape)
    if axis is None or axis < 0:
        return 1, 1, int(np.prod(shape, dtype=np.int64))
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, shape[axis], inner


def quantize_v2(x, mn, mx, T, mode, axis=None, classic=False, ensure_minimum_range=0.01):
    """Returns (status, q, out_min, out_max)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    outer, slices, inner = _split(x.shape, axis)
    mn, mx = _f32(mn), _f32(mx)
    assert mn.size == slices and mx.size == slices
    q = np.zeros(x.shape, NP_OF[T])
    omn, omx = np.zeros(slices, np.float32), np.zeros(slices, np.float32)
    st = lib().orc_quantize_v2(_p(x), C.c_int64(outer), C.c_int64(slices), C.c_int64(inner), T, mode,
                               int(classic), C.c_float(ensure_minimum_range), _p(mn), _p(mx), _p(q),
                               _p(omn), _p(omx))
    return st, q, omn, omx


def dequantize(q, mn, mx, T, mode, axis=None):
    q = np.ascontiguousarray(q, dtype=NP_OF[T])
    outer, slices, inner = _split(q.shape, axis)
    mn, mx = _f32(mn), _f32(mx)
    assert mn.size == slices and mx.size == slices
    y = np.zeros(q.shape, np.float32)
    st = lib().orc_dequantize(_p(q), C.c_int64(outer), C.c_int64(slices), C.c_int64(inner), T, mode,
                              _p(mn), _p(mx), _p(y))
    return st, y


def requantize_per_channel(x, in_min, in_max, req_min, req_max, out_type):
    x = np.ascontiguousarray(x, dtype=np.int32)
    depth = x.shape[-1]
    rows = x.size // depth
    in_min, in_max = _f32(in_min), _f32(in_max)
    assert in_min.size == depth and in_max.size == depth
    q = np.zeros(x.shape, NP_OF[out_type])
    omn, omx = C.c_float(), C.c_float()
    st = lib().orc_requantize_per_channel(_p(x), C.c_int64(rows), C.c_int64(depth), _p(in_min),
                                          _p(in_max), C.c_float(req_min), C.c_float(req_max),
                                          out_type, _p(q), C.byref(omn), C.byref(omx))
    return st, q, np.float32(omn.value), np.float32(omx.value)


def requantization_range_per_channel(x, in_min, in_max, clip_value_max):
    x = np.ascontiguousarray(x, dtype=np.int32)
    depth = x.shape[-1]
    rows = x.size // depth
    in_min, in_max = _f32(in_min), _f32(in_max)
    omn, omx = C.c_float(), C.c_float()
    st = lib().orc_requantization_range_per_channel(_p(x), C.c_int64(rows), C.c_int64(depth),
                                                    _p(in_min), _p(in_max),
                                                    C.c_float(clip_value_max), C.byref(omn),
                                                    C.byref(omx))
    return st, np.float32(omn.value), np.float32(omx.value)


def int_gemm(a, w, transpose_b=False):
    a = np.ascontiguousarray(a)
    w = np.ascontiguousarray(w, dtype=np.int8)
    a_type = QUINT8 if a.dtype == np.uint8 else QINT8
    M, K = a.shape
    N = w.shape[0] if transpose_b else w.shape[1]
    acc = np.zeros((M, N), np.int32)
    lib().orc_int_gemm(_p(a), a_type, _p(w), int(transpose_b), C.c_int64(M), C.c_int64(K),
                       C.c_int64(N), _p(acc))
    return acc


def weight_colsum(w):
    w = np.ascontiguousarray(w, dtype=np.int8)
    K, N = w.shape
    cs = np.zeros(N, np.int32)
    lib().orc_weight_colsum(_p(w), C.c_int64(K), C.c_int64(N), _p(cs))
    return cs


def matmul_attrs(api=API_V2, t_in=QUINT8, t_out=FLOAT, input_mode=MIN_FIRST, out_min_first=False,
                 activation=ACT_NONE, has_requantize=False, has_dequantize=False, n_fused_ops=1,
                 leakyrelu_alpha=0.2, add_position=0, t_bias=0):
    return MatmulAttrs(api, t_in, t_out, input_mode, int(out_min_first), activation,
                       int(has_requantize), int(has_dequantize), n_fused_ops, leakyrelu_alpha,
                       int(add_position), int(t_bias))


def _bias(at, bias):
    """The bias vector as the C side reads it (a bfloat16 bias is given as uint16 bit patterns)."""
    if at.t_bias == QINT32:
        return np.ascontiguousarray(bias, dtype=np.int32)
    if at.t_bias in (BFLOAT16, HALF):
        return np.ascontiguousarray(bias, dtype=np.uint16)
    return _f32(bias)


def qmatmul_prepare(at, N, colsum, min_a, max_a, min_b, max_b, min_out, max_out, bias):
    """Returns (status, scales[n_scales], scaled_bias[N], EpilogueDesc)."""
    min_b, max_b = _f32(min_b), _f32(max_b)
    nb = min_b.size
    bias = _bias(at, bias)
    colsum = np.ascontiguousarray(colsum, dtype=np.int32)
    scales = np.zeros(max(nb, 1), np.float32)
    sb = np.zeros(N, np.float32)
    ep = EpilogueDesc()
    st = lib().orc_qmatmul_prepare(C.byref(at), C.c_int64(N), _p(colsum), C.c_float(min_a),
                                   C.c_float(max_a), _p(min_b), _p(max_b), C.c_int64(nb),
                                   C.c_float(min_out), C.c_float(max_out), _p(bias), _p(scales),
                                   _p(sb), C.byref(ep))
    return st, scales[:ep.n_scales].copy(), sb, ep


def qmatmul_epilogue(acc, ep, scales, bias, t_out, addend=None):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    scales = _f32(scales) if ep.n_scales else np.zeros(1, np.float32)
    bias = _f32(bias)
    out = np.zeros((M, N), NP_OF[t_out])
    addend = None if addend is None else _f32(addend)
    lib().orc_qmatmul_epilogue(_p(acc), C.c_int64(M), C.c_int64(N), C.byref(ep), _p(scales),
                               _p(bias), _p(addend) if addend is not None else None, t_out, _p(out))
    return out


def qmatmul_output_minmax(at, min_a, max_a, min_b, max_b, b_rank, min_out, max_out):
    min_b, max_b = _f32(min_b), _f32(max_b)
    nb = min_b.size
    omn, omx = np.zeros(max(nb, 1), np.float32), np.zeros(max(nb, 1), np.float32)
    n_out = C.c_int64()
    st = lib().orc_qmatmul_output_minmax(C.byref(at), C.c_float(min_a), C.c_float(max_a), _p(min_b),
                                         _p(max_b), C.c_int64(nb), b_rank, C.c_float(min_out),
                                         C.c_float(max_out), _p(omn), _p(omx), C.byref(n_out))
    return st, omn[:n_out.value].copy(), omx[:n_out.value].copy()


def qmatmul(at, a, w, bias, min_a, max_a, min_b, max_b, min_out=0.0, max_out=0.0,
            transpose_b=False, addend=None):
    """Whole op.  Returns (status, out[M,N])."""
    a = np.ascontiguousarray(a)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = a.shape
    N = w.shape[0] if transpose_b else w.shape[1]
    min_b, max_b = _f32(min_b), _f32(max_b)
    bias = _bias(at, bias)
    addend = None if addend is None else _f32(addend)
    out = np.zeros((M, N), NP_OF[at.t_out])
    st = lib().orc_qmatmul(C.byref(at), _p(a), _p(w), int(transpose_b), C.c_int64(M), C.c_int64(K),
                           C.c_int64(N), _p(bias), _p(addend) if addend is not None else None,
                           C.c_float(min_a), C.c_float(max_a), _p(min_b),
                           _p(max_b), C.c_int64(min_b.size), C.c_float(min_out), C.c_float(max_out),
                           _p(out))
    return st, out


class BmmBinary(C.Structure):
    _fields_ = [("alg", C.c_int), ("data", C.c_void_p), ("rank", C.c_int), ("dims", C.c_int64 * 8)]


BIN_MUL, BIN_ADD = 1, 2
ELT_RELU, ELT_CLIP, ELT_LINEAR, ELT_GELU_TANH, ELT_GELU_ERF, ELT_SUM = 1, 2, 3, 4, 5, 6
ELT_ELU, ELT_LOGISTIC, ELT_TANH, ELT_SWISH, ELT_MISH = 7, 8, 9, 10, 11


def qbatch_matmul(x, y, min_x, max_x, min_y, max_y, adj_x=False, adj_y=False, binary=(), t_out=FLOAT):
    """binary: sequence of (BIN_MUL | BIN_ADD, array); 16-bit operands are uint16 bit patterns.  Returns (status, out)."""
    x = np.ascontiguousarray(x, dtype=np.int8)
    y = np.ascontiguousarray(y, dtype=np.int8)
    xm = x.shape[-2:][::-1] if adj_x else x.shape[-2:]
    ym = y.shape[-2:][::-1] if adj_y else y.shape[-2:]
    try:
        batch = np.broadcast_shapes(x.shape[:-2], y.shape[:-2])
    except ValueError:
        return INVALID_ARGUMENT, None
    oshape = tuple(batch) + (xm[0], ym[1])
    out = np.zeros(oshape, NP_OF[t_out])
    bins = (BmmBinary * max(len(binary), 1))()
    keep = []
    for i, (alg, arr) in enumerate(binary):
        arr = np.ascontiguousarray(arr, dtype=np.float32 if t_out == FLOAT else np.uint16)
        keep.append(arr)
        bins[i].alg = alg
        bins[i].data = arr.ctypes.data
        bins[i].rank = 0 if arr.size == 1 else arr.ndim
        for d, v in enumerate(arr.shape if arr.size != 1 else ()):
            bins[i].dims[d] = v
    xd = (C.c_int64 * 8)(*x.shape)
    yd = (C.c_int64 * 8)(*y.shape)
    od = (C.c_int64 * 8)(*oshape)
    f = lib().orc_qbatch_matmul
    f.restype = C.c_int
    st = f(_p(x), x.ndim, xd, _p(y), y.ndim, yd, int(bool(adj_x)), int(bool(adj_y)), C.c_float(min_x), C.c_float(max_x),
           C.c_float(min_y), C.c_float(max_y), len(binary), bins, t_out, _p(out), len(oshape), od)
    return st, out


# ---- quantized Conv2D ------------------------------------------------------------------------------
PAD_VALID, PAD_SAME, PAD_EXPLICIT = 0, 1, 2


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("batch", "in_h", "in_w", "in_c", "k_h", "k_w", "out_c")] + \
               [(n, C.c_int) for n in ("stride_h", "stride_w", "dil_h", "dil_w", "padding", "pad_top", "pad_bottom", "pad_left",
                                       "pad_right")]


class ConvAttrs(C.Structure):
    _fields_ = [("t_in", C.c_int), ("t_out", C.c_int), ("t_bias", C.c_int), ("activation", C.c_int), ("alpha", C.c_float)]


def conv_geom(x_shape, w_shape, strides=(1, 1), dilations=(1, 1), padding=PAD_SAME, explicit=(0, 0, 0, 0)):
    b, h, w_, c = x_shape
    kh, kw, ci, co = w_shape
    assert ci == c
    return ConvGeom(b, h, w_, c, kh, kw, co, strides[0], strides[1], dilations[0], dilations[1], padding, *explicit)


def qconv_prepare(at, N, min_in, max_in, min_f, max_f, min_out, max_out, bias):
    min_f, max_f = _f32(min_f), _f32(max_f)
    depth = min_f.size
    scales = np.zeros(max(depth, 1), np.float32)
    sb = np.zeros(N, np.float32)
    ep = EpilogueDesc()
    b = None if bias is None else (np.ascontiguousarray(bias, np.int32) if at.t_bias == QINT32 else _f32(bias))
    f = lib().orc_qconv_prepare
    f.restype = C.c_int
    st = f(C.byref(at), C.c_int64(N), C.c_float(min_in), C.c_float(max_in), _p(min_f), _p(max_f), C.c_int64(depth),
           C.c_float(min_out), C.c_float(max_out), _p(b) if b is not None else None, _p(scales), _p(sb), C.byref(ep))
    return st, scales, sb, ep


class ConvSum(C.Structure):
    _fields_ = [("position", C.c_int), ("t_summand", C.c_int), ("min_summand", C.c_float), ("max_summand", C.c_float)]


def qconv2d(at, g, x, w, bias, min_in, max_in, min_f, max_f, min_out=0.0, max_out=0.0, sum=None, summand=None):
    """x: [B, H, W, C] uint8 / int8, w: [KH, KW, C, O] int8.  Returns (status, out [B, OH, OW, O]).
    sum: ConvSum(position, t_summand, min, max) with `summand` an array of the output's shape (int8 / uint8)."""
    x = np.ascontiguousarray(x, dtype=np.uint8 if at.t_in == QUINT8 else np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    min_f, max_f = _f32(min_f), _f32(max_f)
    b = None if bias is None else (np.ascontiguousarray(bias, np.int32) if at.t_bias == QINT32 else _f32(bias))
    oh, ow = C.c_int64(), C.c_int64()
    f = lib().orc_qconv2d_sum
    f.restype = C.c_int
    if sum is not None:
        summand = np.ascontiguousarray(summand, dtype=np.uint8 if sum.t_summand == QUINT8 else np.int8)
    args = lambda out: (C.byref(at), C.byref(g), _p(x), _p(w), _p(b) if b is not None else None, C.c_float(min_in),
                        C.c_float(max_in), _p(min_f), _p(max_f), C.c_int64(min_f.size), C.c_float(min_out), C.c_float(max_out),
                        C.byref(sum) if sum is not None else None, _p(summand) if sum is not None else None,
                        out, C.byref(oh), C.byref(ow))
    st = f(*args(None))
    if st != OK:
        return st, None
    out = np.zeros((g.batch, oh.value, ow.value, g.out_c), NP_OF[at.t_out])
    st = f(*args(_p(out)))
    return st, out


def qdepthwise_conv2d(at, g, x, w, bias, min_in, max_in, min_f, max_f, min_out=0.0, max_out=0.0):
    """x: [B, H, W, C] uint8 / int8, w: [KH, KW, C, mult] int8 (g built with conv_geom(x.shape, (KH, KW, C, mult))).
    Returns (status, out [B, OH, OW, C * mult])."""
    x = np.ascontiguousarray(x, dtype=np.uint8 if at.t_in == QUINT8 else np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    mult = w.shape[3]
    min_f, max_f = _f32(min_f), _f32(max_f)
    b = None if bias is None else (np.ascontiguousarray(bias, np.int32) if at.t_bias == QINT32 else _f32(bias))
    oh, ow = C.c_int64(), C.c_int64()
    f = lib().orc_qdepthwise_conv2d
    f.restype = C.c_int
    args = lambda out: (C.byref(at), C.byref(g), C.c_int64(mult), _p(x), _p(w), _p(b) if b is not None else None,
                        C.c_float(min_in), C.c_float(max_in), _p(min_f), _p(max_f), C.c_int64(min_f.size), C.c_float(min_out),
                        C.c_float(max_out), out, C.byref(oh), C.byref(ow))
    st = f(*args(None))
    if st != OK:
        return st, None
    out = np.zeros((g.batch, oh.value, ow.value, g.in_c * mult), NP_OF[at.t_out])
    st = f(*args(_p(out)))
    return st, out
