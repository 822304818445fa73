"""Pins the CPU oracle's quantized Conv2D restatement.  The reference's own conv tests
(test/tensorflow/python/kernel_tests/native_quantized_conv_test.py) draw unseeded random inputs and compare with the
fp32 convolution at rtol = atol = 0.3, so they hold no vectors; what pins the oracle here:

  * integer convolution and geometry (SAME / VALID / EXPLICIT, strides, dilations): an independent numpy evaluation
    on the explicitly padded input (sliding windows + tensordot in int64);
  * TensorFlow's output-size / padding rule on known cases (the extra SAME padding goes to the end);
  * scales and bias handling: the reference test's four pipelines on seeded inputs of the same distributions must
    reproduce the fp32 convolution within its 0.3 tolerance and within what the quantization steps allow -- a dropped
    factor, a missing bias scale or a wrong limit (255 vs 127) misses that bound by far;
  * the qint32-bias and qint32-output forms through their closed forms.
"""
import numpy as np
import pytest

from oracle import pyoracle as orc


def ref_int_conv(x, w, strides, dilations, pads):
    """Direct convolution of integer tensors in int64: pad explicitly, gather windows, contract."""
    (pt, pb), (pl, pr) = pads
    xp = np.pad(x.astype(np.int64), ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    kh, kw, ci, co = w.shape
    eh, ew = (kh - 1) * dilations[0] + 1, (kw - 1) * dilations[1] + 1
    oh = (xp.shape[1] - eh) // strides[0] + 1
    ow = (xp.shape[2] - ew) // strides[1] + 1
    out = np.zeros((x.shape[0], oh, ow, co), np.int64)
    for i in range(kh):
        for j in range(kw):
            win = xp[:, i * dilations[0]: i * dilations[0] + (oh - 1) * strides[0] + 1: strides[0],
                     j * dilations[1]: j * dilations[1] + (ow - 1) * strides[1] + 1: strides[1], :]
            out += np.tensordot(win, w[i, j].astype(np.int64), axes=([3], [0]))
    return out


def same_pads(n, k, s, d):
    eff = (k - 1) * d + 1
    out = -(-n // s)
    need = max((out - 1) * s + eff - n, 0)
    return need // 2, need - need // 2


@pytest.mark.parametrize("x_dtype", [np.uint8, np.int8])
@pytest.mark.parametrize("shape,wshape,strides,dil,padding,explicit", [
    ((1, 6, 6, 4), (3, 3, 4, 4), (1, 1), (1, 1), orc.PAD_SAME, None),
    ((2, 7, 9, 3), (3, 3, 3, 5), (2, 2), (1, 1), orc.PAD_SAME, None),
    ((2, 8, 8, 3), (3, 3, 3, 5), (2, 2), (1, 1), orc.PAD_SAME, None),       # odd total padding: the extra row goes last
    ((1, 9, 9, 2), (3, 3, 2, 3), (1, 1), (2, 2), orc.PAD_SAME, None),       # dilation
    ((2, 7, 9, 3), (3, 2, 3, 5), (2, 1), (1, 1), orc.PAD_VALID, None),
    ((1, 5, 5, 8), (1, 1, 8, 6), (1, 1), (1, 1), orc.PAD_VALID, None),      # pointwise
    ((1, 10, 10, 3), (7, 7, 3, 4), (2, 2), (1, 1), orc.PAD_EXPLICIT, (3, 2, 1, 4)),
])
def test_integer_convolution_against_numpy(x_dtype, shape, wshape, strides, dil, padding, explicit):
    rng = np.random.default_rng(sum(shape) + sum(wshape))
    x = rng.integers(0, 256, shape).astype(np.uint8) if x_dtype == np.uint8 else rng.integers(-128, 128, shape).astype(np.int8)
    w = rng.integers(-128, 128, wshape).astype(np.int8)
    g = orc.conv_geom(shape, wshape, strides, dil, padding, explicit or (0, 0, 0, 0))
    at = orc.ConvAttrs(orc.QUINT8 if x_dtype == np.uint8 else orc.QINT8, orc.QINT32, 0, orc.ACT_NONE, 0.0)
    st, out = orc.qconv2d(at, g, x, w, None, -1.0, 1.0, np.float32([-1]), np.float32([1]))
    assert st == orc.OK
    if padding == orc.PAD_SAME:
        pads = (same_pads(shape[1], wshape[0], strides[0], dil[0]), same_pads(shape[2], wshape[1], strides[1], dil[1]))
    elif padding == orc.PAD_VALID:
        pads = ((0, 0), (0, 0))
    else:
        pads = ((explicit[0], explicit[1]), (explicit[2], explicit[3]))
    np.testing.assert_array_equal(out, ref_int_conv(x, w, strides, dil, pads))


def test_tensorflow_padding_rule_known_cases():
    import ctypes as C
    f = orc.lib().orc_conv_out_dim
    f.restype = C.c_int

    def dim(n, k, s, d, padding, before=0, after=0):
        out, lead = C.c_int64(), C.c_int64()
        st = f(C.c_int64(n), C.c_int64(k), s, d, padding, before, after, C.byref(out), C.byref(lead))
        return st, out.value, lead.value
    assert dim(6, 3, 1, 1, orc.PAD_SAME) == (orc.OK, 6, 1)
    assert dim(7, 3, 2, 1, orc.PAD_SAME) == (orc.OK, 4, 1)
    assert dim(8, 3, 2, 1, orc.PAD_SAME) == (orc.OK, 4, 0)         # one row of padding in total, placed after
    assert dim(224, 7, 2, 1, orc.PAD_SAME) == (orc.OK, 112, 2)     # ResNet stem: 2 before, 3 after
    assert dim(7, 3, 2, 1, orc.PAD_VALID) == (orc.OK, 3, 0)
    assert dim(5, 3, 1, 2, orc.PAD_VALID) == (orc.OK, 1, 0)
    assert dim(224, 7, 2, 1, orc.PAD_EXPLICIT, 3, 3) == (orc.OK, 112, 3)
    assert dim(6, 3, 1, 1, orc.PAD_SAME)[1:] == dim(6, 3, 1, 1, orc.PAD_EXPLICIT, 1, 1)[1:]


def quant_in(x, T):
    _, q, mn, mx = orc.quantize_v2(x, x.min(), x.max(), T, orc.SCALED)
    return q, float(mn[0]), float(mx[0])


def quant_filter(w):
    mn, mx = w.min(axis=(0, 1, 2)).astype(np.float32), w.max(axis=(0, 1, 2)).astype(np.float32)
    _, q, fmn, fmx = orc.quantize_v2(w, mn, mx, orc.QINT8, orc.SCALED, axis=3)
    return q, fmn, fmx


def fp32_conv(x, w):
    pads = (same_pads(x.shape[1], w.shape[0], 1, 1), same_pads(x.shape[2], w.shape[1], 1, 1))
    xp = np.pad(x.astype(np.float64), ((0, 0), pads[0], pads[1], (0, 0)))
    out = np.zeros(x.shape[:3] + (w.shape[3],))
    for i in range(w.shape[0]):
        for j in range(w.shape[1]):
            out += np.tensordot(xp[:, i:i + x.shape[1], j:j + x.shape[2], :], w[i, j].astype(np.float64), axes=([3], [0]))
    return out


@pytest.mark.parametrize("case", ["relu_requantize_u8", "bias_requantize_s8", "bias_relu_requantize_u8", "bias_dequantize",
                                  "bias_relu_dequantize_s8_in"])
def test_reference_test_pipelines_on_seeded_inputs(case):
    """testConvRelu / testConvBias / testConvBiasRelu of the reference (x [1,6,6,4] uniform, w [3,3,4,4] uniform(-2, 2),
    bias uniform(-1, 1), SAME, stride 1) and the Dequantize spellings of the new API."""
    rng = np.random.default_rng(sum(map(ord, case)))
    signed_in = case in ("bias_requantize_s8", "bias_relu_dequantize_s8_in")
    x = rng.uniform(-5.0 if signed_in else 0.0, 5.0, (1, 6, 6, 4)).astype(np.float32)
    w = rng.uniform(-2.0, 2.0, (3, 3, 4, 4)).astype(np.float32)
    b = rng.uniform(-1.0, 1.0, 4).astype(np.float32) if "bias" in case else None
    relu = "relu" in case
    ref = fp32_conv(x, w) + (b if b is not None else 0)
    if relu:
        ref = np.maximum(ref, 0)
    T_in = orc.QINT8 if signed_in else orc.QUINT8
    xq, xmn, xmx = quant_in(x, T_in)
    wq, fmn, fmx = quant_filter(w)
    g = orc.conv_geom(x.shape, w.shape)
    deq = "dequantize" in case
    t_out = orc.FLOAT if deq else (orc.QINT8 if case.endswith("s8") else orc.QUINT8)
    at = orc.ConvAttrs(T_in, t_out, orc.FLOAT if b is not None else 0, orc.ACT_RELU if relu else orc.ACT_NONE, 0.0)
    zmn, zmx = float(ref.min()), float(ref.max())
    st, out = orc.qconv2d(at, g, xq, wq, b, xmn, xmx, fmn, fmx, zmn, zmx)
    assert st == orc.OK
    if deq:
        got = out
    else:
        _, got = orc.dequantize(out, zmn, zmx, t_out, orc.SCALED)
    np.testing.assert_allclose(got, ref, rtol=0.3, atol=0.3)            # the reference test's own bar
    # tighter: 36 products, each operand off by at most half a quantization step, plus half an output step
    rx, rw = np.abs(x).max(), np.abs(w).max(axis=(0, 1, 2)).max()
    sx = rx / (127 if signed_in else 255) / 2
    sw = rw / 127 / 2
    bound = 36 * (sx * rw + sw * rx + sx * sw)
    if not deq:
        bound += max(abs(zmn), abs(zmx)) / (127 if t_out == orc.QINT8 else 255) / 2
    assert np.abs(got - ref).max() <= bound * 1.001
    assert np.abs(got - ref).max() > 0


@pytest.mark.parametrize("act", ["elu", "sigmoid"])
def test_elu_and_sigmoid_act_on_the_scaled_value(act):
    """[BiasAdd, Elu | Sigmoid, Requantize | Dequantize] (quantized_conv_ops.h:83, 86, 100, 103): the output scale -
    requantization included - is applied first, the activation (table alpha 1, post-op scale 1, :436-445) sees that
    value.  Checked against the activation-free convolution: float output = act(float output without it) in float64;
    8-bit output = sat(rne(act(v))) with v rebuilt from the activation-free float output times 127 / range_out."""
    rng = np.random.default_rng(9)
    x = rng.integers(0, 256, (1, 6, 5, 8)).astype(np.uint8)
    w = rng.integers(-127, 128, (3, 3, 8, 4)).astype(np.int8)
    bias = rng.standard_normal(4).astype(np.float32)
    fmn, fmx = np.full(4, -0.05, np.float32), np.full(4, 0.05, np.float32)
    g = orc.conv_geom(x.shape, w.shape, (1, 1), (1, 1), orc.PAD_SAME, (0, 0, 0, 0))
    code = orc.ACT_ELU if act == "elu" else orc.ACT_SIGMOID
    f = (lambda v: np.where(v > 0, v, np.expm1(v))) if act == "elu" else (lambda v: 1.0 / (1.0 + np.exp(-v)))
    _, plain = orc.qconv2d(orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.FLOAT, orc.ACT_NONE, 0.0), g, x, w, bias, 0.0, 2.0, fmn, fmx)
    st, got = orc.qconv2d(orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.FLOAT, code, 0.0), g, x, w, bias, 0.0, 2.0, fmn, fmx)
    assert st == orc.OK
    np.testing.assert_allclose(got, f(plain.astype(np.float64)), rtol=1e-6, atol=1e-7)
    r_out = 3.0
    st, q = orc.qconv2d(orc.ConvAttrs(orc.QUINT8, orc.QINT8, orc.FLOAT, code, 0.0), g, x, w, bias, 0.0, 2.0, fmn, fmx, -r_out, r_out)
    assert st == orc.OK
    v = f(plain.astype(np.float64) * (127.0 / r_out))
    want = np.clip(np.rint(v), -128, 127)
    near_tie = np.abs(v - np.floor(v) - 0.5) < 1e-3           # the float32 value may fall on the other side
    assert np.all((q == want) | near_tie) and near_tie.mean() < 0.02
    # the swish spellings are refused (the reference's table has no entry for the name the op looks up)
    st, _ = orc.qconv2d(orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.FLOAT, orc.ACT_SWISH, 0.0), g, x, w, bias, 0.0, 2.0, fmn, fmx)
    assert st == orc.UNIMPLEMENTED


def test_scales_closed_forms_and_qint32_forms():
    rng = np.random.default_rng(4)
    N = 6
    fmn = -(rng.random(N).astype(np.float32) + 0.5)
    fmx = (-fmn * np.float32(0.8)).astype(np.float32)
    rf = np.maximum(np.abs(fmn), np.abs(fmx))
    b32 = rng.integers(-2000, 2000, N).astype(np.int32)
    bf = rng.standard_normal(N).astype(np.float32)
    L = np.float32(255 * 127)
    # float output: scale = (range_in / 255) * (range_filter / 127); a qint32 bias is multiplied by range_in * range_f / L
    at = orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.QINT32, orc.ACT_NONE, 0.0)
    st, sc, sb, ep = orc.qconv_prepare(at, N, 0.0, 4.0, fmn, fmx, 0.0, 0.0, b32)
    assert st == orc.OK and ep.n_scales == N and ep.n_eltwise == 0
    np.testing.assert_array_equal(sc, (np.float32(4.0) / np.float32(255)) * (rf / np.float32(127)))
    np.testing.assert_array_equal(sb, b32.astype(np.float32) * ((np.float32(4.0) * rf) / L))
    # qint8 output from qint8 input: scale = 127 * r_in * r_f / (127 * 127 * r_out); float bias lands as b * 127 / r_out (to rounding)
    at = orc.ConvAttrs(orc.QINT8, orc.QINT8, orc.FLOAT, orc.ACT_RELU, 0.0)
    st, sc, sb, ep = orc.qconv_prepare(at, N, -3.0, 2.0, fmn, fmx, -8.0, 6.0, bf)
    assert st == orc.OK and ep.n_eltwise == 1 and ep.elt[0].alg == orc.ELT_RELU
    np.testing.assert_array_equal(sc, np.float32(127) * np.float32(3.0) * rf / (np.float32(127 * 127) * np.float32(8.0)))
    np.testing.assert_allclose(sb, bf * np.float32(127 / 8.0), rtol=3e-7)
    # qint32 output: unit scales, a qint32 bias is used as it is, a float bias is expressed in accumulator units
    at = orc.ConvAttrs(orc.QUINT8, orc.QINT32, orc.QINT32, orc.ACT_NONE, 0.0)
    st, sc, sb, _ = orc.qconv_prepare(at, N, 0.0, 4.0, fmn, fmx, 0.0, 0.0, b32)
    np.testing.assert_array_equal(sc, np.ones(N, np.float32))
    np.testing.assert_array_equal(sb, b32.astype(np.float32))
    at = orc.ConvAttrs(orc.QUINT8, orc.QINT32, orc.FLOAT, orc.ACT_NONE, 0.0)
    st, sc, sb, _ = orc.qconv_prepare(at, N, 0.0, 4.0, fmn, fmx, 0.0, 0.0, bf)
    np.testing.assert_array_equal(sb, bf * ((L / (np.float32(4.0) * rf)) * np.float32(1.0)))
    # per-tensor filter range: one scale for all channels
    at = orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.FLOAT, orc.ACT_LEAKYRELU, 0.1)
    st, sc, sb, ep = orc.qconv_prepare(at, N, 0.0, 4.0, fmn[:1], fmx[:1], 0.0, 0.0, bf)
    assert st == orc.OK and ep.n_scales == 1 and ep.elt[0].alpha == np.float32(0.1)
    st, _, _, _ = orc.qconv_prepare(at, N, 0.0, 4.0, fmn[:3], fmx[:3], 0.0, 0.0, bf)
    assert st == orc.INVALID_ARGUMENT


@pytest.mark.parametrize("t_out,t_sum,position", [(orc.QUINT8, orc.QUINT8, 1), (orc.QUINT8, orc.QINT8, 1), (orc.QINT8, orc.QINT8, 1),
                                                  (orc.QUINT8, orc.QUINT8, 2), (orc.QINT8, orc.QINT8, 2)])
def test_sum_fusion_against_an_independent_evaluation(t_out, t_sum, position):
    """[BiasAdd, Sum, Relu, Requantize] and [BiasAdd, Relu, Sum, Requantize]: the fused result equals the unfused int32
    convolution taken through the same fp32 steps in numpy (scale, bias, sum scale x summand, ReLU, saturate + round
    half to even), with the sum scale of quantized_conv_ops.h:398-433 written out here from the ranges."""
    rng = np.random.default_rng(7 + t_out + t_sum + position)
    x = rng.integers(0, 256, (2, 7, 6, 8)).astype(np.uint8)
    w = rng.integers(-127, 128, (3, 3, 8, 16)).astype(np.int8)
    bias = rng.uniform(-1, 1, 16).astype(np.float32)
    g = orc.conv_geom(x.shape, w.shape)
    min_in, max_in, min_f, max_f = 0.0, 4.0, np.float32(-0.5), np.float32(0.5)
    min_out, max_out = (0.0, 30.0) if t_out == orc.QUINT8 else (-30.0, 30.0)
    summand = (rng.integers(0, 256, (2, 7, 6, 16)).astype(np.uint8) if t_sum == orc.QUINT8
               else rng.integers(-128, 128, (2, 7, 6, 16)).astype(np.int8))
    min_s, max_s = (0.0, 12.0) if t_sum == orc.QUINT8 else (-9.0, 12.0)
    at = orc.ConvAttrs(orc.QUINT8, t_out, orc.FLOAT, orc.ACT_RELU, 0.0)
    st, got = orc.qconv2d(at, g, x, w, bias, min_in, max_in, min_f, max_f, min_out, max_out,
                          sum=orc.ConvSum(position, t_sum, min_s, max_s), summand=summand)
    assert st == orc.OK
    # independent evaluation
    st, acc = orc.qconv2d(orc.ConvAttrs(orc.QUINT8, orc.QINT32, 0, orc.ACT_NONE, 0.0), g, x, w, None, min_in, max_in, min_f, max_f)
    assert st == orc.OK
    f32 = np.float32
    lim_out = f32(255.0 if t_out == orc.QUINT8 else 127.0)
    scale = lim_out * f32(4.0) * f32(0.5) / (f32(255.0 * 127.0) * f32(30.0))
    bias_scaled = bias * (f32(255.0 * 127.0) / (f32(4.0) * f32(0.5)) * scale)
    s_out, s_sum = f32(30.0), f32(12.0)
    sum_scale = f32(255.0) * s_sum / (s_out * f32(127.0)) if (t_out == orc.QUINT8 and t_sum == orc.QINT8) else s_sum / s_out
    prev = summand.view(np.uint8 if t_out == orc.QUINT8 else np.int8).astype(np.float32)   # read as the output type
    y = acc.astype(np.float32) * scale + bias_scaled
    if position == 1:
        y = np.maximum(y + sum_scale * prev, f32(0))
    else:
        y = np.maximum(y, f32(0)) + sum_scale * prev
    lo, hi = (0, 255) if t_out == orc.QUINT8 else (-128, 127)
    ref = np.clip(np.rint(y), lo, hi).astype(got.dtype)
    np.testing.assert_array_equal(got, ref)
    assert len(np.unique(got)) > 20          # not saturated away


def test_sum_fusion_type_rules():
    x = np.zeros((1, 4, 4, 4), np.uint8)
    w = np.zeros((1, 1, 4, 4), np.int8)
    g = orc.conv_geom(x.shape, w.shape)
    s = np.zeros((1, 4, 4, 4), np.uint8)
    run = lambda t_out, t_sum: orc.qconv2d(orc.ConvAttrs(orc.QUINT8, t_out, 0, orc.ACT_RELU, 0.0), g, x, w, None, 0.0, 1.0,
                                           np.float32(-1), np.float32(1), -1.0, 1.0, sum=orc.ConvSum(1, t_sum, 0.0, 1.0),
                                           summand=s)[0]
    assert run(orc.QINT8, orc.QUINT8) == orc.INVALID_ARGUMENT      # quantized_conv_ops.h:213-218
    assert run(orc.QINT32, orc.QUINT8) == orc.UNIMPLEMENTED        # the qint32 form takes a float summand: not restated
    assert run(orc.QUINT8, orc.QINT8) == orc.OK


@pytest.mark.parametrize("x_dtype", [np.uint8, np.int8])
@pytest.mark.parametrize("shape,kshape,strides,dil", [((2, 7, 6, 8), (3, 3, 8, 1), (1, 1), (1, 1)), ((1, 9, 9, 5), (3, 3, 5, 2), (2, 2), (1, 1)),
                                                      ((1, 8, 8, 4), (5, 3, 4, 3), (1, 2), (2, 1))])
def test_depthwise_integer_convolution_against_numpy(x_dtype, shape, kshape, strides, dil):
    """Depthwise: output channel c * mult + m is the plain convolution of input channel c with filter w[:, :, c, m]; checked
    channel by channel against the independent numpy evaluation used for the full convolution."""
    rng = np.random.default_rng(sum(shape) + sum(kshape))
    info = np.iinfo(x_dtype)
    x = rng.integers(info.min, info.max + 1, shape).astype(x_dtype)
    w = rng.integers(-127, 128, kshape).astype(np.int8)
    g = orc.conv_geom(shape, (kshape[0], kshape[1], kshape[2], kshape[2] * kshape[3]), strides, dil)
    T_in = orc.QUINT8 if x_dtype == np.uint8 else orc.QINT8
    st, got = orc.qdepthwise_conv2d(orc.ConvAttrs(T_in, orc.QINT32, 0, orc.ACT_NONE, 0.0), g, x, w, None, -1.0, 1.0,
                                    np.float32([-1]), np.float32([1]))
    assert st == orc.OK
    pads = (same_pads(shape[1], kshape[0], strides[0], dil[0]), same_pads(shape[2], kshape[1], strides[1], dil[1]))
    C_, mult = kshape[2], kshape[3]
    assert got.shape[3] == C_ * mult
    for c in range(C_):
        for m in range(mult):
            ref = ref_int_conv(x[..., c:c + 1], w[:, :, c:c + 1, m:m + 1], strides, dil, pads)
            np.testing.assert_array_equal(got[..., c * mult + m], ref[..., 0])


def test_depthwise_scales_follow_the_output_channel():
    """Per-channel filter ranges: entry c * mult + m scales output channel c * mult + m (same prepare as the full
    convolution with in_c * mult channels)."""
    rng = np.random.default_rng(3)
    x = rng.integers(0, 256, (1, 5, 5, 3)).astype(np.uint8)
    w = rng.integers(-127, 128, (3, 3, 3, 2)).astype(np.int8)
    g = orc.conv_geom(x.shape, (3, 3, 3, 6))
    mn, mx = -np.arange(1, 7, dtype=np.float32), np.arange(1, 7, dtype=np.float32)
    at = orc.ConvAttrs(orc.QUINT8, orc.FLOAT, 0, orc.ACT_NONE, 0.0)
    st, got = orc.qdepthwise_conv2d(at, g, x, w, None, 0.0, 2.0, mn, mx)
    st2, acc = orc.qdepthwise_conv2d(orc.ConvAttrs(orc.QUINT8, orc.QINT32, 0, orc.ACT_NONE, 0.0), g, x, w, None, 0.0, 2.0, mn, mx)
    assert st == orc.OK and st2 == orc.OK
    scale = (np.float32(2.0) / np.float32(255.0)) * (mx / np.float32(127.0))
    np.testing.assert_array_equal(got, acc.astype(np.float32) * scale)
