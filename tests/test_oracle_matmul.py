"""Pins the CPU oracle's quantized MatMul restatement.

  * integer GEMM: brute force against numpy int64 (exact);
  * MIN_FIRST zero-point compensation and the output scale: the reference-held 2x3 . 3x4 case of
    native_quantized_fused_matmul_test.py must reproduce the fp32 product within the reference's own
    tolerance (0.2) and, tighter, within the bound the quantization steps allow -- a dropped or
    sign-flipped compensation term misses by > 1;
  * requantize scaling: dequantizing the int8 output with the frozen range must reproduce the fp32
    product to half an output step (+ input quantization noise);
  * the documented quirks (bias inflation for SCALED input, lost requantize factor behind an
    activation) are asserted through their observable consequence, not by retyping the formula;
  * epilogue order against the oneDNN bundled in PyTorch (skipped if that op is unavailable).
"""
import numpy as np
import pytest

from oracle import pyoracle as orc


def quant_weights_per_channel(w):
    r = np.max(np.abs(w), axis=0).astype(np.float32)
    _, q, mn, mx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    return q, mn, mx


def quant_weights_per_tensor(w):
    _, q, mn, mx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
    return q, mn, mx


@pytest.mark.parametrize("a_dtype", [np.uint8, np.int8])
@pytest.mark.parametrize("transpose_b", [False, True])
def test_int_gemm_brute_force(a_dtype, transpose_b):
    rng = np.random.default_rng(0)
    for (M, K, N) in [(1, 1, 1), (3, 17, 5), (16, 64, 48), (7, 129, 33)]:
        info = np.iinfo(a_dtype)
        a = rng.integers(info.min, info.max + 1, size=(M, K)).astype(a_dtype)
        w = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
        ref = a.astype(np.int64) @ w.astype(np.int64)
        got = orc.int_gemm(a, np.ascontiguousarray(w.T) if transpose_b else w, transpose_b)
        np.testing.assert_array_equal(got.astype(np.int64), ref)
    # extreme values: no overflow at the largest K of the configs
    K = 14336
    a = np.full((1, K), 255, np.uint8)
    w = np.full((K, 2), -128, np.int8)
    w[:, 1] = 127
    got = orc.int_gemm(a, w)
    assert got.tolist() == [[255 * -128 * K, 255 * 127 * K]]


def test_colsum():
    rng = np.random.default_rng(1)
    w = rng.integers(-128, 128, size=(300, 37)).astype(np.int8)
    np.testing.assert_array_equal(orc.weight_colsum(w), w.astype(np.int64).sum(0))


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("api", [orc.API_V1, orc.API_V2])
def test_reference_fused_matmul_case(golden, per_channel, api):
    g = golden["fused_matmul"]
    x = np.array(g["x"], np.float32)
    w = np.array(g["w"], np.float32)
    b = np.array(g["bias"], np.float32)
    st, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    assert xq.tolist() == [[218, 180, 0], [146, 165, 255]]
    if per_channel:
        # the reference test quantizes with (min, max) per column, axis=1
        _, wq, wmn, wmx = orc.quantize_v2(w, w.min(0), w.max(0), orc.QINT8, orc.SCALED, axis=1)
    else:
        wq, wmn, wmx = quant_weights_per_tensor(w)
    at = orc.matmul_attrs(api=api, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST,
                          has_dequantize=True, n_fused_ops=1)
    st, y = orc.qmatmul(at, xq, wq, b, xmn[0], xmx[0], wmn, wmx)
    assert st == orc.OK
    ref = x @ w + b
    err = np.max(np.abs(y - ref))
    assert err < g["tolerance"]
    # quantization-noise bound: K * (step_x/2 * |w|max + step_w/2 * |x|max) is ~0.1 here
    assert err < 0.06
    # a missing compensation term would be off by about |min_a| * colsum(w) ~ 1
    assert np.max(np.abs(y - ref)) < 0.1 * np.max(np.abs(0.66 * w.sum(0)))


def test_requantize_output_scale_round_trip():
    rng = np.random.default_rng(4)
    M, K, N = 32, 256, 48
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    b = (rng.standard_normal(N) * 0.1).astype(np.float32)
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    wq, wmn, wmx = quant_weights_per_channel(w)
    ref = x @ w + b
    r_out = float(np.max(np.abs(ref)))
    for api in (orc.API_V1, orc.API_V2):
        at = orc.matmul_attrs(api=api, t_in=orc.QUINT8, t_out=orc.QINT8, input_mode=orc.MIN_FIRST,
                              has_requantize=True, n_fused_ops=1)
        st, q = orc.qmatmul(at, xq, wq, b, xmn[0], xmx[0], wmn, wmx, -r_out, r_out)
        assert st == orc.OK
        st, y = orc.dequantize(q, -r_out, r_out, orc.QINT8, orc.SCALED)
        assert np.max(np.abs(y - ref)) < 0.5 * r_out / 127 + 0.08
        st, omn, omx = orc.qmatmul_output_minmax(at, xmn[0], xmx[0], wmn, wmx, 1, -r_out, r_out)
        assert (omn[0], omx[0]) == (np.float32(-r_out), np.float32(r_out))


def test_s32_output_range_and_values():
    rng = np.random.default_rng(9)
    M, K, N = 4, 64, 8
    xq = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    zero_bias = np.zeros(N, np.float32)
    # SCALED input + zero bias: the s32 output is the accumulator (|acc| < 2^24 here -> exact)
    at = orc.matmul_attrs(api=orc.API_V1, t_in=orc.QUINT8, t_out=orc.QINT32, input_mode=orc.SCALED,
                          n_fused_ops=1)
    st, y = orc.qmatmul(at, xq, wq, zero_bias, 0.0, 2.0, [-1.0], [1.0])
    np.testing.assert_array_equal(y, xq.astype(np.int64) @ wq.astype(np.int64))
    st, omn, omx = orc.qmatmul_output_minmax(at, 0.0, 2.0, [-1.0], [1.0], 0, 0, 0)
    lvl = np.float32(np.float32(2.0) / np.float32(255)) * np.float32(np.float32(2.0) / np.float32(254))
    assert omn[0] == np.float32(lvl * np.float32(-2**31)) and omx[0] == np.float32(lvl * np.float32(2**31))
    st, omn, omx = orc.qmatmul_output_minmax(at, 0.0, 2.0, [-1.0] * N, [1.0] * N, 1, 0, 0)
    assert omn.size == N


def test_quirk_scaled_input_inflates_bias():
    # SCALED input + fp32 bias: bias is multiplied by A*127/(r_in*r_w) (oneDNN-2.x-era scaling) while
    # the primitive adds it after scaling.  Observable: doubling the bias moves the fp32 output by
    # bias * bs, not by bias.
    rng = np.random.default_rng(6)
    M, K, N = 4, 32, 8
    xq = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    b = rng.standard_normal(N).astype(np.float32)
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QINT8, t_out=orc.FLOAT, input_mode=orc.SCALED,
                          has_dequantize=True)
    _, y0 = orc.qmatmul(at, xq, wq, np.zeros(N, np.float32), -2.0, 2.0, [-0.5], [0.5])
    _, y1 = orc.qmatmul(at, xq, wq, b, -2.0, 2.0, [-0.5], [0.5])
    bs = 127.0 * 127.0 / (2.0 * 0.5)
    np.testing.assert_allclose(y1 - y0, np.broadcast_to(b * bs, (M, N)), rtol=1e-4, atol=1e-2)
    # per-channel weights: the single scale bs[0] applies to every channel
    mb = np.linspace(0.25, 1.0, N).astype(np.float32)
    _, z0 = orc.qmatmul(at, xq, wq, np.zeros(N, np.float32), -2.0, 2.0, -mb, mb)
    _, z1 = orc.qmatmul(at, xq, wq, b, -2.0, 2.0, -mb, mb)
    bs0 = 127.0 * 127.0 / (2.0 * 0.25)
    np.testing.assert_allclose(z1 - z0, np.broadcast_to(b * bs0, (M, N)), rtol=1e-4, atol=1e-2)


def test_quirk_activation_drops_requantize_factor():
    # [BiasAdd, Relu, Requantize]: the 255/r_out factor is lost, the u8 output is relu(y) in real
    # units (saturated), while [BiasAdd, Requantize] applies it.
    rng = np.random.default_rng(8)
    M, K, N = 8, 64, 16
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.3).astype(np.float32)
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    wq, wmn, wmx = quant_weights_per_channel(w)
    zero = np.zeros(N, np.float32)
    ref = np.maximum(x @ w, 0)
    r_out = float(ref.max())
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST,
                          activation=orc.ACT_RELU, has_requantize=True, n_fused_ops=2)
    _, q = orc.qmatmul(at, xq, wq, zero, xmn[0], xmx[0], wmn, wmx, 0.0, r_out)
    assert np.max(np.abs(q.astype(np.float32) - np.clip(np.rint(ref), 0, 255))) <= 1
    at1 = orc.matmul_attrs(api=orc.API_V1, t_in=orc.QUINT8, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST,
                           activation=orc.ACT_RELU, has_requantize=True, n_fused_ops=2)
    _, q1 = orc.qmatmul(at1, xq, wq, zero, xmn[0], xmx[0], wmn, wmx, 0.0, r_out)
    np.testing.assert_array_equal(q, q1)
    # legacy QuantizedMatMulWithBiasAndReluAndRequantize is not affected (factor lives in the output scale)
    wq1, wmn1, wmx1 = quant_weights_per_tensor(w)
    atl = orc.matmul_attrs(api=orc.API_LEGACY, t_in=orc.QUINT8, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST,
                           activation=orc.ACT_RELU)
    _, ql = orc.qmatmul(atl, xq, wq1, zero, xmn[0], xmx[0], wmn1, wmx1, 0.0, r_out)
    _, yl = orc.dequantize(ql, 0.0, r_out, orc.QUINT8, orc.SCALED)
    # legacy scale uses (max_b-min_b)/254 and (max_a-min_a)/255 levels: a close, not identical, grid
    assert np.max(np.abs(yl - ref)) < 0.03 * r_out + 0.1


def test_min_first_output_linear_overrides_relu_alpha():
    # output_quant_mode=MIN_FIRST + Requantize appends Linear and its alpha/beta overwrite EVERY
    # eltwise in the chain (onednn_post_op_util.cc:251-262)
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST,
                          out_min_first=True, activation=orc.ACT_RELU, has_requantize=True)
    st, sc, sb, ep = orc.qmatmul_prepare(at, 2, [0, 0], 0.0, 1.0, [-1.0], [1.0], -1.0, 3.0, [0.0, 0.0])
    assert ep.n_eltwise == 2
    alpha = np.float32(255.0) / np.float32(4.0)
    beta = np.float32(np.float32(1.0) * np.float32(255.0)) / np.float32(4.0)
    for e in range(2):
        assert ep.elt[e].alpha == alpha and ep.elt[e].beta == beta
    # the output scale carries no requantize factor in that case
    assert sc[0] == np.float32(np.float32(1.0) * np.float32(1.0)) / np.float32(255.0 * 127.0)


def test_epilogue_rounding_and_saturation():
    ep = orc.EpilogueDesc()
    ep.n_scales = 1
    acc = np.array([[1, 3, 5, 7, -1, -3, 600, -600, 2**31 - 1, -2**31]], np.int32)
    out = orc.qmatmul_epilogue(acc, ep, [0.5], np.zeros(10, np.float32), orc.QINT8)
    assert out.tolist() == [[0, 2, 2, 4, 0, -2, 127, -128, 127, -128]]
    out = orc.qmatmul_epilogue(acc, ep, [0.5], np.zeros(10, np.float32), orc.QUINT8)
    assert out.tolist() == [[0, 2, 2, 4, 0, 0, 255, 0, 255, 0]]
    # s32 destination goes through fp32: 2^31-1 -> 2^31 in fp32 -> saturates to 2147483520
    out = orc.qmatmul_epilogue(acc, ep, [1.0], np.zeros(10, np.float32), orc.QINT32)
    assert out[0, 8] == 2147483520 and out[0, 9] == -2**31 and out[0, 6] == 600


def test_epilogue_mul_then_add_not_fused():
    # pick acc, s, b so that fl(fl(acc*s)+b) != fl(acc*s+b)
    rng = np.random.default_rng(12)
    acc = rng.integers(-2**23, 2**23, size=(1, 4096)).astype(np.int32)
    s = np.float32(0.00123457)
    b = rng.standard_normal(4096).astype(np.float32)
    ep = orc.EpilogueDesc()
    ep.n_scales = 1
    out = orc.qmatmul_epilogue(acc, ep, [s], b, orc.FLOAT)
    two_step = ((acc.astype(np.float64) * np.float64(s)).astype(np.float32).astype(np.float64) + b).astype(np.float32)
    fused = (acc.astype(np.float64) * np.float64(s) + b).astype(np.float32)
    assert np.any(two_step != fused)
    np.testing.assert_array_equal(out, two_step)


def test_epilogue_against_torch_onednn():
    """oneDNN 3.x as bundled with PyTorch (a different build than the reference pins; a cross-check
    of operation order, rounding and saturation, not the definition)."""
    torch = pytest.importorskip("torch")
    if not hasattr(torch.ops, "onednn") or not hasattr(torch.ops.onednn, "qlinear_pointwise"):
        pytest.skip("torch.ops.onednn.qlinear_pointwise unavailable")
    rng = np.random.default_rng(13)
    M, K, N = 16, 64, 32
    xq = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    sw = (rng.random(N).astype(np.float32) * 0.01 + 0.001)
    b = rng.standard_normal(N).astype(np.float32)
    try:
        w_t = torch.from_numpy(np.ascontiguousarray(wq.T))  # [N, K]
        packed = torch.ops.onednn.qlinear_prepack(w_t, [M, K])
        outs = {}
        for post, out_dtype in (("none", torch.float32), ("relu", torch.float32), ("none", torch.uint8)):
            outs[(post, out_dtype)] = torch.ops.onednn.qlinear_pointwise(
                torch.from_numpy(xq), 1.0, 0, packed, torch.from_numpy(sw),
                torch.zeros(N, dtype=torch.int64), torch.from_numpy(b), 1.0, 0, out_dtype, post, [], "")
    except Exception as e:  # signature differs between torch builds
        pytest.skip("qlinear_pointwise not callable here: %r" % (e,))
    acc = orc.int_gemm(xq, wq)
    ep = orc.EpilogueDesc()
    ep.n_scales = N
    np.testing.assert_array_equal(outs[("none", torch.float32)].numpy(),
                                  orc.qmatmul_epilogue(acc, ep, sw, b, orc.FLOAT))
    np.testing.assert_array_equal(outs[("none", torch.uint8)].numpy(),
                                  orc.qmatmul_epilogue(acc, ep, sw, b, orc.QUINT8))
    ep.n_eltwise = 1
    ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = 1, 0.0, 0.0
    np.testing.assert_array_equal(outs[("relu", torch.float32)].numpy(),
                                  orc.qmatmul_epilogue(acc, ep, sw, b, orc.FLOAT))


@pytest.mark.parametrize("post", ["sum", "add"])
def test_sum_and_binary_add_post_ops_against_torch_onednn(post):
    """The "Add" fusion (a sum post-op in the MatMul, a binary add in the BatchMatMul) in the oneDNN bundled with
    PyTorch: one more separately rounded fp32 addition after scale and bias, bit for bit the oracle's result."""
    torch = pytest.importorskip("torch")
    if not hasattr(torch.ops, "onednn") or not hasattr(torch.ops.onednn, "qlinear_pointwise"):
        pytest.skip("torch.ops.onednn.qlinear_pointwise unavailable")
    rng = np.random.default_rng(7)
    M, K, N = 32, 64, 48
    xq = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    sw = (rng.random(N).astype(np.float32) * 0.01 + 0.001)
    b = rng.standard_normal(N).astype(np.float32)
    other = rng.standard_normal((M, N)).astype(np.float32)
    try:
        packed = torch.ops.onednn.qlinear_prepack(torch.from_numpy(np.ascontiguousarray(wq.T)), [M, K])
        y = torch.ops.onednn.qlinear_pointwise.binary(torch.from_numpy(xq), 1.0, 0, packed, torch.from_numpy(sw),
                                                      torch.zeros(N, dtype=torch.int64), torch.from_numpy(other.copy()),
                                                      torch.from_numpy(b), 1.0, 0, torch.float32, 1.0, 0, post, 1.0, "none", [], "")
    except Exception as e:
        pytest.skip("qlinear_pointwise.binary not callable here: %r" % (e,))
    ep = orc.EpilogueDesc()
    ep.n_scales, ep.n_eltwise = N, 1
    ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = orc.ELT_SUM, 1.0, 0.0
    np.testing.assert_array_equal(y.numpy(), orc.qmatmul_epilogue(orc.int_gemm(xq, wq), ep, sw, b, orc.FLOAT, addend=other))


@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_16_bit_outputs_against_torch_onednn(T16):
    """bfloat16 / half destination of an int8 inner product in the oneDNN bundled with PyTorch: the fp32 epilogue
    result narrowed with round-to-nearest-even, bit for bit what the oracle stores."""
    torch = pytest.importorskip("torch")
    if not hasattr(torch.ops, "onednn") or not hasattr(torch.ops.onednn, "qlinear_pointwise"):
        pytest.skip("torch.ops.onednn.qlinear_pointwise unavailable")
    rng = np.random.default_rng(5)
    M, K, N = 64, 64, 64
    xq = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    sw = (rng.random(N).astype(np.float32) * 0.01 + 0.001)
    b = rng.standard_normal(N).astype(np.float32)
    try:
        packed = torch.ops.onednn.qlinear_prepack(torch.from_numpy(np.ascontiguousarray(wq.T)), [M, K])
        y = torch.ops.onednn.qlinear_pointwise(torch.from_numpy(xq), 1.0, 0, packed, torch.from_numpy(sw),
                                               torch.zeros(N, dtype=torch.int64), torch.from_numpy(b), 1.0, 0,
                                               torch.bfloat16 if T16 == orc.BFLOAT16 else torch.float16, "none", [], "")
    except Exception as e:
        pytest.skip("qlinear_pointwise with a 16-bit output not callable here: %r" % (e,))
    ep = orc.EpilogueDesc()
    ep.n_scales = N
    np.testing.assert_array_equal(y.view(torch.int16).numpy().view(np.uint16),
                                  orc.qmatmul_epilogue(orc.int_gemm(xq, wq), ep, sw, b, T16))


@pytest.mark.parametrize("algo,alg", [("tanh", orc.ELT_GELU_TANH), ("none", orc.ELT_GELU_ERF)])
def test_gelu_post_ops_against_torch_onednn(algo, alg):
    """The GELU post-ops are the one place where the oracle (libm tanhf / erff) cannot claim oneDNN's bits: oneDNN
    evaluates them with its own polynomial kernels.  Against the oneDNN bundled with PyTorch (3.x, another build than
    the reference pins) the oracle agrees on more than 90 % of the elements bit for bit and everywhere to 1e-6
    absolute - the tolerance the GPU tests use for these two post-ops."""
    torch = pytest.importorskip("torch")
    if not hasattr(torch.ops, "onednn") or not hasattr(torch.ops.onednn, "qlinear_pointwise"):
        pytest.skip("torch.ops.onednn.qlinear_pointwise unavailable")
    rng = np.random.default_rng(13)
    M, K, N = 64, 64, 64
    xq = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    sw = (rng.random(N).astype(np.float32) * 0.0005 + 0.00005)      # pre-activations spread over about [-100, 100]
    b = (rng.standard_normal(N) * 0.5).astype(np.float32)
    try:
        packed = torch.ops.onednn.qlinear_prepack(torch.from_numpy(np.ascontiguousarray(wq.T)), [M, K])
        y = torch.ops.onednn.qlinear_pointwise(torch.from_numpy(xq), 1.0, 0, packed, torch.from_numpy(sw),
                                               torch.zeros(N, dtype=torch.int64), torch.from_numpy(b), 1.0, 0, torch.float32,
                                               "gelu", [], algo).numpy()
    except Exception as e:
        pytest.skip("qlinear_pointwise with a gelu post-op not callable here: %r" % (e,))
    ep = orc.EpilogueDesc()
    ep.n_scales, ep.n_eltwise = N, 1
    ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = alg, 0.0, 0.0
    ref = orc.qmatmul_epilogue(orc.int_gemm(xq, wq), ep, sw, b, orc.FLOAT)
    np.testing.assert_allclose(y, ref, rtol=0, atol=1e-6)
    assert (y.view(np.int32) == ref.view(np.int32)).mean() > 0.9


# ------------------------------------------------------------------------------------------------
# "Add" (sum post-op), GELU post-ops and the qint32 bias
# ------------------------------------------------------------------------------------------------
def _toy(seed=0, M=7, K=48, N=12):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
    _, xq, mn, mx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    r = np.abs(w).max(0).astype(np.float32)
    _, wq, wmn, wmx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    return x, w, xq, float(mn[0]), float(mx[0]), wq, wmn, wmx


def test_add_post_op_is_a_separately_rounded_fp32_add_in_fused_ops_order():
    x, w, xq, mn, mx, wq, wmn, wmx = _toy()
    M, N = x.shape[0], w.shape[1]
    rng = np.random.default_rng(1)
    bias = rng.standard_normal(N).astype(np.float32)
    z = (rng.standard_normal((M, N)) * 3).astype(np.float32)
    base = orc.matmul_attrs(t_out=orc.FLOAT, has_dequantize=True)
    _, y0 = orc.qmatmul(base, xq, wq, bias, mn, mx, wmn, wmx)
    for pos, act in ((1, orc.ACT_NONE), (1, orc.ACT_RELU), (2, orc.ACT_RELU)):
        at = orc.matmul_attrs(t_out=orc.FLOAT, has_dequantize=True, activation=act, add_position=pos)
        st, y = orc.qmatmul(at, xq, wq, bias, mn, mx, wmn, wmx, addend=z)
        assert st == orc.OK
        if act == orc.ACT_NONE:
            expect = y0 + z                              # one fp32 add on the rounded pre-add value
        elif pos == 1:
            expect = np.maximum(y0 + z, np.float32(0))   # [BiasAdd, Add, Relu]
        else:
            expect = np.maximum(y0, np.float32(0)) + z   # [BiasAdd, Relu, Add]
        np.testing.assert_array_equal(y, expect.astype(np.float32))
    # the two orders differ wherever relu clips
    # a quantized addend does not exist upstream: refused, like a missing addend
    at = orc.matmul_attrs(t_out=orc.QINT8, has_requantize=True, add_position=1)
    assert orc.qmatmul(at, xq, wq, bias, mn, mx, wmn, wmx, -1.0, 1.0, addend=z)[0] == orc.UNIMPLEMENTED
    at = orc.matmul_attrs(t_out=orc.FLOAT, has_dequantize=True, add_position=1)
    assert orc.qmatmul(at, xq, wq, bias, mn, mx, wmn, wmx)[0] == orc.INVALID_ARGUMENT


def test_reference_add_post_op_constants(golden):
    """The constants of the reference's _testAddPostop (native_quantized_fused_matmul_test.py:141-193):
    [BiasAdd, Add, Dequantize] within its own tolerance of the fp32 graph."""
    g = golden["fused_matmul"]
    x, w, b = (np.array(g[k], np.float32) for k in ("x", "w", "bias"))
    z = np.array(golden["fused_matmul_addend"], np.float32) * 2     # the test doubles it (z + z)
    _, xq, mn, mx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    _, wq, wmn, wmx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
    for api in (orc.API_V1, orc.API_V2):
        at = orc.matmul_attrs(api=api, t_out=orc.FLOAT, has_dequantize=True, add_position=1, n_fused_ops=2)
        st, y = orc.qmatmul(at, xq, wq, b, mn[0], mx[0], wmn, wmx, addend=z)
        assert st == orc.OK
        np.testing.assert_allclose(y, x @ w + b + z, rtol=g["tolerance"], atol=g["tolerance"])


@pytest.mark.parametrize("act,fn", [
    (orc.ACT_GELU_APPROX, lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))),
    (orc.ACT_GELU_EXACT, lambda v: 0.5 * v * (1 + np.vectorize(__import__("math").erf)(v / np.sqrt(2))))])
def test_gelu_post_ops_against_float64(act, fn):
    """Bit-level parity with oneDNN's own tanh / erf kernels is unpinned; the formula is pinned against a
    float64 evaluation, at 0 and in both tails."""
    x, w, xq, mn, mx, wq, wmn, wmx = _toy(seed=2, M=40, K=64, N=24)
    bias = np.linspace(-3, 3, 24).astype(np.float32)
    base = orc.matmul_attrs(t_out=orc.FLOAT, has_dequantize=True)
    _, y0 = orc.qmatmul(base, xq, wq, bias, mn, mx, wmn, wmx)
    at = orc.matmul_attrs(t_out=orc.FLOAT, has_dequantize=True, activation=act)
    st, y = orc.qmatmul(at, xq, wq, bias, mn, mx, wmn, wmx)
    assert st == orc.OK
    np.testing.assert_allclose(y, fn(y0.astype(np.float64)), rtol=2e-6, atol=2e-7)
    ep = orc.EpilogueDesc()
    ep.n_eltwise = 1
    ep.elt[0].alg = 4 if act == orc.ACT_GELU_APPROX else 5
    acc = np.array([[0, 1 << 20, -(1 << 20), 3, -3]], np.int32)
    out = orc.qmatmul_epilogue(acc, ep, np.zeros(1, np.float32), np.zeros(5, np.float32), orc.FLOAT)
    assert out[0, 0] == 0 and out[0, 1] == np.float32(1 << 20) and abs(out[0, 2]) == 0
    assert 2.99 < out[0, 3] < 3 and -0.01 < out[0, 4] < 0


@pytest.mark.parametrize("mode", [orc.MIN_FIRST, orc.SCALED])
@pytest.mark.parametrize("t_out", [orc.FLOAT, orc.QINT8, orc.QINT32])
@pytest.mark.parametrize("per_channel", [True, False])
def test_qint32_bias_closed_forms(mode, t_out, per_channel):
    """Tbias = qint32: the bias is cast to fp32 and multiplied by the inverse of the fp32 path's factor;
    no zero-point compensation (quantized_matmul_common.h:1204-1271)."""
    N = 9
    rng = np.random.default_rng(3)
    b = rng.integers(-5000, 5000, N).astype(np.int32)
    wmn = -(rng.random(N if per_channel else 1).astype(np.float32) + 0.5)
    wmx = -wmn * np.float32(0.9)
    colsum = rng.integers(-999, 999, N).astype(np.int32)
    min_a, max_a = np.float32(-1.25), np.float32(2.5)
    at = orc.matmul_attrs(t_in=orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8, t_out=t_out, input_mode=mode,
                          has_dequantize=t_out == orc.FLOAT, has_requantize=t_out == orc.QINT8, t_bias=orc.QINT32)
    st, scales, sb, ep = orc.qmatmul_prepare(at, N, colsum, min_a, max_a, wmn, wmx, -3.0, 3.0, b)
    assert st == orc.OK
    A = np.float32(255 if mode == orc.MIN_FIRST else 127)
    r_in = (max_a - min_a) if mode == orc.MIN_FIRST else np.float32(2.5)
    r_w = np.maximum(np.abs(wmn), np.abs(wmx))
    bs = np.broadcast_to(((r_in * r_w) / (A * np.float32(127))).astype(np.float32), (N,))
    bf = b.astype(np.float32)
    if mode == orc.SCALED or t_out == orc.FLOAT:
        expect = bf * bs
    elif t_out == orc.QINT8:
        expect = bf * np.broadcast_to(scales, (N,))
    else:
        expect = bf
    np.testing.assert_array_equal(sb, expect.astype(np.float32))


def _bf16_rne(x, T=orc.BFLOAT16):
    """fp32 -> bfloat16 (or half) bit patterns by PyTorch's / numpy's conversion (round to nearest even), independent
    of the oracle's."""
    import torch
    if T == orc.HALF:
        with np.errstate(over="ignore"):
            return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def _widen(bits, T=orc.BFLOAT16):
    if T == orc.HALF:
        return bits.view(np.float16).astype(np.float32)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_half_conversion_of_the_epilogue_over_the_whole_exponent_range():
    """The oracle's own fp32 -> half rounding (normals, denormals, ties, overflow to infinity) against numpy's."""
    rng = np.random.default_rng(0)
    acc = rng.integers(-2**31, 2**31, (64, 512)).astype(np.int32)
    acc[0, :8] = [65504, 65519, 65520, 65536, -65520, 1, 3, 0]
    ep = orc.EpilogueDesc(1, 0)
    for k in range(0, 60, 3):
        sc = np.float32(2.0 ** -k)
        out = orc.qmatmul_epilogue(acc, ep, np.float32([sc]), np.zeros(512, np.float32), orc.HALF)
        with np.errstate(over="ignore"):
            np.testing.assert_array_equal(out, _bf16_rne(acc.astype(np.float32) * sc, orc.HALF))



@pytest.mark.parametrize("api,kw", [(orc.API_V2, dict(has_dequantize=True)), (orc.API_V2, dict(has_dequantize=True, activation=orc.ACT_RELU)),
                                    (orc.API_V1, dict(n_fused_ops=1)), (orc.API_LEGACY, {})])
@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_bfloat16_output_is_the_rounded_float_output(api, kw, T16):
    """Tout = bfloat16 follows the float branches of the parameter preparation (:577, 1478-1479) and differs from
    Tout = float only in the destination conversion: nearest-even bfloat16 of the same fp32 value."""
    rng = np.random.default_rng(12)
    M, K, N = 33, 96, 50
    a = rng.integers(0, 256, (M, K)).astype(np.uint8)
    w = rng.integers(-127, 128, (K, N)).astype(np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    args = (a, w, bias, -1.5, 2.5, np.float32([-0.7]), np.float32([0.7]), -30.0, 30.0)
    st, y32 = orc.qmatmul(orc.matmul_attrs(api=api, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, **kw), *args)
    assert st == orc.OK
    st, y16 = orc.qmatmul(orc.matmul_attrs(api=api, t_in=orc.QUINT8, t_out=T16, input_mode=orc.MIN_FIRST, **kw), *args)
    assert st == orc.OK and y16.dtype == np.uint16
    np.testing.assert_array_equal(y16, _bf16_rne(y32, T16))
    assert _widen(y16, T16).tolist() != y32.tolist()  # the rounding is not a no-op here


def test_bfloat16_output_ties_round_to_even():
    """Epilogue alone on accumulators whose fp32 results sit exactly between two bfloat16 values."""
    acc = np.int32([[257, 259, 65536 + 128, 65536 + 384, -257, -259]])   # 1 + 2^-8 -> tie, 1 + 3*2^-8 -> tie, ...
    ep = orc.EpilogueDesc(1, 0)
    out = orc.qmatmul_epilogue(acc, ep, np.float32([1.0 / 256]), np.zeros(6, np.float32), orc.BFLOAT16)
    np.testing.assert_array_equal(out, _bf16_rne(acc.astype(np.float32) / 256))
    f = (out.astype(np.uint32) << 16).view(np.float32)[0]
    assert f[0] == 1.0 and f[1] == 1.015625 and f[4] == -1.0 and f[5] == -1.015625


@pytest.mark.parametrize("mode", [orc.MIN_FIRST, orc.SCALED])
@pytest.mark.parametrize("t_out", [orc.FLOAT, orc.QINT8, orc.QINT32])
@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_bfloat16_bias_is_adjusted_in_fp32_and_stored_as_bfloat16(mode, t_out, T16):
    """Tbias = bfloat16: GetScaledBias widens each entry, computes as for fp32 and stores the adjusted bias in
    Tbias again (quantized_matmul_common.h:578-599, 609-617) - so it equals the nearest-even bfloat16 of what the
    fp32 path gives for the widened bias."""
    N = 40
    rng = np.random.default_rng(8)
    b16 = _bf16_rne(rng.standard_normal(N).astype(np.float32), T16)
    b32 = _widen(b16, T16)
    wmn = -(rng.random(N).astype(np.float32) + 0.5)
    wmx = -wmn
    colsum = rng.integers(-999, 999, N).astype(np.int32)
    kw = dict(t_in=orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8, t_out=t_out, input_mode=mode,
              api=orc.API_V2 if t_out != orc.QINT32 else orc.API_V1, n_fused_ops=1,
              has_dequantize=t_out == orc.FLOAT, has_requantize=t_out == orc.QINT8)
    st, _, sb32, _ = orc.qmatmul_prepare(orc.matmul_attrs(**kw), N, colsum, -1.25, 2.5, wmn, wmx, -3.0, 3.0, b32)
    assert st == orc.OK
    st, _, sb16, _ = orc.qmatmul_prepare(orc.matmul_attrs(t_bias=T16, **kw), N, colsum, -1.25, 2.5, wmn, wmx, -3.0, 3.0, b16)
    assert st == orc.OK
    np.testing.assert_array_equal(sb16, _widen(_bf16_rne(sb32, T16), T16))
    assert not np.array_equal(sb16, sb32)


@pytest.mark.parametrize("act,f", [
    (orc.ACT_ELU, lambda x: np.where(x > 0, x, np.expm1(x))),
    (orc.ACT_SIGMOID, lambda x: 1.0 / (1.0 + np.exp(-x))),
    (orc.ACT_TANH, np.tanh),
    (orc.ACT_SWISH, lambda x: x / (1.0 + np.exp(-x))),
    (orc.ACT_MISH, lambda x: x * np.tanh(np.log1p(np.exp(x))))])
def test_transcendental_post_ops_against_float64(act, f):
    """Elu / Sigmoid / Tanh / _ITEXSwish / _ITEXMish of the post-op table (onednn_post_op_util.cc:34-68, alpha 1 where the
    table says kAlphaOne): the oracle's fp32 libm evaluation against the textbook formula in float64."""
    rng = np.random.default_rng(act)
    M, K, N = 9, 64, 40
    a = rng.integers(0, 256, (M, K)).astype(np.uint8)
    w = rng.integers(-127, 128, (K, N)).astype(np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    kw = dict(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.SCALED, has_dequantize=True)
    st, lin = orc.qmatmul(orc.matmul_attrs(**kw), a, w, bias, 0.0, 6.0, np.float32(-1.5), np.float32(1.5))
    st2, got = orc.qmatmul(orc.matmul_attrs(activation=act, **kw), a, w, bias, 0.0, 6.0, np.float32(-1.5), np.float32(1.5))
    assert st == orc.OK and st2 == orc.OK
    assert lin.min() < -3 and lin.max() > 3          # both tails of every function are exercised
    with np.errstate(over="ignore"):                  # e^x overflows to inf in the far tails, as the formulas allow
        want = f(lin.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_add_fusion_with_a_16_bit_result_rounds_the_fp32_sum_once(T16):
    """The addend of a bfloat16 / half result has that type (quantized_matmul_common.h:341-389); widened to float it
    enters the same fp32 chain as a float addend, so the 16-bit result is the float result rounded to nearest even."""
    rng = np.random.default_rng(8)
    M, K, N = 9, 32, 20
    xq = rng.integers(0, 256, (M, K)).astype(np.uint8)
    wq = rng.integers(-127, 128, (K, N)).astype(np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    z = rng.standard_normal((M, N)).astype(np.float32)
    z = ((z.view(np.uint32) >> 16) << 16).view(np.float32) if T16 == orc.BFLOAT16 else z.astype(np.float16).astype(np.float32)
    kw = dict(api=orc.API_V2, t_in=orc.QUINT8, input_mode=orc.MIN_FIRST, has_dequantize=True, add_position=2,
              activation=orc.ACT_RELU)
    mnb, mxb = np.float32(-0.7), np.float32(0.7)
    st, y32 = orc.qmatmul(orc.matmul_attrs(t_out=orc.FLOAT, **kw), xq, wq, bias, -1.5, 2.5, mnb, mxb, addend=z)
    assert st == orc.OK
    st, y16 = orc.qmatmul(orc.matmul_attrs(t_out=T16, **kw), xq, wq, bias, -1.5, 2.5, mnb, mxb, addend=z)
    assert st == orc.OK and y16.dtype == np.uint16
    if T16 == orc.HALF:
        want = y32.astype(np.float16).view(np.uint16)
    else:
        u = y32.view(np.uint32).astype(np.uint64)
        want = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    np.testing.assert_array_equal(y16, want)
    st, _ = orc.qmatmul(orc.matmul_attrs(t_out=orc.QINT8, api=orc.API_V2, t_in=orc.QUINT8, has_requantize=True, add_position=1),
                        xq, wq, bias, -1.5, 2.5, mnb, mxb, -3.0, 3.0, addend=z)
    assert st == orc.UNIMPLEMENTED
