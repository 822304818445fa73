"""Quantized Conv2D on the GPU: the patch matrix (itexhip_im2col8) and bias scaling through the C ABI, and the op
kernels through the plugin, bit-compared with the CPU oracle (int32 / int8 / fp32 outputs alike: the accumulation
is integer and the epilogue is the same fp32 sequence)."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests.mock_tf import host as tf

pytestmark = pytest.mark.gpu
DT = tf.DType


def same_lead(n, k, s, d):
    eff = (k - 1) * d + 1
    out = -(-n // s)
    return out, max((out - 1) * s + eff - n, 0) // 2


@pytest.mark.parametrize("shape,kh,kw,strides,dil", [((2, 7, 9, 3), 3, 3, (2, 2), (1, 1)), ((1, 6, 6, 4), 3, 3, (1, 1), (1, 1)),
                                                     ((2, 9, 9, 8), 3, 2, (1, 2), (2, 1)), ((1, 12, 12, 16), 1, 1, (2, 2), (1, 1)),
                                                     ((3, 5, 5, 5), 5, 5, (1, 1), (1, 1)),
                                                     # channel counts that take the 16-byte-vector kernel
                                                     ((2, 9, 10, 16), 3, 3, (1, 1), (1, 1)), ((1, 8, 7, 32), 3, 2, (2, 1), (1, 2)),
                                                     ((2, 6, 6, 48), 2, 2, (1, 1), (1, 1)), ((1, 20, 20, 64), 3, 3, (1, 1), (1, 1))])
def test_im2col_against_numpy(hip, dev, shape, kh, kw, strides, dil):
    import torch
    rng = np.random.default_rng(sum(shape) + kh)
    x = rng.integers(0, 256, shape).astype(np.uint8)
    B, H, W, C = shape
    oh, pt = same_lead(H, kh, strides[0], dil[0])
    ow, pl = same_lead(W, kw, strides[1], dil[1])
    K = kh * kw * C
    Kp = (K + 15) // 16 * 16
    g = hip.ConvGeometry(B, H, W, C, kh, kw, oh, ow, strides[0], strides[1], dil[0], dil[1], pt, pl)
    for off in (0, 1):        # aligned, and an unaligned input address (byte loads)
        raw = torch.zeros(x.size + 8, dtype=torch.uint8, device=dev)
        raw[off:off + x.size] = torch.from_numpy(x.ravel()).to(dev)
        cols = torch.full((B * oh * ow, Kp), 0xEE, dtype=torch.uint8, device=dev)
        hip.im2col8(raw.data_ptr() + off, g, Kp, cols)
        torch.cuda.synchronize()
        ref = np.zeros((B, oh, ow, Kp), np.uint8)
        for i in range(kh):
            for j in range(kw):
                for a in range(oh):
                    ih = a * strides[0] - pt + i * dil[0]
                    if not 0 <= ih < H:
                        continue
                    for b_ in range(ow):
                        iw = b_ * strides[1] - pl + j * dil[1]
                        if 0 <= iw < W:
                            ref[:, a, b_, (i * kw + j) * C:(i * kw + j + 1) * C] = x[:, ih, iw, :]
        np.testing.assert_array_equal(cols.cpu().numpy(), ref.reshape(-1, Kp))


def test_scale_vector(hip, dev):
    import torch
    rng = np.random.default_rng(1)
    for n in (1, 7, 300):
        bf = rng.standard_normal(n).astype(np.float32)
        bi = rng.integers(-5000, 5000, n).astype(np.int32)
        f = (rng.random(n).astype(np.float32) + 0.1)
        out = torch.empty(n, dtype=torch.float32, device=dev)
        for bias, T in ((bf, hip.FLOAT), (bi, hip.QINT32)):
            hip.scale_vector(torch.from_numpy(bias).to(dev), T, torch.from_numpy(f).to(dev), n, n, out)
            np.testing.assert_array_equal(out.cpu().numpy(), bias.astype(np.float32) * f)
            hip.scale_vector(torch.from_numpy(bias).to(dev), T, torch.from_numpy(f[:1].copy()).to(dev), 1, n, out)
            np.testing.assert_array_equal(out.cpu().numpy(), bias.astype(np.float32) * f[0])


@pytest.mark.parametrize("shape,lead,out_hw,out_c", [((2, 5, 7, 3), (2, 3), (9, 12), 4), ((7, 7, 3, 64), (0, 0), (8, 4), 64),
                                                     ((1, 1, 1, 1), (0, 0), (1, 1), 4), ((3, 4, 4, 8), (1, 0), (5, 4), 8),
                                                     ((2, 0, 3, 2), (1, 1), (2, 5), 4)])
def test_pad_nhwc8_against_numpy(hip, dev, shape, lead, out_hw, out_c):
    import torch
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(1, 256, shape).astype(np.uint8)
    n, h, w, c = shape
    ref = np.zeros((n, out_hw[0], out_hw[1], out_c), np.uint8)
    ref[:, lead[0]:lead[0] + h, lead[1]:lead[1] + w, :c] = x
    xd = torch.from_numpy(x).to(dev) if x.size else torch.zeros(1, dtype=torch.uint8, device=dev)
    out = torch.full(ref.shape, 0x55, dtype=torch.uint8, device=dev)
    hip.pad_nhwc8(xd, n, h, w, c, lead[0], lead[1], out_hw[0], out_hw[1], out_c, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), ref)
    with pytest.raises(hip.ItexHipError):
        hip.pad_nhwc8(xd, n, h, w, c, lead[0], lead[1], out_hw[0], out_hw[1], out_c + 2, out)   # out_c % 4
    with pytest.raises(hip.ItexHipError):
        hip.pad_nhwc8(xd, n, h + 1, w, c, out_hw[0], lead[1], out_hw[0], out_hw[1], out_c, out)  # does not fit


@pytest.mark.parametrize("shape,wshape,strides,dil_h,signed_in", [((2, 30, 26, 3), (7, 7, 3, 64), (2, 2), 1, False),
                                                                  ((1, 12, 9, 4), (3, 3, 4, 32), (1, 1), 2, True),
                                                                  ((2, 9, 9, 7), (3, 2, 7, 48), (1, 2), 1, False),
                                                                  ((1, 6, 5, 1), (5, 5, 1, 16), (1, 1), 1, True)])
def test_implicit_gemm_conv_few_input_channels(hip, dev, shape, wshape, strides, dil_h, signed_in):
    """A SAME convolution with fewer than 16 input channels as the op kernel runs it: input and filter zero-padded
    (itexhip_pad_nhwc8) to 4 / 8 channels, to the windows' spatial padding and to window rows of a multiple of 16 bytes,
    then itexhip_qconv2d on the padded geometry; int32 accumulators against a numpy convolution of the original
    tensors, 8-bit outputs with scales, bias and ReLU against the patch-matrix path on the original tensors."""
    import torch
    from tests.test_oracle_conv import ref_int_conv
    rng = np.random.default_rng(sum(shape) + sum(wshape))
    B, H, W, C = shape
    kh, kw, _, O = wshape
    x = rng.integers(-128, 128, shape).astype(np.int8) if signed_in else rng.integers(0, 256, shape).astype(np.uint8)
    w = rng.integers(-127, 128, wshape).astype(np.int8)
    oh, pt = same_lead(H, kh, strides[0], dil_h)
    ow, pl = same_lead(W, kw, strides[1], 1)
    pb = max((oh - 1) * strides[0] + (kh - 1) * dil_h + 1 - H - pt, 0)
    pr = max((ow - 1) * strides[1] + kw - W - pl, 0)
    ref = ref_int_conv(x, w, strides, (dil_h, 1), ((pt, pb), (pl, pr)))[:, :oh, :ow, :]
    T_in = hip.QINT8 if signed_in else hip.QUINT8
    cn = 4 if C <= 4 else 8
    kwn = (kw * cn + 15) // 16 * 16 // cn
    hp = max(pt + H, (oh - 1) * strides[0] + (kh - 1) * dil_h + 1)
    wp = max(pl + W, (ow - 1) * strides[1] + kwn)
    xd = torch.from_numpy(x).to(dev)
    xp = torch.empty((B, hp, wp, cn), dtype=xd.dtype, device=dev)
    hip.pad_nhwc8(xd, B, H, W, C, pt, pl, hp, wp, cn, xp)
    wpad = torch.empty((kh, kwn, cn, O), dtype=torch.int8, device=dev)
    hip.pad_nhwc8(torch.from_numpy(w).to(dev), kh, kw, C, O, 0, 0, kwn, cn, O, wpad)
    Kn, M = kh * kwn * cn, B * oh * ow
    gn = hip.ConvGeometry(B, hp, wp, cn, kh, kwn, oh, ow, strides[0], strides[1], dil_h, 1, 0, 0)
    acc = torch.full((M, O), 77, dtype=torch.int32, device=dev)
    assert hip.qconv2d_implicit_ok(gn, xp, O, hip.QINT32, acc)
    packed = torch.empty(hip.qgemm_packed_bytes(Kn, O), dtype=torch.int8, device=dev)
    colsum = torch.empty(O, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(wpad, False, Kn, O, packed, colsum)
    one = torch.ones(1, dtype=torch.float32, device=dev)
    zero_bias = torch.zeros(O, dtype=torch.float32, device=dev)
    ep = hip.Epilogue()
    ep.n_scales, ep.n_eltwise = 1, 0
    hip.qconv2d(xp, T_in, gn, packed, colsum, O, one, zero_bias, ep, hip.QINT32, acc)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(acc.cpu().numpy().reshape(B, oh, ow, O), ref)
    # the patch-matrix path on the original tensors
    K = kh * kw * C
    Kp = (K + 15) // 16 * 16
    g = hip.ConvGeometry(B, H, W, C, kh, kw, oh, ow, strides[0], strides[1], dil_h, 1, pt, pl)
    cols = torch.empty((M, Kp), dtype=torch.uint8, device=dev)
    hip.im2col8(xd, g, Kp, cols)
    packed0 = torch.empty(hip.qgemm_packed_bytes(Kp, O), dtype=torch.int8, device=dev)
    colsum0 = torch.empty(O, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(torch.from_numpy(w.reshape(K, O)).to(dev), False, K, O, packed0, colsum0)
    scales = torch.from_numpy((rng.random(O).astype(np.float32) + 0.5) * np.float32(2e-3)).to(dev)
    bias = torch.from_numpy(rng.standard_normal(O).astype(np.float32)).to(dev)
    ep.n_scales, ep.n_eltwise = O, 1
    ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = hip.ELT_RELU, 0.0, 0.0
    for T, dt in ((hip.QUINT8, torch.uint8), (hip.QINT8, torch.int8), (hip.FLOAT, torch.float32)):
        a = torch.empty((M, O), dtype=dt, device=dev)
        b_ = torch.empty((M, O), dtype=dt, device=dev)
        a.view(torch.uint8).fill_(0x55)
        b_.view(torch.uint8).fill_(0xAA)
        hip.qconv2d(xp, T_in, gn, packed, colsum, O, scales, bias, ep, T, a)
        hip.qgemm(cols, T_in, packed0, colsum0, M, Kp, O, scales, bias, ep, T, b_)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.uint8), b_.view(torch.uint8)), T
    # a window that needs padding, a dilated row or a window row that is not a multiple of 16 bytes is refused
    assert not hip.qconv2d_implicit_ok(hip.ConvGeometry(B, hp, wp, cn, kh, kwn, oh, ow, strides[0], strides[1], dil_h, 1, 1, 0), xp, O, hip.QINT32, acc)
    assert not hip.qconv2d_implicit_ok(hip.ConvGeometry(B, hp, wp, cn, kh, kwn, oh, ow, strides[0], strides[1], dil_h, 2, 0, 0), xp, O, hip.QINT32, acc)
    assert not hip.qconv2d_implicit_ok(hip.ConvGeometry(B, hp, wp + 1, cn, kh, kwn + 1, oh, ow, strides[0], strides[1], dil_h, 1, 0, 0), xp, O, hip.QINT32, acc)
    assert not hip.qconv2d_implicit_ok(hip.ConvGeometry(B, hp, (ow - 1) * strides[1] + kwn - 1, cn, kh, kwn, oh, ow, strides[0], strides[1], dil_h, 1, 0, 0),
                                       xp, O, hip.QINT32, acc)


IMPLICIT_CASES = [  # input NHWC, filter HWIO, strides, dilations, leading pads (top, left) or None for SAME
    ((2, 9, 10, 16), (3, 3, 16, 48), (1, 1), (1, 1), None),      # K = 144: a ragged last K step
    ((1, 8, 7, 32), (3, 2, 32, 64), (2, 1), (1, 2), None),       # strides + dilation
    ((2, 6, 6, 48), (2, 2, 48, 112), (1, 1), (1, 1), None),      # 48 channels: pieces of one K step span two pixels
    ((1, 20, 20, 64), (3, 3, 64, 64), (1, 1), (1, 1), None),     # ResNet-like block
    ((3, 13, 11, 16), (5, 5, 16, 80), (2, 2), (1, 1), (3, 1)),   # explicit asymmetric padding, 400-byte patch rows
    ((1, 12, 12, 128), (1, 1, 128, 160), (2, 2), (1, 1), None),  # strided pointwise, 128x128 tiles
    ((1, 3, 3, 16), (3, 3, 16, 16), (1, 1), (1, 1), None),        # fewer output positions than one tile has rows
]


@pytest.mark.parametrize("shape,wshape,strides,dil,lead", IMPLICIT_CASES)
@pytest.mark.parametrize("signed_in,tile_shape", [(False, None), (True, None), (False, 0), (True, 1), (False, 2)])
def test_implicit_gemm_conv(hip, dev, monkeypatch, shape, wshape, strides, dil, lead, signed_in, tile_shape):
    """itexhip_qconv2d (activation tiles gathered from the NHWC input) against a numpy convolution for the int32
    accumulators, and bit for bit against the patch-matrix path (itexhip_im2col8 + itexhip_qgemm) for every output
    type with per-channel scales, bias and ReLU."""
    if tile_shape is not None:   # every tile shape of the kernel on every case, ragged edges included
        hip.force_tile_shape(conv=tile_shape)
    check_implicit_conv(hip, dev, shape, wshape, strides, dil, lead, signed_in, np.random.default_rng(sum(shape) + sum(wshape) + signed_in))


@pytest.mark.parametrize("seed", range(4))
def test_implicit_gemm_conv_random_geometries(hip, dev, monkeypatch, seed):
    """Seeded random geometries (window, strides, dilation, SAME and explicit leading pads, channel counts, batch) on
    random tile shapes, checked like the fixed cases above."""
    rng = np.random.default_rng(2000 + seed)
    done = 0
    while done < 10:
        B, H, W = int(rng.integers(1, 4)), int(rng.integers(3, 24)), int(rng.integers(3, 24))
        C = 16 * int(rng.choice([1, 1, 2, 3, 4, 6]))
        kh, kw = [(1, 1), (3, 3), (2, 2), (5, 5), (1, 3), (3, 1), (7, 7)][int(rng.integers(0, 7))]
        strides = [(1, 1), (2, 2), (2, 1), (3, 3)][int(rng.integers(0, 4))]
        dil = [(1, 1), (1, 1), (2, 2), (1, 2)][int(rng.integers(0, 4))]
        O = int(rng.choice([16, 32, 48, 64, 80, 128, 144, 272]))
        lead = None if rng.random() < 0.6 else (int(rng.integers(0, kh + 1)), int(rng.integers(0, kw + 1)))
        if lead is not None and ((H + 2 * lead[0] - ((kh - 1) * dil[0] + 1)) // strides[0] + 1 <= 0 or
                                 (W + 2 * lead[1] - ((kw - 1) * dil[1] + 1)) // strides[1] + 1 <= 0):
            continue
        tile_shape = int(rng.integers(-1, 3))
        if tile_shape >= 0:
            hip.force_tile_shape(conv=tile_shape)
        else:
            hip.force_tile_shape(conv=-1)
        check_implicit_conv(hip, dev, (B, H, W, C), (kh, kw, C, O), strides, dil, lead, bool(rng.integers(0, 2)), rng)
        done += 1


def check_implicit_conv(hip, dev, shape, wshape, strides, dil, lead, signed_in, rng):
    import torch
    from tests.test_oracle_conv import ref_int_conv
    B, H, W, Cin = shape
    kh, kw, _, O = wshape
    x = rng.integers(-128, 128, shape).astype(np.int8) if signed_in else rng.integers(0, 256, shape).astype(np.uint8)
    w = rng.integers(-127, 128, wshape).astype(np.int8)
    if lead is None:
        oh, pt = same_lead(H, kh, strides[0], dil[0])
        ow, pl = same_lead(W, kw, strides[1], dil[1])
    else:
        pt, pl = lead
        oh = (H + 2 * pt - ((kh - 1) * dil[0] + 1)) // strides[0] + 1
        ow = (W + 2 * pl - ((kw - 1) * dil[1] + 1)) // strides[1] + 1
    # trailing pads: whatever the output extent needs
    pb = max((oh - 1) * strides[0] + (kh - 1) * dil[0] + 1 - H - pt, 0)
    pr = max((ow - 1) * strides[1] + (kw - 1) * dil[1] + 1 - W - pl, 0)
    ref = ref_int_conv(x, w, strides, dil, ((pt, pb), (pl, pr)))[:, :oh, :ow, :]
    K, M = kh * kw * Cin, B * oh * ow
    g = hip.ConvGeometry(B, H, W, Cin, kh, kw, oh, ow, strides[0], strides[1], dil[0], dil[1], pt, pl)
    T_in = hip.QINT8 if signed_in else hip.QUINT8
    xd = torch.from_numpy(x).to(dev)
    acc = torch.full((M, O), 77, dtype=torch.int32, device=dev)
    assert hip.qconv2d_implicit_ok(g, xd, O, hip.QINT32, acc)
    packed = torch.empty(hip.qgemm_packed_bytes(K, O), dtype=torch.int8, device=dev)
    colsum = torch.empty(O, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(torch.from_numpy(w.reshape(K, O)).to(dev), False, K, O, packed, colsum)
    one = torch.ones(1, dtype=torch.float32, device=dev)
    zero_bias = torch.zeros(O, dtype=torch.float32, device=dev)
    ep = hip.Epilogue()
    ep.n_scales, ep.n_eltwise = 1, 0
    hip.qconv2d(xd, T_in, g, packed, colsum, O, one, zero_bias, ep, hip.QINT32, acc)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(acc.cpu().numpy().reshape(B, oh, ow, O), ref)

    cols = torch.empty((M, K), dtype=torch.uint8, device=dev)
    hip.im2col8(xd, g, K, cols)
    scales = torch.from_numpy((rng.random(O).astype(np.float32) + 0.5) * np.float32(2e-4)).to(dev)
    bias = torch.from_numpy(rng.standard_normal(O).astype(np.float32)).to(dev)
    ep.n_scales, ep.n_eltwise = O, 1
    ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = hip.ELT_RELU, 0.0, 0.0
    for T, dt in ((hip.QINT8, torch.int8), (hip.QUINT8, torch.uint8), (hip.FLOAT, torch.float32), (hip.BFLOAT16, torch.bfloat16),
                  (hip.QINT32, torch.int32)):
        a = torch.empty((M, O), dtype=dt, device=dev)
        b_ = torch.empty((M, O), dtype=dt, device=dev)
        a.view(torch.uint8).fill_(0x55)          # different fillers: an element neither path writes shows up
        b_.view(torch.uint8).fill_(0xAA)
        hip.qconv2d(xd, T_in, g, packed, colsum, O, scales, bias, ep, T, a)
        hip.qgemm(cols, T_in, packed, colsum, M, K, O, scales, bias, ep, T, b_)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.uint8), b_.view(torch.uint8)), T


@pytest.mark.parametrize("n_out", [48, 44, 100])
@pytest.mark.parametrize("t_add", ["u8", "s8", "f32"])
@pytest.mark.parametrize("position,alpha", [(1, 0.0), (2, 0.0), (1, 0.2), (2, None)])
def test_sum_post_op_in_conv_and_gemm(hip, dev, t_add, position, alpha, n_out):
    """One sum post-op (y += scale * addend, the addend float / qint8 / quint8) before or after the activation, through
    itexhip_qconv2d_sum (implicit GEMM), itexhip_qgemm_sum on the patch matrix (tile kernel), on 16 rows of it
    (the M <= 16 kernel) and in place (output buffer = addend buffer): all equal to the oracle's epilogue on the
    int32 convolution.  Output channel counts whose rows are 16-byte aligned (48), only 4-byte aligned (44, 100), with
    whole 32-channel tiles (read as row segments when the addend is 8-bit) and a ragged last one."""
    import torch
    from tests.test_oracle_conv import ref_int_conv
    rng = np.random.default_rng(position * 10 + len(t_add))
    shape, wshape = (2, 10, 9, 32), (3, 3, 32, n_out)
    B, H, W, Cin = shape
    O = wshape[3]
    x = rng.integers(0, 256, shape).astype(np.uint8)
    w = rng.integers(-127, 128, wshape).astype(np.int8)
    acc = ref_int_conv(x, w, (1, 1), (1, 1), ((1, 1), (1, 1))).reshape(-1, O).astype(np.int32)
    M, K = acc.shape[0], 9 * Cin
    g = hip.ConvGeometry(B, H, W, Cin, 3, 3, H, W, 1, 1, 1, 1, 1, 1)
    add_np = {"u8": rng.integers(0, 256, (M, O)).astype(np.uint8), "s8": rng.integers(-128, 128, (M, O)).astype(np.int8),
              "f32": (rng.standard_normal((M, O)) * 20).astype(np.float32)}[t_add]
    T_add = {"u8": hip.QUINT8, "s8": hip.QINT8, "f32": hip.FLOAT}[t_add]
    scales = (rng.random(O).astype(np.float32) + 0.5) * np.float32(3e-4)
    bias = rng.standard_normal(O).astype(np.float32)
    chain = [(orc.ELT_SUM, 0.37, 0.0)]
    if alpha is not None:
        act = (orc.ELT_RELU, alpha, 0.0)
        chain = [chain[0], act] if position == 1 else [act, chain[0]]
    oep, ep = orc.EpilogueDesc(), hip.Epilogue()
    oep.n_scales = ep.n_scales = O
    oep.n_eltwise = ep.n_eltwise = len(chain)
    for k, (alg, a_, b_) in enumerate(chain):
        oep.elt[k].alg, oep.elt[k].alpha, oep.elt[k].beta = alg, a_, b_
        ep.elt[k].alg, ep.elt[k].alpha, ep.elt[k].beta = alg, a_, b_
    xd, add_d = torch.from_numpy(x).to(dev), torch.from_numpy(add_np).to(dev)
    packed = torch.empty(hip.qgemm_packed_bytes(K, O), dtype=torch.int8, device=dev)
    colsum = torch.empty(O, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(torch.from_numpy(w.reshape(K, O)).to(dev), False, K, O, packed, colsum)
    sc_d, bi_d = torch.from_numpy(scales).to(dev), torch.from_numpy(bias).to(dev)
    cols = torch.empty((M, K), dtype=torch.uint8, device=dev)
    hip.im2col8(xd, g, K, cols)
    for T, dt, npdt in ((hip.QUINT8, torch.uint8, np.uint8), (hip.QINT8, torch.int8, np.int8), (hip.FLOAT, torch.float32, np.float32)):
        ref = orc.qmatmul_epilogue(acc, oep, scales, bias, T, addend=add_np.astype(np.float32))
        out = torch.zeros((M, O), dtype=dt, device=dev)
        implicit = hip.qconv2d_implicit_ok(g, xd, O, T, out)   # output rows must be 16-byte aligned for it
        assert implicit == ((O * np.dtype(npdt).itemsize) % 16 == 0)
        if implicit:
            hip.qconv2d_sum(xd, hip.QUINT8, g, packed, colsum, O, sc_d, bi_d, ep, add_d, T_add, T, out)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(out.cpu().numpy(), ref)
        out.zero_()
        hip.qgemm_sum(cols, hip.QUINT8, packed, colsum, M, K, O, sc_d, bi_d, ep, add_d, T_add, T, out)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy(), ref)
        out16 = torch.zeros((16, O), dtype=dt, device=dev)
        hip.qgemm_sum(cols, hip.QUINT8, packed, colsum, 16, K, O, sc_d, bi_d, ep, add_d, T_add, T, out16)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out16.cpu().numpy(), ref[:16])
        if implicit and add_np.dtype.itemsize == np.dtype(npdt).itemsize:     # in place: the addend buffer is the output buffer
            both = add_d.clone()
            hip.qconv2d_sum(xd, hip.QUINT8, g, packed, colsum, O, sc_d, bi_d, ep, both, T_add, T, both)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(both.cpu().numpy().view(npdt), ref)
    with pytest.raises(hip.ItexHipError):     # a sum in the chain without an addend
        hip.qgemm(cols, hip.QUINT8, packed, colsum, M, K, O, sc_d, bi_d, ep, hip.FLOAT, torch.zeros((M, O), device=dev))


@pytest.mark.parametrize("shape,kshape,strides,dil", [((2, 14, 13, 32), (3, 3, 32, 1), (1, 1), (1, 1)),   # dword path
                                                      ((1, 9, 9, 5), (3, 3, 5, 2), (2, 2), (1, 1)),       # multiplier 2, odd channels
                                                      ((2, 8, 8, 6), (5, 3, 6, 1), (1, 2), (2, 1)),       # channels not a multiple of 4
                                                      ((1, 6, 6, 4), (3, 3, 4, 3), (1, 1), (1, 1))])
@pytest.mark.parametrize("signed_in", [False, True])
def test_depthwise_conv_against_oracle(hip, dev, shape, kshape, strides, dil, signed_in):
    """itexhip_qdepthwise_conv2d for every output type: per-channel scales, bias, ReLU; bit-equal to the oracle's epilogue
    on the oracle's depthwise accumulators."""
    import torch
    rng = np.random.default_rng(sum(shape) + sum(kshape) + signed_in)
    B, H, W, Cin = shape
    kh, kw, _, mult = kshape
    O = Cin * mult
    x = rng.integers(-128, 128, shape).astype(np.int8) if signed_in else rng.integers(0, 256, shape).astype(np.uint8)
    w = rng.integers(-127, 128, kshape).astype(np.int8)
    oh, pt = same_lead(H, kh, strides[0], dil[0])
    ow, pl = same_lead(W, kw, strides[1], dil[1])
    og = orc.conv_geom(shape, (kh, kw, Cin, O), strides, dil)
    T_in = orc.QINT8 if signed_in else orc.QUINT8
    st, acc = orc.qdepthwise_conv2d(orc.ConvAttrs(T_in, orc.QINT32, 0, orc.ACT_NONE, 0.0), og, x, w, None, -1.0, 1.0,
                                    np.float32([-1]), np.float32([1]))
    assert st == orc.OK and acc.shape == (B, oh, ow, O)
    g = hip.ConvGeometry(B, H, W, Cin, kh, kw, oh, ow, strides[0], strides[1], dil[0], dil[1], pt, pl)
    scales = (rng.random(O).astype(np.float32) + 0.5) * np.float32(2e-3)
    bias = rng.standard_normal(O).astype(np.float32)
    oep, ep = orc.EpilogueDesc(), hip.Epilogue()
    oep.n_scales = ep.n_scales = O
    oep.n_eltwise = ep.n_eltwise = 1
    for e_ in (oep, ep):
        e_.elt[0].alg, e_.elt[0].alpha, e_.elt[0].beta = orc.ELT_RELU, 0.0, 0.0
    xd, wd = torch.from_numpy(x).to(dev), torch.from_numpy(w).to(dev)
    sc_d, bi_d = torch.from_numpy(scales).to(dev), torch.from_numpy(bias).to(dev)
    for T, dt in ((hip.QINT8, torch.int8), (hip.QUINT8, torch.uint8), (hip.FLOAT, torch.float32), (hip.BFLOAT16, torch.int16),
                  (hip.QINT32, torch.int32)):
        ref = orc.qmatmul_epilogue(acc.reshape(-1, O), oep, scales, bias, T)
        out = torch.zeros((B * oh * ow, O), dtype=dt, device=dev)
        hip.qdepthwise_conv2d(xd, T_in, g, mult, wd, sc_d, bi_d, ep, T, out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        np.testing.assert_array_equal(got.view(ref.dtype) if got.dtype != ref.dtype else got, ref)
    # int32 accumulators themselves: no scales, no bias, no post-op
    ep0 = hip.Epilogue()
    out = torch.zeros((B * oh * ow, O), dtype=torch.int32, device=dev)
    hip.qdepthwise_conv2d(xd, T_in, g, mult, wd, None, None, ep0, hip.QINT32, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy().reshape(acc.shape), acc)


def test_conv_empty_and_degenerate_extents(hip, dev, rt):
    """Zero batch / zero output channels launch nothing and succeed; a window larger than the input under VALID gives
    an empty output through the op (TensorFlow's rule: (in - eff + stride) / stride = 0); a 1x1 output position."""
    import torch
    torch_ = rt
    x = torch.zeros(16 * 16, dtype=torch.uint8, device=dev)
    ep = hip.Epilogue()
    ep.n_scales = 1
    one = torch.ones(16, dtype=torch.float32, device=dev)
    out = torch.full((64,), 7, dtype=torch.int32, device=dev)
    g0 = hip.ConvGeometry(0, 4, 4, 16, 3, 3, 4, 4, 1, 1, 1, 1, 1, 1)
    hip.im2col8(x, g0, 144, out)                                       # no rows
    hip.qdepthwise_conv2d(x, hip.QUINT8, g0, 1, x, one, one, ep, hip.QINT32, out)
    torch.cuda.synchronize()
    assert int(out.min()) == 7                                          # nothing written
    # one output position: 3x3 window over a 3x3 input, VALID
    rng = np.random.default_rng(0)
    xs = rng.integers(0, 256, (1, 3, 3, 16)).astype(np.uint8)
    ws = rng.integers(-127, 128, (3, 3, 16, 16)).astype(np.int8)
    g1 = hip.ConvGeometry(1, 3, 3, 16, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    packed = torch.empty(hip.qgemm_packed_bytes(144, 16), dtype=torch.int8, device=dev)
    colsum = torch.empty(16, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(torch.from_numpy(ws.reshape(144, 16)).to(dev), False, 144, 16, packed, colsum)
    acc = torch.zeros((1, 16), dtype=torch.int32, device=dev)
    hip.qconv2d(torch.from_numpy(xs).to(dev), hip.QUINT8, g1, packed, colsum, 16, one[:1], torch.zeros(16, device=dev), ep,
                hip.QINT32, acc)
    torch_.cuda.synchronize()
    np.testing.assert_array_equal(acc.cpu().numpy()[0], xs.reshape(-1).astype(np.int64) @ ws.reshape(144, 16).astype(np.int64))
    # through the op: window larger than the input, VALID -> empty output, ranges still produced
    node = tf.Node("QuantizedConv2D", dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), out_type=DT(tf.QINT32), strides=[1, 1, 1, 1],
                                           padding="VALID", dilations=[1, 1, 1, 1]))
    assert node.code == tf.OK, node.message
    xq = np.zeros((2, 2, 2, 4), np.uint8)
    wq = np.zeros((3, 3, 4, 8), np.int8)
    s = [np.array(v, np.float32) for v in (0.0, 1.0, -1.0, 1.0)]
    got, res = run_conv(torch_, dev, node, xq, wq, None, tf.FLOAT, s, tf.QINT32, np.int32, True)
    assert got.shape == (2, 0, 0, 8)
    node.close()


def test_implicit_gemm_conv_rejects_other_shapes(hip, dev):
    import torch
    x = torch.zeros(4 * 4 * 24 + 16, dtype=torch.uint8, device=dev)
    y = torch.zeros(16 * 16 * 4 + 16, dtype=torch.uint8, device=dev)
    ok = lambda g, xp=x, O=16, T=hip.QINT32, out=y: hip.qconv2d_implicit_ok(g, xp, O, T, out)
    assert not ok(hip.ConvGeometry(1, 4, 4, 24, 3, 3, 4, 4, 1, 1, 1, 1, 1, 1))   # 24 channels
    g16 = hip.ConvGeometry(1, 4, 4, 16, 3, 3, 4, 4, 1, 1, 1, 1, 1, 1)
    assert ok(g16) and not ok(g16, xp=x.data_ptr() + 4)                         # misaligned input
    assert not ok(hip.ConvGeometry(1, 40, 40, 1024, 5, 5, 40, 40, 1, 1, 1, 1, 2, 2))  # 25 KiB window
    assert not ok(g16, O=24, T=hip.QINT8) and ok(g16, O=32, T=hip.QINT8)        # output rows of 24 bytes
    assert not ok(g16, out=y.data_ptr() + 4) and not ok(g16, T=hip.HALF)
    ep = hip.Epilogue()
    with pytest.raises(hip.ItexHipError) as e:
        hip.qconv2d(x.data_ptr() + 4, hip.QUINT8, g16, x, x, 16, x, x, ep, hip.QINT32, y)
    assert e.value.code == hip.INVALID_ARGUMENT


@pytest.fixture(scope="module")
def rt(dev):
    import torch
    tf.load()
    tf.use_torch_allocator(dev)
    return torch


def fetch(torch, out, np_dtype):
    dtype, shape, addr, _ = out
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    torch.cuda.synchronize()
    live = tf._state["alloc_cb"][2]
    if addr in live:
        return live[addr][:n * np.dtype(np_dtype).itemsize].cpu().numpy().view(np_dtype).copy().reshape(shape)
    return tf.read_host(addr, dtype, shape)


def quantize_inputs(x, w, T_in, per_channel=True):
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), T_in, orc.SCALED)
    if per_channel:
        mn, mx = w.min(axis=(0, 1, 2)).astype(np.float32), w.max(axis=(0, 1, 2)).astype(np.float32)
        _, wq, fmn, fmx = orc.quantize_v2(w, mn, mx, orc.QINT8, orc.SCALED, axis=3)
    else:
        _, wq, fmn, fmx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
        fmn, fmx = np.array(fmn[0], np.float32), np.array(fmx[0], np.float32)
    return xq, np.array(xmn[0], np.float32), np.array(xmx[0], np.float32), wq, fmn, fmx


def run_conv(torch, dev, node, xq, wq, bias, bias_dt, host_scalars, out_dt, np_out, with_minmax):
    keep = [torch.from_numpy(np.ascontiguousarray(v)).to(dev) for v in ([xq, wq] + ([bias] if bias is not None else []))]
    ins = [(tf.QUINT8 if xq.dtype == np.uint8 else tf.QINT8, xq.shape, keep[0].data_ptr(), False),
           (tf.QINT8, wq.shape, keep[1].data_ptr(), False)]
    if bias is not None:
        ins.append((bias_dt, bias.shape, keep[2].data_ptr(), False))
    for s in host_scalars:
        ins.append((tf.FLOAT, s.shape, tf.host_array(s), True))
    outs = [(out_dt, False)] + ([(tf.FLOAT, True), (tf.FLOAT, True)] if with_minmax else [])
    code, msg, res = node.run(ins, outs, stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    return fetch(torch, res[0], np_out), res


LEGACY = [  # op, fusions -> (bias, relu, requantize), input type, output type
    ("QuantizedConv2D", False, False, False, tf.QUINT8, tf.QINT32),
    ("QuantizedConv2DPerChannel", False, False, False, tf.QINT8, tf.QINT32),
    ("QuantizedConv2DWithBias", True, False, False, tf.QUINT8, tf.QINT32),
    ("QuantizedConv2DWithBiasAndRelu", True, True, False, tf.QINT8, tf.QINT32),
    ("QuantizedConv2DAndRelu", False, True, False, tf.QUINT8, tf.QINT32),
    ("QuantizedConv2DAndRequantize", False, False, True, tf.QINT8, tf.QINT8),
    ("QuantizedConv2DAndReluAndRequantize", False, True, True, tf.QUINT8, tf.QUINT8),
    ("QuantizedConv2DWithBiasAndRequantize", True, False, True, tf.QINT8, tf.QINT8),
    ("QuantizedConv2DWithBiasAndReluAndRequantize", True, True, True, tf.QUINT8, tf.QUINT8),
]
NP = {tf.QINT32: np.int32, tf.QINT8: np.int8, tf.QUINT8: np.uint8, tf.FLOAT: np.float32}


@pytest.mark.parametrize("op,has_bias,relu,req,t_in,t_out", LEGACY)
def test_legacy_conv_ops_through_plugin(rt, dev, op, has_bias, relu, req, t_in, t_out):
    """The shapes of the reference's native_quantized_conv_test.py (x [1,6,6,4], w [3,3,4,4], SAME, stride 1) plus a
    strided, larger case; outputs and min / max outputs equal the oracle's."""
    torch = rt
    for shape, wshape, strides, padding in (((1, 6, 6, 4), (3, 3, 4, 4), [1, 1, 1, 1], "SAME"),
                                            ((2, 15, 13, 20), (3, 3, 20, 24), [1, 2, 2, 1], "VALID")):
        rng = np.random.default_rng(len(op) + shape[1])
        signed = t_in == tf.QINT8
        x = rng.uniform(-5.0 if signed else 0.0, 5.0, shape).astype(np.float32)
        w = rng.uniform(-2.0, 2.0, wshape).astype(np.float32)
        b = rng.uniform(-1.0, 1.0, wshape[3]).astype(np.float32) if has_bias else None
        xq, xmn, xmx, wq, fmn, fmx = quantize_inputs(x, w, t_in, per_channel=op != "QuantizedConv2D")
        attrs = dict(Tinput=DT(t_in), Tfilter=DT(tf.QINT8), out_type=DT(t_out), strides=strides, padding=padding,
                     dilations=[1, 1, 1, 1])
        if has_bias and req:
            attrs["Tbias"] = DT(tf.FLOAT)
        node = tf.Node(op, attrs)
        assert node.code == tf.OK, node.message
        zmn, zmx = np.array(-37.5 if t_out == tf.QINT8 else 0.0, np.float32), np.array(41.0, np.float32)
        scalars = [xmn, xmx, fmn, fmx] + ([zmn, zmx] if req else [])
        got, res = run_conv(torch, dev, node, xq, wq, b, tf.FLOAT, scalars, t_out, NP[t_out], True)
        at = orc.ConvAttrs(t_in, t_out, orc.FLOAT if has_bias else 0, orc.ACT_RELU if relu else orc.ACT_NONE, 0.0)
        g = orc.conv_geom(shape, wshape, strides[1:3], (1, 1), orc.PAD_SAME if padding == "SAME" else orc.PAD_VALID)
        st, ref = orc.qconv2d(at, g, xq, wq, b, float(xmn), float(xmx), fmn, fmx, float(zmn), float(zmx))
        assert st == orc.OK
        np.testing.assert_array_equal(got, ref)
        mat = orc.matmul_attrs(t_in=t_in, t_out=t_out)
        st, omn, omx = orc.qmatmul_output_minmax(mat, float(xmn), float(xmx), fmn, fmx, fmn.ndim, float(zmn), float(zmx))
        np.testing.assert_array_equal(np.ravel(fetch(torch, res[1], np.float32)), omn)
        np.testing.assert_array_equal(np.ravel(fetch(torch, res[2], np.float32)), omx)
        node.close()


@pytest.mark.parametrize("t_in", [tf.QUINT8, tf.QINT8])
@pytest.mark.parametrize("fused,t_out,t_bias", [(["BiasAdd", "Relu", "Dequantize"], tf.FLOAT, tf.FLOAT),
                                                (["BiasAdd", "Dequantize"], tf.FLOAT, tf.QINT32),
                                                (["BiasAdd", "LeakyRelu", "Requantize"], tf.QINT8, tf.FLOAT),
                                                (["BiasAdd", "Relu", "Requantize"], tf.QUINT8, tf.QINT32),
                                                (["Dequantize"], tf.FLOAT, tf.FLOAT), ([], tf.QINT32, tf.FLOAT)])
def test_new_api_conv_through_plugin(rt, dev, t_in, fused, t_out, t_bias):
    """_QuantizedConv2D with fused_ops, explicit padding, dilation, channel counts that are not multiples of 16 and a
    pointwise case that skips the patch matrix; against the oracle, and against the fp32 convolution where that applies."""
    torch = rt
    cases = [((2, 10, 9, 6), (3, 3, 6, 10), [1, 1, 2, 1], [1, 2, 1, 1], "EXPLICIT", [0, 0, 2, 1, 0, 3, 0, 0]),
             ((1, 8, 8, 32), (1, 1, 32, 48), [1, 1, 1, 1], [1, 1, 1, 1], "SAME", []),
             ((1, 14, 14, 3), (7, 7, 3, 8), [1, 2, 2, 1], [1, 1, 1, 1], "SAME", []),
             # fewer than 16 input channels with 16-byte output rows: input and filter are padded to 4 / 8 channels and the
             # tile kernel gathers pixel runs (first layer of ResNet-50 in small; explicit pads; dilation down the rows)
             ((2, 23, 21, 3), (7, 7, 3, 64), [1, 2, 2, 1], [1, 1, 1, 1], "SAME", []),
             ((1, 9, 11, 8), (3, 3, 8, 16), [1, 1, 1, 1], [1, 2, 1, 1], "EXPLICIT", [0, 0, 1, 2, 3, 0, 0, 0]),
             ((1, 7, 7, 5), (1, 1, 5, 32), [1, 1, 1, 1], [1, 1, 1, 1], "VALID", [])]
    for shape, wshape, strides, dil, padding, explicit in cases:
        rng = np.random.default_rng(shape[1] * 3 + len(fused))
        signed = t_in == tf.QINT8
        x = rng.uniform(-3.0 if signed else 0.0, 3.0, shape).astype(np.float32)
        w = rng.uniform(-1.0, 1.0, wshape).astype(np.float32)
        has_bias = "BiasAdd" in fused
        xq, xmn, xmx, wq, fmn, fmx = quantize_inputs(x, w, t_in)
        if t_bias == tf.QINT32:
            b = rng.integers(-4000, 4000, wshape[3]).astype(np.int32) if has_bias else None
        else:
            b = rng.uniform(-1.0, 1.0, wshape[3]).astype(np.float32) if has_bias else None
        attrs = dict(Tinput=DT(t_in), Tfilter=DT(tf.QINT8), Tbias=DT(t_bias), Tsummand=DT(t_out), out_type=DT(t_out), strides=strides,
                     padding=padding, dilations=dil, fused_ops=fused, alpha=0.2, data_format="NHWC", is_filter_const=True,
                     is_bias_const=True)
        if explicit:
            attrs["explicit_paddings"] = explicit
        node = tf.Node("_QuantizedConv2D", attrs)
        assert node.code == tf.OK, node.message
        req = "Requantize" in fused
        zmn, zmx = np.array(-20.0 if t_out == tf.QINT8 else 0.0, np.float32), np.array(25.0, np.float32)
        scalars = [xmn, xmx, fmn, fmx] + ([zmn, zmx] if req else [])
        with_mm = t_out != tf.FLOAT
        act = orc.ACT_RELU if "Relu" in fused else orc.ACT_LEAKYRELU if "LeakyRelu" in fused else orc.ACT_NONE
        at = orc.ConvAttrs(t_in, t_out, (orc.QINT32 if t_bias == tf.QINT32 else orc.FLOAT) if has_bias else 0, act, 0.2)
        pad = {"SAME": orc.PAD_SAME, "VALID": orc.PAD_VALID, "EXPLICIT": orc.PAD_EXPLICIT}[padding]
        g = orc.conv_geom(shape, wshape, strides[1:3], dil[1:3], pad, tuple(explicit[2:6]) if explicit else (0, 0, 0, 0))
        st, ref = orc.qconv2d(at, g, xq, wq, b, float(xmn), float(xmx), fmn, fmx, float(zmn), float(zmx))
        assert st == orc.OK
        for _ in range(2):      # the second run uses the cached packed filter and parameter vectors
            got, _res = run_conv(torch, dev, node, xq, wq, b, t_bias, scalars, t_out, NP[t_out], with_mm)
            np.testing.assert_array_equal(got, ref)
        node.close()


@pytest.mark.parametrize("fused,t_out", [(["BiasAdd", "Elu", "Dequantize"], tf.FLOAT), (["BiasAdd", "Sigmoid", "Dequantize"], tf.FLOAT),
                                         (["BiasAdd", "Elu", "Requantize"], tf.QINT8), (["BiasAdd", "Sigmoid", "Requantize"], tf.QUINT8)])
def test_elu_and_sigmoid_fusions_through_plugin(rt, dev, fused, t_out):
    """_QuantizedConv2D [BiasAdd, Elu | Sigmoid, Requantize | Dequantize] (quantized_conv_ops.h:83, 86, 100, 103): the
    activation works on the already scaled value (the output scale, requantization included, comes first).  Float
    results within 2e-6 of the oracle (the device evaluates exp with the hardware instruction), 8-bit ones equal or, where
    the float value sits on a rounding boundary, one unit off.  A 3x3 window on 16 channels (would be the implicit
    GEMM) and a 1x1 one."""
    torch = rt
    for shape, wshape in (((2, 9, 8, 16), (3, 3, 16, 32)), ((1, 6, 6, 32), (1, 1, 32, 16))):
        rng = np.random.default_rng(shape[1] + len(fused[1]))
        x = rng.uniform(0.0, 3.0, shape).astype(np.float32)
        w = rng.uniform(-1.0, 1.0, wshape).astype(np.float32)
        xq, xmn, xmx, wq, fmn, fmx = quantize_inputs(x, w, tf.QUINT8)
        b = rng.uniform(-1.0, 1.0, wshape[3]).astype(np.float32)
        node = tf.Node("_QuantizedConv2D", dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(t_out),
                                                out_type=DT(t_out), strides=[1, 1, 1, 1], padding="SAME", dilations=[1, 1, 1, 1],
                                                fused_ops=fused, alpha=0.2, data_format="NHWC", is_filter_const=True,
                                                is_bias_const=True))
        assert node.code == tf.OK, node.message
        req = "Requantize" in fused
        zmn, zmx = np.array(-4.0 if t_out == tf.QINT8 else 0.0, np.float32), np.array(6.0, np.float32)
        scalars = [xmn, xmx, fmn, fmx] + ([zmn, zmx] if req else [])
        at = orc.ConvAttrs(tf.QUINT8, t_out, orc.FLOAT, orc.ACT_ELU if "Elu" in fused else orc.ACT_SIGMOID, 0.2)
        g = orc.conv_geom(shape, wshape, (1, 1), (1, 1), orc.PAD_SAME, (0, 0, 0, 0))
        st, ref = orc.qconv2d(at, g, xq, wq, b, float(xmn), float(xmx), fmn, fmx, float(zmn), float(zmx))
        assert st == orc.OK
        got, _res = run_conv(torch, dev, node, xq, wq, b, tf.FLOAT, scalars, t_out, NP[t_out], req)
        if t_out == tf.FLOAT:
            np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-6)
        else:
            d = np.abs(got.astype(np.int32) - ref.astype(np.int32))
            assert d.max() <= 1 and (d > 0).mean() < 1e-3
        node.close()
    for bad in (["BiasAdd", "_FusedSwish", "Dequantize"], ["BiasAdd", "_FusedHardSwish", "Requantize"]):
        bad_out = tf.QINT8 if "Requantize" in bad else tf.FLOAT
        n = tf.Node("_QuantizedConv2D", dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(bad_out),
                                             out_type=DT(bad_out), strides=[1, 1, 1, 1],
                                             padding="SAME", dilations=[1, 1, 1, 1], fused_ops=bad, alpha=0.2, data_format="NHWC",
                                             is_filter_const=True, is_bias_const=True))
        assert n.code == tf.UNIMPLEMENTED


@pytest.mark.parametrize("op,t_sum,fused", [
    ("QuantizedConv2DWithBiasSumAndReluAndRequantize", tf.QUINT8, None),
    ("QuantizedConv2DWithBiasSignedSumAndReluAndRequantize", tf.QINT8, None),
    ("_QuantizedConv2D", tf.QUINT8, ["BiasAdd", "Sum", "Relu", "Requantize"]),
    ("_QuantizedConv2D", tf.QINT8, ["BiasAdd", "Relu", "Sum", "Requantize"]),
    ("_QuantizedConv2D", tf.QINT8, ["BiasAdd", "Sum", "LeakyRelu", "Requantize"])])
def test_sum_fusions_through_plugin(rt, dev, op, t_sum, fused):
    """The residual-add fusions of a ResNet block: conv + bias + sum (8-bit summand with its own range) + ReLU +
    requantize, legacy spellings and fused_ops of the new API, implicit-GEMM and patch-matrix shapes; equal to the
    oracle (which restates the reference's scale and type rules for the sum post-op)."""
    torch = rt
    new_api = fused is not None
    t_out = tf.QINT8 if (new_api and "LeakyRelu" in fused) else tf.QUINT8
    for shape, wshape in (((2, 9, 8, 16), (3, 3, 16, 32)), ((1, 7, 7, 6), (3, 3, 6, 16))):
        rng = np.random.default_rng(shape[3] + t_sum + (len(fused) if fused else 0))
        x = rng.uniform(0.0, 4.0, shape).astype(np.float32)
        w = rng.uniform(-1.0, 1.0, wshape).astype(np.float32)
        b = rng.uniform(-1.0, 1.0, wshape[3]).astype(np.float32)
        xq, xmn, xmx, wq, fmn, fmx = quantize_inputs(x, w, tf.QUINT8)
        oshape = (shape[0], shape[1], shape[2], wshape[3])
        summand = (rng.integers(0, 256, oshape).astype(np.uint8) if t_sum == tf.QUINT8 else rng.integers(-128, 128, oshape).astype(np.int8))
        smn, smx = np.array(0.0 if t_sum == tf.QUINT8 else -11.0, np.float32), np.array(14.0, np.float32)
        zmn, zmx = np.array(-25.0 if t_out == tf.QINT8 else 0.0, np.float32), np.array(30.0, np.float32)
        attrs = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(t_sum), out_type=DT(t_out),
                     strides=[1, 1, 1, 1], padding="SAME", dilations=[1, 1, 1, 1])
        if new_api:
            attrs.update(fused_ops=fused, alpha=0.25, data_format="NHWC", is_filter_const=True, is_bias_const=True)
        node = tf.Node(op, attrs)
        assert node.code == tf.OK, node.message
        keep = [torch.from_numpy(np.ascontiguousarray(v)).to(dev) for v in (xq, wq, b, summand)]
        dev_in = lambda i, dt, arr: (dt, arr.shape, keep[i].data_ptr(), False)
        host = lambda v: (tf.FLOAT, v.shape, tf.host_array(v), True)
        ins = [dev_in(0, tf.QUINT8, xq), dev_in(1, tf.QINT8, wq), dev_in(2, tf.FLOAT, b)]
        if new_api:
            ins += [dev_in(3, t_sum, summand)] + [host(v) for v in (xmn, xmx, fmn, fmx, smn, smx, zmn, zmx)]
        else:
            ins += [host(v) for v in (xmn, xmx, fmn, fmx, zmn, zmx)] + [dev_in(3, t_sum, summand), host(smn), host(smx)]
        code, msg, res = node.run(ins, [(t_out, False), (tf.FLOAT, True), (tf.FLOAT, True)],
                                  stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        got = fetch(torch, res[0], NP[t_out])
        leaky = new_api and "LeakyRelu" in fused
        position = 2 if (new_api and fused.index("Sum") > 1 and not leaky and fused[1] == "Relu") else 1
        at = orc.ConvAttrs(orc.QUINT8, t_out, orc.FLOAT, orc.ACT_LEAKYRELU if leaky else orc.ACT_RELU, 0.25)
        g = orc.conv_geom(shape, wshape)
        st, ref = orc.qconv2d(at, g, xq, wq, b, float(xmn), float(xmx), fmn, fmx, float(zmn), float(zmx),
                              sum=orc.ConvSum(position, t_sum, float(smn), float(smx)), summand=summand)
        assert st == orc.OK
        np.testing.assert_array_equal(got, ref)
        assert float(np.ravel(fetch(torch, res[1], np.float32))[0]) == float(zmn)
        assert float(np.ravel(fetch(torch, res[2], np.float32))[0]) == float(zmx)
        node.close()


@pytest.mark.parametrize("op,has_bias,relu,req", [("QuantizedDepthwiseConv2D", False, False, False),
                                                  ("QuantizedDepthwiseConv2DWithBias", True, False, False),
                                                  ("QuantizedDepthwiseConv2DWithBiasAndRelu", True, True, False),
                                                  ("QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize", True, True, True),
                                                  ("_QuantizedDepthwiseConv2D", True, True, True),
                                                  ("_QuantizedDepthwiseConv2D", True, False, False)])
def test_depthwise_ops_through_plugin(rt, dev, op, has_bias, relu, req):
    """Depthwise spellings (legacy and new API) against the oracle: multiplier 1 and 2, strides, per-channel filter ranges
    (one per output channel c * multiplier + m)."""
    torch = rt
    new_api = op.startswith("_")
    for shape, kshape, strides in (((2, 12, 11, 16), (3, 3, 16, 1), [1, 1, 1, 1]), ((1, 9, 9, 6), (3, 3, 6, 2), [1, 2, 2, 1])):
        rng = np.random.default_rng(shape[3] + len(op))
        x = rng.uniform(0.0, 4.0, shape).astype(np.float32)
        w = rng.uniform(-1.0, 1.0, kshape).astype(np.float32)
        O = kshape[2] * kshape[3]
        b = rng.uniform(-1.0, 1.0, O).astype(np.float32) if has_bias else None
        _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.SCALED)
        xmn, xmx = np.array(xmn[0], np.float32), np.array(xmx[0], np.float32)
        wf = w.reshape(kshape[0], kshape[1], O)          # ranges per output channel
        mn, mx = wf.min(axis=(0, 1)).astype(np.float32), wf.max(axis=(0, 1)).astype(np.float32)
        _, wq, fmn, fmx = orc.quantize_v2(wf, mn, mx, orc.QINT8, orc.SCALED, axis=2)
        wq = wq.reshape(kshape)
        if new_api and not req:
            t_out = tf.FLOAT
        else:
            t_out = tf.QUINT8 if req else tf.QINT32
        attrs = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), out_type=DT(t_out), strides=strides, padding="SAME",
                     dilations=[1, 1, 1, 1])
        if new_api:
            fused = (["BiasAdd"] if has_bias else []) + (["Relu"] if relu else []) + (["Requantize"] if req else ["Dequantize"])
            attrs.update(Tbias=DT(tf.FLOAT), Tsummand=DT(t_out), fused_ops=fused, alpha=0.0, data_format="NHWC",
                         is_filter_const=True, is_bias_const=True)
        elif has_bias and req:
            attrs["Tbias"] = DT(tf.FLOAT)
        node = tf.Node(op, attrs)
        assert node.code == tf.OK, node.message
        zmn, zmx = np.array(0.0, np.float32), np.array(20.0, np.float32)
        scalars = [xmn, xmx, fmn, fmx] + ([zmn, zmx] if req else [])
        got, _res = run_conv(torch, dev, node, xq, wq, b, tf.FLOAT, scalars, t_out, NP[t_out], t_out != tf.FLOAT)
        at = orc.ConvAttrs(orc.QUINT8, t_out, orc.FLOAT if has_bias else 0, orc.ACT_RELU if relu else orc.ACT_NONE, 0.0)
        g = orc.conv_geom(shape, (kshape[0], kshape[1], kshape[2], O), strides[1:3])
        st, ref = orc.qdepthwise_conv2d(at, g, xq, wq, b, float(xmn), float(xmx), fmn, fmx, float(zmn), float(zmx))
        assert st == orc.OK
        np.testing.assert_array_equal(got, ref)
        if t_out == tf.FLOAT:       # and the fp32 depthwise convolution it stands for, within the quantization steps
            pads = [(1, 1), (1, 1)] if strides[1] == 1 else [(1, 1), (1, 1)]
            xp = np.pad(x, ((0, 0), pads[0], pads[1], (0, 0)))
            oh, ow = ref.shape[1], ref.shape[2]
            f = np.zeros(ref.shape, np.float64)
            for i in range(3):
                for j in range(3):
                    win = xp[:, i:i + (oh - 1) * strides[1] + 1:strides[1], j:j + (ow - 1) * strides[2] + 1:strides[2], :]
                    f += np.repeat(win, kshape[3], axis=3) * w[i, j].reshape(-1)
            f += b if has_bias else 0
            assert np.abs(got - f).max() < 0.3
        node.close()


def test_conv_cached_bias_follows_its_inputs(rt, dev):
    """The op keeps the scaled bias of a constant-bias node; a bias at another address or other ranges (other scaling
    factors) must still give that call's own result."""
    torch = rt
    rng = np.random.default_rng(5)
    shape, wshape = (1, 8, 8, 16), (3, 3, 16, 16)
    x = rng.uniform(0.0, 3.0, shape).astype(np.float32)
    w = rng.uniform(-1.0, 1.0, wshape).astype(np.float32)
    xq, xmn, xmx, wq, fmn, fmx = quantize_inputs(x, w, tf.QUINT8)
    attrs = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(tf.FLOAT), out_type=DT(tf.FLOAT),
                 strides=[1, 1, 1, 1], padding="SAME", dilations=[1, 1, 1, 1], fused_ops=["BiasAdd", "Dequantize"], alpha=0.0,
                 data_format="NHWC", is_filter_const=True, is_bias_const=True)
    node = tf.Node("_QuantizedConv2D", attrs)
    assert node.code == tf.OK, node.message
    at = orc.ConvAttrs(orc.QUINT8, orc.FLOAT, orc.FLOAT, orc.ACT_NONE, 0.0)
    g = orc.conv_geom(shape, wshape)
    hold = []                                  # keep every device buffer alive so that addresses differ between calls
    for bias, in_max in ((rng.uniform(-1, 1, 16).astype(np.float32), xmx), (rng.uniform(-1, 1, 16).astype(np.float32), xmx),
                         (np.zeros(16, np.float32) + 0.5, np.array(float(xmx) * 2, np.float32))):
        keep = [torch.from_numpy(np.ascontiguousarray(v)).to(dev) for v in (xq, wq, bias)]
        hold.append(keep)
        ins = [(tf.QUINT8, xq.shape, keep[0].data_ptr(), False), (tf.QINT8, wq.shape, keep[1].data_ptr(), False),
               (tf.FLOAT, bias.shape, keep[2].data_ptr(), False)]
        ins += [(tf.FLOAT, v.shape, tf.host_array(v), True) for v in (xmn, in_max, fmn, fmx)]
        code, msg, res = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        st, ref = orc.qconv2d(at, g, xq, wq, bias, float(xmn), float(in_max), fmn, fmx)
        assert st == orc.OK
        np.testing.assert_array_equal(fetch(torch, res[0], np.float32), ref)
    node.close()


def test_int8_bottleneck_block_end_to_end(rt, dev):
    """A ResNet bottleneck block chained through the plugin's ops, every tensor between them quint8 on the device:
    1x1 conv (plain GEMM) -> 3x3 conv (implicit GEMM) -> 1x1 conv + residual Sum + ReLU, each with bias and requantize;
    the final tensor equals the same chain through the oracle."""
    torch = rt
    rng = np.random.default_rng(77)
    B, H, W, C, Cm = 2, 14, 14, 64, 16
    x = rng.uniform(0.0, 4.0, (B, H, W, C)).astype(np.float32)
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.SCALED)
    rng_in = (float(xmn[0]), float(xmx[0]))
    layers = [((1, 1, C, Cm), 0, 6.0), ((3, 3, Cm, Cm), 0, 9.0), ((1, 1, Cm, C), 1, 12.0)]   # filter, sum position, frozen output max
    cur_dev = torch.from_numpy(xq).to(dev)
    cur_ref, cur_rng = xq, rng_in
    keep = [cur_dev]
    for wshape, sum_pos, zmax in layers:
        w = rng.uniform(-0.5, 0.5, wshape).astype(np.float32)
        b = rng.uniform(-0.5, 0.5, wshape[3]).astype(np.float32)
        mn, mx = w.min(axis=(0, 1, 2)).astype(np.float32), w.max(axis=(0, 1, 2)).astype(np.float32)
        _, wq, fmn, fmx = orc.quantize_v2(w, mn, mx, orc.QINT8, orc.SCALED, axis=3)
        fused = ["BiasAdd"] + (["Sum"] if sum_pos else []) + ["Relu", "Requantize"]
        attrs = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(tf.QUINT8), out_type=DT(tf.QUINT8),
                     strides=[1, 1, 1, 1], padding="SAME", dilations=[1, 1, 1, 1], fused_ops=fused, alpha=0.0, data_format="NHWC",
                     is_filter_const=True, is_bias_const=True)
        node = tf.Node("_QuantizedConv2D", attrs)
        assert node.code == tf.OK, node.message
        w_d, b_d = torch.from_numpy(wq).to(dev), torch.from_numpy(b).to(dev)
        keep += [w_d, b_d]
        def host(v):            # host scalars must outlive the call: keep the arrays
            arr = np.array(v, np.float32)
            keep.append(arr)
            return (tf.FLOAT, (), tf.host_array(arr), True)
        hostv = lambda v: (tf.FLOAT, v.shape, tf.host_array(v), True)
        shape_in = tuple(cur_ref.shape)
        ins = [(tf.QUINT8, shape_in, cur_dev.data_ptr(), False), (tf.QINT8, wq.shape, w_d.data_ptr(), False),
               (tf.FLOAT, b.shape, b_d.data_ptr(), False)]
        if sum_pos:
            ins.append((tf.QUINT8, xq.shape, keep[0].data_ptr(), False))
        ins += [host(cur_rng[0]), host(cur_rng[1]), hostv(fmn), hostv(fmx)]
        if sum_pos:
            ins += [host(rng_in[0]), host(rng_in[1])]
        ins += [host(0.0), host(zmax)]
        code, msg, res = node.run(ins, [(tf.QUINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)],
                                  stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        got = fetch(torch, res[0], np.uint8)
        at = orc.ConvAttrs(orc.QUINT8, orc.QUINT8, orc.FLOAT, orc.ACT_RELU, 0.0)
        g = orc.conv_geom(shape_in, wshape)
        kw = dict(sum=orc.ConvSum(1, orc.QUINT8, rng_in[0], rng_in[1]), summand=xq) if sum_pos else {}
        st, ref = orc.qconv2d(at, g, cur_ref, wq, b, cur_rng[0], cur_rng[1], fmn, fmx, 0.0, zmax, **kw)
        assert st == orc.OK
        np.testing.assert_array_equal(got, ref, err_msg="layer %s" % (wshape,))
        assert len(np.unique(got)) > 8
        cur_ref, cur_rng = ref, (0.0, zmax)
        cur_dev = torch.from_numpy(got).to(dev)       # the next op reads the device tensor this one produced
        keep.append(cur_dev)
        node.close()


def test_unsupported_fusions_and_formats(rt, dev):
    base = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tsummand=DT(tf.FLOAT), out_type=DT(tf.FLOAT),
                strides=[1, 1, 1, 1], padding="SAME", dilations=[1, 1, 1, 1], alpha=0.0)
    n = tf.Node("_QuantizedConv2D", dict(base, fused_ops=["BiasAdd", "Sum", "Relu", "Dequantize"]))
    assert n.code == tf.UNIMPLEMENTED and "Sum" in n.message
    n.close()
    n = tf.Node("_QuantizedConv2D", dict(base, fused_ops=["Dequantize"], data_format="NCHW"))
    assert n.code == tf.UNIMPLEMENTED
    n.close()
    n = tf.Node("_QuantizedConv2D", dict(base, fused_ops=["Requantize"]))
    assert n.code == tf.INVALID_ARGUMENT and "Requantize" in n.message
    n.close()
    n = tf.Node("_QuantizedConv2D", dict(base, fused_ops=["Dequantize"], strides=[1, 1, 1, 2]))
    assert n.code == tf.UNIMPLEMENTED
    n.close()
