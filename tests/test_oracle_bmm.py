"""Pins the CPU oracle's quantized BatchMatMul restatement.

  * integer products and broadcasting: numpy int64 matmul on broadcast operands (a library routine, exact);
  * the output scale and the post-op order: the three cases held by the reference's
    quantized_batch_matmul_test.py (plain, Mul, Mul + Add) must reproduce the fp32 graph within the reference's
    own tolerance and, tighter, within what the two quantization steps allow -- a dropped factor, a swapped
    Mul / Add or a wrong range misses that bound;
  * separately rounded fp32 post-ops: a case where (v * t) + u differs from fma(v, t, u);
  * 16-bit outputs: nearest-even conversion of the float result (PyTorch / numpy conversions).
"""
import numpy as np
import pytest

from oracle import pyoracle as orc


def quant(x):
    r = np.float32(np.abs(x).max())
    _, q, mn, mx = orc.quantize_v2(x, x.min(), x.max(), orc.QINT8, orc.SCALED)
    return q, np.float32(mn[0]), np.float32(mx[0]), r


@pytest.mark.parametrize("xs,ys,adj_x,adj_y", [
    ((2, 3, 5, 7), (2, 3, 7, 4), False, False),
    ((2, 3, 7, 5), (2, 3, 4, 7), True, True),
    ((4, 1, 6, 9), (1, 5, 9, 3), False, False),      # both operands broadcast
    ((6, 9), (3, 2, 11, 9), False, True),             # rank-2 x against a rank-4 y
    ((3, 8, 2), (8, 5), True, False),
    ((1, 1, 1), (1, 1, 1), False, False),
    ((2, 0, 4), (2, 4, 3), False, False),             # empty M
    ((2, 3, 0), (2, 0, 3), False, False),             # empty K: zeros times the scale
])
def test_integer_product_and_broadcast_against_numpy(xs, ys, adj_x, adj_y):
    rng = np.random.default_rng(sum(xs) + sum(ys))
    x = rng.integers(-128, 128, xs).astype(np.int8)
    y = rng.integers(-128, 128, ys).astype(np.int8)
    st, out = orc.qbatch_matmul(x, y, -2.0, 1.5, -0.25, 0.75, adj_x, adj_y)
    assert st == orc.OK
    xm = np.swapaxes(x, -1, -2) if adj_x else x
    ym = np.swapaxes(y, -1, -2) if adj_y else y
    acc = np.matmul(xm.astype(np.int64), ym.astype(np.int64))
    scale = np.float32(np.float32(2.0) * np.float32(0.75)) / np.float32(127 * 127)
    np.testing.assert_array_equal(out, acc.astype(np.float32) * scale)
    assert out.shape == acc.shape


@pytest.mark.parametrize("case", ["plain", "mul", "mul_add"])
def test_reference_cases(golden, case):
    g = golden["batch_matmul"]
    x, y, add = (np.array(g[k], np.float32) for k in ("x", "y", "add"))
    mul = np.float32(g["mul"])
    xq, xmn, xmx, rx = quant(x)
    yq, ymn, ymx, ry = quant(y)
    binary = {"plain": (), "mul": ((orc.BIN_MUL, np.float32([mul])),),
              "mul_add": ((orc.BIN_MUL, np.float32([mul])), (orc.BIN_ADD, add))}[case]
    st, out = orc.qbatch_matmul(xq, yq, xmn, xmx, ymn, ymx, binary=binary)
    assert st == orc.OK
    ref = np.matmul(x, y)
    if case != "plain":
        ref = ref * mul
    if case == "mul_add":
        ref = ref + add
    np.testing.assert_allclose(out, ref, rtol=g["tolerance"], atol=g["tolerance"])
    # each operand is off by at most half a step; K = 3 products
    K = x.shape[-1]
    bound = K * (rx / 254 * np.abs(y).max() + ry / 254 * np.abs(x).max() + rx * ry / 254 / 254) * (mul if case != "plain" else 1)
    assert np.abs(out - ref).max() <= bound + 1e-6
    assert np.abs(out - ref).max() > 0   # the quantization error is visible: the product did go through int8


def test_post_ops_apply_in_order_and_round_separately():
    rng = np.random.default_rng(5)
    x = rng.integers(-128, 128, (3, 4, 16)).astype(np.int8)
    y = rng.integers(-128, 128, (3, 16, 5)).astype(np.int8)
    t = rng.standard_normal((3, 4, 5)).astype(np.float32)
    u = rng.standard_normal((3, 1, 5)).astype(np.float32)      # broadcast along M
    _, base = orc.qbatch_matmul(x, y, -1.0, 1.0, -1.0, 1.0)
    _, ma = orc.qbatch_matmul(x, y, -1.0, 1.0, -1.0, 1.0, binary=((orc.BIN_MUL, t), (orc.BIN_ADD, u)))
    _, am = orc.qbatch_matmul(x, y, -1.0, 1.0, -1.0, 1.0, binary=((orc.BIN_ADD, u), (orc.BIN_MUL, t)))
    np.testing.assert_array_equal(ma, base * t + u)            # numpy rounds each fp32 operation
    np.testing.assert_array_equal(am, (base + u) * t)
    assert not np.array_equal(ma, am)
    fused = (base.astype(np.float64) * t + u).astype(np.float32)
    assert not np.array_equal(ma, fused)                       # not a fused multiply-add


def test_binary_operand_shapes():
    x = np.ones((2, 3, 4, 8), np.int8)
    y = np.ones((2, 3, 8, 5), np.int8)
    for shape in [(2, 3, 4, 5), (1, 1, 1, 1), (2, 1, 4, 1), (1, 3, 1, 5), (1,)]:
        t = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
        st, out = orc.qbatch_matmul(x, y, -127.0, 127.0, -127.0, 127.0, binary=((orc.BIN_ADD, t),))
        assert st == orc.OK
        np.testing.assert_array_equal(out, np.float32(8) + np.broadcast_to(t.reshape(shape if len(shape) == 4 else (1, 1, 1, 1)),
                                                                         (2, 3, 4, 5)))
    st, _ = orc.qbatch_matmul(x, y, -1.0, 1.0, -1.0, 1.0, binary=((orc.BIN_ADD, np.zeros((4, 5), np.float32)),))
    assert st == orc.INVALID_ARGUMENT     # lower rank than the output and more than one element
    st, _ = orc.qbatch_matmul(x, y, -1.0, 1.0, -1.0, 1.0, binary=((orc.BIN_ADD, np.zeros((2, 3, 4, 2), np.float32)),))
    assert st == orc.INVALID_ARGUMENT
    st, _ = orc.qbatch_matmul(x, np.ones((2, 3, 7, 5), np.int8), -1.0, 1.0, -1.0, 1.0)
    assert st == orc.INVALID_ARGUMENT     # inner dimensions differ
    st, _ = orc.qbatch_matmul(x, np.ones((4, 3, 8, 5), np.int8), -1.0, 1.0, -1.0, 1.0)
    assert st == orc.INVALID_ARGUMENT     # batch dimensions do not broadcast


@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_16_bit_output_and_operands(T16):
    import torch
    tt = torch.bfloat16 if T16 == orc.BFLOAT16 else torch.float16
    rng = np.random.default_rng(9)
    x = rng.integers(-128, 128, (2, 9, 32)).astype(np.int8)
    y = rng.integers(-128, 128, (2, 32, 6)).astype(np.int8)
    t16 = torch.from_numpy(rng.standard_normal((2, 9, 6)).astype(np.float32)).to(tt)
    t32 = t16.to(torch.float32).numpy()
    _, o32 = orc.qbatch_matmul(x, y, -3.0, 3.0, -2.0, 2.0, binary=((orc.BIN_ADD, t32),))
    st, o16 = orc.qbatch_matmul(x, y, -3.0, 3.0, -2.0, 2.0, binary=((orc.BIN_ADD, t16.view(torch.int16).numpy().view(np.uint16)),),
                                t_out=T16)
    assert st == orc.OK
    np.testing.assert_array_equal(o16, torch.from_numpy(o32).to(tt).view(torch.int16).numpy().view(np.uint16))
