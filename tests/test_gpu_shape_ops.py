"""Quantized Transpose / Reshape: itexhip_transpose through the C ABI against numpy's transpose (a library routine,
exact), the two op kernels through the plugin, and a whole INT8 attention block chained through the plugin's ops
against the oracle chain."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests.mock_tf import host as tf

pytestmark = pytest.mark.gpu
DT = tf.DType


def run_transpose(hip, dev, x, perm, off=0):
    import torch
    raw = torch.zeros(x.nbytes + 64, dtype=torch.uint8, device=dev)
    raw[off:off + x.nbytes] = torch.from_numpy(x.view(np.uint8).ravel()).to(dev)
    out = torch.full((max(x.nbytes, 1) + 64,), 0xEE, dtype=torch.uint8, device=dev)
    hip.transpose(raw.data_ptr() + off, out.data_ptr() + off, x.itemsize, x.shape, perm)
    torch.cuda.synchronize()
    got = out[off:off + x.nbytes].cpu().numpy().view(x.dtype).reshape([x.shape[p] for p in perm])
    assert int(out[off + x.nbytes]) == 0xEE            # nothing written past the end
    return got


@pytest.mark.parametrize("dtype", [np.int8, np.int32])
@pytest.mark.parametrize("shape,perm", [
    ((4, 128, 12, 64), (0, 2, 1, 3)),       # [B, S, H, D] -> [B, H, S, D]: 64-byte rows move whole
    ((4, 12, 128, 64), (0, 2, 1, 3)),
    ((3, 5, 7), (2, 1, 0)), ((3, 5, 7), (1, 0, 2)), ((3, 5, 7), (0, 1, 2)), ((3, 5, 7), (2, 0, 1)),
    ((6, 1, 20, 16), (2, 1, 0, 3)), ((2, 3, 4, 5, 6), (4, 2, 0, 3, 1)), ((100, 36), (1, 0)), ((17,), (0,)),
    ((2, 0, 5), (2, 1, 0)), ((1, 1, 1), (2, 0, 1)), ((2, 2, 2, 2, 2, 2, 2, 2), (7, 6, 5, 4, 3, 2, 1, 0)),
    ((5, 8, 20), (1, 0, 2)),                # 20-byte rows: 4-byte units for int8
])
def test_transpose_against_numpy(hip, dev, dtype, shape, perm):
    rng = np.random.default_rng(len(shape) * 10 + sum(perm))
    x = rng.integers(-128, 128, shape).astype(dtype)
    np.testing.assert_array_equal(run_transpose(hip, dev, x, perm), np.transpose(x, perm))


@pytest.mark.parametrize("off", [1, 4, 16])
def test_transpose_at_unaligned_addresses(hip, dev, off):
    x = np.random.default_rng(off).integers(-128, 128, (3, 16, 4, 32)).astype(np.int8)
    np.testing.assert_array_equal(run_transpose(hip, dev, x, (0, 2, 1, 3), off), np.transpose(x, (0, 2, 1, 3)))


def test_transpose_rejects_bad_permutations(hip, dev):
    import torch
    buf = torch.zeros(64, dtype=torch.int8, device=dev)
    with pytest.raises(hip.ItexHipError):
        hip.transpose(buf, buf, 1, (2, 4), (0, 0))
    with pytest.raises(hip.ItexHipError):
        hip.transpose(buf, buf, 2, (2, 4), (1, 0))


@pytest.fixture(scope="module")
def rt(dev):
    import torch
    tf.load()
    tf.use_torch_allocator(dev)
    return torch


def dev_in(torch, dev, a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def fetch(torch, out, np_dtype):
    dtype, shape, addr, _ = out
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    torch.cuda.synchronize()
    live = tf._state["alloc_cb"][2]
    if addr in live:
        return live[addr][:n * np.dtype(np_dtype).itemsize].cpu().numpy().view(np_dtype).copy().reshape(shape)
    return tf.read_host(addr, dtype, shape)


def run_node(torch, node, ins, outs):
    code, msg, res = node.run(ins, outs, stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    return res


def test_transpose_and_reshape_ops_through_plugin(rt, dev):
    torch = rt
    rng = np.random.default_rng(0)
    x = rng.integers(-128, 128, (2, 16, 4, 8)).astype(np.int8)
    mn, mx = np.array(-1.5, np.float32), np.array([2.5], np.float32)     # a scalar and a 1-element vector
    x_d = dev_in(torch, dev, x)
    perm = np.array([0, 2, 1, 3], np.int32)
    node = tf.Node("_QuantizedTranspose", dict(T=DT(tf.QINT8), Tperm=DT(tf.INT32)))
    assert node.code == tf.OK, node.message
    outs = run_node(torch, node, [(tf.QINT8, x.shape, x_d.data_ptr(), False), (tf.INT32, perm.shape, tf.host_array(perm), True),
                                  (tf.FLOAT, mn.shape, tf.host_array(mn), True), (tf.FLOAT, mx.shape, tf.host_array(mx), True)],
                    [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int8), np.transpose(x, perm))
    assert fetch(torch, outs[1], np.float32) == np.float32(-1.5) and fetch(torch, outs[2], np.float32).ravel()[0] == np.float32(2.5)
    assert tuple(outs[2][1]) == (1,)     # the range tensors keep their shape
    bad = np.array([0, 2, 2, 3], np.int32)
    code, msg, _ = node.run([(tf.QINT8, x.shape, x_d.data_ptr(), False), (tf.INT32, bad.shape, tf.host_array(bad), True),
                             (tf.FLOAT, mn.shape, tf.host_array(mn), True), (tf.FLOAT, mx.shape, tf.host_array(mx), True)],
                            [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.INVALID_ARGUMENT and "repeated" in msg
    node.close()

    rs = tf.Node("QuantizedReshape", dict(T=DT(tf.QINT8), Tshape=DT(tf.INT32)))
    assert rs.code == tf.OK, rs.message
    shape = np.array([32, -1], np.int32)
    outs = run_node(torch, rs, [(tf.QINT8, x.shape, x_d.data_ptr(), False), (tf.INT32, shape.shape, tf.host_array(shape), True),
                                (tf.FLOAT, mn.shape, tf.host_array(mn), True), (tf.FLOAT, mx.shape, tf.host_array(mx), True)],
                    [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    assert tuple(outs[0][1]) == (32, 32)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int8), x.reshape(32, 32))
    assert tuple(outs[1][1]) == () and fetch(torch, outs[2], np.float32) == np.float32(2.5)
    # with a forwardable input the output is the same buffer (no copy), as TensorFlow's Reshape
    outs = run_node(torch, rs, [(tf.QINT8, x.shape, x_d.data_ptr(), False, True), (tf.INT32, shape.shape, tf.host_array(shape), True),
                                (tf.FLOAT, mn.shape, tf.host_array(mn), True), (tf.FLOAT, mx.shape, tf.host_array(mx), True)],
                    [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    assert outs[0][2] == x_d.data_ptr() and outs[0][3] == 0 and tuple(outs[0][1]) == (32, 32)
    wrong = np.array([7, -1], np.int32)
    code, msg, _ = rs.run([(tf.QINT8, x.shape, x_d.data_ptr(), False), (tf.INT32, wrong.shape, tf.host_array(wrong), True),
                           (tf.FLOAT, mn.shape, tf.host_array(mn), True), (tf.FLOAT, mx.shape, tf.host_array(mx), True)],
                          [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.INVALID_ARGUMENT and "multiple of 7" in msg
    rs.close()


def test_int8_attention_block_through_the_plugin(rt, dev):
    """QuantizeV2 -> three _QuantizedMatMul [BiasAdd, Requantize] (Q, K, V) -> QuantizedReshape -> _QuantizedTranspose ->
    _QuantizedBatchMatMul [Mul, Add, Dequantize] (Q.K^T, scale, mask) -> softmax on the host -> QuantizeV2 ->
    _QuantizedBatchMatMul (P.V) -> the context in fp32.  Every op runs through its plugin kernel on the GPU; the
    same chain through the oracle must give identical bits at every step, and the result must be close to the
    fp32 attention."""
    torch = rt
    rng = np.random.default_rng(77)
    B, S, H, D = 2, 32, 4, 64
    E = H * D
    stream = torch.cuda.current_stream().cuda_stream
    x = rng.standard_normal((B * S, E)).astype(np.float32)
    W = [(rng.standard_normal((E, E)) * 0.06).astype(np.float32) for _ in range(3)]
    bias = [(rng.standard_normal(E) * 0.05).astype(np.float32) for _ in range(3)]
    mask = np.where(rng.random((B, 1, 1, S)) < 0.2, np.float32(-10000.0), np.float32(0.0)).astype(np.float32)
    keep = []

    def host(v):
        a = np.array(v, np.float32)
        keep.append(a)
        return (tf.FLOAT, a.shape, tf.host_array(a), True)

    def dev_t(a, dtype):
        t = dev_in(torch, dev, a)
        keep.append(t)
        return (dtype, a.shape, t.data_ptr(), False)

    # ---- QuantizeV2 (MIN_FIRST, quint8)
    qn = tf.Node("QuantizeV2", dict(T=DT(tf.QUINT8), mode="MIN_FIRST", round_mode="HALF_AWAY_FROM_ZERO", narrow_range=False, axis=-1,
                                    ensure_minimum_range=0.01))
    outs = run_node(torch, qn, [dev_t(x, tf.FLOAT), host(x.min()), host(x.max())], [(tf.QUINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    xq = fetch(torch, outs[0], np.uint8)
    xmn, xmx = float(fetch(torch, outs[1], np.float32)), float(fetch(torch, outs[2], np.float32))
    _, xq_ref, omn, omx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    np.testing.assert_array_equal(xq, xq_ref)
    assert (xmn, xmx) == (float(omn[0]), float(omx[0]))

    # ---- Q, K, V projections, requantized to qint8
    V2 = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tout=DT(tf.QINT8), transpose_a=False, transpose_b=False,
              is_weight_const=True, is_bias_const=True, input_quant_mode="MIN_FIRST", output_quant_mode="SCALED",
              leakyrelu_alpha=0.2, fused_ops=["BiasAdd", "Requantize"])
    heads, ranges = [], []
    for w, b in zip(W, bias):
        r = np.abs(w).max(0).astype(np.float32)
        _, wq, wmn, wmx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
        full = x @ w + b
        ro = np.float32(np.abs(full).max())
        node = tf.Node("_QuantizedMatMul", V2)
        assert node.code == tf.OK, node.message
        outs = run_node(torch, node, [dev_t(xq, tf.QUINT8), dev_t(wq, tf.QINT8), dev_t(b, tf.FLOAT), host(xmn), host(xmx), host(wmn),
                                      host(wmx), host(-ro), host(ro)], [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
        y = fetch(torch, outs[0], np.int8)
        at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.QINT8, input_mode=orc.MIN_FIRST, has_requantize=True)
        _, y_ref = orc.qmatmul(at, xq, wq, b, xmn, xmx, wmn, wmx, -ro, ro)
        np.testing.assert_array_equal(y, y_ref)
        # [B*S, E] -> [B, S, H, D] -> [B, H, S, D]
        rs = tf.Node("QuantizedReshape", dict(T=DT(tf.QINT8), Tshape=DT(tf.INT32)))
        shp = np.array([B, S, H, D], np.int32)
        keep.append(shp)
        outs = run_node(torch, rs, [dev_t(y, tf.QINT8), (tf.INT32, shp.shape, tf.host_array(shp), True), host(-ro), host(ro)],
                        [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
        y4 = fetch(torch, outs[0], np.int8)
        tr = tf.Node("_QuantizedTranspose", dict(T=DT(tf.QINT8), Tperm=DT(tf.INT32)))
        pm = np.array([0, 2, 1, 3], np.int32)
        keep.append(pm)
        outs = run_node(torch, tr, [dev_t(y4, tf.QINT8), (tf.INT32, pm.shape, tf.host_array(pm), True), host(-ro), host(ro)],
                        [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
        h = fetch(torch, outs[0], np.int8)
        np.testing.assert_array_equal(h, y_ref.reshape(B, S, H, D).transpose(0, 2, 1, 3))
        heads.append(h)
        ranges.append(float(ro))
        for n in (node, rs, tr):
            n.close()
    q, k, v = heads

    # ---- scores = Q.K^T * 1/sqrt(D) + mask, dequantized
    bmm = dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), U=DT(tf.FLOAT), Tout=DT(tf.FLOAT), adj_x=False, input_quant_mode="SCALED",
               output_quant_mode="SCALED")
    mul = np.array([1.0 / np.sqrt(D)], np.float32)
    n1 = tf.Node("_QuantizedBatchMatMul", dict(bmm, adj_y=True, fused_ops=["Mul", "Add", "Dequantize"]))
    assert n1.code == tf.OK, n1.message
    outs = run_node(torch, n1, [dev_t(q, tf.QINT8), dev_t(k, tf.QINT8), dev_t(mul, tf.FLOAT), dev_t(mask, tf.FLOAT), host(-ranges[0]),
                                host(ranges[0]), host(-ranges[1]), host(ranges[1])], [(tf.FLOAT, False)])
    scores = fetch(torch, outs[0], np.float32)
    _, scores_ref = orc.qbatch_matmul(q, k, -ranges[0], ranges[0], -ranges[1], ranges[1], adj_y=True,
                                      binary=((orc.BIN_MUL, mul), (orc.BIN_ADD, mask)))
    np.testing.assert_array_equal(scores, scores_ref)

    # ---- softmax (not part of the INT8 path: host), probabilities requantized SCALED to qint8
    e = np.exp(scores - scores.max(-1, keepdims=True))
    probs = (e / e.sum(-1, keepdims=True)).astype(np.float32)
    qp = tf.Node("QuantizeV2", dict(T=DT(tf.QINT8), mode="SCALED", round_mode="HALF_TO_EVEN", narrow_range=False, axis=-1,
                                    ensure_minimum_range=0.01))
    outs = run_node(torch, qp, [dev_t(probs, tf.FLOAT), host(0.0), host(1.0)], [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    pq = fetch(torch, outs[0], np.int8)
    pmn, pmx = float(fetch(torch, outs[1], np.float32)), float(fetch(torch, outs[2], np.float32))
    _, pq_ref, _, _ = orc.quantize_v2(probs, 0.0, 1.0, orc.QINT8, orc.SCALED)
    np.testing.assert_array_equal(pq, pq_ref)

    # ---- context = P.V
    n2 = tf.Node("_QuantizedBatchMatMul", dict(bmm, adj_y=False, fused_ops=["Dequantize"]))
    outs = run_node(torch, n2, [dev_t(pq, tf.QINT8), dev_t(v, tf.QINT8), host(pmn), host(pmx), host(-ranges[2]), host(ranges[2])],
                    [(tf.FLOAT, False)])
    ctx = fetch(torch, outs[0], np.float32)
    _, ctx_ref = orc.qbatch_matmul(pq, v, pmn, pmx, -ranges[2], ranges[2])
    np.testing.assert_array_equal(ctx, ctx_ref)

    # ---- against fp32 attention
    def split(t):
        return t.reshape(B, S, H, D).transpose(0, 2, 1, 3)
    qf, kf, vf = (split(x @ w + b) for w, b in zip(W, bias))
    sf = qf @ kf.transpose(0, 1, 3, 2) / np.sqrt(D) + mask
    ef = np.exp(sf - sf.max(-1, keepdims=True))
    ref = (ef / ef.sum(-1, keepdims=True)) @ vf
    err = np.abs(ctx - ref).max()
    assert err < 0.06 * np.abs(ref).max(), (err, np.abs(ref).max())
    for n in (qn, n1, qp, n2):
        n.close()
