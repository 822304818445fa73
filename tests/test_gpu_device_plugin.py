"""GPU tests of the StreamExecutor half of the plugin (SE_InitPlugin): device discovery, the arena
allocator over hipMalloc, streams / events / host callbacks, copies and fills, and the quantized op
chain run entirely on memory and a stream that the plugin itself created (no PyTorch tensors)."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests.mock_tf import host as tf

pytestmark = pytest.mark.gpu
DT = tf.DType


@pytest.fixture(scope="module")
def plug(dev):
    rc, p = tf.load_device()
    assert rc == 0, p.error()
    return p


def test_platform_and_device_description(plug):
    d = plug.describe()
    assert d["platform_name"] == d["platform_type"] == tf._state["device"]
    assert d["use_bfc_allocator"] == 0 and d["ordinal"] == 0 and d["vendor"] == "AMD"
    assert "gfx950" in d["hardware_name"] and d["pci_bus_id"]
    assert d["memory_bandwidth"] == 8 * 10 ** 12


def test_copies_fills_and_allocator_accounting(plug):
    before = plug.stats()
    rng = np.random.default_rng(0)
    a = rng.integers(0, 256, 1 << 20, dtype=np.uint8)
    p = plug.upload(a)                 # stream-ordered copy
    q = plug.upload(a[::-1], sync=True)
    assert p % 256 == 0 and q % 256 == 0 and p != q
    np.testing.assert_array_equal(plug.download(p, np.uint8, a.shape), a)
    np.testing.assert_array_equal(plug.download(q, np.uint8, a.shape, sync=True), a[::-1])
    plug.copy(q, p, a.nbytes)          # device to device on the stream
    np.testing.assert_array_equal(plug.download(q, np.uint8, a.shape), a)
    plug.copy(q + 3, p + 1, 1001, sync=True)   # unaligned, synchronous
    expect = a.copy()
    expect[3:1004] = a[1:1002]
    np.testing.assert_array_equal(plug.download(q, np.uint8, a.shape), expect)
    plug.memset(p, 0, 0, 4096)         # mem_zero
    plug.memset(p + 4096 + 1, 8, 0xab, 1003)   # byte fill, unaligned start and length
    plug.memset(p + 8192, 32, 0xdeadbeef, 64)  # 32-bit fill
    got = plug.download(p, np.uint8, a.shape)
    expect = a.copy()
    expect[:4096] = 0
    expect[4097:4097 + 1003] = 0xab
    expect[8192:8256] = np.frombuffer(np.uint32([0xdeadbeef] * 16).tobytes(), np.uint8)
    np.testing.assert_array_equal(got, expect)
    mid = plug.stats()
    assert mid["bytes_in_use"] == before["bytes_in_use"] + 2 * (1 << 20)
    assert mid["num_allocs"] == before["num_allocs"] + 2
    assert mid["bytes_reserved"] >= 1 << 30 and mid["device_total"] > 200 * (1 << 30)
    plug.free(p)
    plug.free(q)
    after = plug.stats()
    assert after["bytes_in_use"] == before["bytes_in_use"]
    assert after["bytes_reserved"] == mid["bytes_reserved"]     # regions are kept for reuse
    r = plug.alloc(1 << 20)
    assert r in (p, q)                 # the freed block is handed out again (best fit)
    plug.free(r)


def test_streams_events_and_host_callback(plug):
    n = 1 << 16
    a, b = plug.alloc(n), plug.alloc(n)
    host = np.zeros(n, np.uint8)
    rc = plug.lib.mock_device_stream_event_test(a, b, n, host.ctypes.data)
    assert rc == 0, (rc, plug.error())
    assert (host == 0x5a).all()
    plug.free(a)
    plug.free(b)


def test_quantized_linear_on_plugin_memory_and_stream(plug):
    """QuantizeV2 -> _QuantizedMatMul [BiasAdd, Relu, Dequantize] with every device tensor, temporary and
    host-pinned min/max tensor allocated by the plugin and all work on the plugin's stream."""
    tf.load()
    plug.use_for_tensors()
    M, K, N = 96, 512, 320
    rng = np.random.default_rng(5)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    r = np.abs(w).max(0).astype(np.float32)
    _, wq, wmn, wmx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    x_d, w_d, b_d = plug.upload(x), plug.upload(wq), plug.upload(bias)
    mn, mx = np.array(x.min(), np.float32), np.array(x.max(), np.float32)

    qnode = tf.Node("QuantizeV2", dict(T=DT(tf.QUINT8), mode="MIN_FIRST", round_mode="HALF_AWAY_FROM_ZERO",
                                        narrow_range=False, axis=-1, ensure_minimum_range=0.01))
    assert qnode.code == tf.OK, qnode.message
    code, msg, outs = qnode.run([(tf.FLOAT, x.shape, x_d, False), (tf.FLOAT, (), tf.host_array(mn), True),
                                 (tf.FLOAT, (), tf.host_array(mx), True)],
                                [(tf.QUINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=plug.stream)
    assert code == tf.OK, msg
    xq_d = outs[0][2]
    plug.sync()
    omn = tf.read_host(outs[1][2], tf.FLOAT, ()).copy()
    omx = tf.read_host(outs[2][2], tf.FLOAT, ()).copy()
    xq = plug.download(xq_d, np.uint8, (M, K))
    _, xq_ref, omn_ref, omx_ref = orc.quantize_v2(x, mn, mx, orc.QUINT8, orc.MIN_FIRST)
    np.testing.assert_array_equal(xq, xq_ref)
    assert omn == omn_ref[0] and omx == omx_ref[0]

    mnode = tf.Node("_QuantizedMatMul", dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tout=DT(tf.FLOAT),
                                              transpose_a=False, transpose_b=False, is_weight_const=True, is_bias_const=True,
                                              input_quant_mode="MIN_FIRST", output_quant_mode="SCALED", leakyrelu_alpha=0.2,
                                              fused_ops=["BiasAdd", "Relu", "Dequantize"]))
    assert mnode.code == tf.OK, mnode.message
    ins = [(tf.QUINT8, (M, K), xq_d, False), (tf.QINT8, (K, N), w_d, False), (tf.FLOAT, (N,), b_d, False),
           (tf.FLOAT, (), tf.host_array(omn), True), (tf.FLOAT, (), tf.host_array(omx), True),
           (tf.FLOAT, (N,), tf.host_array(wmn), True), (tf.FLOAT, (N,), tf.host_array(wmx), True)]
    in_use = []
    for it in range(2):
        code, msg, outs2 = mnode.run(ins, [(tf.FLOAT, False)], stream=plug.stream)
        assert code == tf.OK, msg
        y = plug.download(outs2[0][2], np.float32, (M, N))
        at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST,
                              activation=orc.ACT_RELU, has_dequantize=True)
        _, y_ref = orc.qmatmul(at, xq_ref, wq, bias, omn, omx, wmn, wmx)
        np.testing.assert_array_equal(y, y_ref)
        in_use.append(plug.stats()["bytes_in_use"])
    assert in_use[0] == in_use[1]      # steady state: the second run allocates nothing new
    mnode.close()
    qnode.close()
    for p in (x_d, w_d, b_d):
        plug.free(p)
