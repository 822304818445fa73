"""GPU tests of the kernel plugin through the mock TensorFlow host: the ops are created from node
attributes and run with device tensors and host-memory min/max tensors, exactly as TensorFlow would
call them; results are compared bit for bit with the CPU oracle."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests.mock_tf import host as tf

pytestmark = pytest.mark.gpu
DT = tf.DType


@pytest.fixture(scope="module")
def rt(dev):
    import torch
    tf.load()
    tf.use_torch_allocator(dev)
    return torch


def dev_in(torch, dev, a):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    return t


def fetch(torch, out, np_dtype):
    """Copies an output tensor of the mock (device or host memory) into numpy."""
    dtype, shape, addr, _ = out
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    import ctypes as C
    torch.cuda.synchronize()
    host = np.empty(n, np_dtype)
    # device memory handed out by the torch allocator: wrap it through a uint8 view
    live = tf._state["alloc_cb"][2]
    if addr in live:
        nbytes = n * np.dtype(np_dtype).itemsize
        host = live[addr][:nbytes].cpu().numpy().view(np_dtype).copy()
    else:
        host = tf.read_host(addr, dtype, shape).ravel()
    return host.reshape(shape)


def run_quantize(torch, dev, x, mn, mx, T, mode, axis=-1, classic=None, forward=False, op="QuantizeV2", narrow_range=False):
    attrs = dict(T=DT(T), mode=mode, round_mode="HALF_TO_EVEN" if mode == "SCALED" else "HALF_AWAY_FROM_ZERO",
                 narrow_range=bool(narrow_range), axis=axis, ensure_minimum_range=0.01)
    if op == "_ITEXQuantizeV2":
        attrs["dtype"] = DT(tf.FLOAT)
        if classic is not None:
            attrs["classic_asymmetric_algorithm"] = bool(classic)
    node = tf.Node(op, attrs)
    assert node.code == tf.OK, node.message
    x_d = dev_in(torch, dev, x)
    mn_h = np.atleast_1d(np.float32(mn)).copy() if axis >= 0 else np.array(mn, np.float32)
    mx_h = np.atleast_1d(np.float32(mx)).copy() if axis >= 0 else np.array(mx, np.float32)
    code, msg, outs = node.run(
        [(tf.FLOAT, x.shape, x_d.data_ptr(), False), (tf.FLOAT, mn_h.shape, tf.host_array(mn_h), True, forward),
         (tf.FLOAT, mx_h.shape, tf.host_array(mx_h), True, forward)],
        [(T, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    q = fetch(torch, outs[0], tf.NP_OF[T])
    omn = fetch(torch, outs[1], np.float32)
    omx = fetch(torch, outs[2], np.float32)
    fwd = (outs[1][3], outs[2][3])
    node.close()
    return q, omn, omx, fwd, (mn_h, mx_h)


def test_quantize_golden_through_plugin(rt, dev, golden):
    torch = rt
    T = {"quint8": tf.QUINT8, "qint8": tf.QINT8}
    for case in golden["quantize_v2"]:
        x = np.array(case["x"], np.float32).reshape(case["shape"])
        op = "_ITEXQuantizeV2" if case["classic_asymmetric_algorithm"] else "QuantizeV2"
        q, omn, omx, _, _ = run_quantize(torch, dev, x, case["min_range"], case["max_range"], T[case["T"]], case["mode"],
                                         classic=case["classic_asymmetric_algorithm"] or None, op=op)
        assert q.ravel().tolist() == case["expected"], case["source"]


def test_quantize_axis_golden_through_plugin(rt, dev, golden):
    torch = rt
    g = golden["quantize_v2_axis"]
    shape = np.array(g["shape"])
    values = np.array(g["values"], np.float32)
    quant = np.array(g["quant_values"], np.int32)
    expected = np.take(quant, np.remainder(np.arange(np.prod(shape)), len(quant))).reshape(shape)
    for axis in (1, 2, 3):
        x = np.take(values, np.remainder(np.arange(np.prod(shape)), len(values))).reshape(shape)
        sc = [1] * 4
        sc[axis] = shape[axis]
        x = (x * np.arange(1, shape[axis] + 1).reshape(sc)).astype(np.float32)
        mn = [g["min_unit"] * (s + 1) for s in range(shape[axis])]
        mx = [g["max_unit"] * (s + 1) for s in range(shape[axis])]
        q, omn, omx, _, _ = run_quantize(torch, dev, x, mn, mx, tf.QINT8, "SCALED", axis=axis)
        np.testing.assert_array_equal(q.astype(np.int32), expected)
        np.testing.assert_array_equal(omx, np.abs(np.float32(mn)))
        np.testing.assert_array_equal(omn, -omx)


@pytest.mark.parametrize("forward", [False, True])
def test_quantize_outputs_and_forwarding(rt, dev, forward):
    """output_min/max: adjusted range; with forwarding the kernel overwrites the caller's min/max
    tensors in place (forward_input_or_allocate_output in the reference)."""
    torch = rt
    x = np.random.default_rng(0).standard_normal(4099).astype(np.float32)
    q, omn, omx, fwd, (mn_h, mx_h) = run_quantize(torch, dev, x, 0.5, 2.0, tf.QUINT8, "SCALED", forward=forward)
    _, q_ref, omn_ref, omx_ref = orc.quantize_v2(x, 0.5, 2.0, orc.QUINT8, orc.SCALED)
    np.testing.assert_array_equal(q, q_ref)
    assert omn == omn_ref[0] == 0.0 and omx == omx_ref[0] == 2.0
    if forward:
        assert fwd == (1, 2) and mn_h == 0.0 and mx_h == 2.0  # input buffers were reused and rewritten
    else:
        assert fwd == (-1, -1) and mn_h == np.float32(0.5)


@pytest.mark.parametrize("T,mode,classic", [(tf.QUINT8, "MIN_FIRST", False), (tf.QUINT8, "MIN_FIRST", True), (tf.QINT8, "SCALED", False),
                                            (tf.QUINT8, "SCALED", False)])
def test_dynamic_range_quantize_through_plugin(rt, dev, T, mode, classic):
    """_ITEXQuantizeV2DynamicRange (what the graph pass makes of Min / Max -> QuantizeV2): the range is the tensor's own,
    found on the device; output and output_min / output_max equal QuantizeV2 fed with numpy's min and max."""
    torch = rt
    rng = np.random.default_rng(11)
    for n, shift in ((70001, 0.3), (5, -2.0), (1, 1.5)):
        x = (rng.standard_normal(n) * 3 + shift).astype(np.float32)
        node = tf.Node("_ITEXQuantizeV2DynamicRange",
                       dict(T=DT(T), mode=mode, round_mode="HALF_TO_EVEN" if mode == "SCALED" else "HALF_AWAY_FROM_ZERO",
                            narrow_range=False, axis=-1, ensure_minimum_range=0.01, dtype=DT(tf.FLOAT),
                            classic_asymmetric_algorithm=classic))
        assert node.code == tf.OK, node.message
        x_d = dev_in(torch, dev, x)
        code, msg, outs = node.run([(tf.FLOAT, x.shape, x_d.data_ptr(), False)], [(T, False), (tf.FLOAT, True), (tf.FLOAT, True)],
                                   stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        q = fetch(torch, outs[0], tf.NP_OF[T])
        omode = orc.SCALED if mode == "SCALED" else orc.MIN_FIRST
        _, q_ref, omn_ref, omx_ref = orc.quantize_v2(x, x.min(), x.max(), T, omode, classic=classic)
        np.testing.assert_array_equal(q, q_ref)
        assert float(np.ravel(fetch(torch, outs[1], np.float32))[0]) == omn_ref[0]
        assert float(np.ravel(fetch(torch, outs[2], np.float32))[0]) == omx_ref[0]
        node.close()


@pytest.mark.parametrize("T,mode", [(tf.QUINT8, "MIN_FIRST"), (tf.QINT8, "SCALED")])
@pytest.mark.parametrize("M,K,N", [(100, 256, 200), (8, 1024, 512), (37, 75, 61)])
def test_dynamic_input_matmul_through_plugin(rt, dev, T, mode, M, K, N):
    """_ITEXQuantizedMatMulDynamicInput (what the graph pass makes of _ITEXQuantizeV2DynamicRange -> _ITEXQuantizedMatMul):
    float activations in, the result of the two separate ops out - Dequantize and Requantize outputs, MFMA kernels and
    (K = 75) the kernel on the unpacked weight; the second run reuses the node's cached weight."""
    torch = rt
    x, w, bias, _, _, _, wq, wmn, wmx = make_problem(M, K, N, seed=M + N)
    omode = orc.SCALED if mode == "SCALED" else orc.MIN_FIRST
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), T, omode)
    r_out = np.float32(np.abs(x @ w + bias).max())
    keep = [dev_in(torch, dev, x), dev_in(torch, dev, wq), dev_in(torch, dev, bias)]
    base = [(tf.FLOAT, x.shape, keep[0].data_ptr(), False), (tf.QINT8, wq.shape, keep[1].data_ptr(), False),
            (tf.FLOAT, bias.shape, keep[2].data_ptr(), False)]
    stream = torch.cuda.current_stream().cuda_stream
    for fused, t_out, host in ((["BiasAdd", "Relu", "Dequantize"], tf.FLOAT, [wmn, wmx]),
                               (["BiasAdd", "Requantize"], tf.QINT8, [wmn, wmx, np.float32(-r_out), np.float32(r_out)])):
        node = tf.Node("_ITEXQuantizedMatMulDynamicInput",
                       dict(V2, T1=DT(T), input_quant_mode=mode, Tout=DT(t_out), fused_ops=fused, ensure_minimum_range=0.01))
        assert node.code == tf.OK, node.message
        requant = t_out == tf.QINT8
        at = orc.matmul_attrs(api=orc.API_V2, t_in=T, t_out=t_out, input_mode=omode, has_dequantize=not requant,
                              has_requantize=requant, activation=orc.ACT_NONE if requant else orc.ACT_RELU)
        st, ref = orc.qmatmul(at, xq, wq, bias, xmn[0], xmx[0], wmn, wmx, -r_out if requant else 0.0, r_out if requant else 0.0)
        assert st == orc.OK
        ins = base + [(tf.FLOAT, np.shape(h), tf.host_array(np.asarray(h, np.float32)), True) for h in host]
        outs_spec = [(t_out, False)] + ([(tf.FLOAT, True), (tf.FLOAT, True)] if requant else [])
        for _ in range(2):
            code, msg, outs = node.run(ins, outs_spec, stream=stream)
            assert code == tf.OK, msg
            np.testing.assert_array_equal(fetch(torch, outs[0], tf.NP_OF[t_out]), ref)
        if requant:
            assert float(np.ravel(fetch(torch, outs[1], np.float32))[0]) == -r_out
            assert float(np.ravel(fetch(torch, outs[2], np.float32))[0]) == r_out
        node.close()


def test_quantized_matmul_transpose_a_as_written(rt, dev):
    """transpose_a = true: the reference takes batch and k from the swapped dimensions but describes the buffer as a
    row-major [batch, k] matrix (quantized_matmul_common.h:183-198), i.e. the [k, batch] tensor is reinterpreted, not
    transposed.  The plugin gives what the reference gives."""
    torch = rt
    M, K, N = 24, 64, 48
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=5)
    node = tf.Node("_QuantizedMatMul", dict(V2, transpose_a=True, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Dequantize"]))
    assert node.code == tf.OK, node.message
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True)
    _, ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
    as_k_by_m = xq.reshape(K, M)          # the same bytes, declared [k, batch]
    ins, keep = matmul_inputs(torch, dev, as_k_by_m, wq, bias, [xmn, xmx, wmn, wmx])
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    np.testing.assert_array_equal(fetch(torch, outs[0], np.float32), ref)
    node.close()


def test_graph_pass_output_runs_on_the_kernel(rt, dev):
    """x -> Reshape -> Min / Max -> QuantizeV2 -> _QuantizedMatMul through TF_InitGraph's optimizer, then the one node it
    leaves, built from the attributes and the input order of the rewritten NodeDef, on the device: equal to the two ops
    evaluated by the oracle."""
    import ctypes as C
    from tests.mock_tf import graphdef as gd
    from tests.test_graph_optimizer import dynamic_linear_graph
    torch = rt
    lib = tf.load()
    lib.mock_graph_result.restype = C.c_void_p
    lib.mock_graph_result_size.restype = C.c_size_t
    assert lib.mock_graph_init(tf.PLUGIN_LIB.encode()) == 0
    data = dynamic_linear_graph(emr=0.01).SerializeToString()
    assert lib.mock_graph_optimize(data, C.c_size_t(len(data))) == tf.OK
    out = gd.GraphDef()
    out.ParseFromString(C.string_at(lib.mock_graph_result(), lib.mock_graph_result_size()))
    mm = {n.name: n for n in out.node}["mm"]
    assert mm.op == "_ITEXQuantizedMatMulDynamicInput"
    attrs = {}
    for k, v in mm.attr.items():
        kind = v.WhichOneof("value")
        if kind == "type":
            attrs[k] = DT(v.type)
        elif kind == "s":
            attrs[k] = v.s.decode()
        elif kind in ("b", "f", "i"):
            attrs[k] = getattr(v, kind)
        elif kind == "list" and len(v.list.s):
            attrs[k] = [x.decode() for x in v.list.s]
    node = tf.Node(mm.op, dict(V2, **attrs))      # attributes the graph leaves at their defaults come from V2
    assert node.code == tf.OK, node.message
    M, K, N = 33, 128, 80
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=3)
    tensors = {"x": x, "w": wq, "b": bias, "wmn": wmn, "wmx": wmx}
    keep, ins = [], []
    n_dev = len(mm.attr["Tdevice_inputs"].list.type)
    data_inputs = [i for i in mm.input if not i.startswith("^")]
    assert len(data_inputs) == n_dev + len(mm.attr["Thost_inputs"].list.type)
    for pos, name in enumerate(data_inputs):
        t = tensors[name]
        dt = {np.float32: tf.FLOAT, np.int8: tf.QINT8}[t.dtype.type]
        if pos < n_dev:
            keep.append(dev_in(torch, dev, t))
            ins.append((dt, t.shape, keep[-1].data_ptr(), False))
        else:
            ins.append((dt, t.shape, tf.host_array(t), True))
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True)
    _, ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.float32), ref)
    node.close()


def test_dynamic_input_matmul_attr_validation(rt, dev):
    bad = tf.Node("_ITEXQuantizedMatMulDynamicInput", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Add", "Dequantize"]))
    assert bad.code == tf.INVALID_ARGUMENT
    bad = tf.Node("_ITEXQuantizedMatMulDynamicInput", dict(V2, T1=DT(tf.QINT8), Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Dequantize"]))
    assert bad.code == tf.INVALID_ARGUMENT and "quint8" in bad.message     # MIN_FIRST gives quint8


@pytest.mark.parametrize("fused,act", [("Tanh", orc.ACT_TANH), ("Sigmoid", orc.ACT_SIGMOID), ("_ITEXSwish", orc.ACT_SWISH)])
def test_quantized_matmul_transcendental_post_ops(rt, dev, fused, act):
    """_QuantizedMatMul [BiasAdd, Tanh | Sigmoid | _ITEXSwish, Dequantize] (a BERT pooler, gates): within 2e-6 of the oracle
    (the device evaluates exp with the hardware instruction)."""
    torch = rt
    M, K, N = 50, 256, 96
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=act)
    node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", fused, "Dequantize"]))
    assert node.code == tf.OK, node.message
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True,
                          activation=act)
    st, ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
    assert st == orc.OK
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [xmn, xmx, wmn, wmx])
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    np.testing.assert_allclose(fetch(torch, outs[0], np.float32), ref, rtol=2e-6, atol=1e-6)
    node.close()


def test_dequantize_through_plugin(rt, dev):
    torch = rt
    rng = np.random.default_rng(1)
    for T, mode in ((tf.QINT8, "SCALED"), (tf.QUINT8, "MIN_FIRST")):
        q = rng.integers(np.iinfo(tf.NP_OF[T]).min, np.iinfo(tf.NP_OF[T]).max + 1, 5003).astype(tf.NP_OF[T])
        node = tf.Node("Dequantize", dict(T=DT(T), mode=mode, narrow_range=False, axis=-1, dtype=DT(tf.FLOAT)))
        assert node.code == tf.OK, node.message
        mn, mx = np.array(-2.5, np.float32), np.array(3.25, np.float32)
        q_d = dev_in(torch, dev, q)
        code, msg, outs = node.run([(T, q.shape, q_d.data_ptr(), False), (tf.FLOAT, (), tf.host_array(mn), True),
                                    (tf.FLOAT, (), tf.host_array(mx), True)], [(tf.FLOAT, False)],
                                   stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        y = fetch(torch, outs[0], np.float32)
        _, y_ref = orc.dequantize(q, mn, mx, T, orc.SCALED if mode == "SCALED" else orc.MIN_FIRST)
        np.testing.assert_array_equal(y, y_ref)
        node.close()


def test_narrow_range_attr_changes_nothing_through_plugin(rt, dev):
    """narrow_range is parsed and never used by the reference (quantize_op.h:118; Dequantize reads it as an attribute of
    the op definition only): QuantizeV2 and Dequantize nodes built with narrow_range = true give the bytes, ranges and
    floats of the nodes built with false, -128 included for saturating inputs."""
    torch = rt
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(4099) * 1.5).astype(np.float32)
    x[:3] = [-50.0, 50.0, -1.0]    # saturate on both sides
    for T, mode in ((tf.QINT8, "SCALED"), (tf.QUINT8, "SCALED"), (tf.QUINT8, "MIN_FIRST")):
        a = run_quantize(torch, dev, x, -1.0, 1.0, T, mode, narrow_range=False)
        b = run_quantize(torch, dev, x, -1.0, 1.0, T, mode, narrow_range=True)
        np.testing.assert_array_equal(a[0], b[0])
        assert a[1] == b[1] and a[2] == b[2]
        if T == tf.QINT8:
            assert b[0][0] == -128 and b[0][1] == 127   # full range, not -127
        _, q_ref, omn, omx = orc.quantize_v2(x, -1.0, 1.0, T, orc.SCALED if mode == "SCALED" else orc.MIN_FIRST)
        np.testing.assert_array_equal(b[0], q_ref)
        ys = []
        for nr in (False, True):
            node = tf.Node("Dequantize", dict(T=DT(T), mode=mode, narrow_range=nr, axis=-1, dtype=DT(tf.FLOAT)))
            assert node.code == tf.OK, node.message
            mn, mx = np.array(omn[0], np.float32), np.array(omx[0], np.float32)
            q_d = dev_in(torch, dev, b[0])
            code, msg, outs = node.run([(T, b[0].shape, q_d.data_ptr(), False), (tf.FLOAT, (), tf.host_array(mn), True),
                                        (tf.FLOAT, (), tf.host_array(mx), True)], [(tf.FLOAT, False)],
                                       stream=torch.cuda.current_stream().cuda_stream)
            assert code == tf.OK, msg
            ys.append(fetch(torch, outs[0], np.float32))
            node.close()
        np.testing.assert_array_equal(ys[0], ys[1])
        _, y_ref = orc.dequantize(b[0], omn[0], omx[0], T, orc.SCALED if mode == "SCALED" else orc.MIN_FIRST)
        np.testing.assert_array_equal(ys[1], y_ref)


def make_problem(M, K, N, seed, per_channel=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    if per_channel:
        r = np.abs(w).max(0).astype(np.float32)
        _, wq, wmn, wmx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    else:
        _, wq, wmn, wmx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
        wmn, wmx = np.array(wmn[0], np.float32), np.array(wmx[0], np.float32)
    return x, w, bias, xq, np.array(xmn[0], np.float32), np.array(xmx[0], np.float32), wq, wmn, wmx


def matmul_inputs(torch, dev, xq, wq, bias, scalars):
    keep = [dev_in(torch, dev, xq), dev_in(torch, dev, wq), dev_in(torch, dev, bias)]
    ins = [(tf.QUINT8 if xq.dtype == np.uint8 else tf.QINT8, xq.shape, keep[0].data_ptr(), False),
           (tf.QINT8, wq.shape, keep[1].data_ptr(), False), (tf.FLOAT, bias.shape, keep[2].data_ptr(), False)]
    for s in scalars:
        ins.append((tf.FLOAT, s.shape, tf.host_array(s), True))
    return ins, keep


V2 = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), transpose_a=False, transpose_b=False,
          is_weight_const=True, is_bias_const=True, input_quant_mode="MIN_FIRST", output_quant_mode="SCALED",
          leakyrelu_alpha=0.2)


@pytest.mark.parametrize("M,K,N", [(4, 64, 32), (100, 256, 200), (16, 1024, 512), (2, 3, 4)])
def test_quantized_matmul_v2_dequantize(rt, dev, M, K, N):
    torch = rt
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=M + K)
    node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Relu", "Dequantize"]))
    assert node.code == tf.OK, node.message
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST,
                          activation=orc.ACT_RELU, has_dequantize=True)
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [xmn, xmx, wmn, wmx])
    stream = torch.cuda.current_stream().cuda_stream
    for it in range(2):  # second run exercises the cached weight / parameter state
        code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=stream)
        assert code == tf.OK, msg
        y = fetch(torch, outs[0], np.float32)
        _, y_ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
        np.testing.assert_array_equal(y, y_ref)
    first = node.temp_allocs()
    # a new activation range must be picked up without re-preparing the weight
    xmn2, xmx2 = np.array(xmn * 1.5, np.float32), np.array(xmx * 0.75, np.float32)
    ins2, keep2 = matmul_inputs(torch, dev, xq, wq, bias, [xmn2, xmx2, wmn, wmx])
    ins2[1] = ins[1]  # same weight tensor
    code, msg, outs = node.run(ins2, [(tf.FLOAT, False)], stream=stream)
    assert code == tf.OK, msg
    _, y_ref2 = orc.qmatmul(at, xq, wq, bias, xmn2, xmx2, wmn, wmx)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.float32), y_ref2)
    assert node.temp_allocs() == first  # no new device allocation
    node.close()


def test_quantized_matmul_requantize_and_minmax_outputs(rt, dev):
    torch = rt
    M, K, N = 64, 512, 96
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=9)
    r_out = np.float32(np.abs(x @ w + bias).max())
    mo, xo = np.array(-r_out, np.float32), np.array(r_out, np.float32)
    stream = torch.cuda.current_stream().cuda_stream
    # V2 spelling
    node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.QINT8), fused_ops=["BiasAdd", "Requantize"]))
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [xmn, xmx, wmn, wmx, mo, xo])
    code, msg, outs = node.run(ins, [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=stream)
    assert code == tf.OK, msg
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.QINT8, input_mode=orc.MIN_FIRST, has_requantize=True)
    _, q_ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx, -r_out, r_out)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int8), q_ref)
    assert fetch(torch, outs[1], np.float32) == -r_out and fetch(torch, outs[2], np.float32) == r_out
    node.close()
    # V1 spelling, qint32 product with per-channel ranges out
    v1 = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(tf.FLOAT), Toutput=DT(tf.QINT32), num_args=1, transpose_a=False,
              transpose_b=False, fused_ops=["BiasAdd"], is_filter_const=True, is_bias_const=True,
              input_quant_mode="MIN_FIRST", leakyrelu_alpha=0.2)
    node = tf.Node("_QuantizedFusedMatMul", v1)
    assert node.code == tf.OK, node.message
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [xmn, xmx, wmn, wmx])
    code, msg, outs = node.run(ins, [(tf.QINT32, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=stream)
    assert code == tf.OK, msg
    at = orc.matmul_attrs(api=orc.API_V1, t_in=orc.QUINT8, t_out=orc.QINT32, input_mode=orc.MIN_FIRST, n_fused_ops=1)
    _, acc_ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int32), acc_ref)
    _, omn_ref, omx_ref = orc.qmatmul_output_minmax(at, xmn, xmx, wmn, wmx, 1, 0, 0)
    np.testing.assert_array_equal(fetch(torch, outs[1], np.float32), omn_ref)
    np.testing.assert_array_equal(fetch(torch, outs[2], np.float32), omx_ref)
    node.close()


def test_legacy_matmul_with_bias_and_relu_and_requantize(rt, dev):
    torch = rt
    M, K, N = 32, 256, 64
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=5, per_channel=False)
    r_out = np.float32(np.maximum(x @ w + bias, 0).max())
    mo, xo = np.array(0.0, np.float32), np.array(r_out, np.float32)
    node = tf.Node("QuantizedMatMulWithBiasAndReluAndRequantize",
                   dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Toutput=DT(tf.QUINT8), transpose_a=False,
                        transpose_b=False, input_quant_mode="MIN_FIRST"))
    assert node.code == tf.OK, node.message
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [xmn, xmx, wmn, wmx, mo, xo])
    code, msg, outs = node.run(ins, [(tf.QUINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)],
                               stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    at = orc.matmul_attrs(api=orc.API_LEGACY, t_in=orc.QUINT8, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST,
                          activation=orc.ACT_RELU)
    _, q_ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx, 0.0, r_out)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.uint8), q_ref)
    node.close()


def test_full_chain_config1_shape(rt, dev):
    """QuantizeV2 -> _QuantizedMatMul [BiasAdd, Relu, Dequantize] -> compared with the fp32 graph at the
    reference tests' own tolerance, and with the oracle exactly."""
    torch = rt
    M, K, N = 128, 1024, 1024
    rng = np.random.default_rng(0)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    r = np.abs(w).max(0).astype(np.float32)
    _, wq, wmn, wmx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    xq, xmn, xmx, _, _ = run_quantize(torch, dev, x, x.min(), x.max(), tf.QUINT8, "MIN_FIRST")
    node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Relu", "Dequantize"]))
    ins, keep = matmul_inputs(torch, dev, xq, wq, bias, [np.array(xmn, np.float32), np.array(xmx, np.float32), wmn, wmx])
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    y = fetch(torch, outs[0], np.float32)
    np.testing.assert_allclose(y, np.maximum(x @ w + bias, 0), rtol=0.2, atol=0.2)
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST,
                          activation=orc.ACT_RELU, has_dequantize=True)
    _, y_ref = orc.qmatmul(at, xq, wq, bias, xmn, xmx, wmn, wmx)
    np.testing.assert_array_equal(y, y_ref)
    node.close()


def test_requantize_per_channel_ops(rt, dev):
    torch = rt
    rng = np.random.default_rng(3)
    x = np.rint(rng.standard_normal((2, 4, 8, 64)) * (1 << 20)).astype(np.int32)
    in_min = -(rng.random(64).astype(np.float32) + 0.5)
    in_max = rng.random(64).astype(np.float32) + 0.5
    x_d = dev_in(torch, dev, x)
    stream = torch.cuda.current_stream().cuda_stream
    rng_node = tf.Node("RequantizationRangePerChannel", dict(T=DT(tf.QINT32), clip_value_max=6.0))
    assert rng_node.code == tf.OK, rng_node.message
    code, msg, outs = rng_node.run([(tf.QINT32, x.shape, x_d.data_ptr(), False), (tf.FLOAT, (64,), tf.host_array(in_min), True),
                                    (tf.FLOAT, (64,), tf.host_array(in_max), True)], [(tf.FLOAT, True), (tf.FLOAT, True)],
                                   stream=stream)
    assert code == tf.OK, msg
    _, omn_ref, omx_ref = orc.requantization_range_per_channel(x, in_min, in_max, 6.0)
    omn, omx = fetch(torch, outs[0], np.float32), fetch(torch, outs[1], np.float32)
    assert omn == omn_ref and omx == omx_ref
    rng_node.close()
    node = tf.Node("RequantizePerChannel", dict(T=DT(tf.QINT32), out_type=DT(tf.QINT8)))
    assert node.code == tf.OK, node.message
    rmin, rmax = np.array(omn, np.float32), np.array(omx, np.float32)
    code, msg, outs = node.run([(tf.QINT32, x.shape, x_d.data_ptr(), False), (tf.FLOAT, (64,), tf.host_array(in_min), True),
                                (tf.FLOAT, (64,), tf.host_array(in_max), True), (tf.FLOAT, (), tf.host_array(rmin), True),
                                (tf.FLOAT, (), tf.host_array(rmax), True)],
                               [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=stream)
    assert code == tf.OK, msg
    _, q_ref, _, _ = orc.requantize_per_channel(x, in_min, in_max, float(rmin), float(rmax), orc.QINT8)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int8), q_ref)
    node.close()


def _ref_constants(golden):
    g = golden["fused_matmul"]
    x, w, b = (np.array(g[k], np.float32) for k in ("x", "w", "bias"))
    z = np.array(golden["fused_matmul_addend"], np.float32) * 2
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    _, wq, wmn, wmx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
    f = lambda v: np.array(v[0], np.float32)
    return g, x, w, b, z, xq, f(xmn), f(xmx), wq, f(wmn), f(wmx)


@pytest.mark.parametrize("api", ["V1", "V2"])
def test_reference_add_post_op_case_through_plugin(rt, dev, golden, api):
    """_testAddPostop of the reference's native_quantized_fused_matmul_test.py (K = 3: the unpacked-weight
    path): [BiasAdd, Add] with the addend as an extra device input that shifts the min/max inputs."""
    torch = rt
    g, x, w, b, z, xq, xmn, xmx, wq, wmn, wmx = _ref_constants(golden)
    if api == "V1":
        node = tf.Node("_QuantizedFusedMatMulAndDequantize",
                       dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(tf.FLOAT), Toutput=DT(tf.FLOAT), num_args=2,
                            transpose_a=False, transpose_b=False, fused_ops=["BiasAdd", "Add"], is_filter_const=True,
                            is_bias_const=True, input_quant_mode="MIN_FIRST", leakyrelu_alpha=0.2))
        at = orc.matmul_attrs(api=orc.API_V1, t_out=orc.FLOAT, add_position=1, n_fused_ops=2)
    else:
        node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Add", "Dequantize"]))
        at = orc.matmul_attrs(api=orc.API_V2, t_out=orc.FLOAT, has_dequantize=True, add_position=1)
    assert node.code == tf.OK, node.message
    ins, keep = matmul_inputs(torch, dev, xq, wq, b, [])
    z_d = dev_in(torch, dev, z)
    ins.append((tf.FLOAT, z.shape, z_d.data_ptr(), False))
    for s in (xmn, xmx, wmn, wmx):
        ins.append((tf.FLOAT, s.shape, tf.host_array(s), True))
    for _ in range(2):   # the reference runs it twice "to check the functionality of object cache"
        code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        y = fetch(torch, outs[0], np.float32)
        np.testing.assert_allclose(y, x @ w + b + z, rtol=g["tolerance"], atol=g["tolerance"])
        _, y_ref = orc.qmatmul(at, xq, wq, b, xmn, xmx, wmn, wmx, addend=z)
        np.testing.assert_array_equal(y, y_ref)
    node.close()


@pytest.mark.parametrize("per_channel", [False, True])
def test_reference_gelu_case_through_plugin(rt, dev, golden, per_channel):
    """_testGeluPerTensorPostop / _testGeluPerchannelPostop: [BiasAdd, GeluApproximate, Dequantize] within the
    reference's tolerance of the fp32 graph; close to the oracle (the transcendental is unpinned at bit level)."""
    torch = rt
    g, x, w, b, z, xq, xmn, xmx, wq, wmn, wmx = _ref_constants(golden)
    if per_channel:
        _, wq, wmn, wmx = orc.quantize_v2(w, w.min(0), w.max(0), orc.QINT8, orc.SCALED, axis=1)
    node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "GeluApproximate", "Dequantize"]))
    assert node.code == tf.OK, node.message
    ins, keep = matmul_inputs(torch, dev, xq, wq, b, [xmn, xmx, wmn, wmx])
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    y = fetch(torch, outs[0], np.float32)
    pre = (x @ w + b).astype(np.float64)
    gelu = 0.5 * pre * (1 + np.tanh(np.sqrt(2 / np.pi) * (pre + 0.044715 * pre ** 3)))
    np.testing.assert_allclose(y, gelu, rtol=g["tolerance"], atol=g["tolerance"])
    at = orc.matmul_attrs(api=orc.API_V2, t_out=orc.FLOAT, has_dequantize=True, activation=orc.ACT_GELU_APPROX)
    _, y_ref = orc.qmatmul(at, xq, wq, b, xmn, xmx, wmn, wmx)
    np.testing.assert_allclose(y, y_ref, rtol=2e-6, atol=1e-6)
    node.close()


def test_reference_qint32_bias_case_through_plugin(rt, dev, golden):
    """The qint32-bias variant of _testAddPostop (run there without an assertion): Tbias = qint32 selects the
    second kernel registration; result bit-equal to the oracle's as-written semantics."""
    torch = rt
    g, x, w, b, z, xq, xmn, xmx, wq, wmn, wmx = _ref_constants(golden)
    b32 = np.array(golden["fused_matmul_bias_qint32"], np.int32)
    node = tf.Node("_QuantizedMatMul", dict(V2, Tbias=DT(tf.QINT32), Tout=DT(tf.FLOAT), fused_ops=["BiasAdd", "Add", "Dequantize"]))
    assert node.code == tf.OK, node.message
    keep = [dev_in(torch, dev, v) for v in (xq, wq, b32, z)]
    ins = [(tf.QUINT8, xq.shape, keep[0].data_ptr(), False), (tf.QINT8, wq.shape, keep[1].data_ptr(), False),
           (tf.QINT32, b32.shape, keep[2].data_ptr(), False), (tf.FLOAT, z.shape, keep[3].data_ptr(), False)]
    for s in (xmn, xmx, wmn, wmx):
        ins.append((tf.FLOAT, s.shape, tf.host_array(s), True))
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    at = orc.matmul_attrs(api=orc.API_V2, t_out=orc.FLOAT, has_dequantize=True, add_position=1, t_bias=orc.QINT32)
    _, y_ref = orc.qmatmul(at, xq, wq, b32, xmn, xmx, wmn, wmx, addend=z)
    np.testing.assert_array_equal(fetch(torch, outs[0], np.float32), y_ref)
    node.close()


def test_bfloat16_quantize_and_16_bit_dequantize_through_plugin(rt, dev):
    """_ITEXQuantizeV2 with dtype = bfloat16 and Dequantize with dtype = bfloat16 / half
    (itex/core/kernels/gpu/quantize_op.cc:38-51, dequantize_op.cc:24-48)."""
    torch = rt
    BF16, HALF = 14, 19
    rng = np.random.default_rng(12)
    x32 = (rng.standard_normal(3001) * 2).astype(np.float32)
    xb = torch.from_numpy(x32).to(dev).to(torch.bfloat16)
    xw = xb.to(torch.float32).cpu().numpy()          # the exactly widened values
    node = tf.Node("_ITEXQuantizeV2", dict(T=DT(tf.QINT8), dtype=DT(BF16), mode="SCALED", round_mode="HALF_TO_EVEN",
                                            narrow_range=False, axis=-1, ensure_minimum_range=0.01))
    assert node.code == tf.OK, node.message
    mn, mx = np.array(xw.min(), np.float32), np.array(xw.max(), np.float32)
    code, msg, outs = node.run([(BF16, xw.shape, xb.data_ptr(), False), (tf.FLOAT, (), tf.host_array(mn), True),
                                (tf.FLOAT, (), tf.host_array(mx), True)],
                               [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    q = fetch(torch, outs[0], np.int8)
    _, q_ref, omn, omx = orc.quantize_v2(xw, mn, mx, orc.QINT8, orc.SCALED)
    np.testing.assert_array_equal(q, q_ref)
    node.close()
    q_d = dev_in(torch, dev, q_ref)
    _, y32 = orc.dequantize(q_ref, omn[0], omx[0], orc.QINT8, orc.SCALED)
    for dtype, tdt_ in ((BF16, torch.bfloat16), (HALF, torch.float16)):
        dn = tf.Node("Dequantize", dict(T=DT(tf.QINT8), mode="SCALED", narrow_range=False, axis=-1, dtype=DT(dtype)))
        assert dn.code == tf.OK, dn.message
        dmn, dmx = np.array(omn[0], np.float32), np.array(omx[0], np.float32)
        code, msg, outs = dn.run([(tf.QINT8, q_ref.shape, q_d.data_ptr(), False), (tf.FLOAT, (), tf.host_array(dmn), True),
                                  (tf.FLOAT, (), tf.host_array(dmx), True)], [(dtype, False)],
                                 stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        bits = fetch(torch, outs[0], np.int16)
        expect = torch.from_numpy(y32).to(tdt_).view(torch.int16).numpy()   # torch rounds to nearest even as well
        np.testing.assert_array_equal(bits, expect)
        dn.close()


@pytest.mark.parametrize("op,M,K,N", [("_QuantizedMatMul", 5, 128, 72), ("_QuantizedMatMul", 90, 256, 203),
                                      ("_QuantizedFusedMatMulAndDequantize", 33, 64, 40),
                                      ("QuantizedMatMulWithBiasAndDequantize", 20, 96, 48)])
@pytest.mark.parametrize("T16", [tf.BFLOAT16, tf.HALF])
def test_bfloat16_output_and_bias_through_plugin(rt, dev, op, M, K, N, T16):
    """Tout / Toutput and Tbias / Targs = bfloat16 or half select their own kernel registrations
    (itex/core/kernels/gpu/quantized_matmul.cc:84-88, 123-129, 147-152, 187-191); bit patterns equal the oracle's."""
    torch = rt
    legacy = op.startswith("Quantized")
    if op == "_QuantizedMatMul" and T16 == tf.HALF:
        # the V2 op has no half OUTPUT registration upstream (:181-195); a half bias with a float output exists
        node = tf.Node(op, dict(V2, Tbias=DT(tf.HALF), Tout=DT(tf.HALF), fused_ops=["BiasAdd", "Dequantize"]))
        assert node.code != tf.OK
        return
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=N, per_channel=not legacy)
    b16 = torch.from_numpy(bias * 30).to(torch.bfloat16 if T16 == tf.BFLOAT16 else torch.float16).view(torch.int16).numpy()
    for bias_type, b in ((tf.FLOAT, bias), (T16, b16)):
        if legacy and bias_type == T16:
            continue   # the legacy ops take float and qint32 biases only (:44-46)
        if op == "_QuantizedMatMul":
            node = tf.Node(op, dict(V2, Tbias=DT(bias_type), Tout=DT(T16), fused_ops=["BiasAdd", "Dequantize"]))
            at = orc.matmul_attrs(api=orc.API_V2, t_out=T16, has_dequantize=True)
            scalars = [xmn, xmx, wmn, wmx]
        elif legacy:
            node = tf.Node(op, dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(bias_type), Toutput=DT(T16),
                                    transpose_a=False, transpose_b=False, input_quant_mode="MIN_FIRST"))
            at = orc.matmul_attrs(api=orc.API_LEGACY, t_out=T16)
            lo, hi = np.array(-9.0, np.float32), np.array(9.0, np.float32)
            scalars = [xmn, xmx, wmn, wmx, lo, hi]
        else:
            node = tf.Node(op, dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(bias_type), Toutput=DT(T16), num_args=1,
                                    transpose_a=False, transpose_b=False, fused_ops=["BiasAdd"], is_filter_const=True,
                                    is_bias_const=True, input_quant_mode="MIN_FIRST", leakyrelu_alpha=0.2))
            at = orc.matmul_attrs(api=orc.API_V1, t_out=T16, n_fused_ops=1)
            scalars = [xmn, xmx, wmn, wmx]
        assert node.code == tf.OK, node.message
        at.t_bias = T16 if bias_type == T16 else orc.FLOAT
        ins, keep = matmul_inputs(torch, dev, xq, wq, b, scalars)
        ins[2] = (bias_type, b.shape, keep[2].data_ptr(), False)
        code, msg, outs = node.run(ins, [(T16, False)], stream=torch.cuda.current_stream().cuda_stream)
        assert code == tf.OK, msg
        st, y_ref = orc.qmatmul(at, xq, wq, b.view(np.uint16) if bias_type == T16 else b, xmn, xmx, wmn, wmx,
                                -9.0 if legacy else 0.0, 9.0 if legacy else 0.0)
        assert st == orc.OK
        np.testing.assert_array_equal(fetch(torch, outs[0], np.int16).view(np.uint16), y_ref)
        node.close()
    # the args list of the Add fusion (bias, addend) must have the output's type: the addend is read as the destination
    bad = tf.Node("_QuantizedFusedMatMulAndDequantize",
                  dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(tf.BFLOAT16), Toutput=DT(tf.FLOAT), num_args=2,
                       transpose_a=False, transpose_b=False, fused_ops=["BiasAdd", "Add"], is_filter_const=True,
                       is_bias_const=True, input_quant_mode="MIN_FIRST", leakyrelu_alpha=0.2))
    assert bad.code == tf.INVALID_ARGUMENT
    bad.close()


@pytest.mark.parametrize("api", ["V1", "V2"])
def test_add_fusion_with_bfloat16_output_through_plugin(rt, dev, api):
    """[BiasAdd, Add] with a bfloat16 result: the addend is a bfloat16 tensor (it is read as the destination,
    quantized_matmul_common.h:341-389; V1 passes bias and addend in one bfloat16 args list); bit patterns equal the
    oracle's, which gets the addend widened to float."""
    torch = rt
    M, K, N = 40, 128, 96
    x, w, bias, xq, xmn, xmx, wq, wmn, wmx = make_problem(M, K, N, seed=21)
    z = (np.random.default_rng(2).standard_normal((M, N)) * 2).astype(np.float32)
    zbits = (z.view(np.uint32) >> 16).astype(np.uint16)
    zwide = (zbits.astype(np.uint32) << 16).view(np.float32)
    if api == "V1":
        bbits = (bias.view(np.uint32) >> 16).astype(np.uint16)
        node = tf.Node("_QuantizedFusedMatMulAndDequantize",
                       dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(tf.BFLOAT16), Toutput=DT(tf.BFLOAT16), num_args=2,
                            transpose_a=False, transpose_b=False, fused_ops=["BiasAdd", "Add"], is_filter_const=True,
                            is_bias_const=True, input_quant_mode="MIN_FIRST", leakyrelu_alpha=0.2))
        at = orc.matmul_attrs(api=orc.API_V1, t_out=orc.BFLOAT16, add_position=1, n_fused_ops=2, t_bias=orc.BFLOAT16)
        b_host, b_dt = bbits, tf.BFLOAT16
    else:
        node = tf.Node("_QuantizedMatMul", dict(V2, Tout=DT(tf.BFLOAT16), fused_ops=["BiasAdd", "Add", "Dequantize"]))
        at = orc.matmul_attrs(api=orc.API_V2, t_out=orc.BFLOAT16, has_dequantize=True, add_position=1)
        b_host, b_dt = bias, tf.FLOAT
    assert node.code == tf.OK, node.message
    keep = [dev_in(torch, dev, xq), dev_in(torch, dev, wq), dev_in(torch, dev, b_host.view(np.int16) if b_dt == tf.BFLOAT16 else b_host),
            dev_in(torch, dev, zbits.view(np.int16))]
    ins = [(tf.QUINT8, xq.shape, keep[0].data_ptr(), False), (tf.QINT8, wq.shape, keep[1].data_ptr(), False),
           (b_dt, bias.shape, keep[2].data_ptr(), False), (tf.BFLOAT16, z.shape, keep[3].data_ptr(), False)]
    for s_ in (xmn, xmx, wmn, wmx):
        ins.append((tf.FLOAT, s_.shape, tf.host_array(s_), True))
    code, msg, outs = node.run(ins, [(tf.BFLOAT16, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    st, y_ref = orc.qmatmul(at, xq, wq, b_host, xmn, xmx, wmn, wmx, addend=zwide)
    assert st == orc.OK
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int16).view(np.uint16), y_ref)
    node.close()


@pytest.mark.parametrize("api", ["V1", "V2"])
@pytest.mark.parametrize("case", ["plain", "mul", "mul_add"])
def test_reference_batch_matmul_cases_through_plugin(rt, dev, golden, api, case):
    """_testQuantizeBMM / _testQuantizeBMMMul / _testQuantizeBMMMulAdd of the reference's
    quantized_batch_matmul_test.py in both spellings: within its tolerance of the fp32 graph, bit-equal to the oracle."""
    torch = rt
    g = golden["batch_matmul"]
    x, y, add = (np.array(g[k], np.float32) for k in ("x", "y", "add"))
    mul = np.array(g["mul"], np.float32)                       # a scalar tensor, as in the reference test
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QINT8, orc.SCALED)
    _, yq, ymn, ymx = orc.quantize_v2(y, y.min(), y.max(), orc.QINT8, orc.SCALED)
    args = {"plain": [], "mul": [mul], "mul_add": [mul, add]}[case]
    fused = {"plain": [], "mul": ["Mul"], "mul_add": ["Mul", "Add"]}[case]
    if api == "V1" and not args:
        node = tf.Node("_QuantizedBatchMatMulV2AndDequantize",
                       dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), Toutput=DT(tf.FLOAT), adj_x=False, adj_y=False, is_filter_const=False))
    elif api == "V1":
        node = tf.Node("_QuantizedFusedBatchMatMulV2AndDequantize",
                       dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), T=DT(tf.FLOAT), Toutput=DT(tf.FLOAT), adj_x=False, adj_y=False,
                            num_args=len(args), fused_ops=fused, is_filter_const=False))
    else:
        node = tf.Node("_QuantizedBatchMatMul",
                       dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), U=DT(tf.FLOAT), Tout=DT(tf.FLOAT), adj_x=False, adj_y=False,
                            fused_ops=fused + ["Dequantize"], input_quant_mode="SCALED", output_quant_mode="SCALED"))
    assert node.code == tf.OK, node.message
    keep = [dev_in(torch, dev, v) for v in [xq, yq] + args]
    ins = [(tf.QINT8, xq.shape, keep[0].data_ptr(), False), (tf.QINT8, yq.shape, keep[1].data_ptr(), False)]
    for a, k in zip(args, keep[2:]):
        ins.append((tf.FLOAT, a.shape, k.data_ptr(), False))
    scal = [np.array(v[0], np.float32) for v in (xmn, xmx, ymn, ymx)]
    for s in scal:
        ins.append((tf.FLOAT, (), tf.host_array(s), True))
    code, msg, outs = node.run(ins, [(tf.FLOAT, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    got = fetch(torch, outs[0], np.float32)
    ref32 = x @ y
    if args:
        ref32 = ref32 * mul
    if len(args) == 2:
        ref32 = ref32 + add
    np.testing.assert_allclose(got, ref32, rtol=g["tolerance"], atol=g["tolerance"])
    binary = [(orc.BIN_MUL, mul.reshape(1)), (orc.BIN_ADD, add)][:len(args)]
    st, ref = orc.qbatch_matmul(xq, yq, xmn[0], xmx[0], ymn[0], ymx[0], binary=binary)
    assert st == orc.OK
    np.testing.assert_array_equal(got, ref)
    node.close()


def test_batch_matmul_attention_through_plugin(rt, dev):
    """adj_y, broadcast batch dimensions of the mask, bfloat16 output with bfloat16 operands."""
    torch = rt
    rng = np.random.default_rng(2)
    B, H, S, D = 2, 3, 80, 64
    q = rng.integers(-128, 128, (B, H, S, D)).astype(np.int8)
    k = rng.integers(-128, 128, (B, H, S, D)).astype(np.int8)
    mask = torch.from_numpy(np.where(rng.random((B, 1, 1, S)) < 0.3, -10000.0, 0.0).astype(np.float32)).to(torch.bfloat16)
    mul = torch.tensor([0.125], dtype=torch.bfloat16)
    node = tf.Node("_QuantizedBatchMatMul",
                   dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), U=DT(tf.BFLOAT16), Tout=DT(tf.BFLOAT16), adj_x=False, adj_y=True,
                        fused_ops=["Mul", "Add", "Dequantize"], input_quant_mode="SCALED", output_quant_mode="SCALED"))
    assert node.code == tf.OK, node.message
    keep = [dev_in(torch, dev, q), dev_in(torch, dev, k), mul.to(dev), mask.to(dev)]
    ins = [(tf.QINT8, q.shape, keep[0].data_ptr(), False), (tf.QINT8, k.shape, keep[1].data_ptr(), False),
           (tf.BFLOAT16, (1,), keep[2].data_ptr(), False), (tf.BFLOAT16, tuple(mask.shape), keep[3].data_ptr(), False)]
    scal = [np.array(s, np.float32) for s in (-4.0, 3.5, -2.0, 2.5)]   # kept alive: the node reads their memory
    for s in scal:
        ins.append((tf.FLOAT, (), tf.host_array(s), True))
    code, msg, outs = node.run(ins, [(tf.BFLOAT16, False)], stream=torch.cuda.current_stream().cuda_stream)
    assert code == tf.OK, msg
    bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    st, ref = orc.qbatch_matmul(q, k, -4.0, 3.5, -2.0, 2.5, adj_y=True,
                                binary=((orc.BIN_MUL, bits(mul)), (orc.BIN_ADD, bits(mask))), t_out=orc.BFLOAT16)
    assert st == orc.OK
    np.testing.assert_array_equal(fetch(torch, outs[0], np.int16).view(np.uint16), ref)
    node.close()
    # an activation is not a fusion this op knows
    bad = tf.Node("_QuantizedBatchMatMul",
                  dict(T1=DT(tf.QINT8), T2=DT(tf.QINT8), U=DT(tf.FLOAT), Tout=DT(tf.FLOAT), adj_x=False, adj_y=False,
                       fused_ops=["Relu", "Dequantize"], input_quant_mode="SCALED", output_quant_mode="SCALED"))
    assert bad.code == tf.UNIMPLEMENTED and "Fusion is not implemented" in bad.message
    bad.close()
