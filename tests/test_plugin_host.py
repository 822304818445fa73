"""CPU-only tests of the PluggableDevice kernel plugin driven by the mock TensorFlow host:
registration table (op names, type constraints, host-memory arguments as the reference registers
them), op definitions, attribute validation and error messages, input validation in Compute before
any device work."""
import numpy as np
import pytest

from tests.mock_tf import host as tf

DT = tf.DType


@pytest.fixture(scope="module")
def reg():
    return tf.registry()


def kernels_of(reg, op):
    return [k for k in reg["kernels"] if k["op"] == op]


def test_registered_names(reg):
    ops = {k["op"] for k in reg["kernels"]}
    expected = {
        # itex/core/kernels/gpu/quantize_op.cc:24-51, dequantize_op.cc:24-48
        "QuantizeV2", "_ITEXQuantizeV2", "Dequantize", "_ITEXDequantize",
        # itex/core/kernels/gpu/quantized_matmul.cc:52-201
        "QuantizedMatMulWithBias", "QuantizedMatMulWithBiasAndRelu", "QuantizedMatMulWithBiasAndReluAndRequantize",
        "QuantizedMatMulWithBiasAndRequantize", "QuantizedMatMulWithBiasAndDequantize",
        "_ITEXQuantizedMatMulWithBiasAndDequantize", "_QuantizedFusedMatMul", "_QuantizedFusedMatMulAndDequantize",
        "_QuantizedFusedMatMulAndRequantize", "_QuantizedMatMul",
        # CPU-side renames (itex/core/kernels/cpu/quantized_matmul.cc:97-163)
        "_ITEXQuantizedMatMul", "_ITEXQuantizedFusedMatMul", "_ITEXQuantizedFusedMatMulAndDequantize",
        "_ITEXQuantizedFusedMatMulAndRequantize",
        # itex/core/kernels/onednn/block/requantize_per_channel_op.cc:176-191, requantization_range_per_channel_op.cc:172-184
        "RequantizePerChannel", "RequantizationRangePerChannel",
    }
    assert expected <= ops
    assert all(k["device"] == "XPU" for k in reg["kernels"])


def test_host_memory_and_constraints(reg):
    for op in ("QuantizeV2", "_ITEXQuantizeV2"):
        ks = kernels_of(reg, op)
        assert {k["constraints"]["T"] for k in ks} == {tf.QINT8, tf.QUINT8}
        for k in ks:
            assert k["host_memory"] == ["min_range", "max_range", "output_min", "output_max"]
    for k in kernels_of(reg, "Dequantize"):
        assert k["host_memory"] == ["min_range", "max_range"]
    v2 = kernels_of(reg, "_QuantizedMatMul")
    assert {(k["constraints"]["T1"], k["constraints"]["Tout"]) for k in v2} == {
        (a, o) for a in (tf.QINT8, tf.QUINT8) for o in (tf.QINT32, tf.FLOAT, tf.BFLOAT16, tf.QINT8, tf.QUINT8)}
    for k in v2:
        assert k["host_memory"] == ["host_inputs", "host_outputs"] and k["constraints"]["T2"] == tf.QINT8
    req = kernels_of(reg, "_QuantizedFusedMatMulAndRequantize")
    assert all(k["host_memory"] == ["min_a", "max_a", "min_b", "max_b", "min_freezed_output", "max_freezed_output",
                                    "min_product", "max_product"] for k in req)
    deq = kernels_of(reg, "_QuantizedFusedMatMulAndDequantize")
    assert all(k["host_memory"] == ["min_a", "max_a", "min_b", "max_b"] for k in deq)
    legacy = kernels_of(reg, "QuantizedMatMulWithBiasAndReluAndRequantize")
    assert len(legacy) == 2 and {k["constraints"]["Tbias"] for k in legacy} == {tf.FLOAT, tf.QINT32}
    assert all({**k["constraints"], "Tbias": 0} == {"T1": tf.QUINT8, "T2": tf.QINT8, "Tbias": 0, "Toutput": tf.QUINT8}
               for k in legacy)
    # every bias / args type the reference registers for a device (kernels/gpu/quantized_matmul.cc:118-133)
    all_bias = {tf.FLOAT, tf.QINT32, tf.BFLOAT16, tf.HALF, tf.QINT8, tf.QUINT8}
    assert {k["constraints"]["Tbias"] for k in v2} == all_bias
    assert {(k["constraints"]["Targs"], k["constraints"]["Toutput"]) for k in deq} == {
        (b, o) for b in all_bias for o in (tf.FLOAT, tf.BFLOAT16, tf.HALF)}
    ldq = kernels_of(reg, "QuantizedMatMulWithBiasAndDequantize")
    assert {(k["constraints"]["Tbias"], k["constraints"]["Toutput"]) for k in ldq} == {
        (b, o) for b in (tf.FLOAT, tf.QINT32) for o in (tf.FLOAT, tf.BFLOAT16, tf.HALF)}


def test_op_definitions_only_for_missing_ops(reg):
    names = {o["name"] for o in reg["ops"]}
    # the mock's "stock TensorFlow" already has QuantizeV2 & co: the plugin must not redefine them
    assert "QuantizeV2" not in names and "Dequantize" not in names and "QuantizedMatMulWithBias" not in names
    assert {"_ITEXQuantizeV2", "_ITEXDequantize", "_QuantizedMatMul", "_ITEXQuantizedMatMul", "_QuantizedFusedMatMul",
            "_QuantizedFusedMatMulAndRequantize", "_QuantizedFusedMatMulAndDequantize"} <= names
    q = next(o for o in reg["ops"] if o["name"] == "_ITEXQuantizeV2")
    assert q["inputs"] == ["input: dtype", "min_range: float", "max_range: float"]
    assert q["outputs"] == ["output: T", "output_min: float", "output_max: float"]
    assert "classic_asymmetric_algorithm: bool = false" in q["attrs"] and q["shape_fn"]
    m = next(o for o in reg["ops"] if o["name"] == "_QuantizedMatMul")
    assert m["inputs"] == ["device_inputs: Tdevice_inputs", "host_inputs: Thost_inputs"]
    assert "fused_ops: list(string) = []" in m["attrs"]


QATTRS = dict(T=DT(tf.QINT8), mode="SCALED", round_mode="HALF_TO_EVEN", narrow_range=False, axis=-1,
              ensure_minimum_range=0.01)


def test_quantize_attr_validation():
    n = tf.Node("QuantizeV2", dict(QATTRS, mode="BOGUS"))
    assert n.code == tf.INVALID_ARGUMENT
    assert n.message == "Mode string must be 'MIN_COMBINED', 'MIN_FIRST', or 'SCALED', is 'BOGUS'"
    n = tf.Node("QuantizeV2", dict(QATTRS, mode="MIN_COMBINED", round_mode="HALF_AWAY_FROM_ZERO"))
    assert n.code == tf.INVALID_ARGUMENT and n.message == "_ITEXQuantizeV2 only supports SCALED and MIN_FIRST MODE"
    n = tf.Node("QuantizeV2", dict(QATTRS, round_mode="UP"))
    assert n.code == tf.INVALID_ARGUMENT and "Round mode string must be" in n.message and "is 'UP'" in n.message
    n = tf.Node("QuantizeV2", dict(QATTRS, mode="MIN_FIRST", round_mode="HALF_TO_EVEN"))
    assert n.code == tf.INVALID_ARGUMENT
    assert n.message == "Round mode 'HALF_TO_EVEN' only supported for mode 'SCALED', but mode is 'MIN_FIRST'."
    attrs = dict(QATTRS)
    del attrs["axis"]
    n = tf.Node("QuantizeV2", attrs)
    assert n.code == tf.INVALID_ARGUMENT and "axis" in n.message
    # no kernel for an unregistered type combination
    n = tf.Node("QuantizeV2", dict(QATTRS, T=DT(tf.QINT32)))
    assert n.code == tf.NOT_FOUND
    ok = tf.Node("QuantizeV2", QATTRS)
    assert ok.code == tf.OK
    ok.close()


def test_failed_construction_is_deleted():
    lib = tf.load()
    before = lib.mock_delete_calls()
    n = tf.Node("QuantizeV2", dict(QATTRS, mode="BOGUS"))
    assert n.code != tf.OK and lib.mock_delete_calls() == before + 1
    n.close()
    assert lib.mock_delete_calls() == before + 1  # nothing left to delete


def test_quantize_rejects_inverted_range_before_device_work():
    n = tf.Node("QuantizeV2", QATTRS)
    x = np.zeros(8, np.float32)
    mn, mx = np.array(1.0, np.float32), np.array(0.5, np.float32)
    code, msg, outs = n.run([(tf.FLOAT, (8,), tf.host_array(x), False), (tf.FLOAT, (), tf.host_array(mn), True),
                             (tf.FLOAT, (), tf.host_array(mx), True)],
                            [(tf.QINT8, False), (tf.FLOAT, True), (tf.FLOAT, True)])
    assert code == tf.INVALID_ARGUMENT and msg == "input_max_range must be larger than input_min_range."
    n.close()


def test_matmul_attr_validation():
    base = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tout=DT(tf.FLOAT), transpose_a=False,
                transpose_b=False, is_weight_const=True, is_bias_const=True, fused_ops=["BiasAdd", "Dequantize"],
                input_quant_mode="MIN_FIRST", output_quant_mode="SCALED", leakyrelu_alpha=0.2)
    assert tf.Node("_QuantizedMatMul", base).code == tf.OK
    n = tf.Node("_QuantizedMatMul", dict(base, input_quant_mode="MIN_COMBINED"))
    assert n.code == tf.INVALID_ARGUMENT
    assert n.message == "Quantization mode must be either MIN_FIRST or SCALED, but received MIN_COMBINED"
    n = tf.Node("_QuantizedMatMul", dict(base, fused_ops=["BiasAdd", "Bogus", "Dequantize"]))
    assert n.code == tf.INVALID_ARGUMENT and n.message == "Found unsupported fusion in _QuantizedMatMul."
    v1 = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Targs=DT(tf.FLOAT), Toutput=DT(tf.QINT8), num_args=1, transpose_a=False,
              transpose_b=False, fused_ops=["Relu", "BiasAdd"], is_filter_const=True, is_bias_const=True,
              input_quant_mode="SCALED", leakyrelu_alpha=0.2)
    n = tf.Node("_QuantizedFusedMatMulAndRequantize", v1)
    assert n.code == tf.INVALID_ARGUMENT and n.message == "_QuantizedFusedMatMul first post op must be BiasAdd"
    n = tf.Node("_QuantizedFusedMatMulAndRequantize", dict(v1, fused_ops=["BiasAdd", "Relu", "Relu6"]))
    assert n.code == tf.INVALID_ARGUMENT and n.message == "_QuantizedFusedMatMul supports maximum 2 post ops"
    assert tf.Node("_QuantizedFusedMatMulAndRequantize", dict(v1, fused_ops=["BiasAdd", "Relu"])).code == tf.OK


def test_eight_bit_bias_is_placed_and_refused_at_compute():
    """Tbias = qint8 / quint8 is registered (a graph naming it finds a kernel, as on the reference's device) and the
    node is constructed; Compute refuses it with TF_UNIMPLEMENTED before any device work."""
    for tb in (tf.QINT8, tf.QUINT8):
        base = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tb), Tout=DT(tf.FLOAT), transpose_a=False,
                    transpose_b=False, is_weight_const=True, is_bias_const=True, fused_ops=["BiasAdd", "Dequantize"],
                    input_quant_mode="MIN_FIRST", output_quant_mode="SCALED", leakyrelu_alpha=0.2)
        n = tf.Node("_QuantizedMatMul", base)
        assert n.code == tf.OK, n.message
        a = np.zeros((4, 32), np.uint8)
        w = np.zeros((32, 8), np.int8)
        b = np.zeros(8, tf.NP_OF[tb])
        s = [np.array(v, np.float32) for v in (0.0, 1.0)]
        wr = [np.full(8, v, np.float32) for v in (-1.0, 1.0)]
        code, msg, _ = n.run([(tf.QUINT8, a.shape, tf.host_array(a), False), (tf.QINT8, w.shape, tf.host_array(w), False),
                              (tb, b.shape, tf.host_array(b), False)] +
                             [(tf.FLOAT, v.shape, tf.host_array(v), True) for v in s + wr], [(tf.FLOAT, False)])
        assert code == tf.UNIMPLEMENTED and "qint8 or quint8" in msg
        n.close()


def test_matmul_shape_validation_before_device_work():
    base = dict(T1=DT(tf.QUINT8), T2=DT(tf.QINT8), Tbias=DT(tf.FLOAT), Tout=DT(tf.FLOAT), transpose_a=False,
                transpose_b=False, is_weight_const=True, is_bias_const=True, fused_ops=["BiasAdd", "Dequantize"],
                input_quant_mode="MIN_FIRST", output_quant_mode="SCALED", leakyrelu_alpha=0.2)
    n = tf.Node("_QuantizedMatMul", base)
    a = np.zeros((4, 32), np.uint8)
    w = np.zeros((16, 8), np.int8)  # inner dimension mismatch
    b = np.zeros(8, np.float32)
    s = [np.array(v, np.float32) for v in (0.0, 1.0, -1.0, 1.0)]
    ins = [(tf.QUINT8, a.shape, tf.host_array(a), False), (tf.QINT8, w.shape, tf.host_array(w), False),
           (tf.FLOAT, b.shape, tf.host_array(b), False)] + [(tf.FLOAT, (), tf.host_array(v), True) for v in s]
    code, msg, _ = n.run(ins, [(tf.FLOAT, False)])
    assert code == tf.INVALID_ARGUMENT and "Matrix size-incompatible" in msg
    n.close()


def test_se_init_plugin_without_a_gpu():
    """SE_InitPlugin is exported and fills the platform tables; with no GPU in the process the device
    count is 0 and device creation is refused cleanly (rc 4 = no such ordinal)."""
    import torch
    rc, plug = tf.load_device()
    if torch.cuda.is_available():
        assert rc == 0, plug.error()
    else:
        assert rc == 4, (rc, plug.error())


def test_batch_matmul_registrations(reg):
    for op, out_attr, host in (("_QuantizedBatchMatMulV2AndDequantize", "Toutput", ["min_x", "max_x", "min_y", "max_y"]),
                               ("_QuantizedFusedBatchMatMulV2AndDequantize", "Toutput", ["min_x", "max_x", "min_y", "max_y"]),
                               ("_QuantizedBatchMatMul", "Tout", ["host_inputs", "host_outputs"])):
        ks = kernels_of(reg, op)
        assert {k["constraints"][out_attr] for k in ks} == {tf.FLOAT, tf.BFLOAT16, tf.HALF}
        assert all(k["constraints"]["T1"] == tf.QINT8 and k["constraints"]["T2"] == tf.QINT8 and k["host_memory"] == host
                   for k in ks)
    names = {o["name"] for o in reg["ops"]}
    assert {"_QuantizedBatchMatMul", "_QuantizedBatchMatMulV2AndDequantize", "_QuantizedFusedBatchMatMulV2AndDequantize",
            "_ITEXQuantizedBatchMatMulV2AndDequantize"} <= names


def test_shape_op_registrations(reg):
    for op, host in (("_QuantizedTranspose", ["perm", "min_x", "max_x", "min_y", "max_y"]),
                     ("QuantizedReshape", ["shape", "input_min", "input_max", "output_min", "output_max"])):
        ks = kernels_of(reg, op)
        assert {k["constraints"]["T"] for k in ks} == {tf.QINT8, tf.QUINT8, tf.QINT32}
        assert all(k["host_memory"] == host for k in ks)
    names = {o["name"] for o in reg["ops"]}
    assert "_QuantizedTranspose" in names and "_ITEXQuantizedReshape" in names and "QuantizedReshape" not in names


def test_conv_registrations(reg):
    # itex/core/kernels/gpu/quantized_conv_ops.cc:77-310
    plain = ["min_input", "max_input", "min_filter", "max_filter", "min_output", "max_output"]
    req = plain[:4] + ["min_freezed_output", "max_freezed_output", "min_output", "max_output"]
    table = {"QuantizedConv2D": ({tf.QINT8, tf.QUINT8}, {tf.QINT32}, plain),
             "QuantizedConv2DPerChannel": ({tf.QINT8, tf.QUINT8}, {tf.QINT32}, plain),
             "QuantizedConv2DWithBias": ({tf.QINT8, tf.QUINT8}, {tf.QINT32}, plain),
             "QuantizedConv2DWithBiasAndRelu": ({tf.QINT8, tf.QUINT8}, {tf.QINT32}, plain),
             "QuantizedConv2DAndRequantize": ({tf.QINT8, tf.QUINT8}, {tf.QINT8}, req),
             "QuantizedConv2DWithBiasAndRequantize": ({tf.QINT8, tf.QUINT8}, {tf.QINT8}, req),
             "QuantizedConv2DWithBiasAndReluAndRequantize": ({tf.QINT8, tf.QUINT8}, {tf.QUINT8}, req)}
    for name, (tin, tout, host) in table.items():
        for op in (name, "_ITEX" + name):
            ks = kernels_of(reg, op)
            assert ks, op
            assert {k["constraints"]["Tinput"] for k in ks} == tin, op
            assert {k["constraints"]["out_type"] for k in ks} == tout, op
            assert all(k["constraints"]["Tfilter"] == tf.QINT8 and k["host_memory"] == host for k in ks), op
    for op in ("QuantizedConv2DWithBiasAndRequantize", "QuantizedConv2DWithBiasAndReluAndRequantize"):
        assert {k["constraints"]["Tbias"] for k in kernels_of(reg, op)} == {tf.FLOAT, tf.QINT32}
    sum_host = req[:6] + ["min_summand", "max_summand", "min_output", "max_output"]
    for name, t_sum in (("QuantizedConv2DWithBiasSumAndReluAndRequantize", tf.QUINT8),
                        ("QuantizedConv2DWithBiasSignedSumAndReluAndRequantize", tf.QINT8)):
        for op in (name, "_ITEX" + name):
            ks = kernels_of(reg, op)
            assert {k["constraints"]["Tbias"] for k in ks} == {tf.FLOAT, tf.QINT32}, op
            assert all(k["constraints"]["Tinput"] == tf.QUINT8 and k["constraints"]["out_type"] == tf.QUINT8 and
                       k["constraints"]["Tsummand"] == t_sum and k["host_memory"] == sum_host for k in ks), op
    for op in ("_QuantizedConv2D", "_ITEXQuantizedConv2DV2", "_QuantizedDepthwiseConv2D", "_ITEXQuantizedDepthwiseConv2DV2"):
        ks = kernels_of(reg, op)
        assert {k["constraints"]["out_type"] for k in ks} == {tf.QINT8, tf.QUINT8, tf.QINT32, tf.FLOAT, tf.BFLOAT16}
        assert all(k["host_memory"] == ["host_inputs", "host_outputs"] for k in ks)
        # Tsummand as the reference constrains it: either 8-bit type under an 8-bit output, else the output's type
        for k in ks:
            out_t, sum_t = k["constraints"]["out_type"], k["constraints"]["Tsummand"]
            assert sum_t in ((tf.QINT8, tf.QUINT8) if out_t in (tf.QINT8, tf.QUINT8) else (out_t,)), op
    for name, outs in (("QuantizedDepthwiseConv2D", {tf.QINT32}), ("QuantizedDepthwiseConv2DWithBias", {tf.QINT32}),
                       ("QuantizedDepthwiseConv2DWithBiasAndRelu", {tf.QINT32}),
                       ("QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize", {tf.QUINT8})):
        for op in (name, "_ITEX" + name):
            ks = kernels_of(reg, op)
            assert ks and {k["constraints"]["out_type"] for k in ks} == outs and all(k["constraints"]["Tinput"] == tf.QUINT8 for k in ks), op
    # stock TensorFlow defines the legacy names and _QuantizedConv2D; the plugin must define the renamed ones only
    names = {o["name"] for o in reg["ops"]}
    assert "_ITEXQuantizedConv2DV2" in names and "_ITEXQuantizedConv2DWithBiasAndRequantize" in names
    assert "QuantizedConv2D" not in names


def test_conv_attr_validation():
    base = dict(Tinput=DT(tf.QUINT8), Tfilter=DT(tf.QINT8), out_type=DT(tf.QINT32), strides=[1, 1, 1, 1], dilations=[1, 1, 1, 1],
                padding="SAME", padding_list=[])
    assert tf.Node("QuantizedConv2D", base).code == tf.OK
    for bad, code, msg in ((dict(strides=[1, 1, 1]), tf.INVALID_ARGUMENT, "Sliding window strides field must specify 4 dimensions"),
                           (dict(dilations=[1, 1]), tf.INVALID_ARGUMENT, "Sliding window dilations field must specify 4 dimensions"),
                           (dict(strides=[1, 0, 1, 1]), tf.INVALID_ARGUMENT, "Row and column strides should be larger than 0."),
                           (dict(dilations=[1, 1, 0, 1]), tf.INVALID_ARGUMENT, "Dilated rates should be larger than 0."),
                           (dict(padding="EXPLICIT", padding_list=[0, 0, 1]), tf.INVALID_ARGUMENT, None),
                           (dict(strides=[2, 1, 1, 1]), tf.UNIMPLEMENTED, None)):
        n = tf.Node("QuantizedConv2D", dict(base, **bad))
        assert n.code == code, (bad, n.code, n.message)
        if msg:
            assert n.message == msg
