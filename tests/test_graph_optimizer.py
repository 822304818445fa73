"""TF_InitGraph through the mock host: registration as TensorFlow checks it, and the quantized subset of the
reference's native-format rewrite (itex/core/graph/native_layout/native_layout.cc:113-198, layout_utils.cc:315-355,
497-545) on GraphDefs serialized and parsed by google.protobuf."""
import ctypes as C
import os

import pytest

from tests.mock_tf import graphdef as gd
from tests.mock_tf import host as tf

QINT8, QUINT8, QINT32, FLOAT = 11, 12, 13, 1
DEV = "/job:localhost/replica:0/task:0/device:XPU:0"
CPU = "/job:localhost/replica:0/task:0/device:CPU:0"


@pytest.fixture(scope="module")
def opt():
    lib = tf.load()
    lib.mock_graph_device_type.restype = C.c_char_p
    lib.mock_graph_result.restype = C.c_void_p
    lib.mock_graph_result_size.restype = C.c_size_t
    assert lib.mock_graph_init(tf.PLUGIN_LIB.encode()) == 0
    return lib


def run(opt, graph):
    data = graph.SerializeToString()
    code = opt.mock_graph_optimize(data, C.c_size_t(len(data)))
    assert code == tf.OK
    out = gd.GraphDef()
    out.ParseFromString(C.string_at(opt.mock_graph_result(), opt.mock_graph_result_size()))
    return out


def run_with_item(opt, graph, preserve="", fetch=""):
    """The same with a grappler item: comma-separated names the session asked to preserve / fetches."""
    data = graph.SerializeToString()
    code = opt.mock_graph_optimize_item(data, C.c_size_t(len(data)), preserve.encode(), fetch.encode())
    assert code == tf.OK
    out = gd.GraphDef()
    out.ParseFromString(C.string_at(opt.mock_graph_result(), opt.mock_graph_result_size()))
    return out


def by_name(g):
    return {n.name: n for n in g.node}


def test_registration(opt):
    assert opt.mock_graph_device_type() == b"XPU"
    TF_TriState_Off = 1
    assert opt.mock_graph_config(b"remapping") == TF_TriState_Off          # xpu_graph.cc:146-148
    assert opt.mock_graph_config(b"layout_optimizer") == TF_TriState_Off
    assert opt.mock_graph_config(b"constant_folding") == 0                 # left at TensorFlow's default


def qdq_graph():
    g = gd.GraphDef()
    g.versions.producer = 1645
    gd.node(g, "x", "Placeholder", device=DEV, dtype=("type", FLOAT))
    for c in ("mn", "mx"):
        gd.node(g, c, "Const", device=CPU, dtype=("type", FLOAT))
    # q1 feeds only a Dequantize: the classic zero-point algorithm; q2 feeds a matmul: the legacy one
    gd.node(g, "q1", "QuantizeV2", ["x", "mn", "mx"], DEV, T=("type", QUINT8), mode="MIN_FIRST", round_mode="HALF_AWAY_FROM_ZERO",
            narrow_range=False, axis=-1, ensure_minimum_range=0.01)
    gd.node(g, "dq1", "Dequantize", ["q1", "q1:1", "q1:2"], DEV, T=("type", QUINT8), mode="MIN_FIRST", narrow_range=False, axis=-1,
            dtype=("type", FLOAT))
    gd.node(g, "q2", "QuantizeV2", ["x", "mn", "mx", "^dq1"], DEV, T=("type", QUINT8), mode="MIN_FIRST",
            round_mode="HALF_AWAY_FROM_ZERO", narrow_range=False, axis=-1, ensure_minimum_range=0.01)
    gd.node(g, "mm", "_QuantizedMatMul", ["q2", "w", "b", "q2:1", "q2:2", "wmn", "wmx"], DEV, T1=("type", QUINT8), T2=("type", QINT8),
            Tbias=("type", FLOAT), Tout=("type", FLOAT), fused_ops=["BiasAdd", "Dequantize"], input_quant_mode="MIN_FIRST")
    return g


def test_quantize_rename_and_classic_algorithm_flag(opt):
    out = by_name(run(opt, qdq_graph()))
    assert out["q1"].op == "_ITEXQuantizeV2" and out["q2"].op == "_ITEXQuantizeV2"
    assert out["dq1"].op == "_ITEXDequantize" and out["mm"].op == "_ITEXQuantizedMatMul"
    assert out["q1"].attr["classic_asymmetric_algorithm"].b is True
    assert out["q2"].attr["classic_asymmetric_algorithm"].b is False
    assert out["q2"].attr["classic_asymmetric_algorithm"].WhichOneof("value") == "b"    # present, not defaulted
    assert out["q1"].attr["dtype"].type == FLOAT                                         # added for QuantizeV2
    # everything else is carried over: inputs incl. the control edge, device, the other attributes, other nodes
    assert list(out["q2"].input) == ["x", "mn", "mx", "^dq1"] and out["q2"].device == DEV
    assert out["q1"].attr["mode"].s == b"MIN_FIRST" and out["q1"].attr["T"].type == QUINT8
    assert abs(out["q1"].attr["ensure_minimum_range"].f - 0.01) < 1e-9 and out["q1"].attr["axis"].i == -1
    assert list(out["mm"].attr["fused_ops"].list.s) == [b"BiasAdd", b"Dequantize"]
    assert out["x"].op == "Placeholder" and out["mn"].op == "Const"
    assert run(opt, qdq_graph()).versions.producer == 1645


def test_rules_that_block_the_rewrite(opt):
    g = gd.GraphDef()
    common = dict(narrow_range=False, axis=-1, ensure_minimum_range=0.01)
    gd.node(g, "on_cpu", "QuantizeV2", ["x", "a", "b"], CPU, T=("type", QINT8), mode="SCALED", round_mode="HALF_TO_EVEN", **common)
    gd.node(g, "unplaced", "QuantizeV2", ["x", "a", "b"], "", T=("type", QINT8), mode="SCALED", round_mode="HALF_TO_EVEN", **common)
    gd.node(g, "min_combined", "QuantizeV2", ["x", "a", "b"], DEV, T=("type", QINT8), mode="MIN_COMBINED",
            round_mode="HALF_AWAY_FROM_ZERO", **common)
    gd.node(g, "scaled_away", "QuantizeV2", ["x", "a", "b"], DEV, T=("type", QINT8), mode="SCALED", round_mode="HALF_AWAY_FROM_ZERO",
            **common)
    gd.node(g, "qint32", "QuantizeV2", ["x", "a", "b"], DEV, T=("type", QINT32), mode="SCALED", round_mode="HALF_TO_EVEN", **common)
    gd.node(g, "ok", "QuantizeV2", ["x", "a", "b"], DEV, T=("type", QINT8), mode="SCALED", round_mode="HALF_TO_EVEN", **common)
    gd.node(g, "relu", "Relu", ["ok"], DEV, T=("type", FLOAT))
    out = by_name(run(opt, g))
    for name in ("on_cpu", "unplaced", "min_combined", "scaled_away", "qint32"):
        assert out[name].op == "QuantizeV2", name
        assert "classic_asymmetric_algorithm" not in out[name].attr
    assert out["ok"].op == "_ITEXQuantizeV2" and out["ok"].attr["classic_asymmetric_algorithm"].b is False   # feeds a Relu
    assert out["relu"].op == "Relu"


def test_every_renamed_op_has_a_kernel_and_an_op_definition(opt):
    reg = tf.registry()
    kernels = {k["op"] for k in reg["kernels"]}
    defined = {o["name"] for o in reg["ops"]}
    ops = ["Dequantize", "QuantizeV2", "QuantizedMatMulWithBias", "QuantizedMatMulWithBiasAndDequantize",
           "QuantizedMatMulWithBiasAndRelu", "QuantizedMatMulWithBiasAndReluAndRequantize", "QuantizedMatMulWithBiasAndRequantize",
           "_QuantizedBatchMatMul", "_QuantizedBatchMatMulV2AndDequantize", "_QuantizedFusedBatchMatMulV2AndDequantize",
           "_QuantizedFusedMatMul", "_QuantizedFusedMatMulAndDequantize", "_QuantizedFusedMatMulAndRequantize", "_QuantizedMatMul",
           "QuantizedReshape", "_QuantizedTranspose", "QuantizedConv2D", "QuantizedConv2DAndRequantize",
           "QuantizedConv2DPerChannel", "QuantizedConv2DWithBias", "QuantizedConv2DWithBiasAndRelu",
           "QuantizedConv2DWithBiasAndReluAndRequantize", "QuantizedConv2DWithBiasAndRequantize",
           "QuantizedConv2DWithBiasSumAndReluAndRequantize", "QuantizedConv2DWithBiasSignedSumAndReluAndRequantize",
           "QuantizedDepthwiseConv2D", "QuantizedDepthwiseConv2DWithBias", "QuantizedDepthwiseConv2DWithBiasAndRelu",
           "QuantizedDepthwiseConv2DWithBiasAndReluAndRequantize"]
    g = gd.GraphDef()
    for i, op in enumerate(ops):
        gd.node(g, "n%d" % i, op, ["x"], DEV, mode="SCALED", T=("type", QINT8))
    out = run(opt, g)
    for n, op in zip(out.node, ops):
        assert n.op == "_ITEX" + op.lstrip("_"), (op, n.op)
        assert n.op in kernels, n.op
        assert n.op in defined, n.op


def test_conv_rows(opt):
    # legacy names get data_format = "NHWC" added (layout_utils.cc:471-495); the new API op becomes ...V2 with its
    # attributes copied unchanged (native_layout.cc:178-179)
    g = gd.GraphDef()
    gd.node(g, "c1", "QuantizedConv2DWithBiasAndRequantize", ["x", "w", "b"], DEV, Tinput=("type", QUINT8), padding="SAME")
    gd.node(g, "c2", "_QuantizedConv2D", ["x", "w"], DEV, Tinput=("type", QINT8), data_format="NHWC", padding="VALID")
    gd.node(g, "c3", "QuantizedConv2D", ["x", "w"], CPU, Tinput=("type", QUINT8))
    out = by_name(run(opt, g))
    assert out["c1"].op == "_ITEXQuantizedConv2DWithBiasAndRequantize"
    assert out["c1"].attr["data_format"].s == b"NHWC" and out["c1"].attr["padding"].s == b"SAME"
    assert out["c1"].attr["Tinput"].type == QUINT8 and list(out["c1"].input) == ["x", "w", "b"]
    assert out["c2"].op == "_ITEXQuantizedConv2DV2" and out["c2"].attr["padding"].s == b"VALID"
    assert out["c3"].op == "QuantizedConv2D" and "data_format" not in out["c3"].attr
    g = gd.GraphDef()
    gd.node(g, "d", "_QuantizedDepthwiseConv2D", ["x", "w"], DEV, Tinput=("type", QUINT8))
    assert by_name(run(opt, g))["d"].op == "_ITEXQuantizedDepthwiseConv2DV2"


def dynamic_range_graph(shape_vals=(-1,), shape_dims=(1,), axis_vals=(0,), axis_dims=(), keep_dims=False, q_axis=-1,
                        max_src="flat", as_content=False, dtype=3, q_device=DEV):
    g = gd.GraphDef()
    gd.node(g, "x", "Placeholder", [], DEV)
    gd.node(g, "other", "Placeholder", [], DEV)
    gd.node(g, "shape", "Const", [], CPU, value=("tensor", dtype, shape_dims, list(shape_vals), as_content))
    gd.node(g, "axis", "Const", [], CPU, value=("tensor", dtype, axis_dims, list(axis_vals), as_content))
    gd.node(g, "flat", "Reshape", ["x", "shape"], DEV)
    gd.node(g, "flat2", "Reshape", ["other", "shape"], DEV)
    gd.node(g, "mn", "Min", ["flat:0", "axis"], DEV, keep_dims=keep_dims)
    gd.node(g, "mx", "Max", [max_src, "axis"], DEV, keep_dims=keep_dims)
    gd.node(g, "q", "QuantizeV2", ["x:0", "mn", "mx", "^flat"], q_device, T=("type", QUINT8), mode="MIN_FIRST",
            round_mode="HALF_AWAY_FROM_ZERO", axis=q_axis)
    gd.node(g, "mm", "_QuantizedMatMul", ["q", "w", "q:1", "q:2"], DEV)
    return g


@pytest.mark.parametrize("as_content,dtype", [(False, 3), (True, 3), (False, 9), (True, 9)])
def test_min_max_feeding_quantize_become_a_dynamic_range_quantize(opt, as_content, dtype):
    """QuantizeV2(x, Min(Reshape(x, [-1]), 0), Max(same, 0)) -> _ITEXQuantizeV2DynamicRange(x): the range is computed on
    the device by the op; the range inputs go, control inputs stay, attributes as for _ITEXQuantizeV2."""
    out = by_name(run(opt, dynamic_range_graph(as_content=as_content, dtype=dtype)))
    q = out["q"]
    assert q.op == "_ITEXQuantizeV2DynamicRange" and list(q.input) == ["x:0", "^flat"]
    assert q.attr["mode"].s == b"MIN_FIRST" and q.attr["dtype"].type == FLOAT and q.attr["T"].type == QUINT8
    assert q.attr["classic_asymmetric_algorithm"].b is False        # its consumer is a MatMul, not a Dequantize
    assert out["mn"].op == "Min" and out["mx"].op == "Max" and out["flat"].op == "Reshape"   # left for other readers / pruning
    reg = tf.registry()
    assert "_ITEXQuantizeV2DynamicRange" in {k["op"] for k in reg["kernels"]}
    assert "_ITEXQuantizeV2DynamicRange" in {o["name"] for o in reg["ops"]}


@pytest.mark.parametrize("kw", [dict(shape_vals=(2, -1), shape_dims=(2,)),      # not flattened to one dimension
                                dict(axis_vals=(1,)),                          # another reduction index
                                dict(axis_vals=(0, 1), axis_dims=(2,)),
                                dict(keep_dims=True),
                                dict(q_axis=0),                                # per-channel quantization
                                dict(max_src="flat2")],                        # Max of another tensor
                         ids=["shape", "axis", "two_axes", "keep_dims", "per_channel", "other_tensor"])
def test_dynamic_range_patterns_that_do_not_match(opt, kw):
    out = by_name(run(opt, dynamic_range_graph(**kw)))
    assert out["q"].op == "_ITEXQuantizeV2" and list(out["q"].input) == ["x:0", "mn", "mx", "^flat"]


def test_dynamic_range_switch_and_placement(opt, monkeypatch):
    out = by_name(run(opt, dynamic_range_graph(q_device=CPU)))
    assert out["q"].op == "QuantizeV2"
    monkeypatch.setenv("ITEX_AMD_FUSE_DYNAMIC_RANGE", "0")
    out = by_name(run(opt, dynamic_range_graph()))
    assert out["q"].op == "_ITEXQuantizeV2" and len(out["q"].input) == 4


def dynamic_linear_graph(fused_ops=("BiasAdd", "Dequantize"), q_mode="MIN_FIRST", m_mode="MIN_FIRST", t_q=QUINT8, t1=QUINT8,
                         extra_reader=False, with_out_range=False, mm_device=DEV, emr=0.02):
    """x -> Reshape -> Min / Max -> QuantizeV2 -> _QuantizedMatMul, as a dynamically quantized linear arrives"""
    g = gd.GraphDef()
    gd.node(g, "x", "Placeholder", [], DEV)
    gd.node(g, "shape", "Const", [], CPU, value=("tensor", 3, (1,), [-1], False))
    gd.node(g, "axis", "Const", [], CPU, value=("tensor", 3, (), [0], False))
    gd.node(g, "flat", "Reshape", ["x", "shape"], DEV)
    gd.node(g, "mn", "Min", ["flat", "axis"], DEV, keep_dims=False)
    gd.node(g, "mx", "Max", ["flat", "axis"], DEV, keep_dims=False)
    gd.node(g, "q", "QuantizeV2", ["x", "mn", "mx", "^ctl_q"], DEV, T=("type", t_q), mode=q_mode,
            round_mode="HALF_TO_EVEN" if q_mode == "SCALED" else "HALF_AWAY_FROM_ZERO", axis=-1, ensure_minimum_range=emr)
    host = ["q:1", "q:2", "wmn", "wmx"] + (["omn", "omx"] if with_out_range else [])
    gd.node(g, "mm", "_QuantizedMatMul", ["q", "w", "b"] + host + ["^ctl_m"], mm_device, T1=("type", t1), T2=("type", QINT8),
            Tbias=("type", FLOAT), Tout=("type", QINT8 if with_out_range else FLOAT), fused_ops=list(fused_ops),
            input_quant_mode=m_mode, Tdevice_inputs=("types", [t1, QINT8, FLOAT]), Thost_inputs=("types", [FLOAT] * len(host)),
            Tdevice_outputs=("types", [QINT8 if with_out_range else FLOAT]),
            Thost_outputs=("types", [FLOAT, FLOAT] if with_out_range else []))
    if extra_reader:
        gd.node(g, "spy", "Identity", ["q:1"], CPU)
    return g


@pytest.mark.parametrize("with_out_range", [False, True])
def test_dynamic_quantize_and_matmul_become_one_node(opt, with_out_range):
    """_ITEXQuantizeV2DynamicRange(x) read only by an _ITEXQuantizedMatMul -> _ITEXQuantizedMatMulDynamicInput(x, w, bias,
    min_b, max_b[, min_out, max_out]): the quantize node goes, its range floor and control inputs move over, the type
    lists follow the inputs."""
    fused = ("BiasAdd", "Relu", "Requantize") if with_out_range else ("BiasAdd", "Dequantize")
    out = by_name(run(opt, dynamic_linear_graph(fused_ops=fused, with_out_range=with_out_range)))
    assert "q" not in out
    mm = out["mm"]
    assert mm.op == "_ITEXQuantizedMatMulDynamicInput"
    tail = ["omn", "omx"] if with_out_range else []
    assert list(mm.input) == ["x", "w", "b", "wmn", "wmx"] + tail + ["^ctl_m", "^ctl_q"]
    assert list(mm.attr["Tdevice_inputs"].list.type) == [FLOAT, QINT8, FLOAT]
    assert list(mm.attr["Thost_inputs"].list.type) == [FLOAT] * (2 + len(tail))
    assert mm.attr["T1"].type == QUINT8 and mm.attr["input_quant_mode"].s == b"MIN_FIRST"
    assert abs(mm.attr["ensure_minimum_range"].f - 0.02) < 1e-9
    assert [f.decode() for f in mm.attr["fused_ops"].list.s] == list(fused)
    reg = tf.registry()
    assert "_ITEXQuantizedMatMulDynamicInput" in {k["op"] for k in reg["kernels"]}
    assert "_ITEXQuantizedMatMulDynamicInput" in {o["name"] for o in reg["ops"]}


@pytest.mark.parametrize("kw", [dict(extra_reader=True),                                  # someone else reads the range
                                dict(fused_ops=("BiasAdd",)),                             # qint32 result: its range is host math
                                dict(fused_ops=("BiasAdd", "Add", "Dequantize")),         # an addend shifts the inputs
                                dict(q_mode="SCALED", t_q=QINT8, t1=QINT8),               # modes disagree
                                dict(t_q=QUINT8, t1=QINT8),                               # types disagree
                                dict(mm_device=CPU)],                                     # the MatMul is not ours
                         ids=["other_reader", "s32_out", "addend", "mode", "type", "placement"])
def test_dynamic_quantize_matmul_pairs_that_stay_apart(opt, kw):
    out = by_name(run(opt, dynamic_linear_graph(**kw)))
    assert out["q"].op == "_ITEXQuantizeV2DynamicRange"
    assert out["mm"].op in ("_ITEXQuantizedMatMul", "_QuantizedMatMul") and out["mm"].input[0] == "q"


@pytest.mark.parametrize("item", [dict(preserve="q"), dict(fetch="q:1"), dict(fetch="q"), dict(preserve="w,q,b")])
def test_preserved_or_fetched_quantize_node_is_not_fused_away(opt, item):
    """A quantize node whose tensor or range the session fetches (or asked to preserve) has no reader inside the graph
    besides the MatMul, yet it must survive: the fusion reads the grappler item and leaves such a pair alone."""
    out = by_name(run_with_item(opt, dynamic_linear_graph(), **item))
    assert out["q"].op == "_ITEXQuantizeV2DynamicRange"
    assert out["mm"].op in ("_ITEXQuantizedMatMul", "_QuantizedMatMul") and out["mm"].input[0] == "q"
    # an item that names other nodes only does not stand in the way
    out = by_name(run_with_item(opt, dynamic_linear_graph(), preserve="w", fetch="mm"))
    assert "q" not in out and out["mm"].op == "_ITEXQuantizedMatMulDynamicInput"


def test_dynamic_quantize_matmul_scaled_and_switch(opt, monkeypatch):
    out = by_name(run(opt, dynamic_linear_graph(q_mode="SCALED", m_mode="SCALED", t_q=QINT8, t1=QINT8)))
    assert "q" not in out and out["mm"].op == "_ITEXQuantizedMatMulDynamicInput"
    monkeypatch.setenv("ITEX_AMD_FUSE_QUANTIZE_MATMUL", "0")
    out = by_name(run(opt, dynamic_linear_graph()))
    assert out["q"].op == "_ITEXQuantizeV2DynamicRange" and out["mm"].op == "_ITEXQuantizedMatMul"


@pytest.mark.parametrize("make", ["qdq", "dynamic_range", "dynamic_linear", "dynamic_linear_requantize"])
def test_the_pass_is_idempotent(opt, make):
    """Grappler may run a custom optimizer more than once: the second run leaves the first run's output as it is."""
    g = {"qdq": qdq_graph, "dynamic_range": dynamic_range_graph, "dynamic_linear": dynamic_linear_graph,
         "dynamic_linear_requantize": lambda: dynamic_linear_graph(fused_ops=("BiasAdd", "Requantize"), with_out_range=True)}[make]()
    once = run(opt, g)
    twice = run(opt, once)
    view = lambda gr: [(n.name, n.op, list(n.input), n.device, {k: v.SerializeToString() for k, v in n.attr.items()})
                       for n in gr.node]       # attribute maps carry no order
    assert view(twice) == view(once)


def test_reshape_is_only_renamed_for_qint8(opt):
    g = gd.GraphDef()
    gd.node(g, "a", "QuantizedReshape", ["x", "s", "mn", "mx"], DEV, T=("type", QINT8))
    gd.node(g, "b", "QuantizedReshape", ["x", "s", "mn", "mx"], DEV, T=("type", QUINT8))   # layout_utils.cc:392-400
    out = by_name(run(opt, g))
    assert out["a"].op == "_ITEXQuantizedReshape" and out["b"].op == "QuantizedReshape"


def test_switch_and_malformed_input(opt, monkeypatch):
    monkeypatch.setenv("ITEX_AMD_NATIVE_FORMAT", "0")
    out = by_name(run(opt, qdq_graph()))
    assert out["q1"].op == "QuantizeV2" and out["mm"].op == "_QuantizedMatMul"
    monkeypatch.delenv("ITEX_AMD_NATIVE_FORMAT")
    bad = b"\x0a\xff\xff\xff\x0f" + b"x" * 8      # a node whose length runs past the buffer
    assert opt.mock_graph_optimize(bad, C.c_size_t(len(bad))) == tf.INVALID_ARGUMENT


def test_unknown_fields_survive(opt):
    g = qdq_graph()
    data = g.SerializeToString() + b"\x18\x07"      # GraphDef.version = 3 (varint), unknown to the subset messages
    assert opt.mock_graph_optimize(data, C.c_size_t(len(data))) == tf.OK
    raw = C.string_at(opt.mock_graph_result(), opt.mock_graph_result_size())
    assert raw.endswith(b"\x18\x07")
