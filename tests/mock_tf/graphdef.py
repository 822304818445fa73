"""GraphDef / NodeDef / AttrValue messages for the graph-optimizer tests, built at run time from descriptors
(TensorFlow's generated classes are not available): the subset of tensorflow/core/framework/{graph,node_def,
attr_value}.proto the tests need, with the same field numbers, so that google.protobuf - not the plugin's own
wire codec - produces the input bytes and parses the output bytes."""
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

_F = descriptor_pb2.FieldDescriptorProto


def _build():
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name = "itex_amd_test_graph.proto"
    fd.package = "tensorflow_subset"
    fd.syntax = "proto3"

    lst = fd.message_type.add()
    lst.name = "ListValue"
    for name, num, typ in (("s", 2, _F.TYPE_BYTES), ("i", 3, _F.TYPE_INT64), ("f", 4, _F.TYPE_FLOAT), ("b", 5, _F.TYPE_BOOL),
                           ("type", 6, _F.TYPE_INT32)):
        f = lst.field.add()
        f.name, f.number, f.type, f.label = name, num, typ, _F.LABEL_REPEATED

    # tensor.proto / tensor_shape.proto: what a Const node's "value" needs
    shp = fd.message_type.add()
    shp.name = "TensorShapeProto"
    dim = shp.nested_type.add()
    dim.name = "Dim"
    f = dim.field.add()
    f.name, f.number, f.type, f.label = "size", 1, _F.TYPE_INT64, _F.LABEL_OPTIONAL
    f = shp.field.add()
    f.name, f.number, f.type, f.label, f.type_name = "dim", 2, _F.TYPE_MESSAGE, _F.LABEL_REPEATED, ".tensorflow_subset.TensorShapeProto.Dim"
    tp = fd.message_type.add()
    tp.name = "TensorProto"
    for name, num, typ, label, tn in (("dtype", 1, _F.TYPE_INT32, _F.LABEL_OPTIONAL, None),
                                      ("tensor_shape", 2, _F.TYPE_MESSAGE, _F.LABEL_OPTIONAL, ".tensorflow_subset.TensorShapeProto"),
                                      ("tensor_content", 4, _F.TYPE_BYTES, _F.LABEL_OPTIONAL, None),
                                      ("int_val", 7, _F.TYPE_INT32, _F.LABEL_REPEATED, None),
                                      ("int64_val", 10, _F.TYPE_INT64, _F.LABEL_REPEATED, None)):
        f = tp.field.add()
        f.name, f.number, f.type, f.label = name, num, typ, label
        if tn:
            f.type_name = tn

    av = fd.message_type.add()
    av.name = "AttrValue"
    av.oneof_decl.add().name = "value"
    for name, num, typ, tn in (("s", 2, _F.TYPE_BYTES, None), ("i", 3, _F.TYPE_INT64, None), ("f", 4, _F.TYPE_FLOAT, None),
                               ("b", 5, _F.TYPE_BOOL, None), ("type", 6, _F.TYPE_INT32, None),
                               ("list", 1, _F.TYPE_MESSAGE, ".tensorflow_subset.ListValue"),
                               ("tensor", 8, _F.TYPE_MESSAGE, ".tensorflow_subset.TensorProto")):
        f = av.field.add()
        f.name, f.number, f.type, f.label = name, num, typ, _F.LABEL_OPTIONAL
        f.oneof_index = 0
        if tn:
            f.type_name = tn

    nd = fd.message_type.add()
    nd.name = "NodeDef"
    entry = nd.nested_type.add()
    entry.name = "AttrEntry"
    entry.options.map_entry = True
    k = entry.field.add()
    k.name, k.number, k.type, k.label = "key", 1, _F.TYPE_STRING, _F.LABEL_OPTIONAL
    v = entry.field.add()
    v.name, v.number, v.type, v.label, v.type_name = "value", 2, _F.TYPE_MESSAGE, _F.LABEL_OPTIONAL, ".tensorflow_subset.AttrValue"
    for name, num, typ, label, tn in (("name", 1, _F.TYPE_STRING, _F.LABEL_OPTIONAL, None),
                                      ("op", 2, _F.TYPE_STRING, _F.LABEL_OPTIONAL, None),
                                      ("input", 3, _F.TYPE_STRING, _F.LABEL_REPEATED, None),
                                      ("device", 4, _F.TYPE_STRING, _F.LABEL_OPTIONAL, None),
                                      ("attr", 5, _F.TYPE_MESSAGE, _F.LABEL_REPEATED, ".tensorflow_subset.NodeDef.AttrEntry")):
        f = nd.field.add()
        f.name, f.number, f.type, f.label = name, num, typ, label
        if tn:
            f.type_name = tn

    ver = fd.message_type.add()
    ver.name = "VersionDef"
    f = ver.field.add()
    f.name, f.number, f.type, f.label = "producer", 1, _F.TYPE_INT32, _F.LABEL_OPTIONAL

    gd = fd.message_type.add()
    gd.name = "GraphDef"
    f = gd.field.add()
    f.name, f.number, f.type, f.label, f.type_name = "node", 1, _F.TYPE_MESSAGE, _F.LABEL_REPEATED, ".tensorflow_subset.NodeDef"
    f = gd.field.add()
    f.name, f.number, f.type, f.label, f.type_name = "versions", 4, _F.TYPE_MESSAGE, _F.LABEL_OPTIONAL, ".tensorflow_subset.VersionDef"

    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    if get is None:
        factory = message_factory.MessageFactory(pool)
        get = factory.GetPrototype
    return {n: get(pool.FindMessageTypeByName("tensorflow_subset." + n)) for n in ("GraphDef", "NodeDef", "AttrValue")}


_M = _build()
GraphDef, NodeDef, AttrValue = _M["GraphDef"], _M["NodeDef"], _M["AttrValue"]


def node(graph, name, op, inputs=(), device="", **attrs):
    """Adds a node; attribute values: str -> s, bool -> b, int -> i, float -> f, ("type", n) -> type, ("types", [n, ...]) -> list.type,
    list of str -> list.s, ("tensor", dtype, shape, values, as_content) -> an int32 (3) / int64 (9) tensor"""
    n = graph.node.add()
    n.name, n.op, n.device = name, op, device
    n.input.extend(inputs)
    for k, v in attrs.items():
        a = n.attr[k]
        if isinstance(v, bool):
            a.b = v
        elif isinstance(v, str):
            a.s = v.encode()
        elif isinstance(v, int):
            a.i = v
        elif isinstance(v, float):
            a.f = v
        elif isinstance(v, tuple) and v[0] == "type":
            a.type = v[1]
        elif isinstance(v, tuple) and v[0] == "types":      # ("types", [n, ...]) -> list.type
            a.list.SetInParent()
            a.list.type.extend(v[1])
        elif isinstance(v, list):
            a.list.s.extend(x.encode() for x in v)
        elif isinstance(v, tuple) and v[0] == "tensor":     # ("tensor", dtype, shape, values, as_content)
            _, dtype, shape, values, as_content = v
            a.tensor.dtype = dtype
            for d in shape:
                a.tensor.tensor_shape.dim.add().size = d
            if as_content:
                import struct
                a.tensor.tensor_content = b"".join(struct.pack("<i" if dtype == 3 else "<q", x) for x in values)
            elif dtype == 3:
                a.tensor.int_val.extend(values)
            else:
                a.tensor.int64_val.extend(values)
        else:
            raise TypeError(k)
    return n
