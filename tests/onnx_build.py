"""Test helper: writes ONNX model files with the protobuf runtime (google.protobuf, an encoder independent of the reader under
test) from message descriptors typed in here after src/main/protobuf/onnx-ml.proto of the reference (field numbers: ModelProto
:187-230, GraphProto :246-267, NodeProto :161-178, AttributeProto :88-132, TensorProto :281-373, ValueInfoProto :145-151,
TypeProto :412-461, TensorShapeProto :393-406).  No model is downloaded: graphs are assembled node by node."""
import numpy as np
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

_F = descriptor_pb2.FieldDescriptorProto
_T = {"int64": _F.TYPE_INT64, "int32": _F.TYPE_INT32, "float": _F.TYPE_FLOAT, "string": _F.TYPE_STRING, "bytes": _F.TYPE_BYTES}


def _build():
    fdp = descriptor_pb2.FileDescriptorProto()
    fdp.name = "onnx_subset_for_tests.proto"; fdp.package = "onnxt"; fdp.syntax = "proto2"

    def message(name, fields, parent=None):
        m = (parent.nested_type if parent is not None else fdp.message_type).add()
        m.name = name
        for fname, number, ftype, repeated, packed in fields:
            f = m.field.add()
            f.name, f.number = fname, number
            f.label = _F.LABEL_REPEATED if repeated else _F.LABEL_OPTIONAL
            if ftype in _T:
                f.type = _T[ftype]
            else:
                f.type = _F.TYPE_MESSAGE; f.type_name = ".onnxt." + ftype
            if packed:
                f.options.packed = True
        return m

    message("TensorProto", [("dims", 1, "int64", True, False), ("data_type", 2, "int32", False, False), ("float_data", 4, "float", True, True),
                            ("int32_data", 5, "int32", True, True), ("int64_data", 7, "int64", True, True), ("name", 8, "string", False, False),
                            ("raw_data", 9, "bytes", False, False)])
    message("AttributeProto", [("name", 1, "string", False, False), ("f", 2, "float", False, False), ("i", 3, "int64", False, False), ("s", 4, "bytes", False, False),
                               ("t", 5, "TensorProto", False, False), ("floats", 7, "float", True, False), ("ints", 8, "int64", True, False), ("type", 20, "int32", False, False)])
    message("NodeProto", [("input", 1, "string", True, False), ("output", 2, "string", True, False), ("name", 3, "string", False, False),
                          ("op_type", 4, "string", False, False), ("attribute", 5, "AttributeProto", True, False)])
    shape = message("TensorShapeProto", [("dim", 1, "TensorShapeProto.Dimension", True, False)])
    message("Dimension", [("dim_value", 1, "int64", False, False), ("dim_param", 2, "string", False, False)], parent=shape)
    tp = message("TypeProto", [("tensor_type", 1, "TypeProto.Tensor", False, False)])
    message("Tensor", [("elem_type", 1, "int32", False, False), ("shape", 2, "TensorShapeProto", False, False)], parent=tp)
    message("ValueInfoProto", [("name", 1, "string", False, False), ("type", 2, "TypeProto", False, False)])
    message("GraphProto", [("node", 1, "NodeProto", True, False), ("name", 2, "string", False, False), ("initializer", 5, "TensorProto", True, False),
                           ("input", 11, "ValueInfoProto", True, False), ("output", 12, "ValueInfoProto", True, False)])
    message("ModelProto", [("ir_version", 1, "int64", False, False), ("producer_name", 2, "string", False, False), ("producer_version", 3, "string", False, False),
                           ("domain", 4, "string", False, False), ("model_version", 5, "int64", False, False), ("doc_string", 6, "string", False, False),
                           ("graph", 7, "GraphProto", False, False)])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fdp)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("onnxt." + n)) for n in ("ModelProto", "GraphProto", "NodeProto", "TensorProto", "ValueInfoProto")}


_CLS = _build()
FLOAT, INT64 = 1, 7


class GraphBuilder:
    """model = GraphBuilder("x", [N, C, H, W]); model.conv(...); ...; model.save(path, output_name, output_dims)"""

    def __init__(self, input_name, input_dims, typed_data=False):
        self.model = _CLS["ModelProto"]()
        self.model.ir_version = 3; self.model.producer_name = "lantern_amd tests"; self.model.producer_version = "1"; self.model.model_version = 1
        self.g = self.model.graph
        self.g.name = "test_graph"
        self.typed_data = typed_data                   # initialisers in float_data / int64_data instead of raw_data
        self._value(self.g.input.add(), input_name, input_dims, FLOAT)
        self.counter = 0

    @staticmethod
    def _value(v, name, dims, elem):
        v.name = name
        v.type.tensor_type.elem_type = elem
        for d in dims:
            v.type.tensor_type.shape.dim.add().dim_value = int(d)

    def fresh(self, stem):
        self.counter += 1
        return "%s_%d" % (stem, self.counter)

    def init(self, name, arr):
        """A float (or, for integer arrays, INT64) initialiser; like the exporters of that era it is also listed as a graph input."""
        arr = np.asarray(arr)
        t = self.g.initializer.add()
        t.name = name
        t.dims.extend(int(d) for d in arr.shape)
        if arr.dtype.kind == "f":
            t.data_type = FLOAT
            if self.typed_data: t.float_data.extend(float(v) for v in arr.astype("<f4").ravel())
            else: t.raw_data = arr.astype("<f4").tobytes()
        else:
            t.data_type = INT64
            if self.typed_data: t.int64_data.extend(int(v) for v in arr.ravel())
            else: t.raw_data = arr.astype("<i8").tobytes()
        self._value(self.g.input.add(), name, arr.shape, t.data_type)
        return name

    def node(self, op_type, inputs, outputs, **attrs):
        n = self.g.node.add()
        n.op_type = op_type
        n.input.extend(inputs); n.output.extend(outputs)
        for k, v in attrs.items():
            a = n.attribute.add()
            a.name = k
            if isinstance(v, float): a.f = v; a.type = 1
            elif isinstance(v, (bool, int, np.integer)): a.i = int(v); a.type = 2
            elif isinstance(v, (bytes, str)): a.s = v.encode() if isinstance(v, str) else v; a.type = 3
            elif isinstance(v, dict):                                      # a tensor attribute: {"dims": [...], "int64": [...]} or {"float": [...]}
                a.type = 4
                a.t.dims.extend(v.get("dims", []))
                if "int64" in v: a.t.data_type = INT64; a.t.raw_data = np.asarray(v["int64"], "<i8").tobytes()
                else: a.t.data_type = FLOAT; a.t.raw_data = np.asarray(v["float"], "<f4").tobytes()
            else: a.ints.extend(int(x) for x in v); a.type = 7
        return outputs[0]

    def save(self, path, output_name, output_dims):
        self._value(self.g.output.add(), output_name, output_dims, FLOAT)
        with open(path, "wb") as f:
            f.write(self.model.SerializeToString())
        return path


def export_module_tree(builder, model_kind, model, x_name):
    """The hand-built application networks (lantern_amd.apps.resnet50.ResNet50 with the 32x32 stem, apps.squeezenet.SqueezeNet)
    written out as the ONNX graphs a PyTorch export of the reference's model files gives: same node order as the modules' calls,
    parameters as initialisers.  Returns the output name."""
    b = builder

    def conv(x, m, name):
        ins = [x, b.init(name + ".weight", m.kernel.x.toCPU())]
        if m.bias is not None:
            ins.append(b.init(name + ".bias", m.bias.x.toCPU()))
        return b.node("Conv", ins, [b.fresh("conv")], kernel_shape=list(m.kernel.x.shape[2:]), strides=list(m.stride), pads=[m.pad[0], m.pad[1], m.pad[0], m.pad[1]], group=1,
                      dilations=[1, 1])

    def bn(x, m, name):
        ins = [x, b.init(name + ".weight", m.scale.x.toCPU()), b.init(name + ".bias", m.bias.x.toCPU()),
               b.init(name + ".running_mean", m.runningMean.toCPU()), b.init(name + ".running_var", m.runningVar.toCPU())]
        return b.node("BatchNormalization", ins, [b.fresh("bn")], epsilon=1e-5, momentum=0.9)

    relu = lambda x: b.node("Relu", [x], [b.fresh("relu")])
    pool = lambda x: b.node("MaxPool", [x], [b.fresh("pool")], kernel_shape=[2, 2], strides=[2, 2], pads=[0, 0, 0, 0])
    if model_kind == "resnet":
        h = pool(relu(bn(conv(x_name, model.conv1, "conv1"), model.bn1, "bn1")))
        for i, blk in enumerate(model.blocks):
            p = "layer%d" % i
            o = relu(bn(conv(h, blk.conv1, p + ".conv1"), blk.bn1, p + ".bn1"))
            o = relu(bn(conv(o, blk.conv2, p + ".conv2"), blk.bn2, p + ".bn2"))
            o = bn(conv(o, blk.conv3, p + ".conv3"), blk.bn3, p + ".bn3")
            idt = h if blk.down is None else bn(conv(h, blk.down[0], p + ".down.0"), blk.down[1], p + ".down.1")
            h = relu(b.node("Add", [o, idt], [b.fresh("add")]))
        return h
    # squeezenet
    h = pool(relu(conv(x_name, model.conv1, "conv1")))
    for i, st in enumerate(model.stages):
        if st is None:
            h = pool(h)
            continue
        p = "fire%d" % i
        s = relu(conv(h, st.squeeze, p + ".squeeze"))
        h = b.node("Concat", [relu(conv(s, st.e1, p + ".expand1x1")), relu(conv(s, st.e3, p + ".expand3x3"))], [b.fresh("cat")], axis=1)
    return conv(h, model.head, "conv10")
