"""ONNX front door: a model file -> the sequence of Tensor / TensorR operator calls the reference builds from it.

Mirrors src/main/scala/lantern/ONNXLib.scala: `readONNX(model_file)` (:209-253) parses the ModelProto, writes every float
initialiser back to back into `<model_file>.bin` (`ParameterWriter`, :157-185; offsets counted in floats) and keeps the
INT64 initialisers as shape values (`intMap`, :226-232); `inference_func` (:597-830) and `training_func` (:833-1071) map
the 22 node types onto the operator surface (Conv -> conv2D_batch / convBBP, Relu -> relu / relu(inPlace), MaxPool ->
maxPool2D_batch with its pads / maxPoolBK WITHOUT them (:876-877), Softmax -> softmax_batch / logSoftmaxB, Gemm ->
gemm(alpha) + bias[*beta], BatchNormalization -> batchNormInference / batchNorm, shape arithmetic on `intMap`, ...).

The reference reads the protobuf through javacpp's ONNX bindings; here the wire format is decoded directly (no protobuf
runtime, no onnx package): varints, 64-/32-bit scalars and length-delimited fields of the messages of
src/main/protobuf/onnx-ml.proto that the reference touches (ModelProto :187-230, GraphProto :246-267, NodeProto :161-178,
AttributeProto :88-132, TensorProto :281-373, ValueInfoProto :145-151, TypeProto :412-461, TensorShapeProto :393-406).
"""
import os
import struct

import numpy as np

from .tensor import Tensor, TensorR

FLOAT, INT64 = 1, 7                    # TensorProto.DataType values the reference accepts (ONNXLib.scala:114-135)


# ---- protobuf wire format ----------------------------------------------------------------------------------------
def _varint(buf, pos):
    result, shift = 0, 0
    while True:
        if pos >= len(buf):
            raise ValueError("truncated varint")
        b = buf[pos]; pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7
        if shift > 63:
            raise ValueError("varint longer than 10 bytes")


def _fields(buf):
    """Yields (field number, wire type, value) of one message: int for varint / fixed, bytes for length-delimited."""
    pos, n = 0, len(buf)
    while pos < n:
        key, pos = _varint(buf, pos)
        field, wire = key >> 3, key & 7
        if wire == 0:
            val, pos = _varint(buf, pos)
        elif wire == 1:
            if pos + 8 > n: raise ValueError("truncated 64-bit field")
            val = bytes(buf[pos:pos + 8]); pos += 8
        elif wire == 2:
            ln, pos = _varint(buf, pos)
            if pos + ln > n: raise ValueError("length-delimited field runs past the end of its message")
            val = bytes(buf[pos:pos + ln]); pos += ln
        elif wire == 5:
            if pos + 4 > n: raise ValueError("truncated 32-bit field")
            val = bytes(buf[pos:pos + 4]); pos += 4
        else:
            raise ValueError("unsupported wire type %d (groups are not used by ONNX)" % wire)
        yield field, wire, val


def _sint64(v):
    """int64 fields travel as unsigned varints of their two's complement."""
    return v - (1 << 64) if v >= (1 << 63) else v


def _packed_varints(val, wire):
    if wire == 0:
        return [_sint64(val)]
    out, pos = [], 0
    while pos < len(val):
        v, pos = _varint(val, pos)
        out.append(_sint64(v))
    return out


class TensorProto:
    def __init__(self, buf):
        self.dims, self.data_type, self.name, self.raw_data = [], 0, "", None
        floats, int64s, int32s = [], [], []
        for f, w, v in _fields(buf):
            if f == 1: self.dims += _packed_varints(v, w)
            elif f == 2: self.data_type = v
            elif f == 4: floats += list(struct.unpack("<%df" % (len(v) // 4), v)) if w == 2 else [struct.unpack("<f", v)[0]]
            elif f == 5: int32s += _packed_varints(v, w)
            elif f == 7: int64s += _packed_varints(v, w)
            elif f == 8: self.name = v.decode("utf-8")
            elif f == 9: self.raw_data = v
        # The reference reads raw_data only (ONNXLib.scala:116-133); exporters that fill the typed fields instead are accepted too.
        if self.raw_data is None:
            if self.data_type == FLOAT: self.raw_data = np.asarray(floats, "<f4").tobytes()
            elif self.data_type == INT64: self.raw_data = np.asarray(int64s, "<i8").tobytes()
            else: self.raw_data = b""

    def values(self):
        """extract_init (ONNXLib.scala:110-139): little-endian floats, or int64 shape values as floats."""
        n = int(np.prod(self.dims, dtype=np.int64)) if self.dims else 1
        if self.data_type == FLOAT:
            arr = np.frombuffer(self.raw_data, "<f4")
        elif self.data_type == INT64:
            arr = np.frombuffer(self.raw_data, "<i8").astype(np.float32)
        else:
            raise RuntimeError("data type not Float, Not handling yet: %d" % self.data_type)
        assert arr.size == n, "%d != %s" % (arr.size, self.dims)
        return arr


class Attribute:
    def __init__(self, buf):
        self.name, self.f, self.i, self.s, self.t, self.ints, self.floats = "", 0.0, 0, b"", None, [], []
        for f, w, v in _fields(buf):
            if f == 1: self.name = v.decode("utf-8")
            elif f == 2: self.f = struct.unpack("<f", v)[0]
            elif f == 3: self.i = _sint64(v)
            elif f == 4: self.s = v
            elif f == 5: self.t = TensorProto(v)
            elif f == 7: self.floats += list(struct.unpack("<%df" % (len(v) // 4), v)) if w == 2 else [struct.unpack("<f", v)[0]]
            elif f == 8: self.ints += _packed_varints(v, w)


class NodeProto:
    def __init__(self, buf):
        self.input, self.output, self.name, self.op_type, self.attribute = [], [], "", "", []
        for f, w, v in _fields(buf):
            if f == 1: self.input.append(v.decode("utf-8"))
            elif f == 2: self.output.append(v.decode("utf-8"))
            elif f == 3: self.name = v.decode("utf-8")
            elif f == 4: self.op_type = v.decode("utf-8")
            elif f == 5: self.attribute.append(Attribute(v))


def _value_info(buf):
    """extract_value (ONNXLib.scala:142-152): name -> (dims, elem_type)."""
    name, dims, elem = "", [], 0
    for f, w, v in _fields(buf):
        if f == 1: name = v.decode("utf-8")
        elif f == 2:                                            # TypeProto
            for f2, w2, v2 in _fields(v):
                if f2 == 1:                                     # tensor_type
                    for f3, w3, v3 in _fields(v2):
                        if f3 == 1: elem = v3
                        elif f3 == 2:                           # TensorShapeProto
                            for f4, w4, v4 in _fields(v3):
                                if f4 == 1:                     # Dimension
                                    dv = 0
                                    for f5, w5, v5 in _fields(v4):
                                        if f5 == 1: dv = _sint64(v5)
                                    dims.append(int(dv))
    return name, (dims, elem)


class GraphProto:
    def __init__(self, buf):
        self.node, self.name, self.initializer, self.input, self.output = [], "", [], [], []
        for f, w, v in _fields(buf):
            if f == 1: self.node.append(NodeProto(v))
            elif f == 2: self.name = v.decode("utf-8")
            elif f == 5: self.initializer.append(TensorProto(v))
            elif f == 11: self.input.append(_value_info(v))
            elif f == 12: self.output.append(_value_info(v))


class ModelProto:
    def __init__(self, buf):
        self.ir_version, self.producer_name, self.producer_version, self.domain, self.model_version, self.doc_string, self.graph = 0, "", "", "", 0, "", None
        for f, w, v in _fields(buf):
            if f == 1: self.ir_version = v
            elif f == 2: self.producer_name = v.decode("utf-8")
            elif f == 3: self.producer_version = v.decode("utf-8")
            elif f == 4: self.domain = v.decode("utf-8")
            elif f == 5: self.model_version = v
            elif f == 6: self.doc_string = v.decode("utf-8")
            elif f == 7: self.graph = GraphProto(v)
        if self.graph is None:
            raise ValueError("not an ONNX model: no graph")


# ---- the `<model>.onnx.bin` parameter file (ONNXLib.scala:157-185) ------------------------------------------------
class ParameterWriter:
    """Float initialisers written back to back as they come; an initialiser's offset is counted in floats."""

    def __init__(self, filename):
        self.output = open(filename, "wb")
        self.off = 0

    def addParams(self, data):
        self.output.write(data)
        offset = self.off
        self.off += len(data)
        return offset // 4

    def record_init(self, init):
        if init.data_type != FLOAT:
            raise RuntimeError("data type not Float, Not handling yet: %d" % init.data_type)
        return init.name, (list(init.dims), init.data_type, self.addParams(init.raw_data))

    def close(self):
        self.output.close()


class ParameterReader:
    def __init__(self, filename):
        self.parameters = np.fromfile(filename, "<f4")

    def getOffset(self, offset, count):
        return self.parameters[offset:offset + count]


def readTensor(tensor_file):
    """A TensorProto file (the model zoo's test_data_set_*/input_0.pb, output_0.pb) as a host array with its dims (ONNXLib.scala:144-155)."""
    with open(tensor_file, "rb") as f:
        t = TensorProto(f.read())
    return t.values().reshape(t.dims)


def _conv_pool_attrs(attributes):
    """getConvMaxPAvPAttr (ONNXLib.scala:283-294)."""
    atts = {a.name: ([int(a.i)] if a.name == "group" else [int(v) for v in a.ints]) for a in attributes}
    assert "strides" in atts, "attributes of a conv/maxP/avP node should have strides"
    assert "kernel_shape" in atts, "attributes of a conv/maxP/avP node should have kernel_shape"
    assert len(atts["strides"]) == 2, "strides should be length 2"
    assert len(atts["kernel_shape"]) == 2, "kernel_shape should be length 2"
    atts.setdefault("pads", [0, 0, 0, 0])
    return atts


class readONNX:
    """ONNXLib.scala:209-1071.  `allNodes` holds (kind, ...) records in graph order."""

    def __init__(self, model_file):
        with open(model_file, "rb") as f:
            self.model = ModelProto(f.read())
        graph = self.graph = self.model.graph
        float_init = [t for t in graph.initializer if t.data_type == FLOAT]
        int_init = [t for t in graph.initializer if t.data_type != FLOAT]
        # shape-valued tensors: name -> (dims of the tensor: [n] or [], the values)
        self.intMap = {t.name: (list(t.dims), [int(v) for v in t.values()]) for t in int_init}
        self.parameterFileName = model_file + ".bin"
        writer = ParameterWriter(self.parameterFileName)
        self.byteMap = dict(writer.record_init(t) for t in float_init)
        writer.close()
        self.reader = ParameterReader(os.path.abspath(self.parameterFileName))
        self.input_map = dict(graph.input)
        self.output_map = dict(graph.output)
        self.x_name, self.x_dims = self.real_input()
        self.y_name, self.y_dims = self.real_output()
        self.allNodes = [self._node(n) for n in graph.node]
        self.modelMap = {"irversion:": self.model.ir_version, "producer name:": self.model.producer_name, "producer version:": self.model.producer_version,
                         "domain:": self.model.domain, "model version:": self.model.model_version, "doc string:": self.model.doc_string,
                         "name of graph:": graph.name, "number of initializer:": len(graph.initializer), "number of inputs:": len(graph.input),
                         "number of outputs:": len(graph.output), "number of nodes:": len(graph.node), "all nodes:": self.allNodes}

    def real_input(self):
        """The one graph input that is not an initialiser (:234-242)."""
        rest = [k for k in self.input_map if k not in self.byteMap and k not in self.intMap]
        assert len(rest) == 1, "there should be one uninitialized input, got %s" % rest
        return rest[0], [int(v) for v in self.input_map[rest[0]][0]]

    def real_output(self):
        keys = list(self.output_map)
        assert len(keys) == 1, "we hope that there is only one output for the model"
        return keys[0], [int(v) for v in self.output_map[keys[0]][0]]

    def _node(self, node):
        """The `allNodes` match (:308-574), arity checks included."""
        op, ins, outs, atts = node.op_type, node.input, node.output, node.attribute
        def one_out():
            assert len(outs) == 1, "number of outputs of a %s node should be 1, got %d" % (op, len(outs))
        if op == "Conv":
            assert len(ins) in (2, 3), "number of inputs of a conv node should always be 2 or 3, got %d" % len(ins)
            one_out()
            return ("conv", ins, outs[0], _conv_pool_attrs(atts))
        if op == "BatchNormalization":
            assert len(ins) == 5, "Number of inputs for a batch normalization layer should be 5, got %d" % len(ins)
            one_out()
            am = {}
            for a in atts:
                if a.name == "epsilon": am["epsilon"] = float(a.f)
                elif a.name == "is_test": am["is_test"] = float(a.i)
                elif a.name == "momentum": am["momentum"] = float(a.f)
                else: raise NotImplementedError("not yet handling BatchNormalization attributes %s" % a.name)
            return ("bn", ins, outs[0], am)
        if op in ("Sum", "Add"):
            assert len(ins) == 2, "number of inputs for %s layer should be 2, got %d" % (op, len(ins))
            one_out()
            return ("sum" if op == "Sum" else "add", ins, outs[0])
        if op == "Relu":
            assert len(ins) == 1, "number of inputs of a relu node should always be 1"
            one_out()
            return ("relu", ins[0], outs[0])
        if op in ("MaxPool", "AveragePool"):
            assert len(ins) == 1, "number of inputs of a %s node should always be 1" % op
            one_out()
            return ("maxpool" if op == "MaxPool" else "averagePool", ins[0], outs[0], _conv_pool_attrs(atts))
        if op == "Concat":
            assert len(ins) > 1, "number of inputs for concat node should be larger than 1"
            one_out()
            assert len(atts) == 1, "number of attributes of a concat node should be 1"
            return ("concat", ins, outs[0], int(atts[0].i))
        if op == "Dropout":
            assert len(ins) == 1, "number of inputs for dropout node should always be 1"
            assert len(outs) == 2, "number of outputs for dropout node should always be 2"
            assert len(atts) == 1, "number of attributes for drop out node should be 1"
            return ("dropout", ins[0], outs, float(atts[0].f))
        if op == "GlobalAveragePool":
            assert len(ins) == 1; one_out()
            return ("globalAveragePool", ins[0], outs[0])
        if op == "Softmax":
            assert len(ins) == 1; one_out()
            return ("softmax", ins[0], outs[0])
        if op == "Reshape":
            assert len(ins) == 2, "number of inputs for Reshape layer should be 2"
            one_out()
            return ("reshape", ins, outs[0])
        if op == "Gemm":
            assert len(ins) == 3, "number of inputs for Gemm layer should be 3, got %d" % len(ins)
            one_out()
            ai = {a.name: int(a.i) for a in atts if a.name in ("transA", "transB")}
            af = {a.name: float(a.f) for a in atts if a.name in ("alpha", "beta")}
            return ("gemm", ins, outs[0], ai, af)
        if op == "Flatten":
            assert len(ins) == 1; one_out()
            assert len(atts) == 1, "number of attributes of a Flatten node should be 1"
            return ("flatten", ins[0], outs[0], int(atts[0].i))
        if op == "Pad":
            assert len(ins) == 1; one_out()
            assert len(atts) == 3, "number of attributes of a Pad node should be 3, got %d" % len(atts)
            by = {a.name: a for a in atts}
            return ("pad", ins[0], outs[0], by["mode"].s.decode("utf-8"), [int(v) for v in by["pads"].ints], float(by["value"].f))
        if op == "Shape":
            assert len(ins) == 1; one_out()
            return ("shape", ins[0], outs[0])
        if op == "Slice":
            assert len(ins) == 1; one_out()
            return ("slice", ins[0], outs[0], {a.name: [int(v) for v in a.ints] for a in atts})
        if op in ("Squeeze", "Unsqueeze"):
            assert len(ins) == 1; one_out()
            assert len(atts) == 1, "size of attributes should be 1 for %sNode, got %d" % (op.lower(), len(atts))
            return (op.lower(), ins[0], outs[0], [int(v) for v in atts[0].ints])
        if op == "Constant":
            one_out()
            assert len(atts) == 1, "size of attributes should be 1 for constantNode, got %d" % len(atts)
            vals = atts[0].t.values()
            assert vals.size == 1, "constant node should have tensor with single value, got %s" % atts[0].t.dims
            return ("constant", outs[0], float(vals[0]))
        if op == "Gather":
            # the reference's Gather takes ONE input and uses its integer attribute as the index into a shape value (:563-570)
            assert len(ins) == 1, "inputs should be size 1 for GatherNode, got %d" % len(ins)
            one_out()
            assert len(atts) == 1, "attributes size should be 1 for GatherNode, got %d" % len(atts)
            return ("gather", ins[0], outs[0], int(atts[0].i))
        raise RuntimeError("Node %s not yet implemented" % op)

    def initializer_map_tensor(self):
        """name -> Tensor over the parameter file's floats, in backend memory (the reference mmaps the file and uploads: :591-592,
        resnet50FromOnnx.scala:151)."""
        out = {}
        for name, (dims, _, offset) in self.byteMap.items():
            n = int(np.prod(dims, dtype=np.int64)) if dims else 1
            out[name] = Tensor.fromNumpy(np.ascontiguousarray(self.reader.getOffset(offset, n), np.float32).reshape(dims if dims else (1,)))
        return out

    # ---- shape arithmetic shared by both mappings (:783-818 and :989-1056) ----
    def _shape_node(self, node, has_tensor, shape_of):
        kind = node[0]
        im = self.intMap
        if kind == "shape":
            s = list(shape_of(node[1])); im[node[2]] = ([len(s)], s)
        elif kind == "constant":
            im[node[1]] = ([], [int(node[2])])
        elif kind == "slice":
            if has_tensor(node[1]): raise NotImplementedError("Slice of a data tensor")
            _, vals = im[node[1]]
            att = node[3]
            axes, starts, ends = att.get("axes", []), att.get("starts", []), att.get("ends", [])
            assert axes == [0], "for slice shape tensor, axes must be 0, axes got %s" % axes
            assert len(starts) == 1 and len(ends) == 1, "for slice shape tensor, starts and ends must be size 1"
            im[node[2]] = ([ends[0] - starts[0]], vals[:ends[0]][starts[0]:])
        elif kind == "squeeze":
            if has_tensor(node[1]): raise NotImplementedError("Squeeze of a data tensor")
            dims, vals = im[node[1]]
            assert node[3] == [0] and dims == [1] and len(vals) == 1, "squeeze on shape tensor must be on dim 0 of a one-element value"
            im[node[2]] = ([], vals)
        elif kind == "unsqueeze":
            if has_tensor(node[1]): raise NotImplementedError("Unsqueeze of a data tensor")
            dims, vals = im[node[1]]
            assert node[3] == [0] and dims == [] and len(vals) == 1, "unsqueeze on shape tensor must be on dim 0 of a scalar"
            im[node[2]] = ([1], vals)
        elif kind == "gather":
            if has_tensor(node[1]): raise NotImplementedError("Gather of a data tensor")
            _, vals = im[node[1]]
            assert node[3] < len(vals), "axis out of bound, got %d, but array size is %d" % (node[3], len(vals))
            im[node[2]] = ([], [vals[node[3]]])
        else:
            return False
        return True

    def _concat_shapes(self, ins, out, axis):
        parts = [self.intMap[k] for k in ins]
        for d, _ in parts:
            assert len(d) == 1, "shape tensors should have rank 1, got %s" % d
        assert axis == 0, "concatenating shape tensors should only be on dim 0, got %d" % axis
        self.intMap[out] = ([sum(d[0] for d, _ in parts)], [v for _, a in parts for v in a])

    def inference_func(self, initializer_map_tensor, allNodesPassed=None):
        """Tensor -> Tensor (:597-830)."""
        nodes = self.allNodes if allNodesPassed is None else allNodesPassed

        def run(x):
            assert list(x.shape) == self.x_dims, "input tensor is not of the correct dimensions: %s, expected %s" % (list(x.shape), self.x_dims)
            inter = {self.x_name: x}
            def get(k): return initializer_map_tensor[k] if k in initializer_map_tensor else inter[k]
            def has(k): return k in initializer_map_tensor or k in inter
            for node in nodes:
                kind = node[0]
                if kind == "conv":
                    _, ins, out, atts = node
                    bias = get(ins[2]) if len(ins) == 3 else None
                    inter[out] = get(ins[0]).conv2D_batch(get(ins[1]), bias, atts["strides"], atts["pads"])[0]
                elif kind == "relu":
                    inter[node[2]] = get(node[1]).relu()
                elif kind == "maxpool":
                    _, i, out, atts = node
                    inter[out] = get(i).maxPool2D_batch(atts["kernel_shape"], atts["strides"], atts["pads"])[0]
                elif kind == "averagePool":
                    _, i, out, atts = node
                    inter[out] = get(i).averagePool2D_batch(atts["kernel_shape"], atts["strides"], atts["pads"])
                elif kind == "concat":
                    _, ins, out, axis = node
                    if has(ins[0]):
                        ts = [get(k) for k in ins]
                        inter[out] = ts[0].concat(axis, *ts[1:])
                    else:
                        self._concat_shapes(ins, out, axis)
                elif kind == "dropout":
                    inter[node[2][0]] = get(node[1])                     # identity at inference
                elif kind == "globalAveragePool":
                    inter[node[2]] = get(node[1]).global_ave_batch()
                elif kind == "softmax":
                    inter[node[2]] = get(node[1]).softmax_batch()
                elif kind == "bn":
                    _, ins, out, _am = node
                    x_, scale, bias, rm, rv = [get(k) for k in ins]
                    inter[out] = x_.batchNormInference(scale, bias, rm, rv)
                elif kind in ("sum", "add"):
                    inter[node[2]] = get(node[1][0]) + get(node[1][1])
                elif kind == "reshape":
                    _, ins, out = node
                    dims, vals = self.intMap[ins[1]]
                    assert len(dims) == 1, "reshape parameter (if presented as a tensor) should be dim 1, got %d" % len(dims)
                    inter[out] = get(ins[0]).resize(*vals)
                elif kind == "gemm":
                    _, ins, out, ai, af = node
                    alpha, beta = af.get("alpha", 1.0), af.get("beta", 1.0)
                    c = get(ins[2])
                    inter[out] = get(ins[0]).gemm(get(ins[1]), ai.get("transA", 0) == 1, ai.get("transB", 0) == 1, alpha) + (c if beta == 1.0 else c * beta)
                elif kind == "flatten":
                    _, i, out, axis = node
                    t = get(i)
                    inter[out] = t.resize(*(list(t.shape[:axis]) + [-1]))
                elif kind == "pad":
                    _, i, out, mode, pads, value = node
                    if not has(i): raise NotImplementedError("Pad of a shape value")
                    assert sum(pads) == 0, "TODO: only supporting no padding so far, got %s" % pads
                    inter[out] = get(i)
                elif not self._shape_node(node, has, lambda k: get(k).shape):
                    raise RuntimeError("not yet implemented, %s" % (node,))
            return inter[self.y_name]
        return run

    def training_func(self, initializer_map_tensor):
        """(TensorR -> TensorR, name -> TensorR of every float initialiser) (:833-1071).  The caller's optimizer steps over
        the whole map, running statistics included (they receive no gradient: resnet50FromOnnx.scala:177-180)."""
        params = {name: TensorR(t) for name, t in initializer_map_tensor.items()}

        def run(x):
            assert list(x.x.shape) == self.x_dims, "input tensor is not of the correct dimensions: %s, expected %s" % (list(x.x.shape), self.x_dims)
            inter = {self.x_name: x}
            def get(k): return params[k] if k in params else inter[k]
            def has(k): return k in params or k in inter
            for node in self.allNodes:
                kind = node[0]
                if kind == "conv":
                    _, ins, out, atts = node
                    bias = get(ins[2]) if len(ins) == 3 else None
                    inter[out] = get(ins[0]).convBBP(get(ins[1]), bias, atts["strides"], atts["pads"])
                elif kind == "relu":
                    inter[node[2]] = get(node[1]).relu(True)
                elif kind == "maxpool":
                    _, i, out, atts = node
                    inter[out] = get(i).maxPoolBK(atts["kernel_shape"], atts["strides"], None)      # the pads are dropped (:876-877)
                elif kind == "concat":
                    _, ins, out, axis = node
                    if has(ins[0]):
                        ts = [get(k) for k in ins]
                        inter[out] = ts[0].concat(axis, *ts[1:])
                    else:
                        self._concat_shapes(ins, out, axis)
                elif kind == "dropout":
                    inter[node[2][0]] = get(node[1]).dropout(node[3])
                elif kind == "globalAveragePool":
                    inter[node[2]] = get(node[1]).global_ave_batch()
                elif kind == "softmax":
                    inter[node[2]] = get(node[1]).logSoftmaxB()
                elif kind == "averagePool":
                    _, i, out, atts = node
                    inter[out] = get(i).averagePoolBK(atts["kernel_shape"], atts["strides"], atts["pads"])
                elif kind == "bn":
                    _, ins, out, _am = node
                    x_, scale, bias, rm, rv = [get(k) for k in ins]
                    inter[out] = x_.batchNorm(scale, bias, rm.x, rv.x)
                elif kind in ("sum", "add"):
                    inter[node[2]] = get(node[1][0]) + get(node[1][1])
                elif kind == "reshape":
                    _, ins, out = node
                    dims, vals = self.intMap[ins[1]]
                    assert len(dims) == 1, "reshape parameter (if presented as a tensor) should be dim 1, got %d" % len(dims)
                    inter[out] = get(ins[0]).resize(*vals)
                elif kind == "gemm":
                    _, ins, out, ai, af = node
                    alpha, beta = af.get("alpha", 1.0), af.get("beta", 1.0)
                    y = get(ins[0]).gemm(get(ins[1]), ai.get("transA", 0) == 1, ai.get("transB", 0) == 1, alpha)
                    inter[out] = (y + get(ins[2])) if beta == 1.0 else (y + get(ins[2]) * beta)
                elif kind == "flatten":
                    _, i, out, axis = node
                    t = get(i)
                    inter[out] = t.resize(*(list(t.x.shape[:axis]) + [-1]))
                elif kind == "pad":
                    _, i, out, mode, pads, value = node
                    if not has(i): raise NotImplementedError("Pad of a shape value")
                    assert sum(pads) == 0, "TODO: only supporting no padding so far, got %s" % pads
                    inter[out] = get(i)
                elif not self._shape_node(node, has, lambda k: get(k).x.shape):
                    raise RuntimeError("node %s is not implemented" % (node,))
            return inter[self.y_name]
        return run, params


class OnnxModel:
    """A model read from an ONNX file with the interface the training loops of `lantern_amd.apps` expect of a Module:
    callable on a TensorR, `namedParameters()` over every float initialiser (the reference's `parameters` map)."""

    def __init__(self, model_file):
        self.onnx = readONNX(model_file)
        self.func, self.params = self.onnx.training_func(self.onnx.initializer_map_tensor())

    def __call__(self, x):
        return self.func(x)

    def namedParameters(self):
        return list(self.params.items())

    def parameters(self):
        return list(self.params.values())
