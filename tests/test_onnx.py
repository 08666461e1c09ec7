"""The ONNX front door (lantern_amd/onnx.py) against the reference's mapping (src/main/scala/lantern/ONNXLib.scala).
Model files are written by tests/onnx_build.py with the protobuf runtime, an encoder independent of the reader under test; no
model is downloaded (the reference's own integration test needs the model zoo's SqueezeNet, TestONNX.scala:479-508, which is not
available offline: parity of the importer against the reference's outputs on that file is unpinned)."""
import os

import numpy as np
import pytest

import lantern_amd as la
from lantern_amd import Tensor, TensorR, gradR_loss, int_array
from lantern_amd.onnx import ModelProto, OnnxModel, readONNX, readTensor, _fields, _varint
from tests.onnx_build import GraphBuilder, export_module_tree


def _small_graph(path, typed_data=False):
    """conv(bias) -> bn -> relu -> maxpool -> conv -> (+ shortcut conv) -> relu -> global shape arithmetic -> reshape -> gemm."""
    rng = np.random.RandomState(0)
    b = GraphBuilder("data", [2, 3, 8, 8], typed_data=typed_data)
    w = {"c1w": rng.randn(4, 3, 3, 3) * 0.3, "c1b": rng.randn(4) * 0.1, "g": rng.rand(4) + 0.5, "be": rng.randn(4) * 0.1, "rm": rng.randn(4) * 0.1, "rv": rng.rand(4) + 0.5,
         "c2w": rng.randn(4, 4, 3, 3) * 0.2, "c3w": rng.randn(4, 4, 1, 1) * 0.5, "fcw": rng.randn(5, 64) * 0.1, "fcb": rng.randn(5) * 0.1}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    h = b.node("Conv", ["data", b.init("c1w", w["c1w"]), b.init("c1b", w["c1b"])], ["c1"], kernel_shape=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1])
    h = b.node("BatchNormalization", [h, b.init("g", w["g"]), b.init("be", w["be"]), b.init("rm", w["rm"]), b.init("rv", w["rv"])], ["bn1"], epsilon=1e-5, momentum=0.9)
    h = b.node("Relu", [h], ["r1"])
    p = b.node("MaxPool", [h], ["p1"], kernel_shape=[2, 2], strides=[2, 2])                        # no pads attribute: defaults to zeros
    m = b.node("Conv", [p, b.init("c2w", w["c2w"])], ["c2"], kernel_shape=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1])
    s = b.node("Conv", [p, b.init("c3w", w["c3w"])], ["c3"], kernel_shape=[1, 1], strides=[1, 1], pads=[0, 0, 0, 0])
    h = b.node("Relu", [b.node("Add", [m, s], ["a1"])], ["r2"])
    # the shape arithmetic a PyTorch export of `x.view(x.size(0), -1)` leaves behind
    b.node("Shape", [h], ["shp"])
    b.node("Gather", ["shp"], ["n0"], axis=0)                                                        # the reference's one-input Gather
    b.node("Unsqueeze", ["n0"], ["n0u"], axes=[0])
    b.node("Constant", [], ["minus1"], value={"dims": [], "int64": [-1]})
    b.node("Unsqueeze", ["minus1"], ["m1u"], axes=[0])
    b.node("Concat", ["n0u", "m1u"], ["newshape"], axis=0)
    h = b.node("Reshape", [h, "newshape"], ["flat"])
    h = b.node("Gemm", [h, b.init("fcw", w["fcw"]), b.init("fcb", w["fcb"])], ["logits"], alpha=1.0, beta=1.0, transB=1)
    b.save(path, "logits", [2, 5])
    return w


def test_wire_format_reader_handles_varints_negative_ints_and_truncation():
    assert _varint(bytes([0xAC, 0x02]), 0) == (300, 2)
    buf = bytes([0x08, 0x96, 0x01, 0x12, 0x03]) + b"abc" + bytes([0x1D]) + np.float32(1.5).tobytes()
    assert list(_fields(buf)) == [(1, 0, 150), (2, 2, b"abc"), (3, 5, np.float32(1.5).tobytes())]
    with pytest.raises(ValueError):
        list(_fields(bytes([0x12, 0x05, 0x61])))                   # a length that runs past the end
    with pytest.raises(ValueError):
        ModelProto(bytes([0x08, 0x03]))                            # no graph


@pytest.mark.parametrize("typed_data", [False, True], ids=["raw_data", "typed_fields"])
def test_model_structure_parameter_file_and_shape_values(tmp_path, typed_data):
    path = str(tmp_path / "small.onnx")
    w = _small_graph(path, typed_data)
    m = readONNX(path)
    assert (m.x_name, m.x_dims, m.y_name, m.y_dims) == ("data", [2, 3, 8, 8], "logits", [2, 5])
    assert m.modelMap["producer name:"] == "lantern_amd tests" and m.modelMap["number of nodes:"] == 16
    assert [n[0] for n in m.allNodes] == ["conv", "bn", "relu", "maxpool", "conv", "conv", "add", "relu", "shape", "gather", "unsqueeze", "constant", "unsqueeze",
                                          "concat", "reshape", "gemm"]
    assert m.allNodes[0][3] == {"kernel_shape": [3, 3], "strides": [1, 1], "pads": [1, 1, 1, 1]}
    assert m.allNodes[3][3]["pads"] == [0, 0, 0, 0]                 # a missing pads attribute defaults to zeros (ONNXLib.scala:293)
    assert m.allNodes[1][3] == {"epsilon": pytest.approx(1e-5), "momentum": pytest.approx(0.9)}
    assert m.allNodes[15][3:] == ({"transB": 1}, {"alpha": 1.0, "beta": 1.0})
    # the parameter file: float initialisers back to back in file order, offsets in floats (ONNXLib.scala:157-185)
    order = ["c1w", "c1b", "g", "be", "rm", "rv", "c2w", "c3w", "fcw", "fcb"]
    flat = np.fromfile(path + ".bin", "<f4")
    off = 0
    for name in order:
        dims, dtype, offset = m.byteMap[name]
        assert dims == list(w[name].shape) and dtype == 1 and offset == off
        np.testing.assert_array_equal(flat[off:off + w[name].size], w[name].ravel())
        off += w[name].size
    assert off == flat.size and os.path.getsize(path + ".bin") == 4 * off


def test_inference_and_training_functions_issue_the_reference_mapping(tmp_path, on_cpu):
    """Against the operator sequence written out by hand (ONNXLib.scala:597-830, 833-1071), on the oracle backend."""
    path = str(tmp_path / "small.onnx")
    w = _small_graph(path)
    rng = np.random.RandomState(1)
    x = rng.randn(2, 3, 8, 8).astype(np.float32)
    m = readONNX(path)
    got = m.inference_func(m.initializer_map_tensor())(Tensor.fromNumpy(x)).toCPU()
    assert m.intMap["newshape"] == ([2], [2, -1]) and m.intMap["n0"] == ([], [2])

    T = lambda k: Tensor.fromNumpy(w[k])
    h = Tensor.fromNumpy(x).conv2D_batch(T("c1w"), T("c1b"), (1, 1), (1, 1, 1, 1))[0].batchNormInference(T("g"), T("be"), T("rm"), T("rv")).relu()
    p = h.maxPool2D_batch((2, 2), (2, 2), (0, 0, 0, 0))[0]
    h = (p.conv2D_batch(T("c2w"), None, (1, 1), (1, 1, 1, 1))[0] + p.conv2D_batch(T("c3w"), None, (1, 1), (0, 0, 0, 0))[0]).relu()
    want = (h.resize(2, -1).gemm(T("fcw"), False, True, 1.0) + T("fcb")).toCPU()
    np.testing.assert_array_equal(got, want)

    # training: convBBP, batchNorm (batch statistics), relu in place, maxPoolBK without pads, + , resize, gemm + bias
    target = int_array([3, 1])
    func, params = readONNX(path).training_func(readONNX(path).initializer_map_tensor())
    xin = TensorR(Tensor.fromNumpy(x), isInput=True)
    loss = gradR_loss(lambda d: func(xin).logSoftmaxB(1).nllLossB(target).mean())(Tensor.zeros(1)).toCPU()
    P = {k: TensorR(T(k)) for k in w}
    xin2 = TensorR(Tensor.fromNumpy(x), isInput=True)

    def by_hand(d):
        h = xin2.convBBP(P["c1w"], P["c1b"], (1, 1), (1, 1, 1, 1)).batchNorm(P["g"], P["be"], P["rm"].x, P["rv"].x).relu(True)
        p = h.maxPoolBK((2, 2), (2, 2), None)
        h = (p.convBBP(P["c2w"], None, (1, 1), (1, 1, 1, 1)) + p.convBBP(P["c3w"], None, (1, 1), (0, 0, 0, 0))).relu(True)
        return (h.resize(2, -1).gemm(P["fcw"], False, True, 1.0) + P["fcb"]).logSoftmaxB(1).nllLossB(target).mean()
    loss2 = gradR_loss(by_hand)(Tensor.zeros(1)).toCPU()
    np.testing.assert_array_equal(loss, loss2)
    assert set(params) == set(w)                                    # every float initialiser is a parameter, running statistics included
    for k in ("c1w", "c1b", "g", "be", "c2w", "c3w", "fcw", "fcb"):
        np.testing.assert_array_equal(params[k].d.toCPU(), P[k].d.toCPU(), err_msg=k)
        assert np.abs(params[k].d.toCPU()).max() > 0, k


def test_gemm_beta_flatten_dropout_softmax_pad_and_unknown_nodes(tmp_path, on_cpu):
    rng = np.random.RandomState(2)
    fw, fb = rng.randn(12, 3).astype(np.float32), rng.randn(3).astype(np.float32)
    b = GraphBuilder("x", [2, 3, 2, 2])
    h = b.node("Pad", ["x"], ["xp"], mode="constant", pads=[0, 0, 0, 0, 0, 0, 0, 0], value=0.0)
    h = b.node("Flatten", [h], ["f"], axis=1)
    h = b.node("Dropout", [h], ["d", "mask"], ratio=0.0)
    h = b.node("Gemm", [h, b.init("w", fw), b.init("b", fb)], ["g"], alpha=0.5, beta=2.0)
    h = b.node("Softmax", [h], ["s"])
    path = b.save(str(tmp_path / "head.onnx"), "s", [2, 3])
    x = rng.randn(2, 3, 2, 2).astype(np.float32)
    m = readONNX(path)
    got = m.inference_func(m.initializer_map_tensor())(Tensor.fromNumpy(x)).toCPU()
    z = 0.5 * (x.reshape(2, 12).astype(np.float64) @ fw) + 2.0 * fb
    e = np.exp(z - z.max(1, keepdims=True))
    np.testing.assert_allclose(got, e / e.sum(1, keepdims=True), rtol=1e-5)
    func, _ = m.training_func(m.initializer_map_tensor())                       # Softmax maps to logSoftmaxB when training (ONNXLib.scala:907-912)
    out = func(TensorR(Tensor.fromNumpy(x), isInput=True)).x.toCPU()
    la.tensor._tape.clear()
    np.testing.assert_allclose(out, np.log(e / e.sum(1, keepdims=True)), rtol=1e-4, atol=1e-5)

    b = GraphBuilder("x", [1, 1])
    b.node("Tanh", ["x"], ["y"])
    with pytest.raises(RuntimeError, match="Tanh not yet implemented"):
        readONNX(b.save(str(tmp_path / "bad.onnx"), "y", [1, 1]))
    b = GraphBuilder("x", [1, 1, 4, 4])
    b.node("Pad", ["x"], ["y"], mode="constant", pads=[0, 0, 1, 1, 0, 0, 1, 1], value=0.0)
    m = readONNX(b.save(str(tmp_path / "pad.onnx"), "y", [1, 1, 6, 6]))
    with pytest.raises(AssertionError, match="only supporting no padding"):
        m.inference_func({})(Tensor.zeros(1, 1, 4, 4))


def test_tensor_file_reader(tmp_path):
    """readTensor (ONNXLib.scala:144-155): the model zoo's input_0.pb / output_0.pb are bare TensorProto messages."""
    from tests.onnx_build import _CLS
    t = _CLS["TensorProto"]()
    arr = np.arange(24, dtype=np.float32).reshape(2, 3, 4) * 0.5
    t.dims.extend(arr.shape); t.data_type = 1; t.raw_data = arr.tobytes(); t.name = "input_0"
    p = tmp_path / "input_0.pb"
    p.write_bytes(t.SerializeToString())
    np.testing.assert_array_equal(readTensor(str(p)), arr)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["resnet", "squeezenet"])
def test_onnx_built_networks_train_like_the_hand_built_applications(tmp_path, hip_backend, kind):
    """The ResNet bottleneck network (every stage, 32x32 stem) and SqueezeNet (all eight Fire modules) exported to ONNX files and
    read back through the front door: three training steps give the hand-built application's losses and parameters bit for bit
    (deterministic mode), including the fused conv + batch-norm + residual-join launches the operator sequence resolves to."""
    from lantern_amd.nn import SGD_Momentum
    be = hip_backend
    la.set_backend(be)
    mark = be.getMallocAddr()
    be.setDeterministic(True)
    try:
        rng = np.random.RandomState(3)
        N = 8
        x = rng.randn(N, 3, 32, 32).astype(np.float32); y = rng.randint(0, 10, size=N).astype(np.int32)
        if kind == "resnet":
            from lantern_amd.apps.resnet50 import ResNet50
            model = ResNet50(num_classes=10, imagenet_stem=False, layers=(1, 1, 1, 1))
        else:
            from lantern_amd.apps.squeezenet import SqueezeNet
            model = SqueezeNet(10)
        b = GraphBuilder("input", [N, 3, 32, 32])
        h = export_module_tree(b, kind, model, "input")
        if kind == "resnet":
            hw = 2
            h = b.node("AveragePool", [h], ["avg"], kernel_shape=[hw, hw], strides=[1, 1], pads=[0, 0, 0, 0])
            h = b.node("Flatten", [h], ["flat"], axis=1)
            h = b.node("Gemm", [h, b.init("fc.weight", model.fc_w.x.toCPU()), b.init("fc.bias", model.fc_b.x.toCPU())], ["out"], alpha=1.0, beta=1.0, transB=1)
        else:
            h = b.node("Reshape", [h, b.init("shape", np.array([N, -1], np.int64))], ["out"])
        path = b.save(str(tmp_path / (kind + ".onnx")), "out", [N, 10])
        onnx_model = OnnxModel(path)

        def train(net, steps=3):
            opt = SGD_Momentum(net, 0.005, 0.9)
            xt, tgt = Tensor.fromNumpy(x), int_array(y)
            m2 = be.getMallocAddr()
            losses = []
            for _ in range(steps):
                xin = TensorR(xt, isInput=True)
                loss = gradR_loss(lambda d: net(xin).logSoftmaxB(1).nllLossB(tgt).mean())(Tensor.zeros(1))
                losses.append(float(loss.toCPU()[0]))
                opt.step()
                be.resetMallocAddr(m2)
            return losses

        want = train(model)
        got = train(onnx_model)
        assert got == want and want[0] != want[-1]
        by_name = dict(onnx_model.namedParameters())
        name = "conv1.weight"
        np.testing.assert_array_equal(by_name[name].x.toCPU(), model.conv1.kernel.x.toCPU())
        last = "fc.weight" if kind == "resnet" else "conv10.weight"
        np.testing.assert_array_equal(by_name[last].x.toCPU(), (model.fc_w if kind == "resnet" else model.head.kernel).x.toCPU())
    finally:
        be.setDeterministic(False)
        be.sync(); be.resetMallocAddr(mark)


def _export(tmp_path, kind, N, cpu_backend, unit_variance=False):
    """The hand-built application, initialised on the oracle backend, written out as an ONNX file; returns the path.
    `unit_variance`: running variances of one instead of the initial zeros (NN:168-182), so that the inference function
    (which divides by sqrt(runningVar + 1e-5)) gives values of ordinary size."""
    from lantern_amd.nn import BatchNorm2D
    la.set_backend(cpu_backend)
    if kind == "resnet":
        from lantern_amd.apps.resnet50 import ResNet50
        model = ResNet50(num_classes=10, imagenet_stem=False, layers=(1, 1, 1, 1))
    else:
        from lantern_amd.apps.squeezenet import SqueezeNet
        model = SqueezeNet(10)
    if unit_variance:
        todo = [model]
        while todo:
            m = todo.pop()
            todo += list(m._children)
            if isinstance(m, BatchNorm2D):
                m.runningVar.fillInPlace(1.0)
    b = GraphBuilder("input", [N, 3, 32, 32])
    h = export_module_tree(b, kind, model, "input")
    if kind == "resnet":
        h = b.node("AveragePool", [h], ["avg"], kernel_shape=[2, 2], strides=[1, 1], pads=[0, 0, 0, 0])
        h = b.node("Flatten", [h], ["flat"], axis=1)
        h = b.node("Gemm", [h, b.init("fc.weight", model.fc_w.x.toCPU()), b.init("fc.bias", model.fc_b.x.toCPU())], ["out"], alpha=1.0, beta=1.0, transB=1)
    else:
        h = b.node("Reshape", [h, b.init("shape", np.array([N, -1], np.int64))], ["out"])
    return b.save(str(tmp_path / (kind + ".onnx")), "out", [N, 10])


class _OnnxTrainer:
    """The reference's training loop over a model read from a file (resnet50FromOnnx.scala:150-191), in the shape the tracking
    tests drive: step() returns the loss, end_step() rewinds the arena."""

    def __init__(self, path, x, y, lr):
        from lantern_amd.nn import SGD_Momentum
        be = la.get_backend()
        self.model = OnnxModel(path)
        self.opt = SGD_Momentum(self.model, lr, 0.9)
        self.x, self.target = Tensor.fromNumpy(x), int_array(y)
        self.mark = be.getMallocAddr()

    def step(self):
        xin = TensorR(self.x, isInput=True)
        loss = gradR_loss(lambda d: self.model(xin).logSoftmaxB(1).nllLossB(self.target).mean())(Tensor.zeros(1))
        self.opt.step()
        return loss

    def end_step(self):
        la.get_backend().resetMallocAddr(self.mark)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["resnet", "squeezenet"])
def test_onnx_built_networks_track_the_oracle_on_the_device(tmp_path, hip_backend, cpu_backend, kind):
    """The same readONNX program (training_func: ONNXLib.scala:833-1071) on the device and on the oracle backend, five steps
    of momentum SGD: every loss and every parameter within the tracking bounds of tests/test_training_parity.py."""
    from tests.test_training_parity import _compare
    N = 8
    rng = np.random.RandomState(3)
    x = rng.randn(N, 3, 32, 32).astype(np.float32); y = rng.randint(0, 10, size=N).astype(np.int32)
    path = _export(tmp_path, kind, N, cpu_backend)
    _compare(lambda: _OnnxTrainer(path, x, y, 0.005), hip_backend, cpu_backend, steps=5, self_calibrate=True, flip_tol=2e-2)


@pytest.mark.gpu
def test_onnx_inference_func_on_the_device_against_the_oracle(tmp_path, hip_backend, cpu_backend):
    """inference_func (ONNXLib.scala:597-830) on the device: batchNormInference, a max-pool and an average pool WITH pads,
    a residual add, Flatten, Gemm with alpha / beta and softmax_batch, against the same program on the oracle backend; then the
    ResNet and SqueezeNet files' inference functions."""
    from tests.util import assert_close
    rng = np.random.RandomState(7)
    f32 = lambda a: np.asarray(a, np.float32)
    b = GraphBuilder("x", [4, 3, 17, 17])
    h = b.node("Conv", ["x", b.init("w1", f32(rng.randn(8, 3, 3, 3) * 0.3)), b.init("b1", f32(rng.randn(8) * 0.1))], ["c1"], kernel_shape=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1])
    h = b.node("BatchNormalization", [h, b.init("g", f32(rng.rand(8) + 0.5)), b.init("be", f32(rng.randn(8) * 0.1)), b.init("rm", f32(rng.randn(8) * 0.1)),
                                      b.init("rv", f32(rng.rand(8) + 0.5))], ["bn"], epsilon=1e-5, momentum=0.9)
    h = b.node("Relu", [h], ["r1"])
    p = b.node("MaxPool", [h], ["mp"], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1])                    # 17 -> 9, real padding
    m = b.node("Conv", [p, b.init("w2", f32(rng.randn(8, 8, 3, 3) * 0.2))], ["c2"], kernel_shape=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1])
    h = b.node("Relu", [b.node("Add", [m, p], ["a1"])], ["r2"])
    h = b.node("AveragePool", [h], ["ap"], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1])              # 9 -> 5, divisor counts the image only
    h = b.node("Flatten", [h], ["fl"], axis=1)
    h = b.node("Gemm", [h, b.init("fw", f32(rng.randn(200, 6) * 0.1)), b.init("fb", f32(rng.randn(6) * 0.1))], ["gm"], alpha=0.5, beta=2.0)
    h = b.node("Softmax", [h], ["sm"])
    path = b.save(str(tmp_path / "infer.onnx"), "sm", [4, 6])
    x = rng.randn(4, 3, 17, 17).astype(np.float32)

    def infer(be, path, x):
        la.set_backend(be)
        mark = be.getMallocAddr()
        try:
            m = readONNX(path)
            return m.inference_func(m.initializer_map_tensor())(Tensor.fromNumpy(x)).toCPU().copy()
        finally:
            be.resetMallocAddr(mark)
    want, got = infer(cpu_backend, path, x), infer(hip_backend, path, x)
    assert want.shape == (4, 6) and np.allclose(want.sum(1), 1.0, atol=1e-5)
    assert_close(got, want, rtol=1e-4, what="inference_func: bn inference, padded pools, gemm alpha/beta, softmax")
    # the two application networks as files: logits of the inference function (running statistics as initialised)
    for kind in ("resnet", "squeezenet"):
        path = _export(tmp_path, kind, 4, cpu_backend, unit_variance=True)
        xs = rng.randn(4, 3, 32, 32).astype(np.float32)
        want, got = infer(cpu_backend, path, xs), infer(hip_backend, path, xs)
        assert np.isfinite(want).all() and np.abs(want).max() > 0
        assert_close(got, want, rtol=1e-4, what="inference_func of the %s file" % kind)
