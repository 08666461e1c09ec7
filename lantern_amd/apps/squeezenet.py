"""SqueezeNet on 32x32 images: training step.

Network of src/out/PLDI19evaluation/squeezenet/pytorch/pytorch_squeeze_cifar10.py:44-83
(conv 3->96 k3 p1, relu, max-pool; eight Fire modules with two more max-pools; conv 512->10 k4;
every conv has a bias, relu after every conv but the last), issued with the op mapping of the ONNX
training path (src/main/scala/lantern/ONNXLib.scala:847-1066: Conv -> convBBP, Relu ->
relu(inPlace), MaxPool -> maxPoolBK, Concat -> concat(1)), loss and optimizer as
src/main/scala/lantern/PLDI19APP/squeezenetFromOnnx.scala trains it: logSoftmaxB, nllLossB, mean,
SGD with momentum 0.9, learning rate 0.005.

`avgpool_head=True` gives the v1.1-style classifier instead: 1x1 conv 512->classes, relu,
averagePool over the remaining 4x4 map.
"""
import numpy as np

from ..nn import Module, Conv2D, SGD_Momentum
from ..tensor import Tensor, TensorR, gradR_loss, get_backend, int_array


class Fire(Module):
    def __init__(self, inplanes, squeeze, expand1, expand3, rng, name):
        super().__init__(name)
        self.squeeze = self.add(Conv2D(inplanes, squeeze, (1, 1), name="squeeze", rng=rng))
        self.e1 = self.add(Conv2D(squeeze, expand1, (1, 1), name="expand1x1", rng=rng))
        self.e3 = self.add(Conv2D(squeeze, expand3, (3, 3), (1, 1), (1, 1), name="expand3x3", rng=rng))

    def __call__(self, x):
        s = self.squeeze(x).relu(True)
        return self.e1(s).relu(True).concat(1, self.e3(s).relu(True))


FIRES = [(96, 16, 64, 64), (128, 16, 64, 64), (128, 32, 128, 128), None,
         (256, 32, 128, 128), (256, 48, 192, 192), (384, 48, 192, 192), (384, 64, 256, 256), None,
         (512, 64, 256, 256)]


class SqueezeNet(Module):
    def __init__(self, num_classes=10, seed=42, avgpool_head=False):
        super().__init__("squeezenet")
        rng = np.random.RandomState(seed)
        self.conv1 = self.add(Conv2D(3, 96, (3, 3), (1, 1), (1, 1), name="conv1", rng=rng))
        self.stages = []
        for i, f in enumerate(FIRES):
            self.stages.append(None if f is None else self.add(Fire(*f, rng=rng, name="fire%d" % i)))
        self.avgpool_head = avgpool_head
        # the last conv is drawn from N(0, 0.01) (pytorch_squeeze_cifar10.py:71-73); all biases start at zero
        self.head = self.add(Conv2D(512, num_classes, (1, 1) if avgpool_head else (4, 4), name="conv10",
                                    init=lambda dims: (rng.standard_normal(dims) * 0.01).astype(np.float32)))

    def __call__(self, x):
        h = self.conv1(x).relu(True).maxPoolBK((2, 2), (2, 2), None)
        for st in self.stages:
            h = h.maxPoolBK((2, 2), (2, 2), None) if st is None else st(h)
        h = self.head(h)
        if self.avgpool_head:
            hw = h.x.shape[2]
            h = h.relu(True).averagePoolBK((hw, hw), (1, 1), None)
        return h.resize(h.x.shape[0], -1)


class Trainer:
    """Parameters and the batch live below the arena mark; a step's tensors are released by rewinding to it."""

    def __init__(self, batch=64, hw=32, num_classes=10, lr=0.005, momentum=0.9, seed=42, avgpool_head=False):
        be = get_backend()
        rng = np.random.RandomState(seed + 1)
        self.model = SqueezeNet(num_classes, seed, avgpool_head)
        self.opt = SGD_Momentum(self.model, lr, momentum)
        self.x = Tensor.fromNumpy(rng.standard_normal((batch, 3, hw, hw)).astype(np.float32))
        self.target = int_array(rng.randint(0, num_classes, size=batch).astype(np.int32))
        self.mark = be.getMallocAddr()

    def step(self):
        xin = TensorR(self.x, isInput=True)
        loss = gradR_loss(lambda dummy: self.model(xin).logSoftmaxB().nllLossB(self.target).mean())(Tensor.zeros(1))
        self.opt.step()
        return loss

    def end_step(self):
        get_backend().resetMallocAddr(self.mark)
