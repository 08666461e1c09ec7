"""LeNet-style MNIST CNN training step (config 1).

Reference: src/main/scala/lantern/NIPS18App/MnistCNN.scala:38-59 -- conv1(1->10,k5) relu maxPool2,
conv2(10->20,k5) relu maxPool2, resize(-1,320), Linear1D(320,50), dropout(0.5), Linear1D(50,10),
logSoftmaxB, nllLossB, sum; SGD lr 5e-4.  Weights are drawn with the glibc rand() sequence from
srand(42) in the reference's module order (conv1, conv2, linear1, linear2), as the emitted
program does (src/out/NIPS18evaluation/evaluationCNN/Lantern/Lantern.cpp:96-140).
`pytorch_order=True` gives the ordering of the competitor script (pool before relu, relu after
linear1, dropout after conv2: src/out/NIPS18evaluation/evaluationCNN/PyTorch/PyTorch.py:38-46).
"""
import numpy as np

from ..nn import Module, Conv2D, Linear1D, SGD
from ..tensor import Tensor, TensorR, gradR_loss, get_backend, int_array


class MNIST(Module):
    def __init__(self, seed=42, pytorch_order=False):
        super().__init__("mnist")
        Tensor.randseed(seed)
        self.conv1 = self.add(Conv2D(1, 10, (5, 5), name="conv1"))
        self.conv2 = self.add(Conv2D(10, 20, (5, 5), name="conv2"))
        self.linear1 = self.add(Linear1D(320, 50, name="linear1"))
        self.linear2 = self.add(Linear1D(50, 10, name="linear2"))
        self.pytorch_order = pytorch_order

    def __call__(self, x):
        if self.pytorch_order:
            h = self.conv1(x).maxPoolBK((2, 2), (2, 2), None).relu()
            h = self.conv2(h).dropout(0.5).maxPoolBK((2, 2), (2, 2), None).relu()
            h = self.linear1(h.resize(-1, 320)).relu()
            return self.linear2(h)
        h = self.conv1(x).relu().maxPoolBK((2, 2), (2, 2), None)
        h = self.conv2(h).relu().maxPoolBK((2, 2), (2, 2), None)
        h = self.linear1(h.resize(-1, 320)).dropout(0.5)
        return self.linear2(h)


class Trainer:
    def __init__(self, batch=100, lr=0.0005, seed=42, pytorch_order=False):
        be = get_backend()
        self.model = MNIST(seed, pytorch_order)
        self.opt = SGD(self.model, lr, gradClip=1000.0)
        rng = np.random.RandomState(seed)
        self.x_host = rng.random_sample((batch, 1, 28, 28)).astype(np.float32)
        self.y_host = rng.randint(0, 10, size=batch).astype(np.int32)
        self.x = Tensor.fromNumpy(self.x_host)
        self.target = int_array(self.y_host)
        self.mark = be.getMallocAddr()

    def step(self):
        xin = TensorR(self.x, isInput=True)
        loss = gradR_loss(lambda dummy: self.model(xin).logSoftmaxB(1).nllLossB(self.target).sum())(Tensor.zeros(4))
        self.opt.step()
        return loss

    def end_step(self):
        get_backend().resetMallocAddr(self.mark)
