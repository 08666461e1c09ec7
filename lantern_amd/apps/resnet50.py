"""ResNet-50 training step (the headline configuration).

Network: bottleneck blocks [3,4,6,3], widths 64..2048, stride on the 3x3, no conv bias
(reference: src/out/PLDI19evaluation/resnet50/pytorch/resnet50.py:56-93, 162-219 for the
ImageNet-shape class; :95-148 for the 32x32 variant the reference trains).  Op mapping as the
ONNX training path emits it (src/main/scala/lantern/ONNXLib.scala:847-1066): Conv -> convBBP,
BatchNormalization -> batchNorm, Relu -> relu(inPlace = true), MaxPool -> maxPoolBK, Add -> +,
AveragePool -> averagePoolBK, Reshape -> resize, Gemm(transB) -> gemm(.., false, true, 1) + bias,
then logSoftmaxB / nllLossB / mean (src/main/scala/lantern/PLDI19APP/resnet50FromOnnx.scala:172-191).
"""
import math

import numpy as np

from ..nn import Module, Conv2D, BatchNorm2D, SGD_Momentum
from ..tensor import Tensor, TensorR, gradR_loss, get_backend, int_array


def _kaiming_normal_fan_out(rng):
    def init(dims):
        fan_out = dims[0] * dims[2] * dims[3]
        return (rng.standard_normal(dims) * math.sqrt(2.0 / fan_out)).astype(np.float32)
    return init


class Bottleneck(Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride, downsample, rng, name):
        super().__init__(name)
        ini = _kaiming_normal_fan_out(rng)
        self.conv1 = self.add(Conv2D(inplanes, planes, (1, 1), useBias=False, name="conv1", init=ini))
        self.bn1 = self.add(BatchNorm2D(planes, "bn1"))
        self.conv2 = self.add(Conv2D(planes, planes, (3, 3), (stride, stride), (1, 1), useBias=False, name="conv2", init=ini))
        self.bn2 = self.add(BatchNorm2D(planes, "bn2"))
        self.conv3 = self.add(Conv2D(planes, planes * 4, (1, 1), useBias=False, name="conv3", init=ini))
        self.bn3 = self.add(BatchNorm2D(planes * 4, "bn3"))
        self.down = None
        if downsample:
            self.down = (self.add(Conv2D(inplanes, planes * 4, (1, 1), (stride, stride), useBias=False, name="down_conv", init=ini)),
                         self.add(BatchNorm2D(planes * 4, "down_bn")))

    def __call__(self, x):
        out = self.bn1(self.conv1(x)).relu(True)
        out = self.bn2(self.conv2(out)).relu(True)
        out = self.bn3(self.conv3(out))
        idt = x if self.down is None else self.down[1](self.down[0](x))
        return (out + idt).relu(True)


class ResNet50(Module):
    def __init__(self, num_classes=1000, imagenet_stem=True, seed=42, layers=(3, 4, 6, 3)):
        super().__init__("resnet50")
        rng = np.random.RandomState(seed)
        ini = _kaiming_normal_fan_out(rng)
        self.imagenet_stem = imagenet_stem
        if imagenet_stem:
            self.conv1 = self.add(Conv2D(3, 64, (7, 7), (2, 2), (3, 3), useBias=False, name="conv1", init=ini))
        else:   # the reference's CIFAR variant: 3x3 stride-1 stem and a 2x2 max-pool (resnet50.py:101-104)
            self.conv1 = self.add(Conv2D(3, 64, (3, 3), (1, 1), (1, 1), useBias=False, name="conv1", init=ini))
        self.bn1 = self.add(BatchNorm2D(64, "bn1"))
        self.blocks = []
        inplanes = 64
        for li, (planes, n, stride) in enumerate(zip((64, 128, 256, 512), layers, (1, 2, 2, 2))):
            for b in range(n):
                s = stride if b == 0 else 1
                down = b == 0 and (s != 1 or inplanes != planes * 4)
                self.blocks.append(self.add(Bottleneck(inplanes, planes, s, down, rng, "layer%d_%d" % (li + 1, b))))
                inplanes = planes * 4
        bound = 1.0 / math.sqrt(inplanes)
        self.fc_w = self.param("fc_weight", Tensor.fromNumpy(rng.uniform(-bound, bound, (num_classes, inplanes)).astype(np.float32)))
        self.fc_b = self.param("fc_bias", Tensor.fromNumpy(rng.uniform(-bound, bound, (num_classes,)).astype(np.float32)))

    def __call__(self, x):
        h = self.bn1(self.conv1(x)).relu(True)
        if self.imagenet_stem:
            h = h.maxPoolBK((3, 3), (2, 2), (1, 1, 1, 1))
        else:                       # resnet50.py:104: MaxPool2d(2, 2), 32x32 -> 16x16 before layer1
            h = h.maxPoolBK((2, 2), (2, 2), None)
        for blk in self.blocks:
            h = blk(h)
        hw = h.x.shape[2]
        h = h.averagePoolBK((hw, hw), (1, 1), None)
        h = h.resize(h.x.shape[0], -1)
        return h.gemm(self.fc_w, False, True, 1.0) + self.fc_b


class Trainer:
    """One emitted training loop: parameters and the batch live below the arena mark; everything a
    step allocates is released by rewinding to it (resnet50FromOnnx.scala:162-191).

    `streamed`: the loop body as the reference's program runs it, with a fresh batch uploaded from the host for every step
    and the loss read back after every step (resnet50FromOnnx.scala:172-176), but without the two stalls: batches alternate
    between two device buffers, the upload of batch i+1 runs on the copy stream while step i computes, and the loss is read
    back into a ring of pinned host slots that the host looks at later (`losses()`)."""

    LOSS_RING = 64

    def __init__(self, model, batch, hw, num_classes, lr=0.1, momentum=0.9, seed=42, streamed=False):
        be = get_backend()
        rng = np.random.RandomState(seed + 1)
        self.model = model
        self.opt = SGD_Momentum(model, lr, momentum)
        self.x_host = rng.standard_normal((batch, 3, hw, hw)).astype(np.float32)
        self.y_host = rng.randint(0, num_classes, size=batch).astype(np.int32)
        self.streamed = streamed
        if streamed:
            shape = (batch, 3, hw, hw)
            self.hx = [be.hostArray(shape), be.hostArray(shape)]
            self.hy = [be.hostArray((batch,), np.int32), be.hostArray((batch,), np.int32)]
            self.hx[0][...] = self.x_host; self.hy[0][...] = self.y_host
            self.hx[1][...] = rng.standard_normal(shape).astype(np.float32); self.hy[1][...] = rng.randint(0, num_classes, size=batch)
            self.dx = [Tensor(be.mallocArray(self.x_host.size, zero=False), shape) for _ in range(2)]
            self.dt = [be.mallocArray(batch, zero=False) for _ in range(2)]
            self.hloss = be.hostArray((self.LOSS_RING,))
            self.hloss[...] = np.nan
            self.i = 0
            be.uploadAsync(self.dx[0].data, self.hx[0]); be.uploadAsync(self.dt[0], self.hy[0])
            self.x, self.target = self.dx[0], self.dt[0]
        else:
            self.x = Tensor.fromNumpy(self.x_host)
            self.target = int_array(self.y_host)
        self.mark = be.getMallocAddr()

    def step(self):
        be = get_backend()
        if self.streamed:
            k = self.i % 2
            be.copyJoin()                     # batch i has arrived (its upload was issued during step i-1)
            self.x, self.target = self.dx[k], self.dt[k]
            # batch i+1 travels while this step computes: the last reader of its buffer, step i-1, has been issued already
            be.uploadAsync(self.dx[1 - k].data, self.hx[1 - k]); be.uploadAsync(self.dt[1 - k], self.hy[1 - k])
        xin = TensorR(self.x, isInput=True)
        target = self.target
        loss = gradR_loss(lambda dummy: self.model(xin).logSoftmaxB().nllLossB(target).mean())(Tensor.zeros(1))
        if self.streamed:
            slot = self.i % self.LOSS_RING
            be.downloadAsync(self.hloss[slot:slot + 1], loss.data)
            self.i += 1
        self.opt.step()
        self.last_loss = loss
        return loss

    def losses(self):
        """The losses of the last LOSS_RING streamed steps, oldest first (waits for the device)."""
        get_backend().sync()
        n = min(self.i, self.LOSS_RING)
        return np.array([self.hloss[(self.i - n + j) % self.LOSS_RING] for j in range(n)], np.float32)

    def end_step(self):
        get_backend().resetMallocAddr(self.mark)
