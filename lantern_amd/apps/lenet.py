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


def train_from_files(result_path, root="../data/bin", nbEpoch=4, batchSize=100, lr=0.0005, seed=42, out=print):
    """The reference program's main loop on dataset files (MnistCNN.scala:60-115): load and normalize `mnist_train.bin`,
    train nbEpoch epochs of full batches, print the progress lines, write the result file.  Returns the per-epoch losses."""
    import time
    from ..data import DataLoader, write_result_file
    be = get_backend()
    t0 = time.time()
    model = MNIST(seed)
    opt = SGD(model, lr, gradClip=1000.0)
    train = DataLoader("mnist", True, 0.1307, 0.3081, (1, 28, 28), root=root)
    train.normalize()
    prepare = time.time() - t0
    out("Data normalized (all prepare time) in %f sec" % prepare)
    loss_save = []
    addr = be.getMallocAddr()
    for epoch in range(nbEpoch):
        state = {"img": 0, "loss": 0.0}
        out("Start training epoch %d" % (epoch + 1))
        t1 = time.time()

        def batch(batchIndex, x, target):
            state["img"] += batchSize
            xin = TensorR(Tensor.fromNumpy(np.ascontiguousarray(x)), isInput=True)
            tgt = int_array(np.ascontiguousarray(target))
            loss = gradR_loss(lambda dummy: model(xin).logSoftmaxB(1).nllLossB(tgt).sum())(Tensor.zeros(4))
            state["loss"] += float(loss.toCPU()[0])
            opt.step()
            if train.length >= 10 and state["img"] % (train.length // 10) == 0:
                out("Train epoch %d: [%d/%d (%.0f%%)]\tAverage Loss: %.6f" % (epoch, state["img"], train.length,
                                                                           100.0 * state["img"] / train.length, state["loss"] / state["img"]))
            be.resetMallocAddr(addr)

        train.foreachBatch(batchSize, batch)
        delta = (time.time() - t1) * 1e6
        out("Training completed in %dms (%d us/images)" % (delta // 1000, delta // max(train.length, 1)))
        loss_save.append(state["loss"] / max(train.length, 1))
    total = time.time() - t0
    write_result_file(result_path, loss_save, prepare, (total - prepare) / max(nbEpoch, 1))
    return loss_save


if __name__ == "__main__":
    import sys
    from .. import BackendHIP, set_backend
    hip = BackendHIP()
    hip.setup()
    set_backend(hip)
    train_from_files(sys.argv[1] if len(sys.argv) > 1 else "result_Lantern.txt", *(sys.argv[2:3]))
    hip.cleanup()

