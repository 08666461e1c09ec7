"""The epoch loop of the reference's CIFAR-10 training programs on a dataset file.

Mirrors src/main/scala/lantern/PLDI19APP/resnet50FromOnnx.scala:137-213 and squeezenetFromOnnx.scala:115-187 (the same loop
around different networks): Cifar10DataLoader over `data_batch_*.bin` records, batches of 64, loss = mean of nllLoss over
logSoftmax, plain SGD `x -= lr * d` followed by clear_grad, a progress line every tenth of an epoch, the arena rewound after
every batch, and a result file holding the per-epoch losses and the median epoch time.  With `device_decode` the raw records
are uploaded and decoded on the device (same floats, a quarter of the copy); otherwise the host decodes as the reference does.

    python -m lantern_amd.apps.cifar_loop squeezenet|resnet50|path/to/model.onnx result.txt path/to/data_batch_1.bin

With a `.onnx` path the network comes from the file through lantern_amd.onnx (readONNX + training_func, as the reference's programs
build theirs: resnet50FromOnnx.scala:150-157), its float initialisers being the parameters.
"""
import time

import numpy as np

from ..data import Cifar10DataLoader, write_result_file
from ..nn import SGD
from ..tensor import Tensor, TensorR, get_backend, gradR_loss, int_array


def train_from_file(model, result_path, data_file, nbEpoch=4, batchSize=64, learning_rate=0.005, dims=(3, 32, 32), out=print,
                    device_decode=True):
    be = get_backend()
    t0 = time.time()
    train = Cifar10DataLoader(data_file, True, dims)
    on_device = device_decode and hasattr(be, "cifar_decode")
    if not on_device:
        train.x                                                       # host decode happens here, as in the reference's constructor
    prepare = time.time() - t0
    out("Data normalized (all prepare time) in %f sec" % prepare)
    opt = SGD(model, learning_rate)
    loss_save, time_save = [], []
    addr = be.getMallocAddr()
    every = train.length // batchSize // 10

    def run_batch(state, epoch, batchIndex, x_tensor, target):
        xin = TensorR(x_tensor, isInput=True)
        loss = gradR_loss(lambda dummy: model(xin).logSoftmaxB(1).nllLossB(target).mean())(Tensor.zeros(1))
        state["loss"] += float(loss.toCPU()[0])
        opt.step()
        if every > 0 and (batchIndex + 1) % every == 0:
            trained, total = batchIndex * batchSize, train.length
            avg = np.float32(state["loss"]) / np.float32(batchIndex)                      # the reference divides by the index: inf at 0
            out("Train epoch %d: [%d/%d (%.0f%%)] Average Loss: %.6f" % (epoch, trained, total, 100.0 * trained / total, avg))
        be.resetMallocAddr(addr)

    for epoch in range(nbEpoch):
        state = {"loss": 0.0}
        out("Start training epoch %d" % (epoch + 1))
        t1 = time.time()
        with np.errstate(divide="ignore", invalid="ignore"):
            if on_device:
                for b, x, y in train.device_batches(batchSize, be):
                    run_batch(state, epoch, b, Tensor(x, (batchSize,) + tuple(dims)), y)
            else:
                train.foreachBatch(batchSize, lambda b, x, y: run_batch(state, epoch, b, Tensor.fromNumpy(np.ascontiguousarray(x)),
                                                                          int_array(np.ascontiguousarray(y))))
        delta = (time.time() - t1) * 1e6
        time_save.append(float(int(delta) // 1000000))                                    # whole seconds, as the reference stores them
        out("Training completed in %dms (%d us/images)" % (delta // 1000, delta // max(train.length, 1)))
        loss_save.append(state["loss"] / max(train.length, 1))
    median_time = sorted(time_save)[nbEpoch // 2] if nbEpoch else 0.0
    write_result_file(result_path, loss_save, prepare, median_time)
    return loss_save


def main(argv):
    from .. import BackendHIP, set_backend
    which, result, data_file = argv[0], argv[1], argv[2]
    hip = BackendHIP()
    hip.setup()
    set_backend(hip)
    if which.endswith(".onnx"):
        from ..onnx import OnnxModel
        model = OnnxModel(which)
    elif which == "squeezenet":
        from .squeezenet import SqueezeNet
        model = SqueezeNet(10)
    else:
        from .resnet50 import ResNet50
        model = ResNet50(num_classes=10, imagenet_stem=False)
    train_from_file(model, result, data_file)
    hip.cleanup()


if __name__ == "__main__":
    import sys
    main(sys.argv[1:])
