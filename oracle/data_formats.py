"""TEST INFRASTRUCTURE, NOT PRODUCT: the reference's dataset and result file formats, restated element by element.

Plain Python loops over `struct`, written from the reference's loops so that a test of the product's loaders
(lantern_amd/data.py, lh_cifar_decode) compares two independent readings of the same bytes:

* `cifar_decode`      src/main/scala/lantern/TensorDataLoader.scala:109-127
* `mnist_batches`     TensorDataLoader.scala:63-107 with normalize = TensorDifferentiation.scala:936-939
* `deepspeech_read`   TensorDataLoader.scala:141-216 (batch count taken from the caller, as the reference fixes it)
* `result_file_text`  src/main/scala/lantern/NIPS18App/MnistCNN.scala:108-114

Pins (tests/test_data_formats.py): the 256 possible pixel values against exact rational arithmetic rounded once; the
file layouts against files assembled field by field with `struct.pack`; the result file against a literal text.
Only small inputs: these loops are slow on purpose.
"""
import struct

import numpy as np


def cifar_decode(raw, count):
    entry = count + 1
    n = len(raw) // entry
    x = np.empty(n * count, dtype=np.float32)
    y = np.empty(n, dtype=np.int32)
    k255 = np.float32(255.0)
    for i in range(n):
        y[i] = raw[i * entry]
        for j in range(count):
            x[i * count + j] = np.float32(raw[i * entry + 1 + j]) / k255
    return x, y


def mnist_batches(data_bytes, target_bytes, dims, batch, mean=None, std=None):
    count = int(np.prod(dims))
    n = len(target_bytes) // 4
    data = list(struct.unpack("<%df" % (len(data_bytes) // 4), data_bytes))
    target = struct.unpack("<%di" % n, target_bytes)
    assert n * count == len(data), "Data length doesn't match"
    vals = np.array(data, dtype=np.float32)
    if mean is not None:
        m, s = np.float32(mean), np.float32(std)
        for i in range(vals.size):
            vals[i] = (vals[i] - m) / s
    out = []
    off = 0
    for b in range(n // batch):
        out.append((vals[off:off + batch * count].reshape((batch,) + tuple(dims)), np.array(target[b * batch:(b + 1) * batch], dtype=np.int32)))
        off += batch * count
    return out


def deepspeech_read(raw, num_batches):
    pos = 0

    def ints(k):
        nonlocal pos
        v = struct.unpack_from("<%di" % k, raw, pos); pos += 4 * k
        return v

    def floats(k):
        nonlocal pos
        v = struct.unpack_from("<%df" % k, raw, pos); pos += 4 * k
        return v

    batch_size, header_batches = ints(2)
    batches = []
    for _ in range(num_batches):
        freq, maxlen = ints(2)
        inp = np.array(floats(batch_size * freq * maxlen), dtype=np.float32).reshape(batch_size, 1, freq, maxlen)
        percent = np.array(floats(batch_size), dtype=np.float32)
        tsize = np.array(ints(batch_size), dtype=np.int32)
        targets = np.array(ints(int(tsize.sum())), dtype=np.int32)
        batches.append((inp, percent, targets, tsize))
    return batch_size, header_batches, batches


def result_file_text(losses, prepare_time, time_per_epoch, unit="1 epoch"):
    text = "unit: %s\n" % unit
    for v in losses:
        text += "%.6f\n" % v          # C's %lf prints six decimals
    return text + "run time: %.6f %.6f\n" % (prepare_time, time_per_epoch)
