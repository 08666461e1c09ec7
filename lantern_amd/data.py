"""Dataset files and the result file of the reference's training programs, read and written in the reference's formats.

Mirrors src/main/scala/lantern/TensorDataLoader.scala (same class and method names):

* `DataLoader` (TensorDataLoader.scala:63-107): `<root>/<name>_{train,test}.bin` holds float32 images back to back,
  `<root>/<name>_{train,test}_target.bin` one int32 label per image; both are memory-mapped.  `normalize()` rewrites
  every pixel as `(x - mean) / std` in fp32 (TensorDifferentiation.scala:936-939); `foreachBatch` hands out
  consecutive full batches and drops the remainder (TensorDataLoader.scala:97-106).
* `Cifar10DataLoader` (TensorDataLoader.scala:109-139): records of one label byte followed by `prod(dims)` pixel
  bytes; a pixel becomes `(float)byte / 255.0f`, a label `(int32)byte`.  `device_batches` uploads the raw records and
  decodes them on the GPU (`lh_cifar_decode`: a quarter of the upload, same bits).
* `DeepSpeechDataLoader` (TensorDataLoader.scala:141-216): int32 batchSize, int32 numBatches, then per batch int32
  freqSize, int32 maxLength, float32 [batchSize, 1, freqSize, maxLength], float32 percent[batchSize], int32
  targetSize[batchSize], int32 targets[sum(targetSize)].  The reference reads 200 batches whatever the header says
  (TensorDataLoader.scala:171-173); here the header's count is the default and `num_batches` overrides it.
* `write_result_file` (NIPS18App/MnistCNN.scala:108-114): "unit: ..", one "%lf" loss per epoch, "run time: %lf %lf".

Host-side code (numpy); the device work is the decode kernel and whatever the caller does with the batches.
"""
import os

import numpy as np


def _map(path, dtype, mode="r"):
    """np.memmap, except that an empty file (which mmap refuses) reads as an empty array."""
    if os.path.getsize(path) < np.dtype(dtype).itemsize:
        return np.zeros(0, dtype=dtype)
    return np.memmap(path, dtype=dtype, mode=mode)


class DataLoader:
    def __init__(self, name, train, mean, std, dims, root="../data/bin"):
        split = "train" if train else "test"
        self.mean, self.std, self.dims = np.float32(mean), np.float32(std), tuple(int(d) for d in dims)
        self.data = _map(os.path.join(root, f"{name}_{split}.bin"), np.float32, "c")   # copy-on-write, as mmap PROT_WRITE|MAP_PRIVATE
        self.target = _map(os.path.join(root, f"{name}_{split}_target.bin"), np.int32)
        self.dLength = int(self.data.size)
        self.length = int(self.target.size)
        self.count = int(np.prod(self.dims))

    def _check(self):
        if self.length * self.count != self.dLength:
            raise ValueError("Data length doesn't match")                                   # assertC of TensorDataLoader.scala:94

    def normalize(self):
        self._check()
        d = self.data
        step = 1 << 24
        for o in range(0, d.size, step):                                                     # in place, bounded temporaries
            d[o:o + step] = (d[o:o + step] - self.mean) / self.std

    def foreach(self, f):
        self._check()
        for i in range(self.length):
            f(i, self.data[i * self.count:(i + 1) * self.count].reshape(self.dims), int(self.target[i]))

    def foreachBatch(self, batchSize, f):
        per = batchSize * self.count
        for b in range(self.length // batchSize):
            f(b, self.data[b * per:(b + 1) * per].reshape((batchSize,) + self.dims), self.target[b * batchSize:(b + 1) * batchSize])


class Cifar10DataLoader:
    def __init__(self, name, train, dims):
        self.dims = tuple(int(d) for d in dims)
        self.count = int(np.prod(self.dims))
        self.entrySize = self.count + 1
        raw = _map(name, np.uint8)
        self.dLength = self.length = int(raw.size // self.entrySize)
        self.records = raw[:self.dLength * self.entrySize].reshape(self.dLength, self.entrySize)
        self._x = self._y = None

    def _decode(self):
        if self._x is None:
            self._y = self.records[:, 0].astype(np.int32)
            self._x = self.records[:, 1:].astype(np.float32) / np.float32(255.0)
        return self._x, self._y

    @property
    def x(self):
        return self._decode()[0]

    @property
    def y(self):
        return self._decode()[1]

    def foreachBatch(self, batchSize, f):
        x, y = self._decode()
        for b in range(self.dLength // batchSize):
            f(b, x[b * batchSize:(b + 1) * batchSize].reshape((batchSize,) + self.dims), y[b * batchSize:(b + 1) * batchSize])

    def device_batches(self, batchSize, backend):
        """Yields (batchIndex, x, y) with x a float32 device array [batchSize, *dims] and y an int32 device array, decoded on
        the device from the uploaded records.  Arrays come from the backend's arena: the caller rewinds it per batch."""
        for b in range(self.dLength // batchSize):
            rec = np.ascontiguousarray(self.records[b * batchSize:(b + 1) * batchSize])
            yield (b,) + backend.cifar_decode(rec, self.count)


class DeepSpeechDataLoader:
    def __init__(self, name, train=True, num_batches=None):
        raw = _map(name, np.uint8)
        if raw.size < 8:
            raise ValueError("DeepSpeech batch file: no header")
        self._i32 = raw[:raw.size // 4 * 4].view(np.int32)
        self._f32 = raw[:raw.size // 4 * 4].view(np.float32)
        self.batchSize, header_batches = int(self._i32[0]), int(self._i32[1])
        pos = 2
        self.numBatches = header_batches if num_batches is None else int(num_batches)
        self.length = self.batchSize * self.numBatches
        self.freqSizes, self.maxLengths, self.inputs, self.percents, self.targetSizes, self.targets = [], [], [], [], [], []
        B = self.batchSize
        for _ in range(self.numBatches):
            if pos + 2 > self._i32.size:
                raise ValueError("DeepSpeech batch file ends before batch %d" % len(self.inputs))
            freq, maxlen = int(self._i32[pos]), int(self._i32[pos + 1]); pos += 2
            n = B * freq * maxlen
            if freq <= 0 or maxlen <= 0 or pos + n + 2 * B > self._i32.size:
                raise ValueError("DeepSpeech batch file: bad header or short batch %d" % len(self.inputs))
            self.freqSizes.append(freq); self.maxLengths.append(maxlen)
            self.inputs.append(self._f32[pos:pos + n].reshape(B, 1, freq, maxlen)); pos += n
            self.percents.append(self._f32[pos:pos + B]); pos += B
            ts = self._i32[pos:pos + B]; pos += B
            total = int(ts.sum())
            if (ts < 0).any() or pos + total > self._i32.size:
                raise ValueError("DeepSpeech batch file: bad target sizes in batch %d" % len(self.inputs))
            self.targetSizes.append(ts)
            self.targets.append(self._i32[pos:pos + total]); pos += total

    def foreachBatch(self, f):
        for b in range(self.numBatches):
            f(b, self.inputs[b], self.percents[b], self.targets[b], self.targetSizes[b])


def write_result_file(path, losses, prepare_time, time_per_epoch, unit="1 epoch"):
    with open(path, "w") as fp:
        fp.write("unit: %s\n" % unit)
        for v in losses:
            fp.write("%f\n" % float(v))
        fp.write("run time: %f %f\n" % (float(prepare_time), float(time_per_epoch)))
