"""Dataset and result files in the reference's formats (src/main/scala/lantern/TensorDataLoader.scala:63-216,
NIPS18App/MnistCNN.scala:108-114): the product's loaders against the element-by-element restatement in
oracle/data_formats.py, the restatement against exact arithmetic and literal files, and the device decode bit for bit."""
import struct
from fractions import Fraction

import numpy as np
import pytest

from lantern_amd import data as D
from oracle import data_formats as O


def _cifar_file(tmp_path, n, count, seed=0, tail=0):
    rng = np.random.RandomState(seed)
    rec = rng.randint(0, 256, size=(n, count + 1)).astype(np.uint8)
    rec[:, 0] = rng.randint(0, 10, size=n)
    path = tmp_path / "data_batch.bin"
    path.write_bytes(rec.tobytes() + bytes(tail))
    return str(path), rec


def test_pixel_values_are_the_correctly_rounded_quotients():
    """Pins the restatement: byte / 255 rounded once to fp32, from exact rationals (all 256 values)."""
    raw = bytes([3]) + bytes(range(256))
    x, y = O.cifar_decode(raw, 256)
    assert y.tolist() == [3]
    for b in range(256):
        q = Fraction(b, 255)
        f = float(x[b])                                     # exact in double
        lo, hi = np.nextafter(np.float32(f), np.float32(-1)), np.nextafter(np.float32(f), np.float32(2))
        assert abs(Fraction(f) - q) <= abs(Fraction(float(lo)) - q) and abs(Fraction(f) - q) <= abs(Fraction(float(hi)) - q), b


@pytest.mark.parametrize("n,count,tail", [(5, 12, 0), (3, 7, 5), (0, 12, 0), (2, 3072, 100)])
def test_cifar_loader_matches_restatement(tmp_path, n, count, tail):
    path, rec = _cifar_file(tmp_path, n, count, tail=tail)      # a trailing partial record is ignored (integer division, DL:117)
    dl = D.Cifar10DataLoader(path, True, (count,))
    x, y = O.cifar_decode(open(path, "rb").read(), count)
    assert dl.length == n
    assert np.array_equal(dl.x.reshape(-1).view(np.uint32), x.view(np.uint32)) and np.array_equal(dl.y, y)
    if n >= 2:
        seen = []
        dl.foreachBatch(2, lambda b, t, tg: seen.append((b, t.copy(), tg.copy())))
        assert len(seen) == n // 2 and seen[0][1].shape == (2, count)
        assert np.array_equal(seen[-1][1].reshape(-1), x[(n // 2 - 1) * 2 * count:(n // 2) * 2 * count])


def test_mnist_loader_normalizes_and_batches_like_the_restatement(tmp_path):
    rng = np.random.RandomState(1)
    dims, n, batch = (1, 4, 3), 7, 2
    data = rng.random_sample((n,) + dims).astype(np.float32)
    target = rng.randint(0, 10, size=n).astype(np.int32)
    (tmp_path / "mnist_train.bin").write_bytes(data.tobytes())
    (tmp_path / "mnist_train_target.bin").write_bytes(target.tobytes())
    dl = D.DataLoader("mnist", True, 0.1307, 0.3081, dims, root=str(tmp_path))
    dl.normalize()
    got = []
    dl.foreachBatch(batch, lambda b, t, tg: got.append((np.array(t), np.array(tg))))
    want = O.mnist_batches(data.tobytes(), target.tobytes(), dims, batch, 0.1307, 0.3081)
    assert len(got) == len(want) == 3                                   # the seventh image is dropped (DL:99)
    for (gx, gt), (wx, wt) in zip(got, want):
        assert np.array_equal(gx.view(np.uint32), wx.view(np.uint32)) and np.array_equal(gt, wt)
    assert np.array_equal(np.frombuffer((tmp_path / "mnist_train.bin").read_bytes(), np.float32), data.reshape(-1))   # file untouched
    singles = []
    dl.foreach(lambda i, t, d: singles.append((i, t.shape, d)))
    assert len(singles) == n and singles[3][1] == dims and singles[3][2] == int(target[3])


def test_mnist_loader_rejects_mismatched_lengths(tmp_path):
    (tmp_path / "mnist_test.bin").write_bytes(np.zeros(13, np.float32).tobytes())
    (tmp_path / "mnist_test_target.bin").write_bytes(np.zeros(2, np.int32).tobytes())
    dl = D.DataLoader("mnist", False, 0.0, 1.0, (1, 2, 3), root=str(tmp_path))
    with pytest.raises(ValueError, match="Data length"):
        dl.normalize()


def _deepspeech_bytes(rng, batch_size, shapes):
    """Assembles a batch file field by field; returns (bytes, the fields)."""
    out = struct.pack("<2i", batch_size, len(shapes))
    fields = []
    for freq, maxlen in shapes:
        inp = rng.standard_normal((batch_size, 1, freq, maxlen)).astype(np.float32)
        percent = rng.random_sample(batch_size).astype(np.float32)
        tsize = rng.randint(1, 5, size=batch_size).astype(np.int32)
        targets = rng.randint(1, 29, size=int(tsize.sum())).astype(np.int32)
        out += struct.pack("<2i", freq, maxlen) + inp.tobytes() + percent.tobytes() + tsize.tobytes() + targets.tobytes()
        fields.append((inp, percent, targets, tsize))
    return out, fields


def test_deepspeech_loader_reads_the_batch_file(tmp_path):
    rng = np.random.RandomState(2)
    raw, fields = _deepspeech_bytes(rng, 3, [(5, 7), (5, 11), (4, 2)])
    path = tmp_path / "deepspeech_train.bin"
    path.write_bytes(raw)
    dl = D.DeepSpeechDataLoader(str(path), True)
    bs, nb, want = O.deepspeech_read(raw, 3)
    assert (dl.batchSize, dl.numBatches, dl.length) == (3, 3, 9) and (bs, nb) == (3, 3)
    assert dl.freqSizes == [5, 5, 4] and dl.maxLengths == [7, 11, 2]
    got = []
    dl.foreachBatch(lambda b, inp, pc, tg, ts: got.append((inp, pc, tg, ts)))
    for g, w, f in zip(got, want, fields):
        for a, b, c in zip(g, w, f):
            assert np.array_equal(np.asarray(a), b) and np.array_equal(b, c)
    assert D.DeepSpeechDataLoader(str(path), True, num_batches=2).length == 6      # the reference fixes the count itself (DL:171-173)
    with pytest.raises(ValueError):
        D.DeepSpeechDataLoader(str(path), True, num_batches=4)                      # past the end of the file
    short = tmp_path / "short.bin"
    short.write_bytes(raw[:-8])
    with pytest.raises(ValueError):
        D.DeepSpeechDataLoader(str(short), True)


def test_result_file_text(tmp_path):
    path = tmp_path / "result.txt"
    D.write_result_file(str(path), [2.301234567, 0.5], 1.25, 10.0)
    text = path.read_text()
    assert text == "unit: 1 epoch\n2.301235\n0.500000\nrun time: 1.250000 10.000000\n"
    assert text == O.result_file_text([2.301234567, 0.5], 1.25, 10.0)


@pytest.mark.gpu
@pytest.mark.parametrize("n,count", [(64, 3072), (5, 7), (1, 256), (0, 12), (33, 4), (1000, 3072)])
def test_device_decode_is_bit_exact(hip_backend, tmp_path, n, count):
    be = hip_backend
    path, rec = _cifar_file(tmp_path, n, count, seed=n + count)
    if n and count == 256:
        rec[0, 1:] = np.arange(256, dtype=np.uint8)                                 # every pixel value once
    mark = be.getMallocAddr()
    x, y = be.cifar_decode(rec, count)
    gx = be.toHost(x, n * count) if n else np.zeros(0, np.float32)
    gy = be.toHost(y, n, dtype=np.int32) if n else np.zeros(0, np.int32)
    want_x = rec[:, 1:].astype(np.float32) / np.float32(255.0)
    assert np.array_equal(gx.view(np.uint32), want_x.reshape(-1).view(np.uint32))
    assert np.array_equal(gy, rec[:, 0].astype(np.int32))
    if 0 < n <= 5:
        ox, oy = O.cifar_decode(rec.tobytes(), count)
        assert np.array_equal(gx.view(np.uint32), ox.view(np.uint32)) and np.array_equal(gy, oy)
    be.resetMallocAddr(mark)


@pytest.mark.gpu
def test_device_batches_walk_the_file(hip_backend, tmp_path):
    be = hip_backend
    path, rec = _cifar_file(tmp_path, 10, 48, seed=9)
    dl = D.Cifar10DataLoader(path, True, (3, 4, 4))
    mark = be.getMallocAddr()
    n_seen = 0
    for b, x, y in dl.device_batches(4, be):
        gx, gy = be.toHost(x, 4 * 48), be.toHost(y, 4, dtype=np.int32)
        assert np.array_equal(gx, dl.x[b * 4:(b + 1) * 4].reshape(-1)) and np.array_equal(gy, dl.y[b * 4:(b + 1) * 4])
        be.resetMallocAddr(mark)
        n_seen += 1
    assert n_seen == 2


def _mnist_files(root, n, seed=3):
    rng = np.random.RandomState(seed)
    (root / "mnist_train.bin").write_bytes(rng.random_sample((n, 1, 28, 28)).astype(np.float32).tobytes())
    (root / "mnist_train_target.bin").write_bytes(rng.randint(0, 10, size=n).astype(np.int32).tobytes())


@pytest.mark.gpu
def test_mnist_program_from_files_matches_the_oracle_run(hip_backend, cpu_backend, tmp_path):
    """The reference program's main loop (MnistCNN.scala:60-115) on a small file set, dropout included (both backends
    draw the same counter-based positions): per-epoch losses within 1e-4 relative, same progress lines, same file layout."""
    import lantern_amd as la
    from lantern_amd.apps.lenet import train_from_files
    _mnist_files(tmp_path, 45)
    runs = {}
    for name, be in (("cpu", cpu_backend), ("hip", hip_backend)):
        la.set_backend(be)
        be.dropout_seed, be.dropout_offset = 42, 0
        mark = be.getMallocAddr()
        lines = []
        losses = train_from_files(str(tmp_path / (name + ".txt")), root=str(tmp_path), nbEpoch=2, batchSize=10, lr=0.002, out=lines.append)
        be.resetMallocAddr(mark)
        runs[name] = (losses, lines, (tmp_path / (name + ".txt")).read_text().splitlines())
    lc, lh = runs["cpu"][0], runs["hip"][0]
    assert len(lc) == len(lh) == 2
    np.testing.assert_allclose(lh, lc, rtol=1e-4)
    progress = [l for l in runs["hip"][1] if l.startswith("Train epoch")]
    assert len(progress) == 2 * 2 and progress[0].startswith("Train epoch 0: [20/45 (44%)]")    # reports where imgIdx % (45 / 10) == 0: 20 and 40
    text = runs["hip"][2]
    assert text[0] == "unit: 1 epoch" and len(text) == 4 and text[3].startswith("run time: ")
    assert [float(v) for v in text[1:3]] == pytest.approx(lh, abs=1e-6)


@pytest.mark.gpu
def test_cifar_program_from_file_matches_the_oracle_run(hip_backend, cpu_backend, tmp_path):
    """The CIFAR training loop of the reference's SqueezeNet program (squeezenetFromOnnx.scala:115-187) on a synthetic record
    file: per-epoch losses on the device against the oracle's (2e-3 relative for the first epoch of ten steps), with the records decoded on the device and on
    the host; progress lines and the result file in the reference's layout."""
    import lantern_amd as la
    from lantern_amd.apps.cifar_loop import train_from_file
    from lantern_amd.apps.squeezenet import SqueezeNet
    path, rec = _cifar_file(tmp_path, 85, 3072, seed=5)
    runs = {}
    for name, be, dev in (("cpu", cpu_backend, False), ("hip", hip_backend, True), ("hip_host_decode", hip_backend, False)):
        la.set_backend(be)
        be.dropout_seed, be.dropout_offset = 42, 0
        mark = be.getMallocAddr()
        lines = []
        losses = train_from_file(SqueezeNet(10), str(tmp_path / (name + ".txt")), path, nbEpoch=2, batchSize=8, learning_rate=0.005,
                                 out=lines.append, device_decode=dev)
        be.resetMallocAddr(mark)
        runs[name] = (losses, lines, (tmp_path / (name + ".txt")).read_text().splitlines())
    lc, lh, lhh = runs["cpu"][0], runs["hip"][0], runs["hip_host_decode"][0]
    assert len(lh) == 2 and all(np.isfinite(lh))
    np.testing.assert_allclose(lh[0], lc[0], rtol=2e-3)          # mean over the first ten steps
    np.testing.assert_allclose(lh[1], lc[1], rtol=1e-2)          # steps 11-20: rounding differences grown through relu / max-pool flips (2e-3 measured)
    # two device runs do not repeat to the last bit (fp32 atomic adds in the split reductions arrive in any order, and ten SGD
    # steps through relu / max-pool amplify that to ~3e-4 of the epoch mean, measured): the first batches must agree as printed
    np.testing.assert_allclose(lh, lhh, rtol=1e-2)
    first = [[float(l.split()[-1]) for l in runs[k][1] if l.startswith("Train epoch 0")][1:4] for k in ("hip", "hip_host_decode")]
    np.testing.assert_allclose(first[0][:1], first[1][:1], rtol=1e-5)        # same input bits: the first two losses agree
    np.testing.assert_allclose(first[0], first[1], rtol=1e-3)
    progress = [l for l in runs["hip"][1] if l.startswith("Train epoch")]
    assert len(progress) == 2 * 10 and progress[0].startswith("Train epoch 0: [0/85 (0%)] Average Loss: inf")   # 85 / 8 / 10 = 1: every batch reports
    assert progress[1].startswith("Train epoch 0: [8/85 (9%)] Average Loss: ")
    text = runs["hip"][2]
    assert text[0] == "unit: 1 epoch" and len(text) == 4 and text[3].startswith("run time: ")
    assert [float(v) for v in text[1:3]] == pytest.approx(lh, abs=1e-6)
