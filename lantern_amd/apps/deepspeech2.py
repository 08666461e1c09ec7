"""DeepSpeech2-style training step.

Follows src/main/scala/lantern/PLDI19APP/DeepSpeech.scala:33-170: two convolutions over the
spectrogram (1->32 k41x11 stride 2x2, 32->32 k21x11 stride 2x1, no bias), each followed by batch
norm and hardTanh(0, 20) in place; [B, C, D, T] -> [T, B, C*D]; a stack of bidirectional tanh RNN
layers whose two directions are summed; BatchNorm1D + Linear (no bias) onto the alphabet; softmax;
CTC loss; SGD with Nesterov momentum 0.9, learning rate 3e-4, gradient clip 400.

`rnn_batch_norm`: sequence-wise BatchNorm1D in front of every RNN layer but the first (the
reference program constructs its BatchRNN modules with useBatchNorm = false, :97-100; the
deepspeech.pytorch model it cites normalises, and so does the default here).
"""
import numpy as np

from ..nn import Module, Conv2D, BatchNorm2D, BatchNorm1D, Linear1D, RNNBase, Lookahead, SGD_Momentum
from ..tensor import Tensor, TensorR, gradR_loss, get_backend


class BatchRNN(Module):
    def __init__(self, inputSize, hiddenSize, mode="tanh", bidirectional=True, useBatchNorm=False, name="batch_rnn"):
        super().__init__(name)
        self.bidirectional = bidirectional
        self.batchNorm = self.add(BatchNorm1D(inputSize, "batch_norm")) if useBatchNorm else None
        self.rnn = self.add(RNNBase(mode, inputSize, hiddenSize, bidirectional=bidirectional))

    def __call__(self, x):
        T, Bn, F = x.x.shape
        if self.batchNorm is not None:
            x = self.batchNorm(x.resize(T * Bn, F)).resize(T, Bn, F)
        out = self.rnn(x)
        if self.bidirectional:
            out = out.resize(T, Bn, 2, out.x.shape[2] // 2).sum(2)
        return out


class DeepSpeech(Module):
    def __init__(self, labels="_'ABCDEFGHIJKLMNOPQRSTUVWXYZ ", rnnHiddenSize=1024, numLayers=3, freq=161, mode="tanh", rnn_batch_norm=True, seed=42,
                 bidirectional=True, context=20):
        super().__init__("deepspeech")
        Tensor.randseed(seed)
        rng = np.random.RandomState(seed)
        self.numClasses = len(labels)
        self.conv1 = self.add(Conv2D(1, 32, (41, 11), (2, 2), useBias=False, name="conv1", rng=rng))
        self.bn1 = self.add(BatchNorm2D(32, "bn1"))
        self.conv2 = self.add(Conv2D(32, 32, (21, 11), (2, 1), useBias=False, name="conv2", rng=rng))
        self.bn2 = self.add(BatchNorm2D(32, "bn2"))
        d = (freq - 41) // 2 + 1
        d = (d - 21) // 2 + 1
        self.rnnInputSize = 32 * d
        self.rnns = [self.add(BatchRNN(self.rnnInputSize if i == 0 else rnnHiddenSize, rnnHiddenSize, mode, bidirectional,
                                       useBatchNorm=rnn_batch_norm and i > 0, name="batch_rnn%d" % i)) for i in range(numLayers)]
        # one-directional model: a look-ahead convolution over `context` future steps, then hardTanh (DeepSpeech.scala:108, 140)
        self.lookahead = None if bidirectional else self.add(Lookahead(rnnHiddenSize, context))
        self.fc_bn = self.add(BatchNorm1D(rnnHiddenSize, "fc_bn"))
        self.fc = self.add(Linear1D(rnnHiddenSize, self.numClasses, bias=False, name="fc", rng=rng))

    def __call__(self, x):                                    # x: [B, 1, D, T]
        h = self.bn1(self.conv1(x)).hardTanh(0.0, 20.0, True)
        h = self.bn2(self.conv2(h)).hardTanh(0.0, 20.0, True)
        Bn, C, Dd, T = h.x.shape
        h = h.resize(Bn, C * Dd, T).permute(2, 0, 1)          # [T, B, C*D]
        for r in self.rnns:
            h = r(h)
        if self.lookahead is not None:
            h = self.lookahead(h).hardTanh(0.0, 20.0, True)
        T, Bn, Hd = h.x.shape
        out = self.fc(self.fc_bn(h.resize(T * Bn, Hd)))
        return out.resize(T, Bn, self.numClasses)


class Trainer:
    def __init__(self, batch=32, freq=161, frames=400, hidden=1024, layers=3, label_len=50, lr=3e-4, seed=42, rnn_batch_norm=True,
                 bidirectional=True, context=20):
        be = get_backend()
        rng = np.random.RandomState(seed + 1)
        self.model = DeepSpeech(rnnHiddenSize=hidden, numLayers=layers, freq=freq, rnn_batch_norm=rnn_batch_norm, seed=seed,
                                bidirectional=bidirectional, context=context)
        self.opt = SGD_Momentum(self.model, lr, 0.9, gradClip=400.0, nesterov=True)
        self.x = Tensor.fromNumpy(np.exp(rng.standard_normal((batch, 1, freq, frames))).astype(np.float32))
        self.labels = rng.randint(1, self.model.numClasses, size=batch * label_len).astype(np.int32)
        self.label_lengths = np.full(batch, label_len, np.int32)
        self.percent = np.ones(batch, np.float32)             # every utterance spans the whole batch width
        self.mark = be.getMallocAddr()

    def step(self):
        xin = TensorR(self.x, isInput=True)
        def loss_fun(dummy):
            probs = self.model(xin).softmax_batch(2)
            out_len = (self.percent * probs.x.shape[0]).astype(np.int32)          # DeepSpeech.scala:137-138
            return TensorR(probs.ctcLoss(out_len, self.labels, self.label_lengths))
        loss = gradR_loss(loss_fun)(Tensor.zeros(1))
        self.opt.step()
        return loss

    def end_step(self):
        get_backend().resetMallocAddr(self.mark)
