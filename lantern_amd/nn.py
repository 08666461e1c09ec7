"""Model building blocks and optimizers (reference: src/main/scala/lantern/NNModule.scala).

`Module` keeps an ordered registry of parameters (the reference finds them by JVM reflection,
NN:20-110); layers follow NN:112-182 (initialisation scales included); optimizers follow
NN:255-303.  Parameters are TensorR objects living below the arena mark of the training loop.
"""
import math

import numpy as np

from .tensor import Tensor, TensorR, get_backend


class Module:
    def __init__(self, name="module"):
        self.name = name
        self._params = []        # (name, TensorR)
        self._children = []

    def param(self, name, t):
        tr = t if isinstance(t, TensorR) else TensorR(t)
        self._params.append((name, tr))
        return tr

    def add(self, m):
        self._children.append(m)
        return m

    def namedParameters(self, prefix=""):
        out = [("%s%s/%s" % (prefix, self.name, n), p) for n, p in self._params]
        for c in self._children:
            out += c.namedParameters("%s%s/" % (prefix, self.name))
        return out

    def parameters(self):
        return [p for _, p in self.namedParameters()]

    def forEachParameter(self, f):
        for p in self.parameters():
            f(p)


def _uniform_from(rng, dims, scale):
    """(U[0,1) - 0.5) * scale: the distribution of Tensor.rand(dims, scale) (CPU:101-110)."""
    if rng is None:
        return Tensor.rand(tuple(dims), scale)
    return Tensor.fromNumpy(((rng.random_sample(tuple(dims)).astype(np.float32) - np.float32(0.5)) * np.float32(scale)))


class Linear1D(Module):
    """y = x . W + b with W of shape [in, out] (NN:112-117)."""

    def __init__(self, inSize, outSize, bias=True, name="linear1d", rng=None):
        super().__init__(name)
        scale = 1.0 / math.sqrt(inSize)
        self.weight = self.param("weight", _uniform_from(rng, (inSize, outSize), scale))
        self.biasOp = self.param("bias", Tensor.zeros(outSize)) if bias else None

    def __call__(self, x):
        y = x.dot(self.weight)
        return y.plusBias(self.biasOp) if self.biasOp is not None else y


class Conv2D(Module):
    """Kaiming-uniform conv (NN:133-146): scale = 2*sqrt(6/fan_in)."""

    def __init__(self, inChannel, outChannel, kernelSize, stride=(1, 1), pad=(0, 0), useBias=True, name="conv2d", rng=None, init=None):
        super().__init__(name)
        kh, kw = kernelSize
        dims = (outChannel, inChannel, kh, kw)
        if init is not None:
            k = Tensor.fromNumpy(init(dims))
        else:
            k = _uniform_from(rng, dims, 2.0 * math.sqrt(6.0 / (inChannel * kh * kw)))
        self.kernel = self.param("kernel", k)
        self.bias = self.param("bias", Tensor.zeros(outChannel)) if useBias else None
        self.stride, self.pad = tuple(stride), tuple(pad)

    def __call__(self, x):
        return x.convBBP(self.kernel, self.bias, self.stride, self.pad)


class BatchNorm2D(Module):
    """NN:168-182: scale ones, bias zeros, running mean/var zeros (not parameters)."""

    def __init__(self, num_features, name="batch_norm_2d"):
        super().__init__(name)
        self.scale = self.param("scale", Tensor.ones(num_features))
        self.bias = self.param("bias", Tensor.zeros(num_features))
        self.runningMean = Tensor.zeros(num_features)
        self.runningVar = Tensor.zeros(num_features)

    def __call__(self, x):
        return x.batchNorm(self.scale, self.bias, self.runningMean, self.runningVar)


class BatchNorm1D(BatchNorm2D):
    """NN:158-166: per-activation statistics over the rows of a rank-2 input."""

    def __call__(self, x):
        assert x.x.rank == 2
        return x.batchNorm1D(self.scale, self.bias, self.runningMean, self.runningVar)


class RNNBase(Module):
    """NN:332-417: one parameter buffer holding, per layer and direction, w_ih [gate, in], w_hh [gate, hidden],
    b_ih, b_hh (forward direction first), initialised with Tensor.rand(size, 0.01).  Modes "relu", "tanh", "lstm", "gru"
    (1, 1, 4 and 3 gates of hiddenSize rows each).  Layers after the first read the previous layer's output, which is
    numDirections * hiddenSize wide (what cuDNN expects; the reference's size formula, NN:357, leaves the factor out and
    so only works for one direction).  `apply(input, hx, cx)`: optional initial hidden / cell states
    [numLayers * numDirections, batch, hidden] (TensorR or Tensor; values only, no gradient: CDN:1843-1844 pass NULL for
    dhx / dcx).  `dropout`: applied to the output of every layer but the last, as cuDNN does, with the backend's own
    dropout operator (cuDNN's generator is its own; the masks are not comparable, their statistics are)."""
    MODES = {"relu": (0, 1), "tanh": (1, 1), "lstm": (2, 4), "gru": (3, 3)}

    def __init__(self, mode, inputSize, hiddenSize, numLayers=1, dropout=0.0, bidirectional=False, name="rnn"):
        super().__init__(name)
        assert mode in self.MODES, "RNN mode %r (relu, tanh, lstm, gru)" % (mode,)
        assert inputSize >= 1, "Input size must be at least 1"
        assert hiddenSize >= 1, "Hidden size must be at least 1"
        assert numLayers >= 1, "Number of layers must be at least 1"
        assert 0.0 <= dropout <= 1.0, "Dropout must be between 0 and 1"
        self.dropout = float(dropout)
        self.mode, self.numGates = self.MODES[mode]
        self.inputSize, self.hiddenSize, self.numLayers, self.bidirectional = inputSize, hiddenSize, numLayers, bidirectional
        self.numDirections = 2 if bidirectional else 1
        self.gateSize = hiddenSize * self.numGates
        self.offsets, total = [], 0
        for layer in range(numLayers):
            self.offsets.append(total)
            total += self.numDirections * self._dir_size(self._layer_input(layer))
        self.parameterBuffer = self.param("parameterBuffer", Tensor.rand((total,), 0.01))

    def _layer_input(self, layer):
        return self.inputSize if layer == 0 else self.hiddenSize * self.numDirections

    def _dir_size(self, layerInputSize):
        return self.gateSize * layerInputSize + self.gateSize * self.hiddenSize + 2 * self.gateSize

    def getParameterSize(self):
        return self.parameterBuffer.x.scalarCount

    def __call__(self, x, hx=None, cx=None):
        assert x.x.rank == 3, "RNN input should have rank 3: [seqLength x batchSize x inputSize]"
        D, Bn, H = self.numDirections, x.x.shape[1], self.hiddenSize
        states = []
        for name, s in (("hidden", hx), ("cell", cx)):
            t = s.x if isinstance(s, TensorR) else s
            if t is not None:
                assert t.rank == 3, "RNN %s state should have rank 3: [numLayers * numDirections x batchSize x hiddenSize]" % name
                assert t.shape[1] == Bn, "RNN %s state second dimension should equal input second dimension (batch size)" % name
                assert t.shape[0] == self.numLayers * D and t.shape[2] == H, "RNN %s state should be [%d, %d, %d]" % (name, self.numLayers * D, Bn, H)
            states.append(t)
        for layer in range(self.numLayers):
            h0, c0 = [None if t is None else t.data.offset(layer * D * Bn * H) if layer else t.data for t in states]
            x = x.rnn(self.mode, self.parameterBuffer, self.hiddenSize, self.bidirectional, offset=self.offsets[layer], hx=h0, cx=c0)
            if self.dropout > 0.0 and layer + 1 < self.numLayers:
                x = x.dropout(self.dropout)
        return x


def RNNRelu(inputSize, hiddenSize, numLayers=1, dropout=0.0, bidirectional=False, name="rnn_relu"):      # NN:316-330
    return RNNBase("relu", inputSize, hiddenSize, numLayers, dropout, bidirectional, name)


def RNNTanh(inputSize, hiddenSize, numLayers=1, dropout=0.0, bidirectional=False, name="rnn_tanh"):
    return RNNBase("tanh", inputSize, hiddenSize, numLayers, dropout, bidirectional, name)


def LSTM(inputSize, hiddenSize, numLayers=1, dropout=0.0, bidirectional=False, name="lstm"):
    return RNNBase("lstm", inputSize, hiddenSize, numLayers, dropout, bidirectional, name)


def GRU(inputSize, hiddenSize, numLayers=1, dropout=0.0, bidirectional=False, name="gru"):
    return RNNBase("gru", inputSize, hiddenSize, numLayers, dropout, bidirectional, name)


class Lookahead(Module):
    """The look-ahead convolution of the one-directional DeepSpeech model (src/main/scala/lantern/PLDI19APP/DeepSpeech.scala:54-66):
    y[t, b, f] = sum_{k <= context} x[t + k, b, f] * weight[f, k], the sequence padded with `context` zero steps.  Built from
    concat, repeat0, permute, a broadcast product and a sum over the last axis, as the reference builds it."""

    def __init__(self, numFeatures, context, name="lookahead"):
        super().__init__(name)
        assert context >= 1, "Context size must be at least 1"
        self.numFeatures, self.context = numFeatures, context
        self.weight = self.param("weight", Tensor.rand((numFeatures, context + 1), math.sqrt(context + 1)))

    def __call__(self, x):
        padding = TensorR(Tensor.zeros(self.context, *x.x.shape[1:]), isInput=True)
        xs = x.concat(0, padding).repeat0(self.context).permute(0, 2, 3, 1)
        return (xs * self.weight).sum(3)


# ---- optimizers (NN:255-303) -------------------------------------------------------------------
class Optim:
    def __init__(self, module):
        self.module = module
        self.params = module.parameters()

    def zero_grad(self):
        for p in self.params:
            p.clear_grad()


class SGD(Optim):
    """x = 1*x + (-lr)*d via geam, then clear_grad (NN:265-287; gradClip is ignored there too), as one backend call per
    parameter (the HIP backend's `sgd_update`; its library gathers a run of them into one launch).
    `fused=True` hands all tensors to the backend in one multi-tensor call instead."""

    def __init__(self, module, learning_rate, gradClip=1.0, descent=True, fused=False):
        super().__init__(module)
        self.lr = learning_rate if descent else -learning_rate
        self.fused = fused

    def step(self):
        be = get_backend()
        if self.fused:
            be.multi_sgd_update([(p.x.data, p.d.data, p.x.scalarCount) for p in self.params], self.lr)
        else:
            for p in self.params:
                be.sgd_update(p.x.data, p.d.data, self.lr, p.x.scalarCount)


class SGD_Momentum(Optim):
    """NN:296-303 + CPU:1232-1246: clip, v = mu*v + g, (nesterov), x -= lr*g, d = 0; one `momentum_update` per parameter,
    as the reference's `step_func` issues them (`fused=True`: one multi-tensor backend call instead)."""

    def __init__(self, module, learning_rate, momentum=0.9, gradClip=400.0, nesterov=False, descent=True, fused=False):
        super().__init__(module)
        assert descent
        self.lr, self.mu, self.clip, self.nesterov, self.fused = learning_rate, momentum, gradClip, nesterov, fused
        self.moment = [Tensor.zeros_like(p.x) for p in self.params]      # enrichParameter (NN:74-84)

    def step(self):
        be = get_backend()
        if self.fused:
            be.multi_momentum_update([(p.x.data, p.d.data, m.data, p.x.scalarCount) for p, m in zip(self.params, self.moment)],
                                     self.lr, self.mu, self.clip, self.nesterov)
        else:
            for p, m in zip(self.params, self.moment):
                be.momentum_update(p.x.data, p.d.data, m.data, self.lr, self.mu, self.clip, self.nesterov, p.x.scalarCount)


class Adagrad(Optim):
    """NN:289-294 + CPU:1217-1230."""

    def __init__(self, module, learning_rate, gradClip=1.0, descent=True):
        super().__init__(module)
        assert descent
        self.lr, self.clip = learning_rate, gradClip
        self.moment = [Tensor.zeros_like(p.x) for p in self.params]

    def step(self):
        be = get_backend()
        for p, m in zip(self.params, self.moment):
            be.adagrad_update(p.x.data, p.d.data, m.data, self.lr, self.clip, p.x.scalarCount)
