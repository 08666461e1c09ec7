"""Sentiment TreeLSTM: one training step per tree (binary constituency trees, Adagrad).

Follows src/main/scala/lantern/PLDI19APP/SentimentTreeLSTM.scala:242-318 (the GPU variant; the CPU
variant :67-140 is the same program with plusBias in place of plusEqual): Leaf = three gemv 150x300
gates, Node = ten gemv 150x150 into five gates, Out = gemv 5x150 + logSoftmax + nll per node, the
losses of the two children added into the parent's, gradR_loss over the root, Adagrad (lr 0.05,
clip 1) after every tree, arena rewound after every tree (:331-345).

Reference behaviour kept on purpose: Leaf and Node return (hidden, cell) but the tree body binds
the pair as (cell, hidden) (:302, :307), so the classifier reads the cell state and the roles of
the two vectors are exchanged on the way up.  `reference_binding=False` gives the textbook wiring.

Tree encoding (src/out/PLDI19evaluation/treelstm/lantern/array_tree.txt): per tree four int arrays
scores[i], words[i] (-1 for internal nodes), lch[i], rch[i] (-1 for leaves); the root is index 0.
"""
import numpy as np

from ..nn import Module, Adagrad
from ..tensor import Tensor, TensorR, gradR_loss, get_backend, int_array


def random_tree(rng, n_leaves, vocab, classes=5):
    """A random full binary tree in the array encoding, nodes numbered in pre-order."""
    scores, words, lch, rch = [], [], [], []

    def build(k):
        i = len(scores)
        scores.append(int(rng.randint(0, classes))); words.append(-1); lch.append(-1); rch.append(-1)
        if k == 1:
            words[i] = int(rng.randint(0, vocab))
        else:
            left = int(rng.randint(1, k))
            lch[i] = build(left)
            rch[i] = build(k - left)
        return i

    build(n_leaves)
    return tuple(np.asarray(a, np.int32) for a in (scores, words, lch, rch))


def read_trees(path):
    """array_tree.txt: first integer = number of trees, then per tree its size and four arrays of that length."""
    vals = np.array(open(path).read().split(), dtype=np.int64)
    n, pos, trees = int(vals[0]), 1, []
    for _ in range(n):
        size = int(vals[pos]); pos += 1
        arrs = []
        for _ in range(4):
            arrs.append(vals[pos:pos + size].astype(np.int32)); pos += size
        trees.append(tuple(arrs))
    return trees


class Leaf(Module):
    def __init__(self, inSize, hSize):
        super().__init__("leaf")
        for g in "iou":
            setattr(self, "W" + g, self.param("W" + g, Tensor.randinit((hSize, inSize), 0.01)))
            setattr(self, "b" + g, self.param("b" + g, Tensor.zeros(hSize)))

    def __call__(self, x):
        i_gate = self.Wi.dot(x).plusBias(self.bi).sigmoid()
        o_gate = self.Wo.dot(x).plusBias(self.bo).sigmoid()
        u_value = self.Wu.dot(x).plusBias(self.bu).tanh()
        cell = i_gate * u_value
        hidden = o_gate * cell.tanh()
        return hidden, cell


class Node(Module):
    NAMES = ["U0i", "U1i", "bbi", "U00f", "U01f", "U10f", "U11f", "bbf", "U0o", "U1o", "bbo", "U0u", "U1u", "bbu"]

    def __init__(self, hSize):
        super().__init__("node")
        for n in self.NAMES:      # creation order = order of the rand() stream (:262-275)
            setattr(self, n, self.param(n, Tensor.zeros(hSize) if n.startswith("bb") else Tensor.randinit((hSize, hSize), 0.01)))

    def __call__(self, hl, cl, hr, cr):
        i_gate = self.U0i.dot(hl).plusEqual(self.U1i.dot(hr)).plusBias(self.bbi).sigmoid()
        fl_gate = self.U00f.dot(hl).plusEqual(self.U01f.dot(hr)).plusBias(self.bbf).sigmoid()
        fr_gate = self.U10f.dot(hl).plusEqual(self.U11f.dot(hr)).plusBias(self.bbf).sigmoid()
        o_gate = self.U0o.dot(hl).plusEqual(self.U1o.dot(hr)).plusBias(self.bbo).sigmoid()
        u_value = self.U0u.dot(hl).plusEqual(self.U1u.dot(hr)).plusBias(self.bbu).tanh()
        cell = (i_gate * u_value).plusEqual(fl_gate * cl).plusEqual(fr_gate * cr)
        hidden = o_gate * cell.tanh()
        return hidden, cell


class Out(Module):
    def __init__(self, hSize, outSize):
        super().__init__("output")
        self.Why = self.param("Why", Tensor.randinit((outSize, hSize), 0.01))
        self.by = self.param("by", Tensor.zeros(outSize))

    def __call__(self, h, score):
        pred = self.Why.dot(h).plusBias(self.by)
        return pred.resize(1, pred.x.shape[0]).logSoftmaxB(1).nllLossB(score)


class TreeNet(Module):
    def __init__(self, inSize=300, hSize=150, outSize=5, reference_binding=True):
        super().__init__("tree")
        self.leaf = self.add(Leaf(inSize, hSize))
        self.node = self.add(Node(hSize))
        self.out = self.add(Out(hSize, outSize))
        self.reference_binding = reference_binding

    def __call__(self, embedding, scores_dev, words, lch, rch):
        def visit(i):                                      # LOOPTM (TD:1719-1761): children first, left before right
            if lch[i] < 0:
                emb = TensorR(embedding(int(words[i])), isInput=True)
                a, b = self.leaf(emb)
                kids = None
            else:
                l, r = visit(int(lch[i])), visit(int(rch[i]))
                a, b = self.node(l[1], l[2], r[1], r[2])
                kids = (l, r)
            hidden, cell = (b, a) if self.reference_binding else (a, b)      # `val ArrayBuffer(cell, hidden) = leaf(..)`
            loss = self.out(hidden, scores_dev.offset(i))
            if kids is not None:
                loss = loss.plusEqual(kids[0][0]).plusEqual(kids[1][0])
            return loss, hidden, cell
        return visit(0)[0]


class Trainer:
    def __init__(self, n_trees=8, vocab=2000, emb=300, hidden=150, classes=5, lr=0.05, seed=42, min_leaves=5, max_leaves=50, trees=None,
                 reference_binding=True, batch_small_ops=True):
        be = get_backend()
        # ~5000 operator calls on 150-element vectors per tree: let the backend run them from a command list
        # instead of one launch each, where it can (BackendHIP.batchSmallOps; `close()` switches it off again)
        self.batching = bool(batch_small_ops) and hasattr(be, "batchSmallOps")
        if self.batching:
            be.batchSmallOps(True)
        rng = np.random.RandomState(seed)
        Tensor.randseed(seed)
        self.model = TreeNet(emb, hidden, classes, reference_binding)
        self.opt = Adagrad(self.model, lr)
        self.embedding = Tensor.fromNumpy((rng.standard_normal((vocab, emb)) * 0.1).astype(np.float32))
        self.trees = trees if trees is not None else [random_tree(rng, int(rng.randint(min_leaves, max_leaves + 1)), vocab, classes) for _ in range(n_trees)]
        if trees is not None:     # real shapes, synthetic tokens inside the table
            self.trees = [(s % classes, np.where(w >= 0, w % vocab, -1).astype(np.int32), l, r) for s, w, l, r in trees]
        self.next = 0
        self.mark = be.getMallocAddr()

    def step(self):
        scores, words, lch, rch = self.trees[self.next % len(self.trees)]
        self.next += 1
        self.nodes = len(scores)
        scores_dev = int_array(scores)                     # scores.toGPU(size) (:336)
        loss = gradR_loss(lambda dummy: self.model(self.embedding, scores_dev, words, lch, rch))(Tensor.zeros(1))
        self.opt.step()
        return loss

    def end_step(self):
        get_backend().resetMallocAddr(self.mark)

    def close(self):
        if self.batching:
            get_backend().batchSmallOps(False)
            self.batching = False


def write_c_program_inputs(directory, trainer):
    """The two input files of the plain-C host program of this training loop (tests/host_c/treelstm_step.c) from a freshly
    built Trainer: params.bin (sizes, embedding table, the 22 parameter tensors in creation order) and trees.txt (the
    reference's array_tree.txt layout).  Returns the parameter TensorRs in file order."""
    import os
    model = trainer.model
    named = model.namedParameters()
    names = [n.split("/", 1)[1] for n, _ in named]
    assert names == ["leaf/Wi", "leaf/bi", "leaf/Wo", "leaf/bo", "leaf/Wu", "leaf/bu"] + ["node/" + n for n in Node.NAMES] + ["output/Why", "output/by"], names
    params = [p for _, p in named]
    emb = trainer.embedding.toCPU()
    vocab, e = emb.shape
    hidden, classes = params[1].x.shape[0], params[-1].x.shape[0]
    with open(os.path.join(str(directory), "params.bin"), "wb") as f:
        np.array([vocab, e, hidden, classes], np.int32).tofile(f)
        emb.astype(np.float32).tofile(f)
        for p in params:
            p.x.toCPU().astype(np.float32).tofile(f)
    with open(os.path.join(str(directory), "trees.txt"), "w") as f:
        f.write("%d\n" % len(trainer.trees))
        for t in trainer.trees:
            f.write("%d\n" % len(t[0]))
            for arr in t:
                f.write(" ".join(str(int(v)) for v in arr) + "\n")
    return params
