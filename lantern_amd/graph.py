"""A training step recorded once into a HIP graph and replayed.

For programs whose kernels are shorter than their launches (LeNet, SqueezeNet on 32x32 images: several hundred
kernels of a few microseconds per step) the host's launch path sets the step time.  The reference pays one launch
per operator (the generated C++ calls a kernel or a cuDNN routine per trait method, TensorDifferentiation.scala:137-379);
here the stream of a whole step -- forward, backward and the optimizer -- is captured after a few eager steps and
enqueued again with one call.

What makes a step replayable: the arena is rewound to the same mark after every step, so every intermediate gets the
address it had when the step was recorded; the inputs stay where they are and are refreshed in place
(`backend.upload(tensor.data, array)` between replays); parameters and optimizer state are updated in place by the recorded kernels;
dropout positions move on inside the graph.  Steps whose shapes change (TreeLSTM's trees) do not qualify.
"""
from .tensor import get_backend


class StepGraph:
    def __init__(self, trainer, eager_steps=3):
        """Runs `eager_steps` ordinary steps (launch plans are measured and scratch buffers grown there, which a
        capture cannot do), then records one `trainer.step(); trainer.end_step()`.  Recording runs nothing: the first
        `launch()` is the step after the eager ones."""
        be = get_backend()
        self.be = be
        for _ in range(eager_steps):
            trainer.step(); trainer.end_step()
        be.sync()
        drawn = be.dropout_offset
        be.captureBegin()
        try:
            self.loss = trainer.step()      # its buffer is written by every replay
            trainer.end_step()
        finally:
            self.graph = be.captureEnd()
        self.drawn = be.dropout_offset - drawn
        be.dropout_offset = drawn           # recording drew nothing

    def launch(self):
        self.be.graphLaunch(self.graph)
        self.be.dropout_offset += self.drawn    # keeps eager steps after a replay on the same stream of positions
        return self.loss

    def close(self):
        if self.graph is not None:
            self.be.graphDestroy(self.graph)
            self.graph = None
