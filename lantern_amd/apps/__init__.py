"""The reference's evaluation programs restated on the Tensor/TensorR surface (one module per
benchmark configuration), each with a `train_step` in the shape of the emitted training loop."""
