"""A one-GPU inference engine for AMD MI355X (gfx950).

From a model folder (config.json + model.safetensors) to generated tokens:
typed configuration and an architecture registry, a by-name weight loader,
layers assembled from registered parts, a paged cache manager, one step
function over ragged batches, a scheduler, sampling and trace replay, with the
forward pass in hand-written HIP kernels.
"""

__version__ = "0.1.0"
