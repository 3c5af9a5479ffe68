"""An inference engine for the dense Llama decoder on one AMD Instinct MI355X (gfx950).

From a model folder (``config.json`` + safetensors) to generated tokens: typed configuration
and architecture registry, weights by tensor name, layers put together from parts, a paged
cache, one step function over mixed batches, a continuous-batching scheduler, greedy and
temperature sampling, and hand-written HIP kernels underneath."""

__version__ = "0.1.0"
