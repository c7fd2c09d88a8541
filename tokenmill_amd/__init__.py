"""tokenmill_amd: a single-GPU inference engine for AMD MI355X (gfx950).

Everything between a request's token ids and its next token: typed configuration and an
architecture registry, a safetensors loader, layers assembled from parts, a paged cache
manager, one step function, a scheduler, a sampler and hand-written HIP kernels.
"""

__version__ = "0.1.0"
