"""tokenmill_amd: a single-GPU inference engine for AMD MI355X (gfx950).

Everything between a request's token ids and its next token: typed configuration and an
architecture registry, a safetensors loader, layers assembled from parts, a paged cache
manager, one step function, a scheduler, a sampler and hand-written HIP kernels.
"""

__version__ = "0.1.0"


def __getattr__(name):          # the public names, imported on first use (torch loads slowly)
    if name in ("LLMEngine", "RequestRejected"):
        from tokenmill_amd.engine import engine
        return getattr(engine, name)
    if name == "EngineConfig":
        from tokenmill_amd.config.engine_config import EngineConfig
        return EngineConfig
    if name == "SamplingParams":
        from tokenmill_amd.sampling.sampler import SamplingParams
        return SamplingParams
    raise AttributeError(name)
