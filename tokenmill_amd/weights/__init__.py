from tokenmill_amd.weights.loader import TensorSpec, WeightsError, read_checkpoint

__all__ = ["TensorSpec", "WeightsError", "read_checkpoint", "random_tensors", "write_random_model"]


def __getattr__(name: str):
    # random_init is also a program (`python -m tokenmill_amd.weights.random_init`): it is imported when one of
    # its functions is asked for, not with the package, so that running it does not find it imported already
    if name in ("random_tensors", "write_random_model"):
        from tokenmill_amd.weights import random_init
        return getattr(random_init, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
