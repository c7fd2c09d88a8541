"""Architectures. Importing this package registers each of them under its config.json name."""
from tokenmill_amd.models import qwen2  # noqa: F401
from tokenmill_amd.models.decoder import DecoderModel, LayerCall

__all__ = ["DecoderModel", "LayerCall"]
