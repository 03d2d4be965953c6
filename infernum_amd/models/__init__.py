"""Importing this package registers the built-in architectures."""
from .model import DecoderModel
from . import llama  # noqa: F401  (registration)
