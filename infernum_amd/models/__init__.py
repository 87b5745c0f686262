"""Importing this package registers the built-in architectures."""
from .model import DecoderModel
from . import llama, malinex, nesilorn, rogizen, sikazen  # noqa: F401  (registration)
