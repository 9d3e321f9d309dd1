"""Architectures.  Importing the package registers the ones it ships."""
from . import llama  # noqa: F401
