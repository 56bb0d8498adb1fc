from .model import Model
from . import llama3_dense, lapevik, segedra  # noqa: F401  (register the architectures)

__all__ = ["Model"]
