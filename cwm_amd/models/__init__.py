from .model import Model
from . import llama3_dense, lapevik, segedra, dogotar, digasun  # noqa: F401  (register the architectures)

__all__ = ["Model"]
