"""Graph rewrites: the fusion passes (``fusion``) and ``parameter_to_transient`` (daceml/transformation/__init__.py)."""
from . import fusion
from .parameter_to_transient import parameter_to_transient

__all__ = ["fusion", "parameter_to_transient"]
