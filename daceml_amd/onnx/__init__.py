"""``donnx`` — the ONNX library: node classes, implementation registry, default implementation.

Usage mirrors daceml.onnx: ``import daceml_amd.onnx as donnx``; ``donnx.ONNXConv(...)``,
``donnx.default_implementation = "hip"`` (module attribute, daceml/onnx/__init__.py:8-9),
``donnx.ONNXConv.default_implementation = ...``, ``node.implementation = ...``.
"""
import sys
import types

from .nodes import *  # noqa: F401,F403
from . import nodes as _nodes
from .forward_implementation_abc import ONNXForward
from .op_implementations.utils import op_implementation
from .op_implementations import hip_implementations  # registers the "hip" implementations


class _Module(types.ModuleType):
    """Makes ``donnx.default_implementation`` a live, assignable module attribute."""
    @property
    def default_implementation(self):
        return _nodes._default_implementation["value"]

    @default_implementation.setter
    def default_implementation(self, value):
        _nodes._default_implementation["value"] = value


sys.modules[__name__].__class__ = _Module

from .onnx_importer import ONNXModel  # noqa: E402,F401  (daceml/onnx/__init__.py:5)
