"""Reverse-mode autodiff over ONNX library nodes (mirror of the daceml.autodiff registry surface)."""
from .base_abc import (AutoDiffException, BackwardContext, BackwardGroup, BackwardImplementation, BackwardResult,
                       autoregister_params, find_backward_implementation)
from .backward_pass_generator import BackwardPassGenerator, add_backward_pass
from . import implementations  # registers the "hip" backward implementations
