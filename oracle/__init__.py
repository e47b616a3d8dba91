"""CPU oracle for the ONNX library-node hot path (test infrastructure only; see oracle/ops.py)."""
from . import ops  # noqa: F401
