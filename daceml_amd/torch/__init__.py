"""PyTorch integration: ``DaceModule`` / ``dace_module`` wrap an ``nn.Module`` so that it runs on the HIP
library-node path (daceml/torch/__init__.py exports the same two names)."""
from .module import DaceModule, HipModule, dace_module, hip_module  # noqa: F401
