"""What a "hip" expansion returns: a tasklet node holding C-ABI call specifications.

In the reference, an expansion that reaches a native library returns a C++ ``Tasklet`` whose body is
the library call, with ``code_init`` / ``code_exit`` and an environment that links the library
(daceml/onnx/op_implementations/cudnn_implementations.py:360-410). ``HipTasklet`` is that node in a
neutral form: a list of ``HipCall``s naming a ``dmlhip_*`` symbol and its arguments in terms of the
node's connectors. The in-tree runtime binds the calls to ctypes (daceml_amd/runtime.py); the DaCe
plugin renders the same calls as the body of a DaCe C++ tasklet (daceml_amd/dace_plugin.py).
"""
import dataclasses
from typing import Any, List, Optional, Sequence

from .sdfg import Node


@dataclasses.dataclass(frozen=True)
class Ptr:
    """Device pointer of the array attached to connector ``conn`` (plus an element offset)."""
    conn: str
    offset: int = 0


@dataclasses.dataclass(frozen=True)
class Null:
    pass


@dataclasses.dataclass(frozen=True)
class I64:
    value: int


@dataclasses.dataclass(frozen=True)
class I32:
    value: int


@dataclasses.dataclass(frozen=True)
class F32:
    value: float


@dataclasses.dataclass(frozen=True)
class USize:
    """A size_t argument."""
    value: int


@dataclasses.dataclass(frozen=True)
class I64Array:
    values: tuple


@dataclasses.dataclass(frozen=True)
class PtrArray:
    """``const void* const*``: pointers of several connectors."""
    conns: tuple


@dataclasses.dataclass
class Struct:
    """Pointer to a filled-in descriptor struct (dmlhip_gemm_desc / dmlhip_conv2d_desc)."""
    value: Any
    c_type: str


@dataclasses.dataclass(frozen=True)
class Workspace:
    """The shared scratch buffer (pointer), ``offset`` bytes in."""
    offset: int = 0


@dataclasses.dataclass(frozen=True)
class WorkspaceBytes:
    """Bytes of the shared scratch buffer that remain after ``offset`` (size_t)."""
    offset: int = 0


@dataclasses.dataclass(frozen=True)
class Stream:
    """The stream the SDFG runs on (``__dace_current_stream`` in a DaCe tasklet)."""


@dataclasses.dataclass
class HipCall:
    symbol: str
    args: List[Any]
    #: algorithmic work of this call alone, for nodes whose calls are separate pieces of work (the two gradients of a
    #: convolution); None: the node's figures go to its first call
    flops: Any = None
    bytes_moved: Any = None


class HipTasklet(Node):
    """Expansion result: same connectors as the library node it replaces."""
    def __init__(self, label: str, inputs: Sequence[str], outputs: Sequence[str], calls: List[HipCall],
                 workspace_bytes: int = 0, flops: int = 0, bytes_moved: int = 0, kind: str = ""):
        super().__init__(label)
        for c in inputs:
            self.add_in_connector(c)
        for c in outputs:
            self.add_out_connector(c)
        self.calls = calls
        self.workspace_bytes = int(workspace_bytes)
        #: algorithmic work of the node, for roofline reporting
        self.flops = int(flops)
        self.bytes_moved = int(bytes_moved)
        self.kind = kind
        #: {output connector: input connector}: the kernels give the right result when the output is the very buffer of
        #: that input (same shape, type and layout); a memory planner may then let the output take over the bytes of an
        #: input that nobody reads afterwards
        self.in_place: dict = {}


class ViewTasklet(Node):
    """Expansion result for nodes that move no data (a Reshape / Transpose folded into a view)."""
    def __init__(self, label: str, inputs: Sequence[str], outputs: Sequence[str]):
        super().__init__(label)
        for c in inputs:
            self.add_in_connector(c)
        for c in outputs:
            self.add_out_connector(c)
        self.calls: List[HipCall] = []
        self.workspace_bytes = 0
        self.flops = 0
        self.bytes_moved = 0
        self.kind = "view"
