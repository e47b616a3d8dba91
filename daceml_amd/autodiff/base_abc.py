"""Abstract base classes of the autodiff registry (mirror of daceml/autodiff/base_abc.py:23-159)."""
import abc
import dataclasses
import logging
import typing

from ..onnx.forward_implementation_abc import _Registry
from ..onnx.nodes import ONNXOp
from ..sdfg import SDFG, Node, SDFGState

log = logging.getLogger(__name__)


class AutoDiffException(Exception):
    """Base class for all exceptions related to automatic differentiation failures."""


@dataclasses.dataclass
class BackwardContext:
    """The graph context required to construct reverse nodes (base_abc.py:23-31)."""
    forward_sdfg: SDFG
    forward_state: SDFGState
    backward_sdfg: SDFG
    backward_state: SDFGState
    backward_generator: "BackwardPassGenerator"  # noqa: F821


class BackwardResult:
    """Names of the gradients a reverse node calculates and requires (base_abc.py:34-60).

    ``passthrough`` is an addition: ``{input connector: output connector}`` says that the gradient of
    that input *is* the gradient given for that output (a residual Add), so no node or copy is needed.
    """
    def __init__(self, required_grad_names, given_grad_names, zero_init=None, passthrough=None):
        #: input connector of the forward node -> connector of the reverse node that outputs its gradient
        self.required_grad_names: typing.Dict[str, str] = required_grad_names
        #: output connector of the forward node -> connector of the reverse node that takes its gradient
        self.given_grad_names: typing.Dict[str, str] = given_grad_names
        #: gradient connector -> whether the array must be zeroed before the reverse node runs
        self.zero_init: typing.Dict[str, bool] = zero_init or {}
        self.passthrough: typing.Dict[str, str] = passthrough or {}

    @staticmethod
    def empty():
        return BackwardResult(given_grad_names={}, required_grad_names={}, zero_init={})


class BackwardGroup(Node):
    """Several reverse nodes that together differentiate one forward node. Its connectors stand for
    connectors of the member nodes; the generator wires edges straight to the members (the role a
    nested SDFG plays for ``backward_program_for_node`` in the reference, autodiff/utils.py)."""
    def __init__(self, label: str):
        super().__init__(label)
        self.inputs: typing.Dict[str, typing.List[typing.Tuple[Node, str]]] = {}
        self.outputs: typing.Dict[str, typing.Tuple[Node, str]] = {}

    def map_input(self, conn: str, node: Node, node_conn: str):
        self.add_in_connector(conn)
        self.inputs.setdefault(conn, []).append((node, node_conn))

    def map_output(self, conn: str, node: Node, node_conn: str):
        self.add_out_connector(conn)
        self.outputs[conn] = (node, node_conn)


class BackwardImplementation(metaclass=_Registry):
    """ABC for backward implementations. Register with ``op=<ONNX name>`` (or ``node_type=<class>``) and
    ``name=<implementation name>`` (base_abc.py:63-112)."""
    @staticmethod
    def backward_can_be_applied(node: Node, state: SDFGState, sdfg: SDFG) -> bool:
        return True

    @staticmethod
    @abc.abstractmethod
    def backward(forward_node: Node, context: BackwardContext, given_gradients: typing.List[typing.Optional[str]],
                 required_gradients: typing.List[typing.Optional[str]]) -> typing.Tuple[Node, BackwardResult]:
        """Add the reverse node(s) of ``forward_node`` to ``context.backward_state`` and return the node
        (or BackwardGroup) plus the gradient connector names. Forward arrays the reverse node needs are
        connected by the implementation itself (``connect_*_from_forward``)."""
        ...


def autoregister_params(**params):
    """dace.registry.autoregister_params for BackwardImplementation subclasses."""
    def dec(cls):
        BackwardImplementation.register(cls, **params)
        return cls
    return dec


def find_backward_implementation(forward_sdfg: SDFG, forward_state: SDFGState,
                                 node: Node) -> typing.Optional[BackwardImplementation]:
    """Selection rule of base_abc.py:114-159: applicable implementations registered for the node's op or
    type; ``node.backward_implementation`` / ``default_backward_implementation`` wins if applicable, else
    the first applicable one."""
    valid = []
    for impl, args in BackwardImplementation.extensions().items():
        if "name" not in args:
            raise ValueError("Expected name in arguments of implementation {}.".format(impl))
        by_type = "node_type" in args and isinstance(node, args["node_type"])
        by_op = isinstance(node, ONNXOp) and args.get("op") == node.schema.name
        if (by_type or by_op) and impl.backward_can_be_applied(node, forward_state, forward_sdfg):
            valid.append((args["name"], impl))
    wanted = None
    if isinstance(node, ONNXOp):
        wanted = node.backward_implementation or type(node).default_backward_implementation
    if wanted:
        chosen = [i for n, i in valid if n == wanted]
        if chosen:
            return chosen[0]
        log.warning("Set backward_implementation %s on %s, but it could not be applied. Falling back to default "
                    "selection.", wanted, node)
    return valid[0][1] if valid else None
