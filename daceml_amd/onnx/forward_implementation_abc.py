"""Registry of forward implementations of ONNX library nodes.

Mirror of daceml/onnx/forward_implementation_abc.py:11-51: an implementation is a class with the
static methods ``forward_can_be_applied(node, state, sdfg)`` and ``forward(node, state, sdfg)``,
registered with the arguments ``op`` (ONNX op name) and ``name`` (implementation name).
"""
import abc
import typing


class _Registry(abc.ABCMeta):
    """Small equivalent of dace.registry.make_registry: keeps ``{class: kwargs}``."""
    def __init__(cls, name, bases, ns):
        super().__init__(name, bases, ns)
        if not any(isinstance(b, _Registry) for b in bases):
            cls._registry_ = {}

    def register(cls, subclass, **kwargs):
        cls._registry_[subclass] = kwargs
        return subclass

    def unregister(cls, subclass):
        cls._registry_.pop(subclass, None)

    def extensions(cls) -> typing.Dict[type, dict]:
        return cls._registry_


class ONNXForward(metaclass=_Registry):
    """ABC for ONNX op forward implementations (register with ``op=<ONNX name>, name=<impl name>``)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        """Whether this expansion can be applied to ``node``; must never raise."""
        return True

    @staticmethod
    @abc.abstractmethod
    def forward(node, state, sdfg):
        """Expand ``node`` and return its expansion (a node or a nested SDFG)."""
        ...

    @classmethod
    def registered_implementations(cls, op_name: str) -> typing.List[typing.Tuple[str, "ONNXForward"]]:
        return [(args["name"], impl) for impl, args in cls.extensions().items()
                if args.get("op") == op_name]
