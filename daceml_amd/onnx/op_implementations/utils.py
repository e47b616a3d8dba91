"""``@op_implementation`` (daceml/onnx/op_implementations/utils.py:19-40).

The reference's decorator only adds the class to the ``ONNXForward`` registry; the node classes pick
registered implementations up once, while ``onnx_op.py`` is imported (onnx_op.py:664-701), so an
implementation registered later is invisible to ``ONNX<Op>.implementations``. Here the decorator
does both registrations, which is what makes a late-registered implementation selectable.
"""
from ..forward_implementation_abc import ONNXForward
from .. import nodes


def op_implementation(op: str, name: str):
    def dec(cls):
        doc = '\n    :Implementation name: ``"{}"``\n'.format(name)
        cls.__doc__ = (cls.__doc__ or "") + doc
        ONNXForward.register(cls, op=op, name=name)
        if nodes.has_onnx_node(op):
            nodes.get_onnx_node(op).register_implementation(name, cls)
        return cls
    return dec
