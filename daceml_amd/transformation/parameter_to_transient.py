"""``parameter_to_transient`` of the reference (daceml/transformation/parameter_to_transient.py:15-103): the array of a
PyTorch parameter stops being an argument of every call and becomes a buffer the compiled program owns for its whole
life, filled once from the parameter when the program is built.

The reference needs this on GPUs because a parameter that stays an argument is copied host to device on each call.
Here parameters are device tensors handed over by pointer, so nothing is copied either way; what the transformation
still gives is the reference's contract — the wrapped module works on a snapshot of the parameter (later changes to
the ``nn.Parameter`` are not seen, no gradient is produced for it) and the call passes one pointer less."""
import logging
import operator

import torch

from ..onnx.onnx_importer import clean_onnx_name
from ..sdfg import AccessNode

log = logging.getLogger(__name__)


def parameter_to_transient(dace_module, parameter_path: str):
    """Convert the array of the parameter found at ``parameter_path`` (dotted, as in ``named_parameters()``) to a
    persistently allocated transient. Call it from a ``post_onnx_hook`` of ``dace_module``, as the reference's tests
    do (tests/transformation/test_param_to_transient.py:32-35, tests/torch/test_bert_encoder.py:27-33)."""
    log.debug("Converting parameter %s to a transient", parameter_path)
    pt_tensor = operator.attrgetter(parameter_path)(dace_module.model)
    array_name = clean_onnx_name(parameter_path)
    sdfg = dace_module.sdfg
    if sdfg is None or dace_module.dace_model is None:
        raise ValueError("parameter_to_transient runs on an imported module: register it as a post_onnx_hook")
    dace_module.dace_model.inputs.remove(parameter_path)     # ValueError if it is not an input, as in the reference

    used = [n for state in sdfg.states() for n in state.nodes() if isinstance(n, AccessNode) and n.data == array_name]
    if not used:
        log.warning("Could not find access node with name '%s', skipping parameter to transient", array_name)
        return
    if array_name not in sdfg.arrays:
        raise ValueError("Could not find parameter %s in sdfg." % array_name)
    desc = sdfg.arrays[array_name]
    if tuple(desc.shape) != tuple(pt_tensor.shape):
        raise ValueError("parameter %s has shape %s, its array %s" % (parameter_path, tuple(pt_tensor.shape), desc.shape))
    desc.transient = True
    desc.persistent = True        # never a candidate for removal or reuse by graph rewrites

    def post_compile_hook(compiled_sdfg):
        buffer = compiled_sdfg.buffers.get(array_name)
        if buffer is None:
            raise ValueError("Could not find the buffer of parameter %s in the compiled program." % array_name)
        with torch.no_grad():
            buffer.copy_(pt_tensor.detach().to(device=buffer.device, dtype=buffer.dtype))

    dace_module.post_compile_hooks["init_" + parameter_path] = post_compile_hook
