"""``torch.onnx.export`` with the settings DaceModule uses (daceml/torch/module.py:266-287): opset 12, constant
folding off so that parameter names survive, initializers kept as graph inputs."""
import contextlib
import copy
import importlib
import io
from typing import Sequence

import torch
from torch.onnx import TrainingMode


@contextlib.contextmanager
def _exporter_without_onnx_package():
    """The TorchScript exporter serialises the graph itself; only its last step — attaching onnxscript functions,
    of which a plain module has none — imports the ``onnx`` package. Where that package is absent the step is
    replaced by the identity for the duration of the export."""
    try:
        importlib.import_module("onnx")
        yield
        return
    except ImportError:
        pass
    utils = None
    for path in ("torch.onnx._internal.torchscript_exporter.onnx_proto_utils", "torch.onnx._internal.onnx_proto_utils"):
        try:
            utils = importlib.import_module(path)
            break
        except ImportError:
            continue
    if utils is None or not hasattr(utils, "_add_onnxscript_fn"):
        raise RuntimeError("cannot export to ONNX: the `onnx` package is not installed and this PyTorch version's "
                           "exporter has no serialisation path without it")
    original = utils._add_onnxscript_fn
    utils._add_onnxscript_fn = lambda model_bytes, custom_opsets: model_bytes
    try:
        yield
    finally:
        utils._add_onnxscript_fn = original


def export_onnx(module: torch.nn.Module, dummy_inputs: Sequence[torch.Tensor], training: bool = False,
                opset_version: int = 12) -> bytes:
    """Serialized ONNX model of ``module`` traced on ``dummy_inputs``; the module's state is restored afterwards
    (tracing in training mode updates e.g. BatchNorm statistics)."""
    state = copy.deepcopy(module.state_dict())
    was_training = module.training
    buf = io.BytesIO()
    try:
        with _exporter_without_onnx_package():
            import warnings
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                torch.onnx.export(module, tuple(dummy_inputs), buf, dynamo=False,
                                  training=TrainingMode.TRAINING if training else TrainingMode.EVAL,
                                  opset_version=opset_version, export_params=True, do_constant_folding=False,
                                  keep_initializers_as_inputs=True)
    finally:
        module.load_state_dict(state)
        module.train(was_training)
    return buf.getvalue()
