"""The ONNX model file the reference's own regression test holds for a Slice (tests/onnx_files/slice.onnx, checked by
tests/test_bert_subgraphs.py:20-30 of the reference: input ones(2), output of shape (1,) holding 1.0), kept here as
tests/golden/reference_slice.onnx. The importer turns the Slice into a view and, because the view is the model's
output, copies it into the caller's buffer with an Identity node."""
import os

import numpy as np
import pytest
import torch


FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_slice.onnx")


def _model():
    from daceml_amd.onnx import ONNXModel
    with open(FIXTURE, "rb") as f:
        return ONNXModel("slice", f.read(), auto_optimize=False)


def test_reference_slice_model_on_the_emulator():
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    model = _model()
    assert model.inputs == ["data"] and model.outputs == ["__return"]
    st = model.sdfg.states()[0]
    assert [n.schema.name for n in st.library_nodes()] == ["Identity"]
    expand_onnx_nodes(model.sdfg)
    arrays = {"data": np.ones(2, np.float32)}
    run_state(model.sdfg, st, arrays)
    out = arrays["__return"]
    assert out.shape == (1, ) and out[0] == 1.0                 # the reference's own assertions
    arrays = {"data": np.array([3.0, 7.0], np.float32)}
    run_state(model.sdfg, st, arrays)
    assert arrays["__return"][0] == 3.0                          # starts [0], ends [1], axes [0]


@pytest.mark.gpu
def test_reference_slice_model_on_gpu():
    out = _model()(data=torch.ones(2).cuda())
    assert out.shape == (1, ) and out[0] == 1.0
