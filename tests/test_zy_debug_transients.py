"""``debug_transients=True`` (daceml/torch/module.py:129-143; the reference's tests/torch/test_debug_transients.py):
every intermediate tensor of the wrapped module becomes an additional output."""
import numpy as np
import pytest
import torch



def _module():
    from daceml_amd.torch import dace_module

    @dace_module(debug_transients=True)
    class Module(torch.nn.Module):
        def forward(self, x):
            y = x + 3
            return y * 5

    return Module()


def test_intermediate_tensors_become_outputs():
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    module = _module()
    x = torch.rand(5, 5)
    model = module._import((x, ))
    assert len(model.outputs) == 2 and not any(model.sdfg.arrays[o].transient for o in model.outputs)
    st = model.sdfg.states()[0]
    expand_onnx_nodes(model.sdfg)
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    run_state(model.sdfg, st, arrays)
    np.testing.assert_allclose(arrays[model.outputs[0]], ((x + 3) * 5).numpy(), rtol=1e-6)
    np.testing.assert_allclose(arrays[model.outputs[1]], (x + 3).numpy(), rtol=1e-6)


def test_exposed_tensors_keep_the_fusion_passes_away():
    """A tensor that is an output has to exist: the chain of a Gelu stays a chain."""
    from daceml_amd.torch import DaceModule
    x = torch.randn(4, 16)
    plain = DaceModule(torch.nn.GELU())._import((x, ))
    exposed = DaceModule(torch.nn.GELU(), debug_transients=True)._import((x, ))
    assert [n.schema.name for n in plain.sdfg.states()[0].library_nodes()] == ["Gelu"]
    assert len(exposed.sdfg.states()[0].library_nodes()) == 5 and len(exposed.outputs) == 5


@pytest.mark.gpu
def test_debug_transients_on_gpu():
    module = _module()
    x = torch.rand(5, 5).cuda()
    output, y = module(x)
    torch.testing.assert_close(output, (x + 3) * 5)
    torch.testing.assert_close(y, x + 3)
