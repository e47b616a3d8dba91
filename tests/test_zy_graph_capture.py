"""``CompiledSDFG.capture``: the launches of a program recorded into a HIP graph and replayed.

Each replay is followed by eager work and a synchronisation and compared
with the eager result on fresh inputs written into the same buffers (a graph holds pointers, not values)."""
import numpy as np
import pytest
import torch

from tests.util import dev, rng

pytestmark = pytest.mark.gpu


def _program(dtype, attention):
    from daceml_amd import graphs
    from daceml_amd.runtime import CompiledSDFG
    from daceml_amd.transformation import fusion
    b, s, h, heads, ffn = 2, 128, 256, 4, 512
    sdfg = graphs.bert_encoder_layer(b, s, h, heads, ffn, dtype, eps=1e-5)
    fusion.auto_optimize(sdfg, attention=attention)
    p = graphs.bert_init_params(h, ffn, 3, bias_std=0.02)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    args = {n: dev(p[n].astype(npdt)) for n in graphs.BERT_PARAM_NAMES}
    args["x"] = dev(rng(1).standard_normal((b, s, h)).astype(npdt))
    args["y"] = torch.empty((b, s, h), dtype=dtype, device="cuda")
    return CompiledSDFG(sdfg), args


@pytest.mark.parametrize("dtype,attention", [(torch.float16, True), (torch.float32, False)])
def test_replays_match_eager_launches(dtype, attention):
    prog, args = _program(dtype, attention)
    prog(**args)
    captured = prog.capture()
    for i in range(4):
        x = torch.randn_like(args["x"])
        args["x"].copy_(x)                       # same buffer, new values
        prog.launch()
        torch.cuda.synchronize()
        eager = args["y"].clone()
        args["y"].fill_(float("nan"))
        captured.replay()
        torch.cuda.synchronize()
        assert torch.equal(args["y"], eager), "replay %d" % i
        (args["y"] * 2).sum().item()             # eager work between the replays


def test_a_graph_belongs_to_its_binding():
    prog, args = _program(torch.float16, True)
    prog(**args)
    captured = prog.capture()
    prog.bind({"y": args["y"]})                  # same tensor: nothing changed
    captured.replay()
    other = torch.empty_like(args["y"])
    prog.bind({"y": other})
    with pytest.raises(RuntimeError):
        captured.replay()
    again = prog.capture()
    again.replay()
    torch.cuda.synchronize()
    replayed = other.clone()
    other.fill_(float("nan"))
    prog.launch()
    torch.cuda.synchronize()
    assert torch.equal(other, replayed)
