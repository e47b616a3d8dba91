"""The executor's memory plan (daceml_amd/memory_plan.py), on the graph alone: the launch order it chooses is a valid
one, transients that are alive at the same time never share bytes, and the benchmarked BERT step - run through the ABI
emulator inside such an arena, in that order - still gives the oracle's results."""
import numpy as np
import pytest
import torch

from daceml_amd import memory_plan
from tests.test_emulated_graphs import B, FFN, H, HEADS, S, _check, _inputs


def _bert_step(dtype=torch.float16, b=B, s=S, h=H, heads=HEADS, ffn=FFN, eps=1e-5):
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    sdfg = graphs.bert_encoder_layer(b, s, h, heads, ffn, dtype, eps=eps)
    fusion.auto_optimize(sdfg, training=True)
    add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + graphs.BERT_PARAM_NAMES,
                      grad_dtypes={n: torch.float32 for n in graphs.BERT_PARAM_NAMES})
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    return sdfg


def _root(sdfg, name):
    while sdfg.arrays[name].view_of is not None:
        name = sdfg.arrays[name].view_of
    return name


def _check_order(sdfg, order):
    """Every node once, states in order, and no node before a node that writes what it touches / reads what it
    writes in the plain topological order."""
    plain = memory_plan.launch_order(sdfg, small_peak=False)
    assert sorted(id(n) for _, n in order) == sorted(id(n) for _, n in plain)
    assert [s.label for s, _ in order] == [s.label for s, _ in plain]
    pos = {id(n): i for i, (_, n) in enumerate(order)}
    touch = {}
    for state, n in plain:
        touch[id(n)] = ({_root(sdfg, e.data.data) for e in state.in_edges(n)},
                        {_root(sdfg, e.data.data) for e in state.out_edges(n)})
    for j, (_, b) in enumerate(plain):
        for _, a in plain[:j]:
            (ra, wa), (rb, wb) = touch[id(a)], touch[id(b)]
            if (wa & (rb | wb)) or (wb & ra):
                assert pos[id(a)] < pos[id(b)], "%s must stay ahead of %s" % (a.label, b.label)


def _check_plan(sdfg, order, plan):
    first, last = memory_plan.lifetimes(sdfg, order)
    assert set(plan) == set(first)
    names = sorted(plan)
    shared_in_place = 0
    for i, a in enumerate(names):
        assert plan[a] % 256 == 0
        for b in names[i + 1:]:
            bytes_overlap = plan[a] < plan[b] + memory_plan.nbytes(sdfg.arrays[b]) and \
                plan[b] < plan[a] + memory_plan.nbytes(sdfg.arrays[a])
            alive_together = first[a] <= last[b] and first[b] <= last[a]
            if bytes_overlap and alive_together:
                # only an output that takes over a dying input of a node that allows it
                early, late = (a, b) if first[a] < first[b] else (b, a)
                assert last[early] == first[late] and plan[a] == plan[b], (a, b)
                state, node = order[first[late]]
                pairs = {(e_out.data.data, e_in.data.data) for e_out in state.out_edges(node) for e_in in state.in_edges(node)
                         if getattr(node, "in_place", {}).get(e_out.src_conn) == e_in.dst_conn}
                assert (late, early) in pairs, (a, b)
                shared_in_place += 1
    return shared_in_place


def test_bert_step_order_and_placement():
    sdfg = _bert_step()
    order = memory_plan.launch_order(sdfg, small_peak=True)
    _check_order(sdfg, order)
    plan = memory_plan.place_transients(sdfg, order)
    assert _check_plan(sdfg, order, plan) == 1          # the Gelu gradient over the gradient it is given
    labels = [n.label for _, n in order]
    # the weight gradient that reads the stored Gelu output last runs before the input gradient that needs a buffer of
    # that size
    assert labels.index("ffn2_matmul_fused_grad_1_hip") < labels.index("ffn2_matmul_fused_grad_0_hip")
    own = sum(memory_plan.nbytes(sdfg.arrays[n]) for n in plan)
    arena = max(off + memory_plan.nbytes(sdfg.arrays[n]) for n, off in plan.items())
    assert arena < 0.56 * own, (arena, own)


def test_benchmarked_shape_fits_the_last_level_cache():
    """[8, 512, 1024] x 16 heads x FFN 4096 in fp16: 252 MB of transients become an arena of 134.5 MB; with the 109 MB of
    caller-owned tensors the step touches less than the 256 MB the last-level cache holds."""
    sdfg = _bert_step(b=8, s=512, h=1024, heads=16, ffn=4096, eps=1e-12)
    order = memory_plan.launch_order(sdfg, small_peak=True)
    plan = memory_plan.place_transients(sdfg, order)
    _check_order(sdfg, order)
    _check_plan(sdfg, order, plan)
    own = sum(memory_plan.nbytes(sdfg.arrays[n]) for n in plan)
    arena = max(off + memory_plan.nbytes(sdfg.arrays[n]) for n, off in plan.items())
    callers = sum(memory_plan.nbytes(d) for n, d in sdfg.arrays.items()
                  if not d.transient and d.view_of is None and n not in sdfg.constants)
    assert 251e6 < own < 253e6 and 134e6 < arena < 135e6 and arena + callers < 245e6


def test_plain_order_is_the_topological_one_and_placement_works_on_it():
    sdfg = _bert_step()
    order = memory_plan.launch_order(sdfg)
    assert [n for _, n in order] == [n for st in sdfg.states() for n in st.topological_sort()]
    _check_plan(sdfg, order, memory_plan.place_transients(sdfg, order))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_bert_step_in_the_arena_gives_the_oracles_results(dtype):
    from tests.abi_emulator import run_sdfg_in_arena
    x, dy, p = _inputs(dtype)
    sdfg = _bert_step(dtype)
    arrays = {"x": x.copy(), "gradient_y": dy.copy(), **{k: v.copy() for k, v in p.items()}}
    labels, plan, total = run_sdfg_in_arena(sdfg, arrays)
    assert len(labels) == (19 if dtype == torch.float16 else 35) and total > 0   # fp32: attention stays a chain of nodes
    _check(arrays, x, dy, p, dtype)
    assert np.array_equal(arrays["x"], x) and all(np.array_equal(arrays[k], v) for k, v in p.items())


def test_placement_of_random_lifetimes_never_overlaps():
    """The free-list itself (split, merge, growth at the end) on random sizes and lifetimes."""
    from daceml_amd.hip_tasklet import HipTasklet
    from daceml_amd.sdfg import SDFG
    rng = np.random.default_rng(3)
    for trial in range(30):
        sdfg = SDFG("t%d" % trial)
        st = sdfg.add_state("s")
        n_nodes = int(rng.integers(3, 25))
        made = []
        for k in range(n_nodes):
            ins = ["i%d" % j for j in range(int(rng.integers(0, min(4, len(made)) + 1)))]
            outs = ["o%d" % j for j in range(int(rng.integers(1, 3)))]
            t = HipTasklet("n%d" % k, ins, outs, [])
            st.add_node(t)
            picked = list(rng.choice(len(made), size=len(ins), replace=False)) if ins else []
            for c, idx in zip(ins, picked):
                st.add_edge(st.add_access(made[idx]), None, t, c, sdfg.make_array_memlet(made[idx]))
            for c in outs:
                name = "a%d_%s" % (k, c)
                sdfg.add_array(name, (int(rng.integers(1, 5000)), ), torch.float16, transient=True)
                st.add_edge(t, c, st.add_access(name), None, sdfg.make_array_memlet(name))
                made.append(name)
        for small in (False, True):
            order = memory_plan.launch_order(sdfg, small_peak=small)
            _check_order(sdfg, order)
            _check_plan(sdfg, order, memory_plan.place_transients(sdfg, order))


def test_transients_left_out_get_no_place_and_the_rest_packs_tighter():
    """What DaceModule does with the buffers a backward call reads: they get fresh memory per forward call, so the arena
    only holds the others."""
    from daceml_amd.runtime import forwarded_transients
    sdfg = _bert_step()
    fwd, bwd = sdfg.states()[0].label, [s.label for s in sdfg.states()[1:]]
    kept = forwarded_transients(sdfg, [fwd], bwd)
    assert "gelu_mulhalf_C_43" in kept and all(sdfg.arrays[n].transient for n in kept)
    order = memory_plan.launch_order(sdfg, small_peak=True)
    everything = memory_plan.place_transients(sdfg, order)
    rest = memory_plan.place_transients(sdfg, order, leave_out=kept)
    assert set(rest) == set(everything) - set(kept) and rest
    size = lambda plan: max(off + memory_plan.nbytes(sdfg.arrays[n]) for n, off in plan.items())  # noqa: E731
    assert size(rest) < 0.5 * size(everything)
    first, last = memory_plan.lifetimes(sdfg, order)
    names = sorted(rest)
    for i, a in enumerate(names):
        for b in names[i + 1:]:
            if rest[a] < rest[b] + memory_plan.nbytes(sdfg.arrays[b]) and rest[b] < rest[a] + memory_plan.nbytes(sdfg.arrays[a]):
                assert last[a] <= first[b] or last[b] <= first[a], (a, b)
