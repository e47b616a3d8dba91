"""``DaceModule``: an ``nn.Module`` that runs the wrapped module on the HIP library-node path.

Mirrors daceml/torch/module.py:46-365 and the ctypes dispatcher (daceml/torch/dispatchers/ctypes_module.py:
21-216): the module is exported to ONNX at opset 12 (on the first call, or at construction when
``dummy_inputs`` are given), imported into an SDFG, run through the ``post_onnx_hooks`` (by default the fusion
pipeline), differentiated when ``backward=True`` (then the ``post_autodiff_hooks`` run, by default the
backward-state rewrites), expanded and bound to the kernels (``post_compile_hooks``). Calls go through a
``torch.autograd.Function`` that allocates outputs with ``torch.empty``, passes the module's live parameters,
enqueues the forward state on the current stream, and in ``backward`` enqueues the backward state and returns
``None`` for inputs that need no gradient.

One difference in structure: forward and backward live in ONE SDFG (two states). ``post_autodiff_hooks`` receive
that SDFG for both arguments. What a backward call reads - the tensors the forward call was bound to, the outputs,
and the SDFG buffers the forward state fills for the backward state - is saved on the autograd context per call
(``ctx.save_for_backward``), so inputs may be dropped or overwritten and several forward calls may be pending.
"""
import collections
import logging
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch
from torch import nn

from ..autodiff import add_backward_pass
from ..onnx.onnx_importer import ONNXModel, clean_onnx_name
from ..runtime import CompiledSDFG, expand_onnx_nodes, forwarded_transients
from ..sdfg import AccessNode
from ..transformation import fusion
from .export import export_onnx

log = logging.getLogger(__name__)


def _unique(existing, name: str) -> str:
    if name not in existing:
        return name
    i = 0
    while "%s_%d" % (name, i) in existing:
        i += 1
    return "%s_%d" % (name, i)


class DaceModule(nn.Module):
    """Wraps ``module``; same constructor vocabulary as the reference (daceml/torch/module.py:86-99).

    :param module: the model to wrap.
    :param dummy_inputs: tensors to trace with; without them the first call's inputs are used.
    :param cuda: must be True or None — the kernels run on a GPU; the module is moved there.
    :param training: trace in training mode.
    :param backward: build the backward pass, so that the result takes part in autograd.
    :param inputs_to_skip: ONNX input names that need no gradient.
    :param auto_optimize: run the fusion pipeline (and the backward-state rewrites).
    :param onnx_simplify, simplify, compile_torch_extension: accepted so that code written for the reference's wrapper
        constructs this one unchanged; they select tools this path does not have (onnx-simplifier, DaCe's simplification
        pass, the generated C++ dispatcher in place of the ctypes one) and change nothing here.
    :param debug_transients: every intermediate tensor of the graph becomes an output, returned after the module's own
        (daceml/torch/module.py:129-143); the fusion passes then leave those tensors in place.
    :param sdfg_name: name of the SDFG (defaults to the module's class name).
    """
    def __init__(self, module: nn.Module, dummy_inputs: Optional[Tuple[torch.Tensor, ...]] = None,
                 cuda: Optional[bool] = None, training: bool = False, backward: bool = False,
                 inputs_to_skip: Optional[List[str]] = None, auto_optimize: bool = True,
                 sdfg_name: Optional[str] = None, debug_transients: bool = False, onnx_simplify: bool = True,
                 simplify: bool = True, compile_torch_extension: bool = True):
        super().__init__()
        if cuda is False:
            raise ValueError("the HIP implementations run on a GPU; cuda=False is not available")
        self.backward = backward
        self.model = module
        self.dace_model: Optional[ONNXModel] = None
        self.training_mode = training
        self.sdfg = None
        self.use_cuda = True
        self.sdfg_name = sdfg_name or type(module).__name__
        self.auto_optimize = auto_optimize
        self.inputs_to_skip = list(inputs_to_skip or [])
        self.function = None
        self.compiled: Optional[CompiledSDFG] = None
        self.optimization_stats: Dict[str, int] = {}

        #: run after the ONNX graph is imported into an SDFG; called with this module
        self.post_onnx_hooks: "collections.OrderedDict[str, Callable]" = collections.OrderedDict()
        #: run after the backward state has been added; called with (forward sdfg, backward sdfg)
        self.post_autodiff_hooks: "collections.OrderedDict[str, Callable]" = collections.OrderedDict()
        #: run after the kernels are bound; called with the CompiledSDFG
        self.post_compile_hooks: "collections.OrderedDict[str, Callable]" = collections.OrderedDict()

        self.debug_transients = debug_transients
        if self.debug_transients:
            def transients_outputs(dace_module):
                # as the reference does it: in node order, everything transient except the statistics side outputs
                sdfg = dace_module.sdfg
                for state in sdfg.states():
                    for node in state.nodes():
                        if not isinstance(node, AccessNode):
                            continue
                        desc = sdfg.arrays[node.data]
                        if desc.transient and desc.view_of is None and node.data not in dace_module.dace_model.outputs \
                                and "mean" not in node.data and "std" not in node.data:
                            dace_module.dace_model.outputs.append(node.data)
                            desc.transient = False

            self.prepend_post_onnx_hook("make_transients_outputs", transients_outputs)

        if self.auto_optimize:
            def optimize_forward(dace_module):
                dace_module.optimization_stats.update(
                    fusion.auto_optimize(dace_module.sdfg, training=dace_module.backward))

            self.append_post_onnx_hook("auto_optimize", optimize_forward)
            if self.backward:
                def optimize_backward(fwd_sdfg, bwd_sdfg):
                    self.optimization_stats.update(fusion.optimize_backward(bwd_sdfg))

                self.append_post_autodiff_hook("auto_optimize", optimize_backward)

        if dummy_inputs is not None:
            self.function = self._initialize_sdfg(dummy_inputs)

    # ------------------------------------------------------------------ hooks (module.py:179-245)
    def reset_sdfg(self):
        """Forget the SDFG so that the next call exports and optimizes again."""
        self.function = None

    def _add_hook(self, table, name, func, first):
        if self.function is not None:
            log.warning("Added a hook after the model was already initialized. This hook (with name %s) will not be "
                        "executed!", name)
        name = _unique(set(table), name)
        table[name] = func
        if first:
            table.move_to_end(name, last=False)

    def prepend_post_onnx_hook(self, name, func):
        self._add_hook(self.post_onnx_hooks, name, func, True)

    def append_post_onnx_hook(self, name, func):
        self._add_hook(self.post_onnx_hooks, name, func, False)

    def prepend_post_autodiff_hook(self, name, func):
        self._add_hook(self.post_autodiff_hooks, name, func, True)

    def append_post_autodiff_hook(self, name, func):
        self._add_hook(self.post_autodiff_hooks, name, func, False)

    def prepend_post_compile_hook(self, name, func):
        self._add_hook(self.post_compile_hooks, name, func, True)

    def append_post_compile_hook(self, name, func):
        self._add_hook(self.post_compile_hooks, name, func, False)

    # ------------------------------------------------------------------ construction
    def _import(self, dummy_inputs: Sequence[torch.Tensor]) -> ONNXModel:
        """Export, import and run the post-ONNX hooks (no GPU needed)."""
        model_bytes = export_onnx(self.model, dummy_inputs, training=self.training_mode)
        self._exported_parameters = dict(self.model.named_parameters())
        self._exported_parameters.update(dict(self.model.named_buffers()))
        self.dace_model = ONNXModel(self.sdfg_name, model_bytes, cuda=True, auto_optimize=False,
                                    parameters_as_inputs=list(self._exported_parameters),
                                    training=self.training_mode)
        self.sdfg = self.dace_model.sdfg
        for hook in self.post_onnx_hooks.values():
            hook(self)
        return self.dace_model

    def _inputs_that_need_gradients(self, model: ONNXModel) -> List[str]:
        """Every tensor input that is not skipped and every parameter that requires a gradient (module.py:333-346 of
        the reference), as far as the graph reads them - directly or through views (the slices of a packed weight)."""
        sdfg, state, params = model.sdfg, model.state, self._exported_parameters
        tensor_inputs = [n for n in model.inputs if n not in params]
        param_inputs = [n for n in model.inputs if n in params]
        buffers = {n for n, _ in self.model.named_buffers()}
        required = [n for n in tensor_inputs if n not in self.inputs_to_skip and
                    sdfg.arrays[clean_onnx_name(n)].dtype.is_floating_point]
        required += [n for n in param_inputs if n not in buffers and params[n].requires_grad]
        used = {e.data.data for e in state.edges()}
        for n in list(used):
            while sdfg.arrays[n].view_of is not None:
                n = sdfg.arrays[n].view_of
                used.add(n)
        return [n for n in required if clean_onnx_name(n) in used]

    def _initialize_sdfg(self, dummy_inputs: Sequence[torch.Tensor]):
        device = next((t.device for t in dummy_inputs if t.is_cuda), None)
        if device is None:
            device = next((p.device for p in self.model.parameters() if p.is_cuda), None)
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.model = self.model.to(device)
        dummy_inputs = tuple(t.to(device) for t in dummy_inputs)
        model = self._import(dummy_inputs)
        sdfg, state = model.sdfg, model.state
        params = self._exported_parameters
        tensor_inputs = [n for n in model.inputs if n not in params]
        param_inputs = [n for n in model.inputs if n in params]
        if len(tensor_inputs) != len(dummy_inputs):
            raise ValueError("the exported graph has %d tensor inputs %s, the module was called with %d" %
                             (len(tensor_inputs), tensor_inputs, len(dummy_inputs)))

        grads: Dict[str, str] = {}
        if self.backward:
            # differentiation works on contractions (as in the reference, where PureMatMul / PureGemm have expanded
            # to Einsum nodes before the backward pass is generated); a no-op after auto_optimize
            fusion.lower_matmul(sdfg)
            # gradients for every input that is not a buffer or skipped, and every parameter that requires one
            # (module.py:333-346)
            required = self._inputs_that_need_gradients(model)
            # a parameter's gradient has the parameter's type, as autograd expects it: the kernels sum over the batch
            # in fp32 and round once when they store (fp32 copies that autograd would get cast anyway cost one more
            # launch per parameter)
            grads = add_backward_pass(sdfg, state, list(model.outputs), [clean_onnx_name(n) for n in required])
            for hook in self.post_autodiff_hooks.values():
                hook(sdfg, sdfg)
        self.required_gradients = grads

        forward_states = [state.label]
        backward_states = [s.label for s in sdfg.states() if s.label != state.label]
        # transients share memory by lifetime (with debug_transients the intermediates are outputs, not transients);
        # those a backward call reads get fresh memory on every forward call (below) and need no place of their own
        expand_onnx_nodes(sdfg)
        outside = forwarded_transients(sdfg, forward_states, backward_states) if self.backward else []
        compiled = CompiledSDFG(sdfg, device=device, reuse_transients=True, outside_arena=outside)
        self.compiled = compiled
        for hook in self.post_compile_hooks.values():
            hook(compiled)

        in_arrays = [clean_onnx_name(n) for n in tensor_inputs + param_inputs]
        out_arrays = list(model.outputs)
        arglist = compiled.arglist()
        grad_of_input = [grads.get(a) for a in in_arrays]
        n_tensor = len(tensor_inputs)

        # what a backward call reads besides the gradients it is given: the tensors the forward call was bound to
        # and the SDFG's own buffers that the forward state fills for the backward state. Both are saved on the
        # autograd context (ctypes_module.py:150-170) - the former keep the memory behind the bound pointers alive,
        # the latter get fresh memory per forward call, so that any number of forward calls may be pending
        forwarded = compiled.forwarded_transients(forward_states, backward_states) if self.backward else []
        self.forwarded_transients = list(forwarded)

        def run_forward(tensors, keep=False):
            call = {}
            for name, t in zip(in_arrays, tensors):
                if name in arglist:
                    call[name] = t.detach().contiguous()
            outs = []
            for name in out_arrays:
                d = sdfg.arrays[name]
                t = torch.empty(d.shape, dtype=d.dtype, device=device)
                call[name] = t
                outs.append(t)
            compiled.bind(call)
            saved = {}
            if keep:
                for name in forwarded:
                    d = sdfg.arrays[name]
                    saved[name] = torch.empty(d.shape, dtype=d.dtype, device=device)
                compiled.rebind_transients(saved, release=True)
            compiled.launch(forward_states)
            return tuple(outs), call, saved

        class DifferentiableFunction(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *tensors):
                outs, call, saved = run_forward(tensors, keep=True)
                ctx.daceml_bound_names = list(call)
                ctx.daceml_saved_names = list(saved)
                ctx.save_for_backward(*call.values(), *saved.values())
                ctx.mark_non_differentiable(*[o for o in outs if not o.dtype.is_floating_point])
                return outs[0] if len(outs) == 1 else outs

            @staticmethod
            def backward(ctx, *grad_outputs):
                kept = ctx.saved_tensors
                nb = len(ctx.daceml_bound_names)
                call = dict(zip(ctx.daceml_bound_names, kept[:nb]))
                compiled.rebind_transients(dict(zip(ctx.daceml_saved_names, kept[nb:])))
                for name, g in zip(out_arrays, grad_outputs):
                    gname = "gradient_" + name
                    if gname not in arglist:
                        continue
                    d = sdfg.arrays[gname]
                    call[gname] = torch.zeros(d.shape, dtype=d.dtype, device=device) if g is None else \
                        g.to(d.dtype).contiguous()
                results = []
                for gname in grad_of_input:
                    if gname is None:
                        results.append(None)
                        continue
                    d = sdfg.arrays[gname]
                    t = torch.empty(d.shape, dtype=d.dtype, device=device)
                    call[gname] = t
                    results.append(t)
                compiled.bind(call)
                compiled.launch(backward_states)
                return tuple(None if r is None else r.to(sdfg.arrays[a].dtype) for r, a in zip(results, in_arrays))

        def function(*args):
            if len(args) != n_tensor:
                raise TypeError("%s takes %d tensors, got %d" % (self.sdfg_name, n_tensor, len(args)))
            tensors = tuple(args) + tuple(params[n] for n in param_inputs)
            if self.backward:
                return DifferentiableFunction.apply(*tensors)
            outs = run_forward(tensors)[0]
            return outs[0] if len(outs) == 1 else outs

        return function

    def forward(self, *actual_inputs):
        """Run the module; the first call traces it with these inputs (module.py:379-396)."""
        if self.function is None:
            self.function = self._initialize_sdfg(actual_inputs)
        return self.function(*actual_inputs)


def dace_module(moduleclass=None, dummy_inputs=None, cuda=None, training=False, backward=False,
                inputs_to_skip=None, onnx_simplify=True, simplify=True, auto_optimize=True, sdfg_name=None,
                compile_torch_extension=True, debug_transients=False):
    """Class decorator: instances of the decorated ``nn.Module`` class are created wrapped in a ``DaceModule``
    (daceml/torch/module.py:399-441)."""
    def wrap(cls):
        def make(*args, **kwargs):
            return DaceModule(cls(*args, **kwargs), dummy_inputs=dummy_inputs, cuda=cuda, training=training,
                              backward=backward, inputs_to_skip=inputs_to_skip, auto_optimize=auto_optimize,
                              sdfg_name=sdfg_name, debug_transients=debug_transients)
        make.__name__ = cls.__name__
        make.__doc__ = cls.__doc__
        return make

    if moduleclass is None:
        return wrap
    return wrap(moduleclass)


# names that say what the wrapper runs on
HipModule = DaceModule
hip_module = dace_module
