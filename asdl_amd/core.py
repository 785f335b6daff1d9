"""Hook engine: the ``extend`` context attaches one Operation per supported leaf module and calls
it from a forward hook and from a hook on the gradient of the module's output
(role of asdl/core.py:20-97, 130-244)."""
import sys
from contextlib import contextmanager, nullcontext

import torch
import torch.nn as nn
from torch.autograd.graph import GradientEdge

from .matrices import *
from .operations import *
from .operations import FWD_OPS, BWD_OPS, BWD_OPS_WITH_INPUTS
from .utils import record_original_requires_grad

_supported_module_classes = (nn.Linear, nn.Conv2d, nn.BatchNorm1d, nn.BatchNorm2d, nn.LayerNorm)

__all__ = ['extend', 'no_centered_cov', 'module_wise_assignments', 'modules_to_assign']


def _model_fingerprint(model):
    """What the module-wise assignments depend on: the module tree (identities, in order) and, for every supported
    leaf, the identities and requires_grad flags of its weight and bias.  ~50 us for a ResNet-50."""
    ids, flags = [], []
    stack = [model]
    while stack:
        m = stack.pop()
        ids.append(id(m))
        if isinstance(m, _supported_module_classes):
            params = m._parameters
            w, b = params.get('weight'), params.get('bias')
            flags.append((id(w), w is not None and w.requires_grad, id(b), b is not None and b.requires_grad))
        children = m._modules
        if children:
            stack.extend(c for c in reversed(children.values()) if c is not None)
    return tuple(ids), tuple(flags)


def _assignment_plan(model, op_names, ignore_modules, map_rule, plan_key):
    """[(module, op names, operation class)] of extend().  With a ``plan_key`` (a hashable that stands for map_rule)
    the list of the previous call with the same arguments is reused as long as the model's fingerprint is the same:
    walking the modules by name and applying the rules costs ten times the fingerprint, once per step."""
    def build():
        plan = []
        for module, names in module_wise_assignments(model, *op_names, ignore_modules=ignore_modules, map_rule=map_rule):
            if len(names) == 0:
                continue
            op_class = get_op_class(module)
            if op_class is None:
                continue
            plan.append((module, [n for n in names if n in op_class.supported_operations], op_class))
        return plan

    if plan_key is None:
        return build()
    try:
        key = (plan_key, tuple(op_names), tuple(m if isinstance(m, (str, type)) else id(m) for m in ignore_modules or ()))
        hash(key)
    except TypeError:
        return build()
    cache = model.__dict__.setdefault('_asdl_amd_assignment_plans', {})
    fingerprint = _model_fingerprint(model)
    hit = cache.get(key)
    if hit is not None and hit[0] == fingerprint:
        return hit[1]
    plan = build()
    cache[key] = (fingerprint, plan)
    return plan


@contextmanager
def extend(model, *op_names, ignore_modules=None, map_rule=None, vectors=None, stream=None,
           factor_stream=None, plan_key=None) -> OperationContext:
    """``stream``: as in the reference, the hook operations run under ``torch.cuda.stream(stream)``.
    ``factor_stream``: a kernels.FactorStream; the hook operations launch on its side stream, ordered after the
    kernels that produced their inputs, so that the statistics kernels overlap the forward / backward kernels that
    follow; OperationContext.join_factor_stream() orders the consumers after them.
    ``plan_key``: see _assignment_plan (callers whose map_rule is a fixed function of the key)."""
    handles = []
    cxt = OperationContext(vectors=vectors)
    use_stream = torch.cuda.is_available() and stream is not None
    cxt.factor_stream = factor_stream if torch.cuda.is_available() else None

    def stream_cxt():
        return torch.cuda.stream(stream) if use_stream else nullcontext()

    def run_hook(fn, *tensors, backward=False):
        fs = cxt.factor_stream
        if fs is None or not tensors[0].is_cuda:
            with stream_cxt():
                fn()
            return
        fs.run(fn, *tensors, backward=backward)

    try:
        for module, names, op_class in _assignment_plan(model, op_names, ignore_modules, map_rule, plan_key):
            op = op_class(module, list(names), model_for_kernel=model)
            cxt.register_operation(module, op)
            has_fwd = any(n in FWD_OPS for n in names)
            has_bwd = any(n in BWD_OPS for n in names)
            if not (has_fwd or has_bwd):
                continue

            # only the stored outputs and the unit-wise statistics look at the module's output
            needs_out = OP_SAVE_OUTPUTS in names or any(n in BWD_OPS_WITH_INPUTS for n in names)

            def forward_hook(_module, in_data, out_data, _has_bwd=has_bwd, _needs_out=needs_out, _op=op):
                x = in_data[0].detach()
                y = out_data.detach() if _needs_out else None
                run_hook(lambda: _op.forward_post_process(x, y), x)
                if _has_bwd and out_data.requires_grad:
                    def grad_hook(grad, _m=_module):
                        if not cxt.is_operation_registered(_m):
                            return None          # context already closed
                        g = grad.detach()
                        run_hook(lambda: _op.backward_pre_process(g, None), g, backward=True)
                        return None
                    handles.append(out_data.register_hook(grad_hook))
                    # the graph edge the hook sits on: a backward pass restricted to these edges still fires
                    # every hook, without the weight-gradient kernels of the layers
                    cxt.grad_edges.append(GradientEdge(out_data.grad_fn, out_data.output_nr))
            handles.append(module.register_forward_hook(forward_hook))
        handles.append(model.register_forward_pre_hook(lambda *_: cxt.grad_edges.clear()))
        if not cxt.is_operation_registered(model):
            cxt.register_operation(model, Operation(model, []))
        yield cxt
    finally:
        for handle in handles:
            handle.remove()
        cxt.clear_operations()
        if hasattr(cxt.factor_stream, 'discard'):
            # factor calls that were recorded but not launched yet: dropped if the pass ended in an exception,
            # launched otherwise (the consumers above all call join_factor_stream() themselves)
            if sys.exc_info()[0] is not None:
                cxt.factor_stream.discard()
            else:
                cxt.factor_stream.join()


def no_centered_cov(model: nn.Module, shapes, ignore_modules=None, cvp=False, vectors=None, stream=None,
                    calc_inv=False, factor_stream=None) -> OperationContext:
    """Maps Fisher shapes to operations (asdl/core.py:83-97): the Kronecker-factored, swift Kronecker-factored and
    unit-wise shapes have kernels here."""
    if cvp:
        raise NotImplementedError('covariance-vector products are not on this path')

    def map_rule(shape):
        if shape == SHAPE_KRON:
            return OP_COV_KRON_INV if calc_inv else OP_COV_KRON
        if shape == SHAPE_SWIFT_KRON:
            return OP_COV_SWIFT_KRON_INV if calc_inv else OP_COV_SWIFT_KRON
        if shape == SHAPE_UNIT_WISE:
            return OP_COV_UNIT_WISE_INV if calc_inv else OP_COV_UNIT_WISE
        raise NotImplementedError(
            f'Fisher shape "{shape}" has no MI355X kernel in this build; only "{SHAPE_KRON}", "{SHAPE_SWIFT_KRON}" and '
            f'"{SHAPE_UNIT_WISE}" are supported. '
            'Exclude such modules with PreconditioningConfig(ignore_modules=[...]).')
    return extend(model, *shapes, ignore_modules=ignore_modules, map_rule=map_rule, vectors=vectors, stream=stream,
                  factor_stream=factor_stream, plan_key=('no_centered_cov', bool(calc_inv)))


def named_supported_modules(model):
    for name, module in model.named_modules():
        if isinstance(module, _supported_module_classes):
            yield name, module


def module_wise_assignments(model, *assign_rules, ignore_modules=None, map_rule=None, named=False):
    """Yields (name,) module, [values] following the rule priorities of asdl/core.py:130-244:
    module instance > name substring > module class > the bare string rules."""
    if any(not isinstance(rule, (str, tuple)) for rule in assign_rules):
        raise TypeError(f'every assign rule has to be {str} or {tuple}.')
    ignore_modules = [] if ignore_modules is None else ignore_modules
    if map_rule is None:
        def map_rule(x):
            return x

    common, specified = [], {}
    for rule in assign_rules:
        if isinstance(rule, str):
            common.append(rule)
            continue
        if len(rule) < 2:
            raise ValueError(f'Tuple length has to be >= 2. Given: {rule}.')
        key, values = rule[0], rule[1:]
        if any(not isinstance(v, str) for v in values):
            raise TypeError(f'All values have to be {str}. Given: {values}.')
        if key in specified:
            raise ValueError(f'({key}, _) is already assigned.')
        specified[key] = list(values)

    ignored_ids = {id(m) for m in ignore_modules if isinstance(m, nn.Module)}
    ignored_classes = tuple(cls for cls in ignore_modules if isinstance(cls, type))
    ignored_keywords = [keyword for keyword in ignore_modules if isinstance(keyword, str)]
    name_rules = [key for key in specified if isinstance(key, str)]
    for name, module in named_supported_modules(model):
        if id(module) in ignored_ids or isinstance(module, ignored_classes):
            continue
        if ignored_keywords and any(keyword in name for keyword in ignored_keywords):
            continue
        requires_grad = False
        for attr in ['weight', 'bias']:
            param = getattr(module, attr, None)
            if param is not None:
                requires_grad = requires_grad or param.requires_grad
                record_original_requires_grad(param)
        if not requires_grad:
            continue
        info = (name, module) if named else (module,)
        if module in specified:
            values = specified[module]
        elif name_rules and any(key in name for key in name_rules):
            values = specified[next(key for key in name_rules if key in name)]
        elif module.__class__ in specified:
            values = specified[module.__class__]
        else:
            if len(common) == 0:
                continue
            values = common
        yield (*info, [map_rule(v) for v in values])


def modules_to_assign(model, value, *assign_rules, ignore_modules=None, named=False):
    for info in module_wise_assignments(model, *assign_rules, ignore_modules=ignore_modules, named=named):
        if value in info[-1]:
            yield (info[0], info[1]) if named else info[0]
