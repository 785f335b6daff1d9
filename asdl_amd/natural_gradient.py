"""K-FAC gradient maker on one GPU (behaviour of asdl/precondition/natural_gradient.py:28-128,
323-543, 859-900 for the Kronecker-factored shape).

Host-side differences from the reference, all result-preserving:
* the EMA pre-scale ``curv *= (1 - ema_decay)`` is folded into the factor kernels,
* inverses of all layers are taken in one batched pass with one host synchronisation,
* layer ownership across ranks (the reference's partitions) does not exist: one process, one GPU.
"""
import sys
from typing import Any, List, Union

import torch
import torch.distributed as dist
from torch import nn

from . import kernels
from .core import module_wise_assignments, modules_to_assign
from .fisher import FisherConfig, get_fisher_maker
from .grad_maker import LOSS_CROSS_ENTROPY
from .matrices import *
from .prec_grad_maker import PreconditionedGradientMaker, PreconditioningConfig
from .symmatrix import Kron, SymMatrix, UnitWise, batched_unit_update_inv, batched_update_inv

_invalid_ema_decay = -1
_module_level_shapes = [SHAPE_LAYER_WISE, SHAPE_KRON, SHAPE_SWIFT_KRON, SHAPE_KFE, SHAPE_UNIT_WISE, SHAPE_DIAG]
_kernel_shapes = [SHAPE_KRON, SHAPE_SWIFT_KRON, SHAPE_UNIT_WISE]
_norm_classes = (nn.BatchNorm1d, nn.BatchNorm2d, nn.LayerNorm)
PRECONDITION_STREAMS = 6      # side streams over which precondition() spreads the layers
OVERLAP_INVERSE_UPDATE = True           # EMA mode: update_preconditioner()'s inverses beside the loss backward pass
PREPARE_PRECONDITION_EARLY = True      # host side of precondition() while the device still works on the inverses
FLAGS_AFTER_PRECONDITION = True        # forward_and_backward(): the zero / not-positive-definite flags of the step's
                                       # inverses are read after the preconditioning has been enqueued instead of
                                       # before, so that the device has that work in its queue while the host waits and
                                       # prepares the next step.  What the caller sees is the reference's behaviour: a
                                       # factor that is not positive definite raises torch.linalg.LinAlgError from
                                       # this call, with the gradients as the backward pass left them (they are
                                       # saved before the preconditioning and put back); an all-zero factor without
                                       # an earlier inverse, for which the reference computes none, has the identity
                                       # while the gradients are preconditioned (its own gradient is zero, as its
                                       # inputs or output gradients are) and none afterwards.
GROUPED_PRECONDITION = True      # all Kronecker-factored modules in three launches instead of one stream-juggled chain per module

__all__ = ['NaturalGradientMaker', 'KfacGradientMaker']


def _bias_requires_grad(module):
    return hasattr(module, 'bias') and module.bias is not None and module.bias.requires_grad


class NaturalGradientMaker(PreconditionedGradientMaker):
    _supported_classes = (nn.Linear, nn.Conv2d, nn.BatchNorm1d, nn.BatchNorm2d, nn.LayerNorm, nn.Embedding)

    def __init__(self, model, config: PreconditioningConfig, fisher_type: str = FISHER_MC,
                 fisher_shape: Union[str, List[Any]] = SHAPE_KRON, loss_type: str = LOSS_CROSS_ENTROPY,
                 scale: float = 1, grad_scale: float = 1, n_mc_samples: int = 1, var: float = 1., seed: int = None):
        from torch.nn.parallel import DistributedDataParallel as DDP
        if isinstance(model, DDP):
            raise TypeError(f'{DDP} is not supported.')
        if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
            raise NotImplementedError('this build runs on one GPU: layer-partitioned preconditioning across ranks '
                                      'is not implemented')
        super().__init__(model, config)
        if isinstance(fisher_shape, str):
            fisher_shape = [fisher_shape]
        if not self.do_accumulate and config.curvature_upd_ratio is not None:
            raise ValueError('curvature_upd_ratio cannot be specified when no curvature accumulation is performed.')

        unsupported = [m for m in self.module_dict.values() if not isinstance(m, (nn.Linear, nn.Conv2d) + _norm_classes)]
        if unsupported:
            kinds = sorted({type(m).__name__ for m in unsupported})
            raise NotImplementedError(
                f'{kinds} modules have no kernels in this build (Linear / Conv2d: Kronecker-factored, BatchNorm / '
                f'LayerNorm: unit-wise). Pass PreconditioningConfig(ignore_modules=[...]) to leave them '
                f'un-preconditioned.')

        self.named_modules_for_curvature = []
        self.modules_for_curvature = []
        self.shape_for = {}
        for name, module, shapes in module_wise_assignments(self.module_dict, *fisher_shape, named=True):
            if len(shapes) != 1:
                raise ValueError(f'Each module has to be assigned one Fisher shape. '
                                 f'{name} is assigned {len(shapes)} shapes.')
            if shapes[0] not in _kernel_shapes:
                raise NotImplementedError(f'Fisher shape "{shapes[0]}" (module {name}) is not on this path.')
            if shapes[0] == SHAPE_UNIT_WISE and not isinstance(module, _norm_classes):
                raise NotImplementedError(f'the unit-wise shape is built for BatchNorm / LayerNorm only (module {name}).')
            self.modules_for_curvature.append(module)
            self.named_modules_for_curvature.append((name, module))
            self.shape_for[module] = shapes[0]
            self.shape_for[name] = shapes[0]
        self._named_modules_for = {}

        fisher_config = FisherConfig(fisher_type=fisher_type, fisher_shapes=fisher_shape, loss_type=loss_type,
                                     n_mc_samples=n_mc_samples, ignore_modules=config.ignore_modules, var=var,
                                     seed=seed)
        self.fisher_maker = get_fisher_maker(model, fisher_config)
        self.fisher_type = fisher_type
        self.fisher_shape = fisher_shape
        self.scale = scale
        self.grad_scale = grad_scale
        self.world_rank = 0
        self.world_size = 1

    def do_forward_and_backward(self, step=None):
        return not self.do_update_curvature(step)

    def named_modules_for(self, shape):
        if shape not in self._named_modules_for:
            self._named_modules_for[shape] = list(modules_to_assign(self.model, shape, *self.fisher_shape,
                                                                    ignore_modules=self.config.ignore_modules,
                                                                    named=True))
        return self._named_modules_for[shape]

    def modules_for(self, shape):
        return [m for _, m in self.named_modules_for(shape)]

    @property
    def late_inverse_flags(self):
        """fisher.LATE_INVERSE_FLAGS for this maker: the flags of an inverse update are read by the next one."""
        return self.fisher_maker.late_inverse_flags

    @late_inverse_flags.setter
    def late_inverse_flags(self, value):
        self.fisher_maker.late_inverse_flags = bool(value)

    def check_late_flags(self):
        """Reads the flags that late_inverse_flags left unread (after the last step, before a checkpoint)."""
        self.fisher_maker.check_late_flags()

    @property
    def _fisher_attr(self):
        return self.fisher_maker.config.fisher_attr

    def _get_module_fisher(self, module):
        return getattr(module, self._fisher_attr, None)

    def _get_module_symmatrix(self, module, shape):
        fisher = self._get_module_fisher(module)
        if fisher is None:
            return None
        if shape in [SHAPE_KRON, SHAPE_SWIFT_KRON]:
            return fisher.kron
        if shape == SHAPE_UNIT_WISE:
            return fisher.unit
        raise ValueError(f'Invalid shape: {shape}.')

    @property
    def do_accumulate(self):
        return self.config.ema_decay != _invalid_ema_decay

    _STATE_TENSORS = (('kron', 'A'), ('kron', 'B'), ('kron', 'A_inv'), ('kron', 'B_inv'), ('unit', 'data'), ('unit', 'inv'))

    def state_dict(self) -> dict:
        """``step`` as in the reference (asdl/precondition/prec_grad_maker.py:129-133) plus, under ``curvature``, the
        curvature state itself so that a resumed run continues where it stopped: per module name a dict
        ``'<kron|unit>.<attribute>' -> tensor`` holding the Kronecker factors A, B (kept in EMA mode only; without EMA
        they live in scratch memory and only the inverses exist), their inverses A_inv, B_inv, and the unit-wise
        blocks and their inverses.  Tensors are clones on the device they live on.  Flags of the last inverse update
        that late_inverse_flags left unread are read first: a checkpoint never holds unchecked inverses."""
        self.check_late_flags()
        state = dict(self.state)
        curvature = {}
        for shape in _kernel_shapes:
            for name, module in self.named_modules_for(shape):
                fisher = self._get_module_fisher(module)
                if fisher is None:
                    continue
                entry = curvature.setdefault(name, {})
                for part, attr in self._STATE_TENSORS:
                    holder = getattr(fisher, part, None)
                    tensor = getattr(holder, attr, None) if holder is not None else None
                    if isinstance(tensor, torch.Tensor):
                        entry[f'{part}.{attr}'] = tensor.detach().clone()
        state['curvature'] = {name: entry for name, entry in curvature.items() if entry}
        return state

    def load_state_dict(self, state_dict: dict):
        """Restores ``step`` and, when present, the curvature state written by state_dict() (a reference-style
        ``{'step': n}`` loads as before).  Factors and inverses are moved to the model's device; modules missing from
        the model raise KeyError."""
        self.state['step'] = state_dict['step']
        curvature = state_dict.get('curvature')
        if curvature is None:
            return
        named = {}
        for shape in _kernel_shapes:
            for name, module in self.named_modules_for(shape):
                named[name] = module
        for name, entry in curvature.items():
            if name not in named:
                raise KeyError(f'the saved curvature names module {name!r}, which this model does not have')
            module = named[name]
            device = next(module.parameters()).device
            fisher = self._get_module_fisher(module)
            if fisher is None:
                fisher = SymMatrix()
                setattr(module, self._fisher_attr, fisher)
            for key, tensor in entry.items():
                part, attr = key.split('.')
                if (part, attr) not in self._STATE_TENSORS:
                    raise KeyError(f'unknown curvature entry {key!r} of module {name!r}')
                holder = getattr(fisher, part, None)
                if holder is None:
                    holder = Kron(A=None, B=None) if part == 'kron' else UnitWise()
                    setattr(fisher, part, holder)
                setattr(holder, attr, tensor.detach().to(device=device, dtype=torch.float32).clone().contiguous())
                if part == 'kron':
                    holder._A_dim = holder._B_dim = None
        self._precond_plan = None

    def update_curvature(self):
        config = self.config
        scale = self.scale
        prescale = 1.0
        ema_decay = config.ema_decay
        if ema_decay != _invalid_ema_decay:
            scale *= ema_decay
            prescale = 1 - ema_decay          # applied to the old factors inside the factor kernels
        self.fisher_maker.before_inverse_wait = self.prepare_precondition if PREPARE_PRECONDITION_EARLY else None
        self.fisher_maker.after_factors = self._update_preconditioner_early \
            if getattr(self, '_inverse_update_follows', False) else None
        try:
            self.delegate_forward_and_backward(self.fisher_maker, data_size=config.data_size, scale=scale,
                                               accumulate=self.do_accumulate, calc_loss_grad=True,
                                               calc_inv=not self.do_accumulate, damping=config.damping,
                                               accumulate_prescale=prescale)
        finally:
            self.fisher_maker.before_inverse_wait = None
            self.fisher_maker.after_factors = None

    def forward_and_backward(self):
        """The template of the base class.  With accumulated (EMA) factors the inverses are a step of their own,
        update_preconditioner(); when that step follows update_curvature() in this very call, its Kronecker part is
        enqueued as soon as the factors are final, beside the loss backward pass, instead of after it."""
        step = self.state['step']
        self._inverse_update_follows = bool(
            OVERLAP_INVERSE_UPDATE and self.do_accumulate and self.do_update_curvature(step)
            and self.do_update_preconditioner(step))
        self._kron_inverses_current = False
        # precondition() follows in this very call: it may read the flags of the inverses once it has launched
        self.fisher_maker.flags_to_caller = bool(FLAGS_AFTER_PRECONDITION)
        try:
            return super().forward_and_backward()
        finally:
            self._inverse_update_follows = False
            self._kron_inverses_current = False
            self.fisher_maker.flags_to_caller = False
            unread = self.fisher_maker.take_caller_flags()
            if unread and sys.exc_info()[0] is None:
                for late in unread:          # no stage read them (precondition() was replaced, say)
                    late.check(when=None)

    def _curvature_matrices(self, module_name=None):
        matrices, units = [], []
        for shape in _kernel_shapes:
            for name, module in self.named_modules_for(shape):
                if module_name is not None and name != module_name:
                    continue
                if module not in self.modules_for_curvature:
                    continue
                matrix = self._get_module_symmatrix(module, shape)
                if matrix is not None:
                    (units if shape == SHAPE_UNIT_WISE else matrices).append(matrix)
        return matrices, units

    def _update_preconditioner_early(self):
        """The Kronecker part of update_preconditioner() with its default arguments, enqueued only: returns the
        pending inverses (finish() reads their flags).  GPU factors only."""
        matrices, _ = self._curvature_matrices()
        if not matrices or not all(k.has_A and k.has_B and k.A.is_cuda for k in matrices):
            return None
        pending = batched_update_inv(matrices, self.config.damping, defer=True)
        self._kron_inverses_current = pending is not None
        return pending

    def update_preconditioner(self, damping=None, module_name=None, kron=None, zero_curvature=False):
        if not self.do_accumulate:
            return
        if kron is None:
            kron = ['A', 'B']
        if damping is None:
            damping = self.config.damping
        matrices, units = self._curvature_matrices(module_name)
        if getattr(self, '_kron_inverses_current', False) and module_name is None and not zero_curvature \
                and set(kron) == {'A', 'B'} and damping == self.config.damping:
            matrices = []        # already inverted beside the loss backward pass of this call
            self._kron_inverses_current = False
        batched_update_inv(matrices, damping, calc_A_inv='A' in kron, calc_B_inv='B' in kron)
        batched_unit_update_inv(units, damping)
        if zero_curvature:
            for unit in units:
                unit.mul_(0)
        if zero_curvature:
            with torch.no_grad():
                for matrix in matrices:
                    if 'A' in kron:
                        matrix.A.mul_(0)
                    if 'B' in kron:
                        matrix.B.mul_(0)

    def precondition(self, vectors=None, grad_scale=None, use_inv=True):
        if vectors is not None:
            raise NotImplementedError('precondition(vectors=...) is not on this path')
        if grad_scale is None:
            grad_scale = self.grad_scale
        work = self._precondition_work()
        unread = self.fisher_maker.take_caller_flags()
        if not unread:
            self._precondition_launch(work, grad_scale, use_inv)
            return
        # FLAGS_AFTER_PRECONDITION: launch on inverses whose flags are still on the device, then read them
        grads = [g for m, _ in work for g in (getattr(getattr(m, 'weight', None), 'grad', None),
                                              getattr(getattr(m, 'bias', None), 'grad', None)) if g is not None]
        saved = self._save_gradients(grads)
        self._precondition_launch(work, grad_scale, use_inv)
        try:
            for late in unread:
                late.check(when=None)
        except torch.linalg.LinAlgError:
            if grads:
                torch._foreach_copy_(grads, saved)      # as the reference leaves them when its Cholesky raises
            raise

    def _save_gradients(self, grads):
        """Copies of ``grads`` in one reusable buffer (one launch per dtype and device).  The views into the buffer
        depend on the gradients' shapes, types and devices only and are kept from step to step."""
        if not grads:
            return []
        key = tuple((g.shape, g.dtype, g.device) for g in grads)
        memo = getattr(self, '_grad_backup_views', None)
        if memo is None or memo[0] != key:
            buffers = getattr(self, '_grad_backup', None)
            if buffers is None:
                buffers = self._grad_backup = {}
            need = {}
            for g in grads:
                k = (g.dtype, g.device)
                need[k] = need.get(k, 0) + g.numel()
            for k, n in need.items():
                if k not in buffers or buffers[k].numel() < n:
                    buffers[k] = torch.empty(n, dtype=k[0], device=k[1])
            used = dict.fromkeys(need, 0)
            views = []
            for g in grads:
                k = (g.dtype, g.device)
                views.append(buffers[k][used[k]:used[k] + g.numel()].view(g.shape))
                used[k] += g.numel()
            memo = self._grad_backup_views = (key, views)
        views = memo[1]
        torch._foreach_copy_(views, grads)
        return views

    def _precondition_launch(self, work, grad_scale, use_inv):
        if use_inv and GROUPED_PRECONDITION:
            work = self._precondition_grouped(work, grad_scale)
        grads = [m.weight.grad for m, _ in work if getattr(m, 'weight', None) is not None and m.weight.grad is not None]
        if len(work) < 4 or not grads or not grads[0].is_cuda:
            for module, shape in work:
                self._precondition_module(module, shape, grad_scale=grad_scale, use_inv=use_inv)
            return
        # The layers are independent and most of their GEMMs are too small to fill the device: spread them
        # over the side streams (largest first) and join.  Everything they touch is waited for before returning.
        from .symmatrix import _side_streams
        dev = grads[0].device
        main = torch.cuda.current_stream(dev)
        side = _side_streams(dev, PRECONDITION_STREAMS)
        start = torch.cuda.Event()
        start.record(main)
        work.sort(key=lambda mw: -(mw[0].weight.numel() * (mw[0].weight.shape[0] + mw[0].weight[0].numel())))
        for st in side:
            st.wait_event(start)
        for i, (module, shape) in enumerate(work):
            with torch.cuda.stream(side[i % len(side)]):
                self._precondition_module(module, shape, grad_scale=grad_scale, use_inv=use_inv)
        for st in side:
            done = torch.cuda.Event()
            done.record(st)
            main.wait_event(done)

    def _precondition_work(self):
        return [(module, shape) for shape in _kernel_shapes for module in self.modules_for(shape)
                if module in self.modules_for_curvature]

    def _plan_grouped(self, work, grad_scale):
        """Collects every Kronecker-factored module whose operands the grouped kernels take into one
        kernels.KronPrecondPlan (B_inv G for every module, (.) A_inv for every module, B_inv bias: a handful of
        launches, same arithmetic per module as Kron.mvp(use_inv=True, inplace=True)).  Returns
        (plan, rest of ``work`` for the per-module path, signature) or None when no module qualifies;
        the signature lists the objects the plan was built from."""
        items, unit_items, rest, signature = [], [], [], []
        for module, shape in work:
            kron = self._get_module_symmatrix(module, shape) if shape in (SHAPE_KRON, SHAPE_SWIFT_KRON) else None
            weight = getattr(module, 'weight', None)
            item = None
            if shape == SHAPE_UNIT_WISE and weight is not None and weight.requires_grad and _bias_requires_grad(module):
                unit = self._get_module_symmatrix(module, shape)
                gw, gb = weight.grad, module.bias.grad
                if unit is not None and unit.has_inv and gw is not None and gb is not None and \
                        all(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() for t in (unit.inv, gw, gb)) \
                        and unit.inv.ndim == 3 and tuple(unit.inv.shape[1:]) == (2, 2) \
                        and gw.numel() == gb.numel() == unit.inv.shape[0]:
                    unit_items.append((unit.inv, gw.data.view(-1), gb.data.view(-1)))
                    signature.append((module, shape, unit, unit.inv, None, gw, gb))
                    continue
            if kron is not None and kron.has_inv and weight is not None and weight.requires_grad \
                    and weight.grad is not None:
                grad_b = None
                has_bias = _bias_requires_grad(module)
                if has_bias:
                    grad_b = module.bias.grad
                if not has_bias or grad_b is not None:
                    if kernels.kron_precond_groupable(kron.B_inv, kron.A_inv, weight.grad, grad_b):
                        item = (kron.B_inv, kron.A_inv, weight.grad.data, None if grad_b is None else grad_b.data)
                        signature.append((module, shape, kron, kron.A_inv, kron.B_inv, weight.grad, grad_b))
            if item is None:
                rest.append((module, shape))
            else:
                items.append(item)
        if len(items) + len(unit_items) < (1 if kernels.HALF_PIECE_PRECONDITION else 2):
            return None      # (a single module still gains from the grouped form's fp16-piece products)
        return kernels.KronPrecondPlan(items, grad_scale, unit_items), rest, signature

    def prepare_precondition(self):
        """Does the host side of the coming precondition() ahead of time.  update_curvature() has this called
        after the loss backward pass is enqueued and before the host waits for the inverses' flags, i.e. while the
        device is busy: when the wait returns, precondition() only has to launch.  precondition() checks that the
        plan still describes the current inverses and gradients and builds a new one if not."""
        self._precond_plan = None
        if not GROUPED_PRECONDITION:
            return
        work = self._precondition_work()
        planned = self._plan_grouped(work, self.grad_scale)
        if planned is not None:
            self._precond_plan = (planned, [m for m, _ in work])

    def _take_plan(self, work, grad_scale):
        """The plan of prepare_precondition() if it still holds (same modules, inverses and gradient tensors)."""
        prepared, self._precond_plan = getattr(self, '_precond_plan', None), None
        if prepared is None:
            return None
        (plan, rest, signature), modules = prepared
        if plan.grad_scale != float(grad_scale) or len(modules) != len(work) or \
                any(m is not w for m, (w, _) in zip(modules, work)):
            return None
        for module, shape, matrix, A_inv, B_inv, grad_w, grad_b in signature:
            if self._get_module_symmatrix(module, shape) is not matrix or module.weight.grad is not grad_w or \
                    (grad_b is not None and module.bias.grad is not grad_b):
                return None
            if shape == SHAPE_UNIT_WISE:
                if matrix.inv is not A_inv:
                    return None
            elif matrix.A_inv is not A_inv or matrix.B_inv is not B_inv:
                return None
        return plan, rest, signature

    def _precondition_grouped(self, work, grad_scale):
        """Preconditions the modules the grouped kernels take and returns the rest of ``work``."""
        planned = self._take_plan(work, grad_scale) or self._plan_grouped(work, grad_scale)
        if planned is None:
            return work
        plan, rest, _ = planned
        plan.launch()
        return rest

    def _precondition_module(self, module, shape=None, vectors=None, vec_weight=None, vec_bias=None,
                             grad_scale=None, use_inv=True):
        if grad_scale is None:
            grad_scale = self.grad_scale
        if shape is None:
            shape = self.shape_for.get(module)
        if shape is None:
            raise ValueError(f'No shape is assigned to module: {module}.')
        matrix = self._get_module_symmatrix(module, shape)
        if matrix is None:
            raise ValueError(f'Matrix of shape {shape} for module {module} has not been calculated.')
        if vec_weight is None and module.weight.requires_grad:
            vec_weight = module.weight.grad
        if vec_weight is None:
            raise ValueError(f'weight gradient for module {module} has not been calculated.')
        if _bias_requires_grad(module):
            if vec_bias is None:
                vec_bias = module.bias.grad
            if vec_bias is None:
                raise ValueError(f'bias gradient for module {module} has not been calculated.')
        if grad_scale != 1:
            vec_weight.data.mul_(grad_scale)
            if vec_bias is not None:
                vec_bias.data.mul_(grad_scale)
        if not use_inv or matrix.has_inv:
            matrix.mvp(vec_weight=vec_weight, vec_bias=vec_bias, use_inv=use_inv, inplace=True)


class KfacGradientMaker(NaturalGradientMaker):
    """K-FAC (https://arxiv.org/abs/1503.05671) behind the GradientMaker interface; same constructor
    arguments as asdl/precondition/natural_gradient.py:883-900.

    BatchNorm1d/2d and LayerNorm modules get the unit-wise shape, as in the reference; ``swift=True`` keeps the
    factors of layers that see fewer samples than they have columns as row matrices (SKFAC).  Embedding modules
    have no kernels in this build (exclude them through ``config.ignore_modules``)."""

    def __init__(self, model, config: PreconditioningConfig, fisher_type: str = FISHER_MC,
                 loss_type: str = LOSS_CROSS_ENTROPY, scale: float = 1, grad_scale: float = 1, n_mc_samples: int = 1,
                 var: float = 1., seed: int = None, swift=False):
        fisher_shape = [SHAPE_SWIFT_KRON if swift else SHAPE_KRON, (nn.BatchNorm1d, SHAPE_UNIT_WISE), (nn.BatchNorm2d, SHAPE_UNIT_WISE),
                        (nn.LayerNorm, SHAPE_UNIT_WISE)]
        super().__init__(model, config, fisher_type=fisher_type, fisher_shape=fisher_shape, loss_type=loss_type,
                         scale=scale, grad_scale=grad_scale, n_mc_samples=n_mc_samples, var=var, seed=seed)
