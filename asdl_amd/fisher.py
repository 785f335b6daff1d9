"""FisherMaker: forward, (sampled / exact / empirical) backward under the hooks, and extraction of
``module.fisher`` (behaviour of asdl/fisher.py:29-205, 419-521 for the Kronecker-factored shape)."""
from dataclasses import dataclass
from typing import Any, List, Tuple, Union

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from .core import no_centered_cov
from .grad_maker import GradientMaker, LOSS_CROSS_ENTROPY, LOSS_MSE
from .profiling import nvtx_range, phase_mark
from .matrices import *
from .operations import OperationContext
from .symmatrix import SymMatrix, batched_unit_update_inv, batched_update_inv
from .utils import skip_param_grad

__all__ = ['FisherConfig', 'get_fisher_maker', 'FisherMaker']

_supported_types = [FISHER_EXACT, FISHER_MC, FISHER_EMP]
_invalid_data_size = -1
GROUPED_FACTORS = True     # the Kronecker factors of a forward + backward pass in one grouped launch (kernels.FactorGroup) instead of one launch per factor
GROUP_FLUSH_EVERY = (-2, 0)  # (forward, backward): launch the group after that many hooks of the pass (0: once, when the pass
                             # has ended; -1: that pass launches its factors one by one; -2: it launches its unfolded
                             # factors one by one and leaves its plain X^T X factors to the group).  The forward pass of
                             # the benchmark sits at the balance of the host's launch rate and the device, so most of its
                             # factor kernels cost nothing where they are, and the grouped plain factors take half the
                             # time of their single launches; the backward pass is bound by the device (ResNet-50 batch
                             # 64 in one process: 26.9 ms per step with single launches, 27.4 with (0, 0), 26.3 with
                             # (-1, 0), 26.0 with (-2, 0))
FACTOR_SIDE_STREAM = False  # statistics kernels of the hooks on a side stream (ordering the two streams costs ~30 us of host time per hook: more than the overlap gains)
PRUNED_FISHER_BACKWARD = True   # sampled / exact Fisher passes skip the weight-gradient kernels (their results are never used)
LATE_INVERSE_FLAGS = False  # Read the zero / not-positive-definite flags of an update with calc_loss_grad only when the next
                            # update reaches the same point (FisherMaker.late_inverse_flags; check_late_flags() after
                            # the last one) instead of waiting for them before the preconditioning is enqueued: the
                            # host then never waits for the device inside a step and prepares the next step while the
                            # device finishes this one.  The price is the reference's error behaviour: a factor
                            # that is not positive definite raises torch.linalg.LinAlgError one update late, and an
                            # all-zero factor, whose inverse the reference skips, preconditions with the identity
                            # until then.  Off by default; bench.py switches it on and says so.
EAGER_INVERSE = True        # start the bulk of the inverses during a single sampled / empirical backward pass: the longest chains get a head start
EAGER_INVERSE_SAMPLED = False   # ... also when a loss backward pass follows the sampled one.  That pass hides the
                                # inverses anyway, and one grouped inverse for all factors after the sampled pass is
                                # faster than an early batch plus a remainder (ResNet-50 batch 64: 27.55 against
                                # 27.96-28.50 ms per step in one process)


@dataclass
class FisherConfig:
    fisher_type: str
    fisher_shapes: List[Any]
    loss_type: str = None
    n_mc_samples: int = 1
    var: float = 1.
    seed: int = None
    fisher_attr: str = 'fisher'
    fvp_attr: str = 'fvp'
    ignore_modules: List[Any] = None
    data_size: int = _invalid_data_size
    scale: float = 1.
    is_distributed: bool = False
    all_reduce: bool = False
    is_master: bool = True
    ignore_index: int = -1


class FisherMaker(GradientMaker):
    _loss_reduction = 'sum'

    def __init__(self, model, config):
        super().__init__(model)
        self.config: FisherConfig = config
        self.late_inverse_flags = LATE_INVERSE_FLAGS
        self._late_flags = []
        self.flags_to_caller = False         # set by a caller that enqueues work between the inverses and their flags
                                             # (the preconditioning) and then reads them itself: take_caller_flags()
        self._caller_flags = None
        self.before_inverse_wait = None      # optional callable, run right before the host waits for the inverses
        self.after_factors = None            # optional callable, run when the factors are final and before the loss
                                             # backward pass is enqueued; may return an object with finish()

    def check_late_flags(self):
        """Reads the flags of the last update whose flags were left unread (late_inverse_flags) and raises
        torch.linalg.LinAlgError for a factor that was not positive definite.  Called by the next update; call it
        after the last one."""
        pending, self._late_flags = self._late_flags, []
        for late in pending:
            late.check()

    def take_caller_flags(self):
        """The unread flags of this call's inverses (flags_to_caller), as a list of objects with check(); None when
        they have been read already."""
        pending, self._caller_flags = self._caller_flags, None
        return pending

    def zero_fisher(self, fvp=False):
        attr = self.config.fvp_attr if fvp else self.config.fisher_attr
        for module in self.model.modules():
            module.__dict__.pop(attr, None)      # a plain attribute: set by setattr(module, attr, SymMatrix)

    def _factor_stream(self):
        """Where the statistics kernels of the hooks go, one object per maker: a group that launches the factors of
        the whole pass together (GROUPED_FACTORS), a side stream of default priority (FACTOR_SIDE_STREAM), or None
        for one launch per factor on the caller's stream."""
        if not (GROUPED_FACTORS or FACTOR_SIDE_STREAM) or not torch.cuda.is_available():
            return None
        p = next(self.model.parameters(), None)
        if p is None or not p.is_cuda:
            return None
        from .kernels import DeferredFactors, FactorStream
        kind = DeferredFactors if GROUPED_FACTORS else FactorStream
        fs = getattr(self, '_factor_stream_obj', None)
        if type(fs) is not kind or fs.device != p.device:
            fs = kind(p.device)
            self._factor_stream_obj = fs
        if GROUPED_FACTORS:
            fs.every = GROUP_FLUSH_EVERY
        return fs

    @property
    def single_backward_pass(self):
        """True when _fisher_loop (or the empirical-Fisher backward) runs exactly one backward pass."""
        return self.is_fisher_emp or (self.config.fisher_type == FISHER_MC and self.config.n_mc_samples == 1)

    @property
    def is_fisher_emp(self):
        return False

    @property
    def do_local_accumulate(self) -> bool:
        raise NotImplementedError

    def forward_and_backward(self, data_size=_invalid_data_size, scale=None, accumulate=False, calc_loss_grad=False,
                             calc_inv=False, fvp=False, damping=None, vec=None,
                             accumulate_prescale=1.0) -> Union[Tuple[Any, Tensor], Any]:
        """Same arguments as asdl/fisher.py:69-77 plus ``accumulate_prescale``: with accumulate=True
        the existing factors are multiplied by it inside the kernel that adds the new statistic
        (the EMA decay), instead of in a separate pass beforehand."""
        if accumulate and calc_inv:
            raise ValueError('accumulate and calc_inv cannot be True at the same time.')
        if fvp:
            raise NotImplementedError('Fisher-vector products are not on this path')
        model = self.model
        config = self.config
        fisher_shapes = config.fisher_shapes
        if isinstance(fisher_shapes, str):
            fisher_shapes = [fisher_shapes]
        if data_size == _invalid_data_size:
            data_size = config.data_size
        if data_size == _invalid_data_size:
            raise ValueError('data_size is not specified.')
        if scale is None:
            scale = config.scale
        scale /= data_size

        if not accumulate:
            self.zero_fisher()
        if config.seed is not None:
            torch.random.manual_seed(config.seed)

        loss_grad_with_fisher = calc_loss_grad and self.is_fisher_emp
        loss_grad_after_fisher = calc_loss_grad and not self.is_fisher_emp
        inv_with_fisher = calc_inv and not self.do_local_accumulate
        inv_after_fisher = calc_inv and self.do_local_accumulate

        with no_centered_cov(model, fisher_shapes, ignore_modules=config.ignore_modules,
                             calc_inv=inv_with_fisher, factor_stream=self._factor_stream()) as cxt:
            if accumulate:
                self._register_fisher(cxt, accumulate_prescale)
            if damping is not None:
                cxt.set_damping(damping)
            cxt.set_cov_scale(scale)
            if inv_with_fisher and self.single_backward_pass and EAGER_INVERSE and \
                    (EAGER_INVERSE_SAMPLED or not loss_grad_after_fisher):
                # every B factor is final when its hook has run: the bulk of the inverses may start behind
                # the backward pass that is still producing the others
                cxt.set_eager_inverse(getattr(self, '_inverse_cost_prev', 0))

            with nvtx_range('fwd'):
                self.call_model()
                loss = None
                if self.is_fisher_emp or calc_loss_grad:
                    self.call_loss()
                    loss = self._loss
            phase_mark('fwd')             # forward pass with the cov_kron_A kernels of its hooks

            def closure(nll_expr, retain_graph=False):
                keep = retain_graph or loss_grad_after_fisher
                if loss_grad_with_fisher or not PRUNED_FISHER_BACKWARD or not cxt.grad_edges:
                    with skip_param_grad(model, disable=loss_grad_with_fisher):
                        nll_expr().backward(retain_graph=keep)
                else:
                    # No parameter takes a gradient from this pass: differentiate with respect to the
                    # hooked module outputs only.  Every hook fires as in a full pass; the autograd
                    # engine leaves out the weight-gradient kernels, whose results would be dropped, and
                    # accumulates into no .grad, so the parameters' requires_grad flags stay as they are.
                    torch.autograd.grad(nll_expr(), list(cxt.grad_edges), retain_graph=keep, allow_unused=True)

            with nvtx_range('bwd'):
                if self.is_fisher_emp:
                    closure(lambda: loss)
                else:
                    self._fisher_loop(closure)
            cxt.join_factor_stream()
            phase_mark('bwd_fisher')      # backward pass that feeds the cov_kron_B kernels (early inverses run beside it)
            cxt.finish_registered()
            # The inverses only need the factors: enqueue them now (side streams) and, when a loss backward
            # pass follows, let that pass run on the main stream meanwhile; the flags are read afterwards.
            deferred = cxt.flush_inverses(defer=loss_grad_after_fisher or self.flags_to_caller)
            self._inverse_cost_prev = cxt.inverse_cost
            self._extract_fisher(cxt)

        if inv_after_fisher:
            self.replace_fisher_with_inv(damping)
        early = None
        if loss_grad_after_fisher:
            if self.after_factors is not None:
                early = self.after_factors()     # e.g. the caller's inverse update, enqueued beside the pass below
            with nvtx_range('bwd'):
                loss.backward()
        if calc_loss_grad:
            # the loss was summed over the batch: divide gradients and loss by the data size (enqueued before the
            # host waits for the inverse flags, so that nothing is left to launch between that wait and the caller)
            grads = [p.grad for p in model.parameters() if p.grad is not None]
            if grads:
                torch._foreach_div_(grads, data_size)     # one launch for all parameters
            loss.div_(data_size)
        phase_mark('bwd_loss')            # loss backward pass (the inverses run beside it on side streams)
        if deferred is not None or early is not None:
            if self.before_inverse_wait is not None:
                self.before_inverse_wait()      # host work of the caller that needs no flags: the device is still busy
            if deferred is not None:
                self.check_late_flags()         # of the previous update: read long ago by the device's clock
                to_caller = self.flags_to_caller and not self.late_inverse_flags
                late = deferred.finish_late(config.fisher_attr, warn=self.late_inverse_flags) if (self.late_inverse_flags or to_caller) else None
                if late is None:
                    deferred.finish(config.fisher_attr)
                elif to_caller:
                    self._caller_flags = late
                else:
                    self._late_flags = late
            if early is not None:
                early.finish()
        phase_mark('upd_inv')             # what is left of the inverses once the loss backward pass has ended
        return self._model_output, loss

    def _register_fisher(self, cxt: OperationContext, prescale=1.0):
        attr = self.config.fisher_attr
        for module in self.model.modules():
            fisher = getattr(module, attr, None)
            if fisher is not None and cxt.is_operation_registered(module):
                cxt.register_symmatrix(module, fisher, first_beta=prescale)

    def _extract_fisher(self, cxt: OperationContext):
        attr = self.config.fisher_attr
        for module in cxt.registered_modules():       # (in the order of model.modules(), which registered them)
            if getattr(module, attr, None) is None:
                fisher = cxt.cov_symmatrix(module, pop=True)
                if fisher is not None:
                    setattr(module, attr, fisher)

    def replace_fisher_with_inv(self, damping):
        attr = self.config.fisher_attr
        krons, units = [], []
        for module in self.model.modules():
            fisher: SymMatrix = getattr(module, attr, None)
            if fisher is not None and fisher.has_kron:
                krons.append(fisher.kron)
            if fisher is not None and fisher.has_unit:
                units.append(fisher.unit)
        batched_unit_update_inv(units, damping, replace=True)
        batched_update_inv(krons, damping=damping, replace=True)

    def _fisher_loop(self, closure):
        raise NotImplementedError

    def get_fisher_tensor(self, module: nn.Module, *keys) -> Union[torch.Tensor, None]:
        data = getattr(module, self.config.fisher_attr, None)
        if data is None:
            return None
        for key in keys:
            data = getattr(data, key, None)
        if data is not None and not isinstance(data, torch.Tensor):
            raise TypeError(f'data have to be {torch.Tensor}, got {type(data)}.')
        return data


class FisherExactCrossEntropy(FisherMaker):
    """asdl/fisher.py:419-440."""

    @property
    def do_local_accumulate(self) -> bool:
        if self._logits is not None:
            return self._logits.shape[-1] > 1
        return True

    def _fisher_loop(self, closure):
        logits = self._logits
        log_probs = F.log_softmax(logits, dim=-1)
        log_probs = log_probs.view(-1, log_probs.size(-1))
        n, n_classes = log_probs.shape
        with torch.no_grad():
            sqrt_probs = torch.sqrt(F.softmax(logits, dim=-1)).view(n, n_classes)
        for i in range(n_classes):
            targets = torch.full((n,), i, device=logits.device, dtype=torch.long)

            def nll_expr():
                nll = F.nll_loss(log_probs, targets, reduction='none', ignore_index=self.config.ignore_index)
                return nll.mul(sqrt_probs[:, i]).sum()
            closure(nll_expr, retain_graph=i < n_classes - 1)


class FisherMCCrossEntropy(FisherMaker):
    """asdl/fisher.py:443-459."""

    @property
    def do_local_accumulate(self) -> bool:
        return self.config.n_mc_samples > 1

    def _fisher_loop(self, closure):
        logits = self._logits
        n_mc_samples = self.config.n_mc_samples
        probs = F.softmax(logits, dim=-1)
        log_probs = F.log_softmax(logits, dim=-1)
        # validate_args=False: the check of the simplex constraint would synchronise the host with the forward
        # pass; the draw itself (normalisation + multinomial) is unchanged
        dist = torch.distributions.Categorical(probs, validate_args=False)
        for i in range(n_mc_samples):
            with torch.no_grad():
                targets = self.sample_targets(dist, i)
            closure(lambda: F.nll_loss(log_probs.view(-1, log_probs.size(-1)), targets.view(-1), reduction='sum',
                                       ignore_index=self.config.ignore_index) / n_mc_samples,
                    retain_graph=i < n_mc_samples - 1)

    def sample_targets(self, dist, i):
        """One draw of the model's predictive distribution; override to replay fixed targets."""
        return dist.sample()


class FisherExactMSE(FisherMaker):
    """asdl/fisher.py:462-473."""

    @property
    def do_local_accumulate(self) -> bool:
        if self._logits is not None:
            return self._logits.shape[-1] > 1
        return True

    def _fisher_loop(self, closure):
        logits = self._logits
        n_dims = logits.size(-1)
        for i in range(n_dims):
            closure(lambda: logits[:, i].sum(), retain_graph=i < n_dims - 1)


class FisherMCMSE(FisherMaker):
    """asdl/fisher.py:476-490."""

    @property
    def do_local_accumulate(self) -> bool:
        return self.config.n_mc_samples > 1

    def _fisher_loop(self, closure):
        logits = self._logits
        n_mc_samples = self.config.n_mc_samples
        dist = torch.distributions.normal.Normal(logits, scale=np.sqrt(self.config.var), validate_args=False)
        for i in range(n_mc_samples):
            with torch.no_grad():
                targets = dist.sample()
            closure(lambda: 0.5 * F.mse_loss(logits, targets, reduction='sum') / n_mc_samples,
                    retain_graph=i < n_mc_samples - 1)


class FisherEmp(FisherMaker):
    """asdl/fisher.py:493-500."""

    @property
    def do_local_accumulate(self) -> bool:
        return False

    @property
    def is_fisher_emp(self):
        return True


def get_fisher_maker(model: nn.Module, config: FisherConfig):
    fisher_type = config.fisher_type
    loss_type = config.loss_type
    if fisher_type not in _supported_types:
        raise ValueError(f'Invalid fisher_type: {fisher_type}. {_supported_types} are supported.')
    if fisher_type == FISHER_EMP:
        return FisherEmp(model, config)
    if loss_type not in [LOSS_CROSS_ENTROPY, LOSS_MSE]:
        raise ValueError(f'Invalid loss_type: {loss_type}. {[LOSS_CROSS_ENTROPY, LOSS_MSE]} are supported.')
    if fisher_type == FISHER_EXACT:
        return FisherExactCrossEntropy(model, config) if loss_type == LOSS_CROSS_ENTROPY else FisherExactMSE(model, config)
    return FisherMCCrossEntropy(model, config) if loss_type == LOSS_CROSS_ENTROPY else FisherMCMSE(model, config)
