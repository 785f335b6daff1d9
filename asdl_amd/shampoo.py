"""Shampoo gradient maker on one GPU (behaviour of asdl/precondition/shampoo.py:21-56, 201-223,
300-367, 465-586, without block partitioning and without the layer-partitioned exchange).

MI355X-first host layout: every statistic of one size n (and one root exponent p) lives in a single
[count, n, n] tensor, so that the inverse roots of all of them are taken by one batched call whose
convergence tests run on the device; Preconditioner.statistics / .preconditioners hold views into
these groups.
"""
from collections import defaultdict

import torch
import torch.distributed as dist

from . import kernels
from .prec_grad_maker import PreconditionedGradientMaker, PreconditioningConfig

__all__ = ['ShampooGradientMaker', 'Preconditioner', 'compute_power']

_invalid = -1


def compute_power(mat_g, p, iter_count=100, error_tolerance=1e-6, ridge_epsilon=1e-6, start_vector=None):
    """(mat_g + r I)^(-1/p), r = ridge_epsilon * lambda_max; mat_g keeps the ridge
    (asdl/precondition/shampoo.py:465-528).  ``start_vector`` replaces the U(-1, 1) draw of the power
    iteration."""
    if mat_g.ndim == 1:
        return torch.pow(mat_g + ridge_epsilon, -1 / p)
    n = mat_g.shape[0]
    if n == 1:
        return torch.eye(1, device=mat_g.device)
    if start_vector is None:
        start_vector = torch.rand(n, device=mat_g.device) * 2 - 1
    out, _ = kernels.inv_root_newton(mat_g, p, ridge_epsilon, start_vector, max_iter=iter_count,
                                     tol=error_tolerance)
    return out


class Preconditioner:
    """Statistics and preconditioners of one parameter (asdl/precondition/shampoo.py:300-367)."""

    def __init__(self, param, config: PreconditioningConfig, statistics, preconditioners, inverse_exponent=_invalid):
        if param.ndim <= 1:
            raise ValueError(f'len(self._transformed_shape) has to be > 1. Got {param.ndim}.')
        self.config = config
        self.param = param
        self.statistics = statistics            # views into the per-size groups
        self.preconditioners = preconditioners
        self.inverse_exponent = inverse_exponent

    @property
    def exponent(self):
        return 2 * self.param.ndim if self.inverse_exponent == _invalid else self.inverse_exponent

    def update_statistics(self):
        grad = self.param.grad
        if grad.dtype != torch.float32:
            raise TypeError('Shampoo statistics are float32: keep parameters (and so their gradients) in float32')
        ema_decay = self.config.ema_decay
        alpha, beta = (1.0, 1.0) if ema_decay == _invalid else (float(ema_decay), 1.0 - float(ema_decay))
        ndim = grad.ndim
        for i in range(ndim):
            stat = self.statistics[i]
            if i == ndim - 1:
                kernels.syrk_tn(grad.reshape(-1, grad.shape[-1]), out=stat, alpha=alpha, beta=beta)
            elif i == 0:
                kernels.syrk_nt(grad.reshape(grad.shape[0], -1), out=stat, alpha=alpha, beta=beta)
            else:
                kernels.syrk_nt(grad.movedim(i, 0).reshape(grad.shape[i], -1).contiguous(), out=stat, alpha=alpha, beta=beta)

    def precondition(self):
        grad = self.param.grad
        cur = grad.detach()
        for j in range(grad.ndim):
            x2d = cur.reshape(cur.shape[0], -1)
            cur = kernels.gemm(x2d, self.preconditioners[j], transA=True).view(*cur.shape[1:], cur.shape[0])
        self.param.grad.data.copy_(cur.reshape(self.param.shape))


class ShampooGradientMaker(PreconditionedGradientMaker):
    """Shampoo (https://arxiv.org/abs/1802.09568) behind the GradientMaker interface; constructor of
    asdl/precondition/shampoo.py:34-35.  ``block_size`` other than -1 is not supported (the reference
    never forwards it to its Preconditioner either)."""

    def __init__(self, model: torch.nn.Module, config: PreconditioningConfig, block_size: int = _invalid,
                 sync_group=None, init_scale: float = 1e-12):
        super().__init__(model, config)
        if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
            raise NotImplementedError('this build runs on one GPU')
        if block_size != _invalid:
            raise NotImplementedError('block partitioning is not on this path')
        self.sync_group = sync_group
        self.block_size = block_size
        self.world_rank, self.world_size = 0, 1
        params = [p for p in model.parameters() if p.ndim > 1 and p.requires_grad]
        for p in params:
            if not p.is_cuda:
                raise RuntimeError('asdl_amd kernels run on a ROCm device only; move the model to the GPU first. '
                                   'There is no CPU fallback.')
        slots = defaultdict(list)      # (n, exponent) -> [(param index, axis)]
        for pi, p in enumerate(params):
            for axis, n in enumerate(p.shape):
                slots[(n, 2 * p.ndim)].append((pi, axis))
        self._groups = {}
        views = {}
        for (n, exp), members in slots.items():
            dev = params[members[0][0]].device
            eye = torch.eye(n, device=dev)
            stats = (init_scale * eye).repeat(len(members), 1, 1).contiguous()
            precs = eye.repeat(len(members), 1, 1).contiguous()
            self._groups[(n, exp)] = (stats, precs)
            for k, (pi, axis) in enumerate(members):
                views[(pi, axis)] = (stats[k], precs[k])
        self.preconditioners = []
        for pi, p in enumerate(params):
            self.preconditioners.append(Preconditioner(p, config, [views[(pi, a)][0] for a in range(p.ndim)],
                                                       [views[(pi, a)][1] for a in range(p.ndim)]))
        self.start_vector_fn = None     # optional: (count, n, device) -> [count, n] start vectors
        self.last_root_stats = {}

    def do_forward_and_backward(self, step=None):
        return True

    def update_curvature(self):
        for preconditioner in self.preconditioners:
            preconditioner.update_statistics()

    def update_preconditioner(self):
        """All inverse roots of one size in one batched call (per matrix:
        asdl/precondition/shampoo.py:341-349)."""
        damping = self.config.damping
        for (n, exp), (stats, precs) in self._groups.items():
            if n == 1:
                continue                 # ComputePower returns the identity for 1 x 1 input
            count = stats.shape[0]
            if self.start_vector_fn is not None:
                v0 = self.start_vector_fn(count, n, stats.device)
            else:
                v0 = torch.rand(count, n, device=stats.device) * 2 - 1
            _, st = kernels.inv_root_newton(stats, exp, damping, v0, out=precs)
            self.last_root_stats[(n, exp)] = st

    def precondition(self):
        for preconditioner in self.preconditioners:
            preconditioner.precondition()
