"""Shampoo gradient maker on one GPU (behaviour of asdl/precondition/shampoo.py:21-56, 201-223,
300-367, 465-586, without block partitioning and without the layer-partitioned exchange).

MI355X-first host layout: every statistic of one size n (and one root exponent p) lives in a single
[count, n, n] tensor, so that the inverse roots of all of them are taken by one batched call whose
convergence tests run on the device; Preconditioner.statistics / .preconditioners hold views into
these groups.
"""
import itertools
from collections import defaultdict

import torch
import torch.distributed as dist

from . import kernels
from .prec_grad_maker import PreconditionedGradientMaker, PreconditioningConfig

__all__ = ['ShampooGradientMaker', 'Preconditioner', 'BlockPartitioner', 'compute_power']

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


def _merge_small_dims(shape_to_merge, max_dim):
    """Collapses runs of neighbouring dimensions whose product stays within ``max_dim``
    (asdl/precondition/shampoo.py:370-395): [1, 2, 512, 1, 2048, 1, 3, 4] -> [1024, 2048, 12] for max_dim 1024."""
    merged, run = [], 1
    for d in shape_to_merge:
        if run * d <= max_dim:
            run *= d
            continue
        if run > 1:
            merged.append(run)
        run = d
    if run > 1:
        merged.append(run)
    return merged


class BlockPartitioner:
    """Cuts a tensor into blocks of at most ``block_size`` along every axis that is longer than that
    (asdl/precondition/shampoo.py:398-462).  Blocks are ordered with the first axis slowest; each block has one
    square statistic per axis."""

    def __init__(self, shape, block_size=_invalid):
        self._shape = tuple(shape)
        self._ranges = []          # per axis: [(start, stop), ...]
        for d in self._shape:
            if block_size != _invalid and d > block_size:
                starts = list(range(0, d, block_size))
                self._ranges.append([(a, min(a + block_size, d)) for a in starts])
            else:
                self._ranges.append([(0, d)])
        self._blocks = list(itertools.product(*self._ranges))      # one tuple of (start, stop) per block

    def kronecker_factor_shapes(self):
        return [[b - a, b - a] for block in self._blocks for a, b in block]

    def num_splits(self):
        """Statistics per block (= number of axes)."""
        return len(self._shape)

    def partition(self, tensor):
        if tuple(tensor.shape) != self._shape:
            raise ValueError(f'tensor shape ({tensor.shape}) does not match self._shape ({self._shape}).')
        return [tensor[tuple(slice(a, b) for a, b in block)] for block in self._blocks]

    def merge_partitions(self, partitions):
        if len(partitions) != len(self._blocks):
            raise ValueError(f'len(partitions) has to be {len(self._blocks)}. Got {len(partitions)}.')
        out = torch.empty(self._shape, dtype=partitions[0].dtype, device=partitions[0].device)
        for block, part in zip(self._blocks, partitions):
            out[tuple(slice(a, b) for a, b in block)] = part
        return out


def _axis_statistic(grad, axis, out, alpha, beta):
    """out <- beta*out + alpha * (grad contracted with itself over every axis but ``axis``)."""
    ndim = grad.ndim
    if axis == ndim - 1:
        kernels.syrk_tn(grad.reshape(-1, grad.shape[-1]), out=out, alpha=alpha, beta=beta)
    elif axis == 0:
        kernels.syrk_nt(grad.reshape(grad.shape[0], -1), out=out, alpha=alpha, beta=beta)
    else:
        kernels.syrk_nt(grad.movedim(axis, 0).reshape(grad.shape[axis], -1).contiguous(), out=out, alpha=alpha, beta=beta)


HALF_PIECE_STATISTICS = True      # the grouped statistics on two fp16 pieces per element instead of true fp32 products,
                                  # summed in chunks of 256 k (the leading products in an accumulator of their own that
                                  # joins a running total): 5.9 -> 1.9 ms per step on the GPT-2-small stack, relative
                                  # error 2.7e-7 (fp32 products: 4.1e-7).  What the matrix instructions' accumulation
                                  # leaves the diagonal low: 1-5 % of a ridge of 1e-6 lambda_max (fp32 products:
                                  # 0.3-1 %; one accumulator for the whole sum: 2-3 % at 2304 columns and up, 10 % at 768)
HALF_PIECE_PRECONDITION = True     # grouped preconditioning on two fp16 pieces per element (kernels.KronPrecondPlan does the same)
GROUPED_PRECONDITION = True      # matrix-shaped parameters: all their preconditioning products in two launches
GROUPED_STATISTIC_MIN_DIM = 768   # statistics of this size and up go into one grouped launch (with GROUPED_PRECONDITION)


def _precondition_block(grad, preconditioners):
    """tensordot(grad, P_j, [[0], [0]]) for every axis in turn (asdl/precondition/shampoo.py:358-364)."""
    cur = grad
    for j in range(grad.ndim):
        x2d = cur.reshape(cur.shape[0], -1)
        cur = kernels.gemm(x2d, preconditioners[j], transA=True).view(*cur.shape[1:], cur.shape[0])
    return cur


class Preconditioner:
    """Statistics and preconditioners of one parameter; constructor arguments of
    asdl/precondition/shampoo.py:300-323.  ``statistics`` / ``preconditioners`` (keyword only) let
    ShampooGradientMaker hand in views into its per-size groups, whose roots it takes in batched calls."""

    def __init__(self, param, config: PreconditioningConfig, block_size: int = _invalid, inverse_exponent: int = _invalid,
                 best_effort_shape_interpretation: bool = False, init_scale: float = 1e-12, *, statistics=None,
                 preconditioners=None):
        self.config = config
        self.param = param
        self._transformed_shape = tuple(param.shape)
        if best_effort_shape_interpretation:
            self._transformed_shape = tuple(_merge_small_dims(param.shape, block_size))
        if len(self._transformed_shape) <= 1:
            raise ValueError(f'len(self._transformed_shape) has to be > 1. Got {len(self._transformed_shape)}.')
        if not param.is_cuda:
            raise RuntimeError('asdl_amd kernels run on a ROCm device only; move the model to the GPU first. '
                               'There is no CPU fallback.')
        self._partitioner = BlockPartitioner(self._transformed_shape, block_size)
        shapes = self._partitioner.kronecker_factor_shapes()
        if statistics is None:
            statistics = [init_scale * torch.eye(s[0], device=param.device) for s in shapes]
            preconditioners = [torch.eye(s[0], device=param.device) for s in shapes]
        if len(statistics) != len(shapes) or len(preconditioners) != len(shapes):
            raise ValueError(f'{len(shapes)} statistics and preconditioners are needed.')
        self.statistics = statistics
        self.preconditioners = preconditioners
        self.inverse_exponent = inverse_exponent
        self.start_vector_fn = None     # optional: n -> [n] start vector of the power iteration

    @property
    def exponent(self):
        return 2 * len(self._transformed_shape) if self.inverse_exponent == _invalid else self.inverse_exponent

    def _blocks_of_grad(self):
        grad = self.param.grad
        if grad.dtype != torch.float32:
            raise TypeError('Shampoo statistics are float32: keep parameters (and so their gradients) in float32')
        return self._partitioner.partition(grad.detach().reshape(self._transformed_shape))

    def update_statistics(self, skip_axes=()):
        """``skip_axes``: axes whose statistic the caller has updated itself (the gradient maker's grouped launch)."""
        ema_decay = self.config.ema_decay
        alpha, beta = (1.0, 1.0) if ema_decay == _invalid else (float(ema_decay), 1.0 - float(ema_decay))
        ndim = len(self._transformed_shape)
        for j, block in enumerate(self._blocks_of_grad()):
            block = block if block.is_contiguous() else block.contiguous()
            for i in range(ndim):
                if i not in skip_axes:
                    _axis_statistic(block, i, self.statistics[j * ndim + i], alpha, beta)

    def update_preconditioners(self):
        """L^(-1/exponent) of every statistic, one at a time (asdl/precondition/shampoo.py:341-349); the gradient
        maker takes the roots of its grouped statistics in batched calls instead."""
        for i, stat in enumerate(self.statistics):
            v0 = self.start_vector_fn(stat.shape[0]) if self.start_vector_fn is not None else None
            root = compute_power(stat, self.exponent, ridge_epsilon=self.config.damping, start_vector=v0)
            if isinstance(self.preconditioners[i], torch.Tensor) and self.preconditioners[i].shape == root.shape:
                self.preconditioners[i].copy_(root)
            else:
                self.preconditioners[i] = root

    def precondition(self):
        ndim = len(self._transformed_shape)
        out = []
        for j, block in enumerate(self._blocks_of_grad()):
            block = block if block.is_contiguous() else block.contiguous()
            out.append(_precondition_block(block, self.preconditioners[j * ndim:(j + 1) * ndim]))
        merged = out[0] if len(out) == 1 else self._partitioner.merge_partitions(out)
        self.param.grad.data.copy_(merged.reshape(self.param.shape))


class ShampooGradientMaker(PreconditionedGradientMaker):
    """Shampoo (https://arxiv.org/abs/1802.09568) behind the GradientMaker interface; constructor of
    asdl/precondition/shampoo.py:34-35.  As in the reference, ``block_size`` is kept but not forwarded to the
    Preconditioner objects (asdl/precondition/shampoo.py:53): there it only enters the cost model of the multi-GPU layer
    assignment.  Preconditioner itself takes ``block_size`` / ``best_effort_shape_interpretation``."""

    def __init__(self, model: torch.nn.Module, config: PreconditioningConfig, block_size: int = _invalid,
                 sync_group=None, init_scale: float = 1e-12):
        super().__init__(model, config)
        if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
            raise NotImplementedError('this build runs on one GPU')
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
            self.preconditioners.append(Preconditioner(p, config, statistics=[views[(pi, a)][0] for a in range(p.ndim)],
                                                       preconditioners=[views[(pi, a)][1] for a in range(p.ndim)]))
        self.start_vector_fn = None     # optional: (count, n, device) -> [count, n] start vectors
        self.last_root_stats = {}

    def state_dict(self) -> dict:
        """``step`` as in the reference (asdl/precondition/prec_grad_maker.py:129-133) plus, under ``shampoo``, the
        statistics and inverse roots of every preconditioned parameter (in the order of model.parameters()): a list of
        ``{'shape': parameter shape, 'statistics': [tensor per axis], 'preconditioners': [tensor per axis]}``."""
        state = dict(self.state)
        state['shampoo'] = [dict(shape=tuple(pc.param.shape),
                                 statistics=[s.detach().clone() for s in pc.statistics],
                                 preconditioners=[q.detach().clone() for q in pc.preconditioners])
                            for pc in self.preconditioners]
        return state

    def load_state_dict(self, state_dict: dict):
        """Restores ``step`` and, when present, the statistics and roots written by state_dict(), in place (the
        per-size group tensors the batched root update works on keep their storage)."""
        self.state['step'] = state_dict['step']
        saved = state_dict.get('shampoo')
        if saved is None:
            return
        if len(saved) != len(self.preconditioners):
            raise ValueError(f'the saved state holds {len(saved)} parameters, this model has {len(self.preconditioners)}')
        with torch.no_grad():
            for pc, entry in zip(self.preconditioners, saved):
                if tuple(entry['shape']) != tuple(pc.param.shape):
                    raise ValueError(f'saved parameter shape {tuple(entry["shape"])} != {tuple(pc.param.shape)}')
                for mine, theirs in ((pc.statistics, entry['statistics']), (pc.preconditioners, entry['preconditioners'])):
                    if len(mine) != len(theirs):
                        raise ValueError('saved state and model disagree on the number of Kronecker factors')
                    for dst, src in zip(mine, theirs):
                        dst.copy_(src)

    def do_forward_and_backward(self, step=None):
        return True

    @staticmethod
    def _groupable(pc):
        """A matrix-shaped, unpartitioned parameter whose gradient, statistics and preconditioners the grouped
        split-bf16 GEMM takes (float32, dense, 16-byte aligned, sizes multiples of 4)."""
        grad = pc.param.grad
        shape = pc._transformed_shape
        if grad is None or len(shape) != 2 or tuple(grad.shape) != shape or grad.dtype != torch.float32 \
                or not grad.is_contiguous() or shape[0] % 4 or shape[1] % 4 or grad.data_ptr() % 16:
            return False
        for mats in (pc.statistics, pc.preconditioners):
            if len(mats) != 2:
                return False
            for q, n in zip(mats, shape):
                if not isinstance(q, torch.Tensor) or tuple(q.shape) != (n, n) or not q.is_contiguous() \
                        or q.dtype != torch.float32 or q.data_ptr() % 16:
                    return False
        return True

    def _split_groupable(self):
        if not GROUPED_PRECONDITION:
            return [], list(self.preconditioners)
        grouped = [pc for pc in self.preconditioners if self._groupable(pc)]
        if len(grouped) < 2:
            return [], list(self.preconditioners)
        taken = set(map(id, grouped))
        return grouped, [pc for pc in self.preconditioners if id(pc) not in taken]

    def update_curvature(self):
        """Statistics of every axis (asdl/precondition/shampoo.py:331-339).  The large ones of matrix-shaped
        parameters (GROUPED_STATISTIC_MIN_DIM and up), G G^T or G^T G, run in one grouped launch (lower tiles, mirrored:
        exactly symmetric; the EMA folded into alpha / beta): on two fp16 pieces per element with the gradient's range
        measured by one pass and sums in chunks (HALF_PIECE_STATISTICS), else with true fp32 products.  Small statistics stay on the fp32
        SYRK kernels, one at a time: the inverse roots of small, ill-conditioned statistics magnify what a different
        summation order changes in the last bits, and the golden runs of the reference pin those."""
        grouped, _ = self._split_groupable()
        done = {}
        if grouped:
            ema_decay = self.config.ema_decay
            alpha, beta = (1.0, 1.0) if ema_decay == _invalid else (float(ema_decay), 1.0 - float(ema_decay))
            specs = []
            half = HALF_PIECE_STATISTICS
            dev = grouped[0].param.device
            if half:
                mx = torch.zeros(len(grouped), dtype=torch.float32, device=dev)
                vectors = []
            for i, pc in enumerate(grouped):
                m, n = pc._transformed_shape
                g = pc.param.grad.data_ptr()
                w = mx.data_ptr() + 4 * i if half else 0
                axes = []
                if m >= GROUPED_STATISTIC_MIN_DIM:
                    specs.append((g, n, g, n, pc.statistics[0].data_ptr(), m, m, m, n, 0, 1, alpha, beta, True, w, w, 0))
                    axes.append(0)
                if n >= GROUPED_STATISTIC_MIN_DIM:
                    specs.append((g, n, g, n, pc.statistics[1].data_ptr(), n, n, n, m, 1, 0, alpha, beta, True, w, w, 0))
                    axes.append(1)
                if half and axes:
                    vectors.append((g, m * n, 1, w))
                done[id(pc)] = tuple(axes)
            if specs:
                if half:
                    kernels.absmax_grouped(vectors, dev)
                kernels.gemm_grouped_raw(specs, dev, pieces=23 if half else 0)
        for preconditioner in self.preconditioners:
            preconditioner.update_statistics(skip_axes=done.get(id(preconditioner), ()))

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
        """P_0^T G P_1 for every matrix-shaped parameter in two grouped launches (all G^T P_0, then all (.)^T P_1:
        the per-axis tensordot chain of asdl/precondition/shampoo.py:351-367, on the split-bf16 kernel with all 24
        mantissa bits); parameters with more axes, blocks or unaligned sizes go one at a time."""
        specs_first, specs_second, off = [], [], 0
        grouped, rest = self._split_groupable()
        if grouped:
            dev = grouped[0].param.device
            buf, _ = kernels.workspace(4 * sum(pc.param.numel() for pc in grouped), dev)
            base = buf.data_ptr()
            half = HALF_PIECE_PRECONDITION
            if half:
                # operand ranges for the fp16 pieces: the roots are symmetric positive definite (largest magnitude on
                # the diagonal), the gradients are measured, the intermediate by the first product's epilogue
                mx = torch.zeros(len(grouped), 4, dtype=torch.float32, device=dev)
                vectors = []
            for i, pc in enumerate(grouped):
                m, n = pc._transformed_shape
                g, t = pc.param.grad.data_ptr(), base + 4 * off
                off += m * n
                p0, p1 = pc.preconditioners[0].data_ptr(), pc.preconditioners[1].data_ptr()
                # T[n, m] = G^T P_0, then G[m, n] <- T^T P_1
                first, second = (g, n, p0, m, t, m, n, m, m, 1, 0, 1.0), (t, m, p1, n, g, n, m, n, n, 1, 0, 1.0)
                if half:
                    w = mx.data_ptr() + 16 * i
                    vectors += [(g, m * n, 1, w), (p0, m, m + 1, w + 4), (p1, n, n + 1, w + 8)]
                    first += (0.0, False, w, w + 4, w + 12)
                    second += (0.0, False, w + 12, w + 8, 0)
                specs_first.append(first)
                specs_second.append(second)
            if half:
                kernels.absmax_grouped(vectors, dev)
            kernels.gemm_grouped_raw(specs_first, dev, pieces=22 if half else 3)
            kernels.gemm_grouped_raw(specs_second, dev, pieces=22 if half else 3)
        for preconditioner in rest:
            preconditioner.precondition()
