"""Per-layer operations of the K-FAC path and the context that stores their results.

Mirrors the operator seam of the reference (asdl/operations/operation.py:87-548 for Operation,
:551-964 for OperationContext, asdl/operations/linear.py, conv.py, batchnorm.py and layernorm.py for the layer
classes) for the operations on this path: OP_COV_KRON(_INV), OP_COV_SWIFT_KRON(_INV) and OP_COV_UNIT_WISE(_INV).
Differences that come from running on the GPU kernels:

* cov_kron_A / cov_kron_B take optional ``out``, ``alpha``, ``beta`` and compute
  ``out <- beta*out + alpha*factor`` in one launch, so the reference's separate
  ``.mul_(cov_scale)``, ``results[key] += value`` and EMA pre-scale passes disappear.
* Conv2d.preprocess_in_data returns a lazy UnfoldedInput; the unfold happens inside the kernel.
* With OP_COV_KRON_INV the inverses are not taken inside the backward hook: the context queues the
  (A, B) pairs and inverts them all in one batched pass (OperationContext.flush_inverses).
"""
import warnings
from typing import Dict

import torch
import torch.nn as nn

from . import kernels
from . import profiling as _profiling
from .profiling import nvtx_range
from .symmatrix import Kron, SymMatrix, UnitWise, batched_update_inv
from .utils import UnfoldedInput, im2col_2d, original_requires_grad

OP_COV_KRON = 'cov_kron'
OP_COV_KRON_INV = 'cov_kron_inv'
OP_COV_SWIFT_KRON = 'cov_swift_kron'            # Kronecker factors kept as n x d row matrices where n < d (SKFAC)
OP_COV_SWIFT_KRON_INV = 'cov_swift_kron_inv'
OP_COV_UNIT_WISE = 'cov_unit_wise'
OP_COV_UNIT_WISE_INV = 'cov_unit_wise_inv'
OP_SAVE_INPUTS = 'save_inputs'
OP_SAVE_OUTPUTS = 'save_outputs'
OP_SAVE_OUTGRADS = 'save_outgrads'

ALL_OPS = [OP_COV_KRON, OP_COV_KRON_INV, OP_COV_SWIFT_KRON, OP_COV_SWIFT_KRON_INV, OP_COV_UNIT_WISE,
           OP_COV_UNIT_WISE_INV, OP_SAVE_INPUTS, OP_SAVE_OUTPUTS, OP_SAVE_OUTGRADS]
BWD_OPS_WITH_INPUTS = [OP_COV_UNIT_WISE, OP_COV_UNIT_WISE_INV]     # the forward hook has to keep the output
FWD_OPS = [OP_SAVE_INPUTS, OP_SAVE_OUTPUTS, OP_COV_KRON, OP_COV_KRON_INV, OP_COV_SWIFT_KRON,
           OP_COV_SWIFT_KRON_INV] + BWD_OPS_WITH_INPUTS
BWD_OPS = [OP_SAVE_OUTGRADS, OP_COV_KRON, OP_COV_KRON_INV, OP_COV_SWIFT_KRON, OP_COV_SWIFT_KRON_INV, OP_COV_UNIT_WISE,
           OP_COV_UNIT_WISE_INV]

__all__ = ['Operation', 'Linear', 'Conv2d', 'BatchNorm', 'LayerNorm', 'OperationContext', 'get_op_class', 'ALL_OPS',
           'FWD_OPS', 'BWD_OPS', 'OP_COV_KRON', 'OP_COV_KRON_INV', 'OP_COV_SWIFT_KRON', 'OP_COV_SWIFT_KRON_INV',
           'OP_COV_UNIT_WISE', 'OP_COV_UNIT_WISE_INV',
           'OP_SAVE_INPUTS', 'OP_SAVE_OUTPUTS', 'OP_SAVE_OUTGRADS']

AUTOCAST_ROUNDS_FP32_OPERANDS = True


def _autocast_rounds(x):
    """True for an fp32 operand of an input factor that is computed inside a bf16 autocast region.  The reference
    forms that factor with torch.matmul in its forward hook (asdl/operations/linear.py:75-77, conv.py:80-88), i.e.
    inside the region, where matmul casts both operands to bf16 (and returns bf16).  Rounding the operand the same
    way gives the statistic of the activation the layer itself consumed, on the bf16 matrix cores; the sums stay in
    fp32.  Output gradients are not concerned: backward hooks run outside the region."""
    return (AUTOCAST_ROUNDS_FP32_OPERANDS and x.dtype == torch.float32 and x.is_cuda
            and torch.is_autocast_enabled('cuda') and torch.get_autocast_dtype('cuda') == torch.bfloat16)


_FACTOR_CACHE_ATTR = '_asdl_amd_factor_cache'

# A module that is called several times in one forward pass (shared weights), factors not accumulated (no EMA).
# True, the reference's behaviour (asdl/operations/operation.py:225-233, 265-279): every backward call pairs the A
# factor of the LAST forward call with the B factor of its own output gradient, takes the pi-damping of that pair,
# inverts both, and the inverses of the calls are ADDED.  False: the A and the B contributions of the calls are
# summed and inverted once, (sum A + lam I)^-1, the curvature block that K-FAC defines and that both forms compute
# when the factors are accumulated.
PER_CALL_INVERSES = True


class Operation:
    supported_operations = {OP_COV_KRON, OP_COV_KRON_INV, OP_COV_SWIFT_KRON, OP_COV_SWIFT_KRON_INV, OP_SAVE_INPUTS,
                            OP_SAVE_OUTPUTS, OP_SAVE_OUTGRADS}

    def __init__(self, module, op_names, model_for_kernel=None):
        if hasattr(module, 'weight'):
            requires_grad = module.weight.requires_grad
            if hasattr(module, 'bias') and module.bias is not None:
                requires_grad = requires_grad or module.bias.requires_grad
            if not requires_grad:
                raise ValueError(f'One of weight or bias has to require grad (module: {module}).')
        self._module = module
        if isinstance(op_names, str):
            op_names = [op_names]
        if not isinstance(op_names, list):
            raise TypeError(f'op_names has to be a list. Got {type(op_names)}.')
        op_names = set(op_names)
        for name in op_names:
            if name not in ALL_OPS:
                raise ValueError(f'Invalid operation name: {name}. {ALL_OPS} are supported.')
        self._op_names = op_names
        self._inv_only = op_names == {OP_COV_KRON_INV}     # the hooks of this combination may repeat remembered calls
        self._op_results = {}
        self._damping = 1.e-7
        self._cov_scale = 1.
        self._first_beta = {}       # 'A' / 'B' -> factor applied to a registered matrix at its first update
        self._n_forward = self._n_backward = 0    # hook calls that contributed to the scratch factors
        self._touched = set()
        self._context = None

    # ---- result store (asdl/operations/operation.py:118-160)
    def accumulate_result(self, value, *keys, extend=False):
        results = self._op_results
        for key in keys[:-1]:
            if results.get(key, None) is None:
                results[key] = {}
            results = results[key]
        key = keys[-1]
        if results.get(key, None) is None:
            results[key] = value
        elif extend:
            results[key].extend(value)
        else:
            results[key] += value

    def get_result(self, *keys, pop=False, default=None):
        results = self._op_results
        for key in keys[:-1]:
            try:
                results = results[key]
            except KeyError:
                return None
        key = keys[-1]
        if pop:
            return results.pop(key, default)
        return results.get(key, default)

    def clear_results(self):
        self._op_results = {}

    def set_damping(self, value):
        self._damping = value

    def set_cov_scale(self, value):
        self._cov_scale = value

    # ---- fused accumulate into the stored factor
    def _update_factor(self, key, compute):
        """compute(out, alpha, beta) writes ``beta*out + alpha*factor`` (allocating when out is None)."""
        existing = self.get_result(OP_COV_KRON, key)
        if existing is None:
            self.accumulate_result(compute(None, self._cov_scale, 0.0), OP_COV_KRON, key)
        else:
            beta = self._first_beta.pop(key, 1.0)
            compute(existing, self._cov_scale, beta)
        self._touched.add(key)

    def _scratch_factor(self, key, dim, device, rows=None):
        """Reusable buffer for a factor that only lives until it has been inverted: [dim, dim], or [rows, dim]
        for a low-rank factor."""
        cache = getattr(self._module, _FACTOR_CACHE_ATTR, None)
        if cache is None:
            cache = {}
            setattr(self._module, _FACTOR_CACHE_ATTR, cache)
        shape = (dim if rows is None else rows, dim)
        buf = cache.get(key)
        if buf is None or tuple(buf.shape) != shape or buf.device != device:
            buf = torch.empty(*shape, dtype=torch.float32, device=device)
            cache[key] = buf
        return buf

    def _remembered_call(self, key, tmp_key, raw, first):
        """The factor call that this module's hook made on the previous pass, made again on ``raw`` (see
        kernels.GroupedCall, kernels.DirectCall): True when the group has taken it or it has been launched.  Only the square scratch factors of the *_INV
        operations are remembered; whatever differs from the remembered call goes through _factor_inv_mode()."""
        cache = getattr(self._module, _FACTOR_CACHE_ATTR, None)
        rec = cache.get('call' + key) if cache is not None else None
        if rec is None or cache.get(key) is not rec.out:
            return False
        if not rec.again(raw, (self._geometry(), self._cov_scale, first, _autocast_rounds(raw))):
            return False
        self._op_results[tmp_key] = rec.out
        self._op_results['_eig_scale_' + key] = 1.0
        return True

    def _geometry(self):
        """What the factor kernels take from the module besides its input (nothing for a Linear layer)."""
        return None

    def _factor_inv_mode(self, key, tmp_key, data, swift, square_fn, low_rank_fn, device, slot=None, raw=None):
        """One contribution to the scratch factor of the *_INV operations.  Swift (asdl/operations/operation.py:
        282-299): a factor with fewer samples than columns is the unscaled [n, d] row matrix; a square one is
        scaled by cov_scale only after the damping has been taken from the unscaled factors, which the damping
        kernel reproduces by un-scaling its eigenvalue mean.  ``slot``: the contribution does not join the
        factor of the earlier calls but is written to a scratch buffer of its own (per-call factors of a module
        that is called several times) and returned instead of stored under ``tmp_key``."""
        n, dim = self.swift_rows_cols(data)
        first = slot is not None or tmp_key not in self._op_results
        cache_key = key if slot is None else f'{key}@{slot}'
        if swift and n < dim:
            buf = self._scratch_factor(cache_key, dim, device, rows=n)
            low_rank_fn(buf, 1.0, 0.0 if first else 1.0)
            self._op_results['_eig_scale_' + key] = 1.0
        else:
            buf = self._scratch_factor(cache_key, dim, device)
            remember = raw is not None and slot is None and not swift
            if remember:
                kernels.GroupedCall.begin()
            square_fn(buf, self._cov_scale, 0.0 if first else 1.0)
            if remember:
                extra = (self._geometry(), self._cov_scale, first, _autocast_rounds(raw))
                rec = kernels.GroupedCall.remember(raw, buf, extra)
                if rec is None:
                    rec = kernels.DirectCall.remember(raw, buf, extra)      # launched at once: that launch, then
                getattr(self._module, _FACTOR_CACHE_ATTR)['call' + key] = rec
            self._op_results['_eig_scale_' + key] = 1.0 / self._cov_scale if swift else 1.0
        if slot is None:
            self._op_results[tmp_key] = buf
        return buf

    def forward_post_process(self, in_data: torch.Tensor, out_data: torch.Tensor):
        if not _profiling._ranges_on:         # (108 hook calls per step: not even an empty context manager)
            return self._forward_post_process(in_data, out_data)
        with nvtx_range('cov_kron_A'):
            self._forward_post_process(in_data, out_data)

    def _forward_post_process(self, in_data: torch.Tensor, out_data: torch.Tensor):
        module = self._module
        op_names = self._op_names
        if OP_SAVE_INPUTS in op_names:
            self.accumulate_result([in_data], OP_SAVE_INPUTS, extend=True)
        if OP_SAVE_OUTPUTS in op_names:
            self.accumulate_result([out_data], OP_SAVE_OUTPUTS, extend=True)
        if OP_COV_KRON in op_names:
            data = self.preprocess_in_data(module, in_data, out_data)
            self._update_factor('A', lambda out, alpha, beta: self.cov_kron_A(module, data, out=out, alpha=alpha, beta=beta))
        elif OP_COV_SWIFT_KRON in op_names:
            data = self.preprocess_in_data(module, in_data, out_data)
            n, dim = self.swift_rows_cols(data)
            fn = self.cov_swift_kron_A if n < dim else self.cov_kron_A
            self._update_factor('A', lambda out, alpha, beta: fn(module, data, out=out, alpha=alpha, beta=beta))
        elif OP_COV_KRON_INV in op_names or OP_COV_SWIFT_KRON_INV in op_names:
            if PER_CALL_INVERSES:
                # the reference's backward hook forms A from the input of the LAST forward call
                # (asdl/operations/operation.py:232): a later call replaces the factor of an earlier one
                self._op_results.pop('_A_tmp', None)
            if OP_COV_KRON_INV in op_names and self._remembered_call('A', '_A_tmp', in_data, '_A_tmp' not in self._op_results):
                self._n_forward += 1
                return
            data = self.preprocess_in_data(module, in_data, out_data)
            self._factor_inv_mode(
                'A', '_A_tmp', data, OP_COV_SWIFT_KRON_INV in op_names,
                lambda out, alpha, beta: self.cov_kron_A(module, data, out=out, alpha=alpha, beta=beta),
                lambda out, alpha, beta: self.cov_swift_kron_A(module, data, out=out, alpha=alpha, beta=beta),
                in_data.device, raw=in_data)
            self._n_forward += 1

    def backward_pre_process(self, out_grads, vector: torch.Tensor = None):
        if not _profiling._ranges_on:
            return self._backward_pre_process(out_grads, vector)
        with nvtx_range('cov_kron_B'):
            self._backward_pre_process(out_grads, vector)

    def _backward_pre_process(self, out_grads, vector: torch.Tensor = None):
        module = self._module
        op_names = self._op_names
        if not any(name in BWD_OPS for name in op_names):
            return
        if self._inv_only and self._n_forward <= 1 and \
                self._remembered_call('B', '_B_tmp', out_grads, '_B_tmp' not in self._op_results):
            self._n_backward += 1
            if self._context is not None:
                self._context.queue_inverse(self)
            return
        grads = self.preprocess_out_grads(module, out_grads)
        if OP_SAVE_OUTGRADS in op_names:
            self.accumulate_result([grads], OP_SAVE_OUTGRADS, extend=True)
        if OP_COV_KRON in op_names:
            self._update_factor('B', lambda out, alpha, beta: self.cov_kron_B(module, grads, out=out, alpha=alpha, beta=beta))
        elif OP_COV_SWIFT_KRON in op_names:
            n, dim = self.swift_rows_cols(grads)
            fn = self.cov_swift_kron_B if n < dim else self.cov_kron_B
            self._update_factor('B', lambda out, alpha, beta: fn(module, grads, out=out, alpha=alpha, beta=beta))
        elif OP_COV_KRON_INV in op_names or OP_COV_SWIFT_KRON_INV in op_names:
            per_call = PER_CALL_INVERSES and self._n_forward > 1
            buf = self._factor_inv_mode(
                'B', '_B_tmp', grads, OP_COV_SWIFT_KRON_INV in op_names,
                lambda out, alpha, beta: self.cov_kron_B(module, grads, out=out, alpha=alpha, beta=beta),
                lambda out, alpha, beta: self.cov_swift_kron_B(module, grads, out=out, alpha=alpha, beta=beta),
                grads.device, slot=self._n_backward % self._n_forward if per_call else None, raw=out_grads)
            if per_call:
                self._op_results.setdefault('_B_calls', []).append(buf)
            self._n_backward += 1
            # a module called several times in the forward pass is complete after as many backward hooks
            if self._context is not None and self._n_backward % max(self._n_forward, 1) == 0:
                self._context.queue_inverse(self)

    def finish_registered(self):
        """Applies the pending pre-scale to registered factors that no hook touched."""
        kron = self._op_results.get(OP_COV_KRON)
        for key, beta in list(self._first_beta.items()):
            if kron is not None and kron.get(key) is not None and beta != 1.0:
                kron[key].mul_(beta)
        self._first_beta = {}

    @staticmethod
    def preprocess_in_data(module, in_data, out_data):
        return in_data

    @staticmethod
    def preprocess_out_grads(module, out_grads):
        return out_grads

    @staticmethod
    def cov_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        raise NotImplementedError

    @staticmethod
    def cov_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        raise NotImplementedError

    @staticmethod
    def swift_rows_cols(data):
        """(samples, columns) of a preprocessed input / output gradient: the swift factors keep the row matrix
        when there are fewer samples than columns."""
        return data.shape[0], data.shape[1]

    @staticmethod
    def cov_swift_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        raise NotImplementedError

    @staticmethod
    def cov_swift_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        raise NotImplementedError


class Linear(Operation):
    """module.weight: f_out x f_in; in_data: n x f_in; out_grads: n x f_out
    (asdl/operations/linear.py:9-42, 75-89)."""

    @staticmethod
    def preprocess_in_data(module, in_data, out_data):
        if in_data.ndim > 2:
            in_data = in_data.flatten(end_dim=in_data.ndim - 2)
        return in_data

    @staticmethod
    def preprocess_out_grads(module, out_grads):
        if out_grads.ndim > 2:
            out_grads = out_grads.flatten(end_dim=out_grads.ndim - 2)
        return out_grads

    @staticmethod
    def cov_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        return kernels.syrk_tn(in_data, out=out, alpha=alpha, beta=beta, round_bf16=_autocast_rounds(in_data))   # f_in x f_in

    @staticmethod
    def cov_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        return kernels.syrk_tn(out_grads, out=out, alpha=alpha, beta=beta)    # f_out x f_out

    @staticmethod
    def cov_swift_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        """The inputs themselves, n x f_in with n < f_in (asdl/operations/linear.py:79-85)."""
        return kernels.conv_patch_sum(in_data, out=out, alpha=alpha, beta=beta)

    @staticmethod
    def cov_swift_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        """n x f_out with n < f_out (asdl/operations/linear.py:91-97)."""
        return kernels.conv_patch_sum(out_grads, out=out, alpha=alpha, beta=beta)


class Conv2d(Operation):
    """module.weight: c_out x c_in x k_h x k_w; in_data: lazy n x (c_in k_h k_w) x out_size;
    out_grads: n x c_out x out_size (asdl/operations/conv.py:9-42, 80-103)."""

    def _geometry(self):
        m = self._module
        return (m.kernel_size, m.stride, m.padding, m.dilation, m.groups)

    @staticmethod
    def preprocess_in_data(module, in_data, out_data):
        if isinstance(in_data, UnfoldedInput):
            return in_data
        if getattr(module, 'groups', 1) != 1:
            raise NotImplementedError('grouped convolutions are not supported by the K-FAC factors')
        return im2col_2d(in_data, module)

    @staticmethod
    def preprocess_out_grads(module, out_grads):
        if kernels._is_channels_last(out_grads):
            # [n, h, w, c_out] in memory: keep it, the rows of B's statistic are the pixels
            return out_grads
        return out_grads.flatten(start_dim=2)

    @staticmethod
    def cov_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        if not isinstance(in_data, UnfoldedInput):
            # already materialised [n, d, out_size] patches
            return kernels.syrk_nt(in_data, out=out, alpha=alpha / in_data.shape[-1], beta=beta)
        return kernels.conv_syrk(in_data.x, in_data.kernel_size, in_data.stride, in_data.padding, out=out,
                                 alpha=alpha / in_data.out_size, beta=beta, round_bf16=_autocast_rounds(in_data.x))

    @staticmethod
    def cov_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        if out_grads.ndim == 4:                                               # channels last
            n, c, h, w = out_grads.shape
            rows = out_grads.permute(0, 2, 3, 1).reshape(n * h * w, c)        # a view
            return kernels.syrk_tn(rows, out=out, alpha=alpha, beta=beta)
        return kernels.syrk_nt(out_grads, out=out, alpha=alpha, beta=beta)    # c_out x c_out

    @staticmethod
    def cov_swift_kron_A(module, in_data, out=None, alpha=1.0, beta=0.0):
        """Per-sample sums of the patches over the output positions, n x (c_in k_h k_w): `in_data.sum(dim=-1)` of the
        unfolded input (asdl/operations/conv.py:90-97), taken straight from the activation."""
        if not isinstance(in_data, UnfoldedInput):
            return kernels.conv_patch_sum(in_data, out=out, alpha=alpha, beta=beta)      # [n, d, out_size] patches
        return kernels.conv_patch_sum(in_data.x, in_data.kernel_size, in_data.stride, in_data.padding, out=out,
                                      alpha=alpha, beta=beta)

    @staticmethod
    def cov_swift_kron_B(module, out_grads, out=None, alpha=1.0, beta=0.0):
        """`out_grads.sum(dim=-1)`, n x c_out (asdl/operations/conv.py:105-111)."""
        return kernels.conv_patch_sum(out_grads, out=out, alpha=alpha, beta=beta)


class _NormOperation(Operation):
    """Unit-wise Fisher of modules with one (weight, bias) pair per feature: 2 x 2 blocks of the per-sample
    gradients (asdl/operations/batchnorm.py:8-108, asdl/operations/layernorm.py:7-84, and the unit-wise branch of
    Operation.backward_pre_process, asdl/operations/operation.py:230-235, 308-321).  As in the reference the
    normalised input is recovered from the module's output, which the forward hook keeps by reference: an
    in-place activation behind the module changes what the backward hook sees there, too."""
    supported_operations = {OP_COV_UNIT_WISE, OP_COV_UNIT_WISE_INV, OP_SAVE_INPUTS, OP_SAVE_OUTPUTS, OP_SAVE_OUTGRADS}

    def forward_post_process(self, in_data, out_data):
        op_names = self._op_names
        if OP_SAVE_INPUTS in op_names:
            self.accumulate_result([in_data], OP_SAVE_INPUTS, extend=True)
        if OP_SAVE_OUTPUTS in op_names:
            self.accumulate_result([out_data], OP_SAVE_OUTPUTS, extend=True)
        if any(n in BWD_OPS_WITH_INPUTS for n in op_names):
            self._op_results['_out_data'] = out_data

    @staticmethod
    def as_samples(module, tensor):
        """[samples, features, *positions] view of an output / output-gradient tensor."""
        return tensor

    def backward_pre_process(self, out_grads, vector=None):
        with nvtx_range('cov_unit_wise'):
            self._backward_pre_process(out_grads, vector)

    def _backward_pre_process(self, out_grads, vector=None):
        module = self._module
        op_names = self._op_names
        if OP_SAVE_OUTGRADS in op_names:
            self.accumulate_result([out_grads], OP_SAVE_OUTGRADS, extend=True)
        if not any(n in BWD_OPS_WITH_INPUTS for n in op_names):
            return
        if not (original_requires_grad(module, 'weight') and original_requires_grad(module, 'bias')):
            raise ValueError(f'Both weight and bias have to require grad for {OP_COV_UNIT_WISE} (module: {module}).')
        out_data = self._op_results.get('_out_data')
        if out_data is None:
            raise RuntimeError(f'{OP_COV_UNIT_WISE}: the forward hook did not run (module: {module})')
        y, g = self.as_samples(module, out_data), self.as_samples(module, out_grads)
        weight, bias = module.weight.detach().flatten(), module.bias.detach().flatten()
        if OP_COV_UNIT_WISE in op_names:
            store = self._op_results.setdefault(OP_COV_UNIT_WISE, {})
            existing = store.get('data')
            if existing is None:
                store['data'] = kernels.unit_wise_stats(y, g, weight, bias, alpha=self._cov_scale)
            else:
                beta = self._first_beta.pop('data', 1.0)
                kernels.unit_wise_stats(y, g, weight, bias, out=existing, alpha=self._cov_scale, beta=beta)
        else:
            first = '_unit_tmp' not in self._op_results
            cache = getattr(module, _FACTOR_CACHE_ATTR, None)
            if cache is None:
                cache = {}
                setattr(module, _FACTOR_CACHE_ATTR, cache)
            buf = cache.get('unit')
            if buf is None or buf.shape[0] != weight.numel() or buf.device != weight.device:
                buf = torch.empty(weight.numel(), 2, 2, dtype=torch.float32, device=weight.device)
                cache['unit'] = buf
            kernels.unit_wise_stats(y, g, weight, bias, out=buf, alpha=self._cov_scale, beta=0.0 if first else 1.0)
            self._op_results['_unit_tmp'] = buf
            self._n_backward += 1
            if self._context is not None:
                self._context.queue_unit_inverse(self)

    def finish_registered(self):
        unit = self._op_results.get(OP_COV_UNIT_WISE)
        beta = self._first_beta.pop('data', 1.0)
        if unit is not None and unit.get('data') is not None and beta != 1.0:
            unit['data'].mul_(beta)
        self._first_beta = {}


class BatchNorm(_NormOperation):
    """BatchNorm1d: [n, f]; BatchNorm2d: [n, c, h, w] in any memory format."""


class LayerNorm(_NormOperation):
    """[n, *, normalized_shape]: every leading index is a sample, the normalized shape is flattened to the
    features (asdl/operations/layernorm.py:20-42)."""

    @staticmethod
    def as_samples(module, tensor):
        f = module.weight.numel()
        return tensor.reshape(-1, f)


EAGER_COST_FRACTION = 0.6
_warned_late_fallback = False


class LateChunk:
    """The unread flags of one chunk of DeferredInverses.finish_late() and the modules its Kron objects belong to."""

    def __init__(self, late, targets, attr):
        self._late, self._targets, self._attr = late, targets, attr

    def check(self, *args, **kwargs):
        zero = self._late.check(*args, **kwargs)
        if zero and self._attr is not None:
            owner = {id(kron): module for module, kron in self._targets}
            for kron, which in zero:
                fisher = getattr(owner.get(id(kron)), self._attr, None)
                if fisher is not None and fisher.has_kron:
                    setattr(fisher.kron, which + '_inv', None)
        return zero


class DeferredInverses:
    """Inverses enqueued by OperationContext.flush_inverses(defer=True), possibly in several chunks.
    finish(attr) waits for them, raises torch.linalg.LinAlgError for a factor that is not positive definite,
    and removes from ``module.<attr>.kron`` the inverse of any all-zero factor (which the reference never
    computes)."""

    def __init__(self, chunks, context=None):
        self._chunks = chunks            # [(PendingInverses, [(module, kron), ...]), ...]
        self._context = context

    def finish_late(self, attr=None, warn=True):
        """finish() without its host synchronisation (PendingInverses.finish_late): returns objects whose check()
        reads the flags later (and, like finish(), removes from ``module.<attr>.kron`` the inverse of an all-zero
        factor that had none before).  None when the context also has unit-wise flags to read, which only finish()
        does."""
        if self._context is not None and self._context._unit_flags:
            global _warned_late_fallback
            if warn and not _warned_late_fallback:
                _warned_late_fallback = True
                warnings.warn('late_inverse_flags: this model has unit-wise (BatchNorm / LayerNorm) blocks, whose flags '
                              'are read at once; the flags of the Kronecker factors are read with them.')
            return None
        if self._context is not None:
            self._context._unit_flags_deferred = False      # nothing was deferred to this object's finish()
        for pending, _ in self._chunks:
            pending.join()
        return [LateChunk(late, targets, attr) for late, targets in
                ((pending.finish_late(), targets) for pending, targets in self._chunks) if late is not None]

    def finish(self, attr):
        if self._context is not None:
            self._context.check_unit_flags()
        for pending, _ in self._chunks:
            pending.join()               # all waits first, then the flag reads
        for pending, targets in self._chunks:
            pending.finish()
            for module, kron in targets:
                fisher = getattr(module, attr, None)
                if fisher is None or not fisher.has_kron:
                    continue
                if kron.A_inv is None:
                    fisher.kron.A_inv = None
                if kron.B_inv is None:
                    fisher.kron.B_inv = None


def get_op_class(module):
    """asdl/operations/__init__.py:60-79, restricted to the layer types on this path."""
    if isinstance(module, nn.Linear):
        return Linear
    elif isinstance(module, nn.Conv2d):
        return Conv2d
    elif isinstance(module, (nn.BatchNorm1d, nn.BatchNorm2d)):
        return BatchNorm
    elif isinstance(module, nn.LayerNorm):
        return LayerNorm
    warnings.warn(f'Failed to lookup operations for Module {module}.')
    return None


class OperationContext:
    def __init__(self, vectors=None):
        self._operations: Dict[nn.Module, Operation] = {}
        self._vectors = vectors
        self._pending_inverse = []
        self._inverse_chunks = []
        self._pending_unit = []
        self._unit_flags = []
        self._unit_flags_deferred = False
        self.factor_stream = None
        self.grad_edges = []       # autograd edges of the hooked module outputs of the latest forward pass
        self._eager_total = 0.0
        self._eager_done = False
        self._inverse_cost = 0.0

    def is_operation_registered(self, module):
        return module in self._operations

    def registered_modules(self):
        return list(self._operations)

    def register_operation(self, module, operation):
        operation._context = self
        self._operations[module] = operation

    def get_operation(self, module) -> Operation:
        try:
            return self._operations[module]
        except KeyError:
            raise KeyError(f'No operation is registered to {module}.')

    def clear_operations(self):
        self._operations.clear()
        self._pending_inverse = []
        self._inverse_chunks = []
        self._pending_unit = []

    def call_operations_in_forward(self, module, in_data, out_data):
        self.get_operation(module).forward_post_process(in_data, out_data)

    def call_operations_in_backward(self, module, out_grads):
        self.get_operation(module).backward_pre_process(out_grads, None)

    def get_result(self, module, *keys, pop=False, default=None):
        try:
            return self.get_operation(module).get_result(*keys, pop=pop, default=default)
        except KeyError:
            return default

    def set_damping(self, value):
        for operation in self._operations.values():
            operation.set_damping(value)

    def set_cov_scale(self, value):
        for operation in self._operations.values():
            operation.set_cov_scale(value)

    def clear_batch_grads(self):
        pass

    def calc_full_cov(self, model, scale=1., calc_inv=False, damping=1e-7):
        pass  # only needed for the full (non layer-wise) shape

    def join_factor_stream(self):
        """Orders the current stream after the statistics kernels that ran on the factor stream."""
        if self.factor_stream is not None:
            self.factor_stream.join()

    # ---- deferred, batched inverses
    def set_eager_inverse(self, total_cost):
        """``total_cost``: sum of d^3 over all factors inverted in the previous step (0 or None: unknown).
        When known, the pairs queued so far are inverted as soon as they hold EAGER_COST_FRACTION of it,
        i.e. while the backward pass that produces the remaining B factors is still running: in a network
        whose widest layers come last, the longest chains of the batched inverse start early and only the
        cheap remainder is left for after the pass.  One early batch only, so that same-size factors still
        share launches.  Only valid when every factor receives a single contribution (one backward pass)."""
        self._eager_total = float(total_cost or 0)
        self._eager_done = False

    @property
    def inverse_cost(self):
        """Sum of d^3 over the factors queued for inversion since the context was created."""
        return self._inverse_cost

    def queue_inverse(self, operation):
        if operation not in self._pending_inverse:
            self._pending_inverse.append(operation)
            for key in ('_A_tmp', '_B_tmp'):
                buf = operation._op_results.get(key)
                if buf is not None:
                    self._inverse_cost += float(buf.shape[0]) ** 3
        if self._eager_total > 0 and not self._eager_done and \
                self._inverse_cost >= EAGER_COST_FRACTION * self._eager_total:
            self._eager_done = True
            # this runs inside a backward hook: with a factor stream the hook's launches are redirected to it, and
            # the factors queued so far were computed there
            with kernels.main_stream_launches():
                self.join_factor_stream()
                self._enqueue_pending()

    def queue_unit_inverse(self, operation):
        if operation not in self._pending_unit:
            self._pending_unit.append(operation)

    def _invert_units(self):
        """Damped inverses of the queued unit-wise blocks (one grouped launch); their singularity flags are read
        together in check_unit_flags()."""
        ops = self._pending_unit
        self._pending_unit = []
        todo = []
        for op in ops:
            blocks = op._op_results.pop('_unit_tmp', None)
            if blocks is None:
                continue
            store = op._op_results.setdefault(OP_COV_UNIT_WISE, {})
            prev = store.get('inv')
            reuse = prev is not None and prev.shape == blocks.shape
            todo.append((op, store, blocks, prev if reuse else None))
        if not todo:
            return
        invs, flags = kernels.unit_wise_inv_grouped([t[2] for t in todo], [t[0]._damping for t in todo],
                                                    outs=[t[3] for t in todo])
        for i, ((op, store, _, _), inv) in enumerate(zip(todo, invs)):
            store['inv'] = inv
            self._unit_flags.append((op._module, flags[i]))

    def check_unit_flags(self):
        """torch.inverse raises for a singular block (asdl/operations/operation.py:317-320); here the flags of all
        modules are read with one copy."""
        pending = self._unit_flags
        self._unit_flags = []
        self._unit_flags_deferred = False
        if not pending:
            return
        host = torch.stack([f for _, f in pending]).cpu().tolist()
        for (module, _), (nonzero, bad) in zip(pending, host):
            if bad != 0x7fffffff:
                raise torch.linalg.LinAlgError(f'unit-wise block {bad - 1} of {module} + damping is singular')

    def _enqueue_pending(self):
        """Starts the batched inverse of every queued pair (side streams, worker threads) and places the
        output tensors in the result store; their flags are read by DeferredInverses.finish()."""
        ops = self._pending_inverse
        self._pending_inverse = []
        if not ops:
            return
        shared = [op for op in ops if op._op_results.get('_B_calls')]
        if shared:
            ops = [op for op in ops if op not in shared]
            for op in shared:
                self._invert_per_call(op)
            if not ops:
                return
        krons = []
        for op in ops:
            A = op._op_results.pop('_A_tmp', None)
            B = op._op_results.pop('_B_tmp', None)
            if A is None or B is None:
                raise RuntimeError('cov_kron_inv: the forward and backward hooks did not both run')
            prev = op._op_results.get(OP_COV_KRON) or {}
            kron = Kron(A, B, prev.get('A_inv'), prev.get('B_inv'))
            scales = (op._op_results.pop('_eig_scale_A', 1.0), op._op_results.pop('_eig_scale_B', 1.0))
            if scales != (1.0, 1.0):
                kron._eig_scale = scales          # swift: the damping is taken from the unscaled factors
            krons.append(kron)
        # every operation in one context shares the damping value
        pending = batched_update_inv(krons, damping=ops[0]._damping, replace=False, defer=True)
        outs = {(id(k), which): out for _, k, which, out in pending._records}
        for op, kron in zip(ops, krons):
            store = op._op_results.setdefault(OP_COV_KRON, {})
            store['A_inv'] = outs[(id(kron), 'A')]
            store['B_inv'] = outs[(id(kron), 'B')]
        self._inverse_chunks.append((pending, [(op._module, kron) for op, kron in zip(ops, krons)]))

    def _invert_per_call(self, op):
        """A module that was called several times (PER_CALL_INVERSES): one (A, B_k) pair per backward call, each with
        its own pi-damping, and the sum of their inverses.  A rare shape of model: the pairs are inverted at once and
        their flags read here, with a host synchronisation."""
        A = op._op_results.pop('_A_tmp', None)
        B_calls = op._op_results.pop('_B_calls', None)
        if A is None or not B_calls:
            raise RuntimeError('cov_kron_inv: the forward and backward hooks did not both run')
        scales = (op._op_results.pop('_eig_scale_A', 1.0), op._op_results.pop('_eig_scale_B', 1.0))
        krons = []
        for B in B_calls:
            kron = Kron(A, B)
            if scales != (1.0, 1.0):
                kron._eig_scale = scales
            krons.append(kron)
        batched_update_inv(krons, damping=op._damping, replace=False, defer=False)
        store = op._op_results.setdefault(OP_COV_KRON, {})
        for which in ('A_inv', 'B_inv'):
            total = None
            for kron in krons:
                inv = getattr(kron, which)
                if inv is not None:
                    total = inv if total is None else total.add_(inv)
            if total is None:
                store.pop(which, None)
            else:
                store[which] = total

    def flush_inverses(self, defer=False):
        """Inverts every queued (A, B) pair in batched passes.  With ``defer=True`` the launches are only
        enqueued: the result store receives the output tensors right away and the returned object's
        finish() must be called before they are used (it reads the zero / not-positive-definite flags)."""
        self._enqueue_pending()
        self._invert_units()
        chunks = self._inverse_chunks
        self._inverse_chunks = []
        if not chunks:
            if not self._unit_flags_deferred:
                self.check_unit_flags()
            return None
        deferred = DeferredInverses(chunks, self)
        if defer:
            self._unit_flags_deferred = True      # read with the other flags in deferred.finish(), not by a later flush
            return deferred
        self.check_unit_flags()
        for pending, _ in chunks:
            pending.join()
        for pending, targets in chunks:
            pending.finish()
            for module, kron in targets:
                store = self.get_operation(module)._op_results.setdefault(OP_COV_KRON, {})
                for which in ('A_inv', 'B_inv'):
                    if getattr(kron, which) is None:
                        store.pop(which, None)       # all-zero factor: the reference computes no inverse
        return None

    # ---- symmatrix exchange (asdl/operations/operation.py:815-876)
    def cov_symmatrix(self, module, pop=False):
        self.flush_inverses()       # no-op when the caller has already flushed (possibly deferred)
        cov_kron = self.get_result(module, OP_COV_KRON, pop=pop)
        cov_unit = self.get_result(module, OP_COV_UNIT_WISE, pop=pop)
        kwargs = {}
        if cov_kron is not None:
            kwargs = dict(kron_A=cov_kron.pop('A', None), kron_B=cov_kron.pop('B', None),
                          kron_A_inv=cov_kron.pop('A_inv', None), kron_B_inv=cov_kron.pop('B_inv', None))
        if cov_unit is not None and not all(v is None for v in cov_unit.values()):
            kwargs['unit'] = UnitWise(data=cov_unit.pop('data', None), inv=cov_unit.pop('inv', None))
        if all(v is None for v in kwargs.values()):
            return None
        return SymMatrix(**kwargs)

    def register_symmatrix(self, module, matrix: SymMatrix, first_beta=1.0):
        """Places the module's existing factors in the result store so that the hooks accumulate
        into them in place; ``first_beta`` is the factor they are scaled by at their first update."""
        operation = self.get_operation(module)
        if matrix.has_kron:
            if matrix.kron.has_A:
                operation.accumulate_result(matrix.kron.A, OP_COV_KRON, 'A')
                operation._first_beta['A'] = first_beta
            if matrix.kron.has_B:
                operation.accumulate_result(matrix.kron.B, OP_COV_KRON, 'B')
                operation._first_beta['B'] = first_beta
        if matrix.has_unit and matrix.unit.has_data:
            operation.accumulate_result(matrix.unit.data, OP_COV_UNIT_WISE, 'data')
            operation._first_beta['data'] = first_beta

    def finish_registered(self):
        for operation in self._operations.values():
            operation.finish_registered()
