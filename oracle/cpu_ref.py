"""CPU oracle for the K-FAC / Shampoo curvature path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain PyTorch CPU ops, the arithmetic that
kazukiosawa/asdl performs on the curvature hot path.  It exists to check the
HIP kernels and to serve as the timed CPU baseline; nothing in the product
package imports it.  Only tests/, __graft_entry__.smoke() and the
``cpu_baseline`` leg of bench.py may use it.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  How each function is pinned (tests/test_oracle.py):

  linear_cov_kron_A/B   closed form vs fp64 matmul, trace = ||X||_F^2, the
                        single-datum kron(B, A) == per-example-gradient Fisher
                        identity of test/grad_maker/test_fisher.py:152-156
  im2col_2d             torch.nn.functional.unfold (library routine) and a
                        6-nested-loop brute force on tiny inputs
  conv_cov_kron_A/B     brute-force loops; single-datum Fisher identity
  ema / scale           linearity (test_fisher.py:215-237)
  kron_damping          the pi formula written out in test_fisher.py:267-273,
                        plus the pi in {0, inf} special cases
  cholesky_inv          (X + damping I) @ inv == I, fp64 torch.linalg.inv
  kron_mvp              (B^-1 kron A^-1) vec(G) identity  -- the reference has no
                        test that calls precondition(); pinned by mathematics
  norm_cov_unit_wise    per-example gradients of (weight, bias) taken one sample at a
                        time by autograd: block f == sum_n g_n g_n^T with
                        g_n = (dL_n/dw_f, dL_n/db_f) (brute force), for BatchNorm1d/2d
                        in eval mode and LayerNorm; golden default-K-FAC runs of a
                        BatchNorm CNN written from the reference
  unit_wise_inv / mvp   (block + damping I) @ inv == I per block; block-diagonal
                        matrix-vector product against an explicit dense matrix
  matrix_to_tril /      the worked 3x3 example in the docstrings of asdl/symmatrix.py:25-54,
  tril_to_matrix        numpy.tril_indices (library routine), pack(unpack(t)) == t
  smw_inv               fp64 inverse of x^T x / n + damping I formed densely (the identity it
                        implements); golden SKFAC runs written from the reference
  *_cov_swift_*         the row sums of F.unfold / of the output gradient (library routines);
                        golden SKFAC runs (swift=True) written from the reference
  merge_small_dims /    the two worked examples in the docstring of asdl/precondition/shampoo.py:370-384;
  block_slices /        partition + merge round trip, block statistics against tensordot on slices; golden
  PartitionedShampoo..  runs of the reference's Preconditioner with block_size and dimension merging
  power_iter            eigvalsh lambda_max (converged limit only)
  compute_power         fp64 eigh closed form (S + rI)^(-1/p), X^p (S + rI) == I;
                        golden trajectories written from the reference
                        (tests/golden/make_golden.py) for iteration counts and
                        the early-break path
  kfac_step / shampoo_step
                        golden multi-step runs written from the reference
                        (tests/golden/make_golden.py)
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = [
    'norm_restore_input', 'norm_cov_unit_wise', 'unit_wise_inv', 'unit_wise_mvp',
    'linear_cov_kron_A', 'linear_cov_kron_B', 'im2col_2d', 'conv_cov_kron_A', 'conv_cov_kron_B',
    'ema_accumulate', 'kron_damping', 'cholesky_inv', 'kron_update_inv', 'kron_mvp',
    'power_iter', 'mat_power', 'compute_power', 'shampoo_statistics', 'shampoo_precondition',
    'matrix_to_tril', 'tril_to_matrix', 'KfacOracle', 'ShampooOracle',
    'merge_small_dims', 'block_slices', 'PartitionedShampooOracle',
    'linear_cov_swift', 'conv_cov_swift_kron_A', 'conv_cov_swift_kron_B', 'swift_kron_damping', 'smw_inv', 'swift_inv',
]


# --------------------------------------------------------------------------- factors
def _flatten_rows(x):
    # asdl/operations/linear.py:20-25, 37-42: n x * x f -> (n*) x f
    return x.flatten(end_dim=x.ndim - 2) if x.ndim > 2 else x


def linear_cov_kron_A(in_data):
    """A = a^T a, no bias column (asdl/operations/linear.py:75-77)."""
    a = _flatten_rows(in_data)
    return a.T @ a


def linear_cov_kron_B(out_grads):
    """B = g^T g (asdl/operations/linear.py:87-89)."""
    g = _flatten_rows(out_grads)
    return g.T @ g


def im2col_2d(x, kernel_size, stride, padding):
    """[n,c,h,w] -> [n, c*kh*kw, h_out*w_out], rows ordered (c, ky, kx), zero padding,
    dilation 1 (asdl/utils.py:51-71)."""
    kh, kw = kernel_size
    sy, sx = stride
    ph, pw = (0, 0) if padding == 'valid' else padding
    if ph + pw > 0:
        x = F.pad(x, (pw, pw, ph, ph))
    x = x.unfold(2, kh, sy).unfold(3, kw, sx)          # n c ho wo kh kw
    x = x.permute(0, 1, 4, 5, 2, 3).contiguous()       # n c kh kw ho wo
    return x.view(x.size(0), x.size(1) * kh * kw, x.size(4) * x.size(5))


def conv_cov_kron_A(x, kernel_size, stride, padding):
    """A = (1/out_size) sum_n X_n X_n^T over unfolded patches
    (asdl/operations/conv.py:24-27, 80-88)."""
    col = im2col_2d(x, kernel_size, stride, padding)
    out_size = col.shape[-1]
    m = col.transpose(0, 1).flatten(start_dim=1)
    return (m @ m.T) / out_size


def conv_cov_kron_B(out_grads):
    """B = sum_{n,pos} g g^T, NOT divided by out_size (asdl/operations/conv.py:39-42, 99-103)."""
    g = out_grads.flatten(start_dim=2)
    m = g.transpose(0, 1).flatten(start_dim=1)
    return m @ m.T


def ema_accumulate(old, new, ema_decay):
    """EMA mode: old <- (1 - ema_decay) * old + new, where ``new`` was already computed with
    the extra factor ``ema_decay`` in its scale; the first call has no ``old``
    (asdl/precondition/natural_gradient.py:397-405, asdl/operations/operation.py:118-137)."""
    if old is None:
        return new
    return old * (1 - ema_decay) + new


# --------------------------------------------------------------------------- damping / inverse
def kron_damping(A, B, damping, eps=1e-7):
    """pi-split of the damping between the two Kronecker factors
    (asdl/symmatrix.py:499-510, asdl/operations/operation.py:457-466)."""
    a_mean = A.trace() / A.shape[-1]
    b_mean = B.trace() / B.shape[-1]
    pi = torch.sqrt(a_mean / b_mean)
    pi_v = float(pi)
    if pi_v != 0 and pi_v != float('inf'):
        r = damping ** 0.5
        return max(float(r * pi), eps), max(float(r / pi), eps)
    return damping, damping


def cholesky_inv(X, damping=1e-7):
    """(X + damping I)^-1 through a lower Cholesky factor; X is left unchanged
    (asdl/utils.py:91-96)."""
    Xd = X.clone()
    Xd.diagonal().add_(damping)
    return torch.cholesky_inverse(torch.linalg.cholesky(Xd))


def kron_update_inv(A, B, damping, eps=1e-7):
    """Returns (A_inv, B_inv); an all-zero factor is skipped and yields None
    (asdl/symmatrix.py:499-534)."""
    dA, dB = kron_damping(A, B, damping, eps)
    A_inv = None if bool(torch.all(A == 0)) else cholesky_inv(A, dA)
    B_inv = None if bool(torch.all(B == 0)) else cholesky_inv(B, dB)
    return A_inv, B_inv


# --------------------------------------------------------------------------- low-rank ("swift") factors
def linear_cov_swift(data):
    """n x f rows themselves when n < f, else the f x f factor (asdl/operations/linear.py:79-97)."""
    data = _flatten_rows(data)
    n, f = data.shape
    return data.clone() if n < f else data.T @ data


def conv_cov_swift_kron_A(x, kernel_size, stride, padding):
    """asdl/operations/conv.py:90-97: per-sample sum of the patches over the output positions when n < c_in k_h k_w
    (not divided by the output size), else the ordinary factor."""
    col = im2col_2d(x, kernel_size, stride, padding)
    n, d, _ = col.shape
    return col.sum(dim=-1) if n < d else conv_cov_kron_A(x, kernel_size, stride, padding)


def conv_cov_swift_kron_B(out_grads):
    """asdl/operations/conv.py:105-111."""
    g = out_grads.flatten(start_dim=2)
    n, c, _ = g.shape
    return g.sum(dim=-1) if n < c else conv_cov_kron_B(out_grads)


def swift_kron_damping(A, B, damping, eps=1e-7):
    """asdl/operations/operation.py:457-466, asdl/symmatrix.py:499-510: the eigenvalue mean of an n x d row matrix
    is sum(x^2) / d."""
    def mean(M):
        return (M.trace() if M.shape[0] == M.shape[1] else (M ** 2).sum()) / M.shape[-1]
    pi = torch.sqrt(mean(A) / mean(B))
    pi_v = float(pi)
    if pi_v != 0 and pi_v != float('inf'):
        r = damping ** 0.5
        return max(float(r * pi), eps), max(float(r / pi), eps)
    return damping, damping


def smw_inv(x, damping=1e-7):
    """(x^T x / n + damping I)^-1 of an n x d matrix through its n x n Gram matrix (asdl/utils.py:107-115)."""
    n, d = x.shape
    G = x @ x.T
    G = G + damping * n * torch.eye(n, dtype=x.dtype)
    Ginv_x = torch.linalg.solve(G, x)
    return (torch.eye(d, dtype=x.dtype) - x.T @ Ginv_x) / damping


def swift_inv(M, damping):
    return cholesky_inv(M, damping) if M.shape[0] == M.shape[1] else smw_inv(M, damping)


def kron_mvp(A_inv, B_inv, grad_w, grad_b=None):
    """W <- B_inv @ view(W, [dB, -1]) @ A_inv ; b <- B_inv @ b (asdl/symmatrix.py:536-548)."""
    dB = B_inv.shape[-1]
    w = (B_inv @ grad_w.reshape(dB, -1) @ A_inv).view_as(grad_w)
    if grad_b is not None:
        return w, B_inv @ grad_b
    return w


# --------------------------------------------------------------------------- Shampoo
def power_iter(mat_g, v0, error_tolerance=1e-6, num_iters=100):
    """Power iteration from the start vector ``v0`` (the reference draws it from
    U(-1, 1)); returns (lambda_max estimate, iterations)
    (asdl/precondition/shampoo.py:531-558)."""
    v = v0
    error = 1
    iters = 0
    singular_val = 0
    while error > error_tolerance and iters < num_iters:
        v = v / torch.norm(v)
        mat_v = torch.mv(mat_g, v)
        s_v = torch.dot(v, mat_v)
        error = torch.abs(s_v - singular_val)
        v = mat_v
        singular_val = s_v
        iters += 1
    return singular_val, iters


def mat_power(mat_m, p):
    """mat_m^p by repeated squaring (asdl/precondition/shampoo.py:561-586)."""
    if p in [1, 2, 4, 8, 16, 32]:
        p_done = 1
        res = mat_m
        while p_done < p:
            res = res @ res
            p_done *= 2
        return res
    power = None
    while p > 0:
        if p % 2 == 1:
            power = mat_m @ power if power is not None else mat_m
        p //= 2
        mat_m = mat_m @ mat_m
    return power


def compute_power(mat_g, p, v0, iter_count=100, error_tolerance=1e-6, ridge_epsilon=1e-6):
    """(mat_g + r I)^(-1/p), r = ridge_epsilon * lambda_max, by the coupled Newton iteration.
    ``mat_g`` is modified in place (the ridge stays in the stored statistic), exactly as in
    asdl/precondition/shampoo.py:465-528.  Returns (root, iterations, final error)."""
    n = mat_g.shape[0]
    identity = torch.eye(n, dtype=mat_g.dtype)
    if n == 1:
        return identity, 0, 0.0
    alpha = -1.0 / p
    max_ev, _ = power_iter(mat_g, v0)
    mat_g += (ridge_epsilon * max_ev) * identity
    z = (1 + p) / (2 * torch.norm(mat_g))
    mat_root = identity * torch.pow(z, 1.0 / p)
    mat_m = mat_g * z
    error = torch.max(torch.abs(mat_m - identity))
    count = 0
    while error > error_tolerance and count < iter_count:
        tmp = (1 - alpha) * identity + alpha * mat_m
        new_root = mat_root @ tmp
        mat_m = mat_power(tmp, p) @ mat_m
        new_error = torch.max(torch.abs(mat_m - identity))
        if new_error > error * 1.2:
            break
        mat_root = new_root
        error = new_error
        count += 1
    return mat_root, count, float(error)


def shampoo_statistics(grad, stats, ema_decay=-1):
    """Per-axis statistics of an N-D gradient, updated in place
    (asdl/precondition/shampoo.py:324-339)."""
    ndim = grad.ndim
    for i in range(ndim):
        axes = list(range(i)) + list(range(i + 1, ndim))
        stat = torch.tensordot(grad, grad, [axes, axes])
        if ema_decay == -1:
            stats[i].add_(stat)
        else:
            stats[i].mul_(1 - ema_decay).add_(stat, alpha=ema_decay)
    return stats


def shampoo_precondition(grad, preconditioners):
    """Chained tensordot over axis 0 with every preconditioner; for a matrix this is
    P_L^T G P_R (asdl/precondition/shampoo.py:351-367)."""
    out = grad
    for P in preconditioners:
        out = torch.tensordot(out, P, [[0], [0]])
    return out


def merge_small_dims(shape, max_dim):
    """asdl/precondition/shampoo.py:370-395."""
    out, prod = [], 1
    for d in shape:
        if prod * d <= max_dim:
            prod *= d
        else:
            if prod > 1:
                out.append(prod)
            prod = d
    if prod > 1:
        out.append(prod)
    return out


def block_slices(shape, block_size):
    """Index ranges of the blocks of BlockPartitioner (asdl/precondition/shampoo.py:405-447), first axis slowest."""
    import itertools
    per_axis = []
    for d in shape:
        if block_size != -1 and d > block_size:
            per_axis.append([slice(a, min(a + block_size, d)) for a in range(0, d, block_size)])
        else:
            per_axis.append([slice(0, d)])
    return list(itertools.product(*per_axis))


class PartitionedShampooOracle:
    """One parameter's Preconditioner with block partitioning and dimension merging
    (asdl/precondition/shampoo.py:300-367)."""

    def __init__(self, shape, block_size=-1, merge=False, damping=1e-7, ema_decay=-1, init_scale=1e-12):
        self.shape = tuple(shape)
        self.tshape = tuple(merge_small_dims(shape, block_size)) if merge else tuple(shape)
        self.blocks = block_slices(self.tshape, block_size)
        self.damping, self.ema_decay = damping, ema_decay
        self.statistics = [init_scale * torch.eye(s.stop - s.start) for blk in self.blocks for s in blk]
        self.preconditioners = [torch.eye(s.stop - s.start) for blk in self.blocks for s in blk]

    def update_statistics(self, grad):
        g = grad.reshape(self.tshape)
        nd = len(self.tshape)
        for j, blk in enumerate(self.blocks):
            shampoo_statistics(g[blk], self.statistics[j * nd:(j + 1) * nd], self.ema_decay)

    def update_preconditioners(self, start_vectors):
        exp = 2 * len(self.tshape)
        for i, stat in enumerate(self.statistics):
            n = stat.shape[0]
            self.preconditioners[i] = compute_power(stat, exp, start_vectors(n), ridge_epsilon=self.damping)[0] \
                if n > 1 else torch.eye(1)

    def precondition(self, grad):
        g = grad.reshape(self.tshape)
        nd = len(self.tshape)
        out = torch.empty(self.tshape)
        for j, blk in enumerate(self.blocks):
            out[blk] = shampoo_precondition(g[blk], self.preconditioners[j * nd:(j + 1) * nd])
        return out.reshape(self.shape)


# --------------------------------------------------------------------------- end-to-end K-FAC
def _update_by_interval(step, interval, warmup=0):
    # asdl/precondition/prec_grad_maker.py:198-201
    return step < warmup or (step - warmup) % interval == 0


def norm_restore_input(module, out_data):
    """Normalised input of a BatchNorm / LayerNorm module recovered from its output
    (asdl/operations/batchnorm.py:11-21, asdl/operations/layernorm.py:20-31)."""
    if isinstance(module, nn.LayerNorm):
        x = (out_data - module.bias).div(module.weight)
        k = len(module.weight.shape)
        if k < x.ndim - 1:
            x = x.flatten(end_dim=-k - 1)
        return x
    shape = (1, module.num_features) + (1,) * (out_data.ndim - 2)
    return (out_data - module.bias.view(shape)).div(module.weight.view(shape))


def norm_cov_unit_wise(module, out_data, out_grads):
    """[f, 2, 2] blocks sum_n [[gw^2, gw gb], [gw gb, gb^2]] of the per-sample gradients of (weight, bias)
    (asdl/operations/batchnorm.py:28-55, 95-108; asdl/operations/layernorm.py:33-84)."""
    x = norm_restore_input(module, out_data)
    if isinstance(module, nn.LayerNorm):
        k = len(module.weight.shape)
        g = out_grads.flatten(end_dim=-k - 1) if k < out_grads.ndim - 1 else out_grads
        gw, gb = x.mul(g).flatten(start_dim=1), g.flatten(start_dim=1)
    else:
        gw, gb = x.mul(out_grads), out_grads
        if gw.ndim > 2:
            dims = tuple(range(2, gw.ndim))
            gw, gb = gw.sum(dim=dims), gb.sum(dim=dims)
    f = gw.shape[1]
    ww, bb, wb = (gw ** 2).sum(0), (gb ** 2).sum(0), (gw * gb).sum(0)
    return torch.vstack([ww, wb, wb, bb]).reshape(2, 2, f).transpose(0, 2).contiguous()


def unit_wise_inv(blocks, damping):
    """(blocks + damping I)^-1 per block; None for an all-zero tensor (asdl/symmatrix.py:687-699)."""
    if torch.all(blocks == 0):
        return None
    eye = torch.eye(blocks.shape[-1], dtype=blocks.dtype)
    return torch.inverse(blocks + damping * eye)


def unit_wise_mvp(mat, vec_weight, vec_bias):
    """asdl/symmatrix.py:701-709: [w, b][f] <- mat[f] @ [w, b][f]."""
    v = torch.stack([vec_weight.flatten(), vec_bias.flatten()], dim=1).unsqueeze(2)
    out = torch.matmul(mat, v).squeeze(2)
    return out[:, 0].view_as(vec_weight), out[:, 1].view_as(vec_bias)


def matrix_to_tril(mat):
    # asdl/symmatrix.py:25-38: rows of the lower triangle one after the other
    return torch.cat([mat[i, :i + 1] for i in range(mat.shape[0])])


def tril_to_matrix(tril):
    # asdl/symmatrix.py:41-54 (n from asdl/symmatrix.py:57-67: n^2 + n = 2 numel)
    n = int(math.sqrt(2 * tril.numel() + 0.25) - 0.5)
    out = torch.zeros(n, n, dtype=tril.dtype)
    k = 0
    for i in range(n):
        out[i, :i + 1] = tril[k:k + i + 1]
        out[:i + 1, i] = tril[k:k + i + 1]
        k += i + 1
    return out


class KfacOracle:
    """Restatement of KfacGradientMaker.forward_and_backward for Linear / Conv2d layers
    (BatchNorm / LayerNorm ignored, as in the reference's training script,
    examples/arxiv_results/train.py:363).

    Follows asdl/precondition/prec_grad_maker.py:135-154,
    asdl/precondition/natural_gradient.py:323-324, 397-543 and asdl/fisher.py:69-152, 443-459.

    ``fisher_type`` is 'fisher_emp' or 'fisher_mc'.  For 'fisher_mc' the sampled targets
    come from ``torch.distributions.Categorical(probs).sample()`` after
    ``torch.random.manual_seed(seed)`` exactly like the reference, or are injected through
    ``mc_targets`` (one tensor per step) so that another device can replay them.
    """

    def __init__(self, model, data_size, damping=1e-7, ema_decay=-1, fisher_type='fisher_emp',
                 scale=1., grad_scale=1., seed=None, curvature_upd_interval=None,
                 preconditioner_upd_interval=1, factor_dtype=None, unit_wise_norm=False, swift=False):
        self.model = model
        self.data_size = data_size
        self.damping = damping
        self.ema_decay = ema_decay
        self.fisher_type = fisher_type
        self.scale = scale
        self.grad_scale = grad_scale
        self.seed = seed
        self.curv_interval = curvature_upd_interval
        self.prec_interval = preconditioner_upd_interval
        self.factor_dtype = factor_dtype
        self.swift = swift        # KfacGradientMaker(swift=True), asdl/precondition/natural_gradient.py:886-887
        self.step = 0
        self.layers = [(n, m) for n, m in model.named_modules()
                       if isinstance(m, (nn.Linear, nn.Conv2d))
                       and any(p.requires_grad for p in m.parameters())]
        # unit_wise_norm: BatchNorm1d/2d and LayerNorm get the unit-wise shape, as in the default
        # KfacGradientMaker (asdl/precondition/natural_gradient.py:886-889); else they are ignored
        self.norm_layers = [(n, m) for n, m in model.named_modules()
                            if unit_wise_norm and isinstance(m, (nn.BatchNorm1d, nn.BatchNorm2d, nn.LayerNorm))]
        self.A = {}
        self.B = {}
        self.A_inv = {}
        self.B_inv = {}
        self.unit = {}
        self.unit_inv = {}
        self.last_mc_targets = None

    # -- schedule (prec_grad_maker.py:174-187)
    def _do_update_preconditioner(self, step):
        return _update_by_interval(step, self.prec_interval)

    def _do_update_curvature(self, step):
        if self.curv_interval is not None:
            return _update_by_interval(step, self.curv_interval)
        return self._do_update_preconditioner(step)

    def _factor(self, module, in_data, out_grads, cov_scale):
        cast = (lambda t: t.to(self.factor_dtype)) if self.factor_dtype is not None else (lambda t: t)
        if isinstance(module, nn.Conv2d):
            A = conv_cov_kron_A(cast(in_data), module.kernel_size, module.stride, module.padding)
            B = conv_cov_kron_B(cast(out_grads))
        else:
            A = linear_cov_kron_A(cast(in_data))
            B = linear_cov_kron_B(cast(out_grads))
        return A * cov_scale, B * cov_scale

    def _swift_factor(self, module, in_data, out_grads):
        """Unscaled swift factors (asdl/operations/operation.py:201-204, 279-285)."""
        cast = (lambda t: t.to(self.factor_dtype)) if self.factor_dtype is not None else (lambda t: t)
        if isinstance(module, nn.Conv2d):
            return (conv_cov_swift_kron_A(cast(in_data), module.kernel_size, module.stride, module.padding),
                    conv_cov_swift_kron_B(cast(out_grads)))
        return linear_cov_swift(cast(in_data)), linear_cov_swift(cast(out_grads))

    def _swift_update_inv(self, A, B):
        """Kron.update_inv with non-square factors (asdl/symmatrix.py:499-534)."""
        dA, dB = swift_kron_damping(A, B, self.damping)
        A_inv = None if bool(torch.all(A == 0)) else swift_inv(A, dA)
        B_inv = None if bool(torch.all(B == 0)) else swift_inv(B, dB)
        return A_inv, B_inv

    def _shared_module_factors(self, name, module, inputs, out_grads, cov_scale, accumulate):
        """A module that is called several times in one forward pass.  With accumulated factors (OP_COV_KRON)
        every forward call adds its A and every backward call its B (asdl/operations/operation.py:196-198,
        262-264 with accumulate_result's ``+=``, :136-137).  Without (OP_COV_KRON_INV, :265-279) every backward
        call forms A from the input of the LAST forward call (:232), B from its own output gradient, takes the
        pi-damping of that pair, inverts both and ADDS THE INVERSES to those of the earlier calls."""
        if accumulate:
            A = sum(self._factor(module, x, out_grads[0], cov_scale)[0] for x in inputs)
            B = sum(self._factor(module, inputs[0], g, cov_scale)[1] for g in out_grads)
            self.A[name] = ema_accumulate(self.A.get(name), A, self.ema_decay)
            self.B[name] = ema_accumulate(self.B.get(name), B, self.ema_decay)
            return
        A_inv = B_inv = None
        for g in out_grads:
            A, B = self._factor(module, inputs[-1], g, cov_scale)
            dA, dB = kron_damping(A, B, self.damping)
            Ai, Bi = cholesky_inv(A, dA), cholesky_inv(B, dB)
            A_inv = Ai if A_inv is None else A_inv + Ai
            B_inv = Bi if B_inv is None else B_inv + Bi
        self.A_inv[name], self.B_inv[name] = A_inv, B_inv

    def forward_and_backward(self, x, t, loss_fn=F.cross_entropy, mc_targets=None):
        model = self.model
        step = self.step
        N = self.data_size
        accumulate = self.ema_decay != -1
        if not self._do_update_curvature(step):
            # plain mean-reduced forward/backward, stale inverses (prec_grad_maker.py:140-142)
            y = model(x)
            loss = loss_fn(y, t)
            loss.backward()
        else:
            scale = self.scale
            if accumulate:
                scale = scale * self.ema_decay      # the (1 - ema_decay) pre-scale is in ema_accumulate
            cov_scale = scale / N
            saved_in, saved_g, saved_out = {}, {}, {}
            handles = []
            for name, m in self.norm_layers:
                # a hook on the output tensor, not a module backward hook: the latter forbids the in-place
                # activations that commonly follow a normalisation layer
                def norm_hook(mod, inp, out, name=name):
                    saved_out[name] = out.detach()
                    if out.requires_grad:
                        out.register_hook(lambda g, name=name: saved_g.__setitem__(name, g.detach()))
                handles.append(m.register_forward_hook(norm_hook))
            # a module may be called several times per forward pass: the inputs are kept in call order, the
            # output gradients in the order the backward hook fires (asdl/operations/operation.py:188, 225-233)
            calls_in, calls_g = {}, {}
            for name, m in self.layers:
                def fwd_hook(mod, inp, out, name=name):
                    saved_in[name] = inp[0].detach()
                    calls_in.setdefault(name, []).append(inp[0].detach())

                def bwd_hook(mod, gin, gout, name=name):
                    saved_g[name] = gout[0].detach()
                    calls_g.setdefault(name, []).append(gout[0].detach())
                handles.append(m.register_forward_hook(fwd_hook))
                handles.append(m.register_full_backward_hook(bwd_hook))
            if self.seed is not None:
                torch.random.manual_seed(self.seed)
            y = model(x)
            loss = loss_fn(y, t, reduction='sum')
            if self.fisher_type == 'fisher_emp':
                loss.backward()
            else:
                probs = F.softmax(y, dim=-1)
                log_probs = F.log_softmax(y, dim=-1)
                if mc_targets is None:
                    with torch.no_grad():
                        mc_targets = torch.distributions.Categorical(probs).sample()
                self.last_mc_targets = mc_targets
                nll = F.nll_loss(log_probs.view(-1, log_probs.size(-1)), mc_targets.view(-1),
                                 reduction='sum', ignore_index=-1)
                req = [p.requires_grad for p in model.parameters()]
                for p in model.parameters():
                    p.requires_grad_(False)
                nll.backward(retain_graph=True)
                for p, r in zip(model.parameters(), req):
                    p.requires_grad_(r)
            for h in handles:
                h.remove()
            for name, m in self.layers:
                if self.swift:
                    A, B = self._swift_factor(m, saved_in[name], saved_g[name])
                    if accumulate:        # OP_COV_SWIFT_KRON: every factor, square or not, times cov_scale
                        self.A[name] = ema_accumulate(self.A.get(name), A * cov_scale, self.ema_decay)
                        self.B[name] = ema_accumulate(self.B.get(name), B * cov_scale, self.ema_decay)
                    else:
                        # OP_COV_SWIFT_KRON_INV (asdl/operations/operation.py:282-299): damping from the unscaled
                        # factors; only the square ones are scaled before the inverse
                        dA, dB = swift_kron_damping(A, B, self.damping)
                        self.A_inv[name] = cholesky_inv(A * cov_scale, dA) if A.shape[0] == A.shape[1] else smw_inv(A, dA)
                        self.B_inv[name] = cholesky_inv(B * cov_scale, dB) if B.shape[0] == B.shape[1] else smw_inv(B, dB)
                    continue
                if len(calls_in[name]) > 1:
                    if self.swift:
                        raise NotImplementedError('swift factors of a module called more than once are not restated')
                    self._shared_module_factors(name, m, calls_in[name], calls_g[name], cov_scale, accumulate)
                    continue
                A, B = self._factor(m, saved_in[name], saved_g[name], cov_scale)
                if accumulate:
                    self.A[name] = ema_accumulate(self.A.get(name), A, self.ema_decay)
                    self.B[name] = ema_accumulate(self.B.get(name), B, self.ema_decay)
                else:
                    self.A_inv[name], self.B_inv[name] = kron_update_inv(A, B, self.damping)
            for name, m in self.norm_layers:
                blocks = norm_cov_unit_wise(m, saved_out[name].float(), saved_g[name].float()) * cov_scale
                if accumulate:
                    self.unit[name] = ema_accumulate(self.unit.get(name), blocks, self.ema_decay)
                else:
                    # asdl/operations/operation.py:317-321: inverted in the hook, no all-zero test
                    self.unit_inv[name] = torch.inverse(blocks + self.damping * torch.eye(2))
            if self.fisher_type != 'fisher_emp':
                loss.backward()
            for p in model.parameters():
                if p.grad is not None:
                    p.grad.div_(N)
            loss = loss.detach() / N
        if accumulate and self._do_update_preconditioner(step):
            for name, _ in self.layers:
                if name in self.A:
                    update = self._swift_update_inv if self.swift else (lambda A, B: kron_update_inv(A, B, self.damping))
                    self.A_inv[name], self.B_inv[name] = update(self.A[name], self.B[name])
            for name, _ in self.norm_layers:
                if name in self.unit:
                    inv = unit_wise_inv(self.unit[name], self.damping)
                    if inv is not None:
                        self.unit_inv[name] = inv
        for name, m in self.norm_layers:
            if self.unit_inv.get(name) is None:
                continue
            if self.grad_scale != 1:
                m.weight.grad.mul_(self.grad_scale)
                m.bias.grad.mul_(self.grad_scale)
            w, b = unit_wise_mvp(self.unit_inv[name], m.weight.grad, m.bias.grad)
            m.weight.grad.copy_(w)
            m.bias.grad.copy_(b)
        for name, m in self.layers:
            if self.A_inv.get(name) is None or self.B_inv.get(name) is None:
                continue
            gw = m.weight.grad
            gb = m.bias.grad if m.bias is not None and m.bias.requires_grad else None
            if self.grad_scale != 1:
                gw.mul_(self.grad_scale)
                if gb is not None:
                    gb.mul_(self.grad_scale)
            Ai, Bi = self.A_inv[name].to(gw.dtype), self.B_inv[name].to(gw.dtype)
            if gb is not None:
                w, b = kron_mvp(Ai, Bi, gw, gb)
                gb.copy_(b)
            else:
                w = kron_mvp(Ai, Bi, gw)
            gw.copy_(w)
        self.step += 1
        return y, loss


class ShampooOracle:
    """Restatement of ShampooGradientMaker for parameters with ndim > 1, no block
    partitioning (asdl/precondition/shampoo.py:34-56, 201-223, 300-367)."""

    def __init__(self, model, damping=1e-7, ema_decay=-1, curvature_upd_interval=None,
                 preconditioner_upd_interval=1, init_scale=1e-12):
        self.model = model
        self.damping = damping
        self.ema_decay = ema_decay
        self.curv_interval = curvature_upd_interval
        self.prec_interval = preconditioner_upd_interval
        self.params = [p for p in model.parameters() if p.ndim > 1 and p.requires_grad]
        self.stats = [[init_scale * torch.eye(s) for s in p.shape] for p in self.params]
        self.precs = [[torch.eye(s) for s in p.shape] for p in self.params]
        self.step = 0
        self.newton_iters = []

    def forward_and_backward(self, x, t, loss_fn=F.cross_entropy, start_vectors=None):
        """``start_vectors``: optional callable n -> U(-1,1) start vector for the power
        iteration; default draws ``torch.rand(n) * 2 - 1`` like the reference."""
        step = self.step
        y = self.model(x)
        loss = loss_fn(y, t)
        loss.backward()
        do_prec = _update_by_interval(step, self.prec_interval)
        do_curv = _update_by_interval(step, self.curv_interval) if self.curv_interval is not None else do_prec
        if do_curv:
            for p, stats in zip(self.params, self.stats):
                shampoo_statistics(p.grad, stats, self.ema_decay)
        if do_prec:
            for i, p in enumerate(self.params):
                exp = 2 * p.ndim
                for j, stat in enumerate(self.stats[i]):
                    n = stat.shape[0]
                    v0 = start_vectors(n) if start_vectors is not None else torch.rand(n) * 2 - 1
                    root, iters, _ = compute_power(stat, exp, v0, ridge_epsilon=self.damping)
                    self.precs[i][j] = root
                    self.newton_iters.append(iters)
        for p, precs in zip(self.params, self.precs):
            p.grad.copy_(shampoo_precondition(p.grad, precs).reshape(p.shape))
        self.step += 1
        return y, loss
