"""Containers of the curvature matrices on the K-FAC path: SymMatrix, its Kronecker part (square factors or the
row matrices of the swift variant) and the unit-wise 2 x 2 blocks, with their packed on-disk form.

Same attributes and call signatures as asdl/symmatrix.py (SymMatrix :94-358, Kron :361-548, UnitWise :617-719,
save / load :25-87, 226-269, 471-492); the arithmetic runs in the HIP kernels.  Full / layer-wise matrices can be
saved and loaded; KFE and diagonal containers are accepted as opaque attributes but have no kernels here.
"""
import os
from collections import defaultdict

import numpy as np
import torch
from torch import Tensor

from . import kernels
from .profiling import nvtx_range

__all__ = ['SymMatrix', 'Kron', 'UnitWise', 'batched_update_inv', 'PendingInverses', 'matrix_to_tril', 'tril_to_matrix',
           'get_n_cols_by_tril']

_default_damping = 1e-5


def matrix_to_tril(mat: Tensor):
    """Lower triangle of a square matrix as a 1-D tensor, row direction: [[1,x,x],[2,3,x],[4,5,6]] ->
    [1,2,3,4,5,6] (asdl/symmatrix.py:25-38).  The matrix has to be on the GPU."""
    if mat.ndim != 2:
        raise ValueError(f'mat.ndim has to be 2. Got {mat.ndim}.')
    if mat.dtype != torch.float32 or mat.stride(1) != 1:
        mat = mat.float().contiguous()
    return kernels.tril_pack(mat)


def get_n_cols_by_tril(tril: Tensor):
    """n with n(n+1)/2 == tril.numel() (asdl/symmatrix.py:57-67)."""
    if tril.ndim != 1:
        raise ValueError(f'tril.ndim has to be 1. Got {tril.ndim}.')
    return int(np.sqrt(2 * tril.numel() + 0.25) - 0.5)


def tril_to_matrix(tril: Tensor):
    """Full symmetric matrix of a packed lower triangle (asdl/symmatrix.py:41-54).  On the GPU."""
    if tril.ndim != 1:
        raise ValueError(f'tril.ndim has to be 1. Got {tril.ndim}.')
    n_cols = get_n_cols_by_tril(tril)
    if n_cols * (n_cols + 1) // 2 != tril.numel():
        raise ValueError(f'{tril.numel()} values are not the lower triangle of a square matrix.')
    return kernels.tril_unpack(tril.float(), n_cols)


def _save_as_numpy(path, tensor):
    """float32 .npy file, directories created on the way (asdl/symmatrix.py:74-78)."""
    dirname = os.path.dirname(path)
    if dirname and not os.path.isdir(dirname):
        os.makedirs(dirname)
    np.save(path, tensor.detach().cpu().numpy().astype('float32'))


def _load_from_numpy(path, device=None):
    """The matrices of this build live on the GPU: ``device`` None means the current one, a CPU device is an
    error rather than a silent host path (the reference defaults to 'cpu', asdl/symmatrix.py:81-83)."""
    device = torch.device('cuda' if device is None else device)
    if device.type != 'cuda':
        raise RuntimeError(f'factors are loaded onto a GPU in this build, got device {device}')
    return torch.from_numpy(np.load(path)).to(device)


_side_stream_cache = {}
N_SIDE_STREAMS = 8     # groups of a batched inverse that may run side by side
GROUPED_INVERSE = True  # all square factors of a call in one merged launch sequence (kernels.chol_inv_grouped);
                        # False: one batched inverse per distinct size, spread over the side streams


def _side_streams(device, n):
    key = device.index if device.index is not None else torch.cuda.current_device()
    pool = _side_stream_cache.setdefault(key, [])
    while len(pool) < n:
        pool.append(torch.cuda.Stream(device=device))
    return pool[:n]


_enqueue_workers = {}
_next_side_stream = 0


def _worker(stream_index):
    """One enqueue thread per side stream.  The launches of a batched inverse are a few dozen small kernels
    issued from C without the interpreter lock, so the caller can go on (with the backward pass) while they are
    being issued; a single thread per stream keeps the jobs of that stream, which share its workspace, in
    order."""
    w = _enqueue_workers.get(stream_index)
    if w is None:
        from concurrent.futures import ThreadPoolExecutor
        w = ThreadPoolExecutor(max_workers=1, thread_name_prefix=f'asdl_amd_inv{stream_index}')
        _enqueue_workers[stream_index] = w
    return w


def _is_all_none(xs):
    return all(x is None for x in xs)


class LateFlags:
    """Flags of a batch of inverses on their way to pinned host memory (PendingInverses.finish_late).  check() waits
    for the copy, which has long arrived when it is called a step later, and raises for a factor that was not
    positive definite."""

    def __init__(self, host, event, records, keep_alive):
        self._host, self._event, self._records, self._keep_alive = host, event, records, keep_alive

    def check(self, when='reported late: the flags of this update were read after the next one'):
        """Raises for a factor that was not positive definite.  Returns the (Kron, 'A' | 'B') whose factor was all
        zero and had no inverse before: the reference computes none for them (asdl/symmatrix.py:517, :527); the
        device has put the identity there, and the caller removes it again."""
        if self._host is None:
            return []
        if self._event is not None:
            self._event.synchronize()
        host, self._host, self._keep_alive = self._host.tolist(), None, None
        n = len(self._records)
        info_host, nz_host = host[:n], host[n:]
        zero = []
        for (flat, k, which, was_fresh), inf in zip(self._records, info_host):
            if not nz_host[flat]:
                if was_fresh:
                    setattr(k, which + '_inv', None)
                    zero.append((k, which))
            elif inf != 0:
                raise torch.linalg.LinAlgError(
                    f'cholesky_inv: the leading minor of order {inf} of kron.{which} + damping was not '
                    f'positive-definite' + (f' ({when})' if when else ''))
        return zero


class PendingInverses:
    """Inverses that have been enqueued (on side streams) but whose flags have not been read yet.
    finish() joins the streams into the current one, reads all flags with one device-to-host copy,
    raises for a matrix that is not positive definite and stores the inverses on the Kron objects."""

    def __init__(self, records, infos, nz_flat, events, replace, keep_alive=None, futures=(), fresh=None):
        self._records, self._infos, self._nz_flat = records, infos, nz_flat
        self._fresh = list(fresh) if fresh is not None else [True] * len(records)   # output buffers that held no inverse
        self._keep_alive = keep_alive      # tensors the side-stream kernels still read
        self._events, self._replace = events, replace
        self._futures = list(futures)      # enqueue jobs running on worker threads; each returns an event
        self._done = False

    def join(self):
        """Makes the current stream wait for the inverses (no host synchronisation beyond the enqueue
        jobs themselves)."""
        events = list(self._events) + [f.result() for f in self._futures]
        self._events, self._futures = [], []
        if events:
            main = torch.cuda.current_stream()
            for ev in events:
                main.wait_event(ev)

    def finish_late(self):
        """finish() without its host synchronisation: the inverses are stored on the Kron objects as if every factor
        was non-zero and positive definite, the copy of the flags to pinned host memory is enqueued, and the returned
        LateFlags reads them when asked (a step later, say).  Until then an all-zero factor, whose inverse was
        skipped, has the identity as its inverse if the buffer is a fresh one (the device fills it in), and its
        previous inverse otherwise, as in the reference, which skips the update (asdl/symmatrix.py:517, :527)."""
        if self._done:
            return None
        self._done = True
        self.join()
        fresh = [(flat, out) for (flat, k, which, out), was_fresh in zip(self._records, self._fresh) if was_fresh]
        if fresh:
            kernels.identity_where_zero([out for _, out in fresh], self._nz_flat, [flat for flat, _ in fresh])
        flags = torch.cat(self._infos + [self._nz_flat])
        event = None
        if flags.is_cuda:
            host = torch.empty(flags.shape, dtype=flags.dtype, pin_memory=True)
            host.copy_(flags, non_blocking=True)
            event = torch.cuda.Event()
            event.record()
        else:
            host = flags.clone()
        for (flat, k, which, out) in self._records:
            setattr(k, which + '_inv', out)
            if self._replace:
                setattr(k, which, None)
        # (flag index, Kron, side, did the buffer hold no inverse before)
        late = LateFlags(host, event, [(flat, k, which, was_fresh) for (flat, k, which, _), was_fresh
                                       in zip(self._records, self._fresh)], (flags, self._keep_alive))
        self._keep_alive = None
        return late

    def finish(self):
        if self._done:
            return
        self._done = True
        self.join()
        host = torch.cat(self._infos + [self._nz_flat]).cpu().tolist()        # the one synchronisation
        n = len(self._records)
        info_host, nz_host = host[:n], host[n:]
        self._keep_alive = None
        for (flat, k, which, out), inf in zip(self._records, info_host):
            if not nz_host[flat]:
                continue                                            # all-zero factor: inverse skipped
            if inf != 0:
                raise torch.linalg.LinAlgError(
                    f'cholesky_inv: the leading minor of order {inf} of kron.{which} + damping is not '
                    f'positive-definite')
            setattr(k, which + '_inv', out)
            if self._replace:
                setattr(k, which, None)


def batched_update_inv(krons, damping=_default_damping, calc_A_inv=True, calc_B_inv=True, eps=1e-7, replace=False,
                       defer=False):
    """Kron.update_inv for many Kron objects at once (asdl/symmatrix.py:499-534 per object).

    One damping launch for all pairs, one batched Cholesky inverse per distinct matrix size, and
    a single device-to-host read at the end for the zero / not-positive-definite flags (the
    reference synchronises three to five times per layer).  With ``defer=True`` the launches are
    enqueued and a PendingInverses is returned: the caller may enqueue unrelated work (the loss
    backward pass) before calling its finish()."""
    krons = [k for k in krons if k is not None]
    if not krons:
        return None
    for k in krons:
        if not k.has_data:
            raise ValueError('data do not exist.')
        if calc_A_inv and not k.has_A:
            raise ValueError('A does not exist.')
        if calc_B_inv and not k.has_B:
            raise ValueError('B does not exist.')
        for m in (k.A, k.B):
            if m is not None and (m.ndim != 2 or m.shape[0] > m.shape[1]):
                raise ValueError('a Kronecker factor is a square matrix or an [n, d] row matrix with n < d')
    dev = (krons[0].A if krons[0].has_A else krons[0].B).device
    mats_on_gpu = dev.type == 'cuda'
    A_list = [k.A if k.has_A else k.B for k in krons]
    B_list = [k.B if k.has_B else k.A for k in krons]
    A_list = [a if a.is_contiguous() else a.contiguous() for a in A_list]
    B_list = [b if b.is_contiguous() else b.contiguous() for b in B_list]
    eig_scale = None
    if any(getattr(k, '_eig_scale', None) is not None for k in krons):
        eig_scale = [getattr(k, '_eig_scale', None) or (1.0, 1.0) for k in krons]
    lam, nonzero = kernels.kron_damping(A_list, B_list, float(damping), float(eps), eig_scale=eig_scale)
    single = [i for i, k in enumerate(krons) if not (k.has_A and k.has_B)]
    if single:
        lam[kernels.device_ints(tuple(single), dev)] = float(damping)      # no pi split without both factors
    lam_flat, nz_flat = lam.view(-1), nonzero.view(-1)

    groups = defaultdict(list)   # d -> [(flat index, matrix, kron, 'A'|'B')]
    low_rank = []                # the same entries for [n, d] row matrices (n < d), inverted through their Gram matrix
    for i, k in enumerate(krons):
        if calc_A_inv:
            entry = (2 * i, A_list[i], k, 'A')
            (groups[A_list[i].shape[0]] if A_list[i].shape[0] == A_list[i].shape[1] else low_rank).append(entry)
        if calc_B_inv:
            entry = (2 * i + 1, B_list[i], k, 'B')
            (groups[B_list[i].shape[0]] if B_list[i].shape[0] == B_list[i].shape[1] else low_rank).append(entry)
    # GROUPED_INVERSE: every square factor of the call goes into one grouped inverse, whose launches carry the steps
    # of all matrices at once.  Otherwise each size group is an independent chain of small launches, and the groups
    # are spread over a few side streams (default priority) so that their launch latencies overlap.  Either way
    # everything joins the caller's stream again.
    if GROUPED_INVERSE and groups:
        merged = [e for d in sorted(groups, reverse=True) for e in groups[d]]
        groups = {-1: merged}
    order = sorted(groups, key=lambda d: sum(e[1].shape[0] ** 3 for e in groups[d]), reverse=True)
    prepared = []
    fresh_of = {}                # id(output buffer) -> it held no inverse before
    for d in order:
        entries = groups[d]
        idx = kernels.device_ints(tuple(e[0] for e in entries), dev)
        outs = []
        for _, mat, k, which in entries:
            old = getattr(k, which + '_inv')
            reuse = old is not None and old.shape == mat.shape and old.is_contiguous() and old.dtype == mat.dtype
            outs.append(old if reuse else torch.empty_like(mat))
            fresh_of[id(outs[-1])] = not reuse
        info = torch.empty(len(entries), dtype=torch.int32, device=dev)
        prepared.append((entries, outs, lam_flat[idx], nz_flat[idx].contiguous(), info))
    for flat, mat, k, which in low_rank:
        # (x^T x / n + lam I)^-1 by Sherman-Morrison-Woodbury (smw_inv, asdl/utils.py:107-115): a group of its own
        d = mat.shape[1]
        old = getattr(k, which + '_inv')
        reuse = old is not None and tuple(old.shape) == (d, d) and old.is_contiguous() and old.dtype == mat.dtype
        out = old if reuse else torch.empty(d, d, dtype=mat.dtype, device=dev)
        fresh_of[id(out)] = not reuse
        info = torch.empty(1, dtype=torch.int32, device=dev)
        prepared.append(([(flat, mat, k, which)], [out], lam_flat[flat:flat + 1], None, info))
    prepared.sort(key=lambda g: -sum(e[1].shape[0] * e[1].shape[1] ** 2 for e in g[0]))
    infos, records, events, futures = [], [], [], []
    use_streams = mats_on_gpu and (len(prepared) > 1 or defer)

    range_name = 'inv_kron' + ('_A' if calc_A_inv else '') + ('_B' if calc_B_inv else '')

    def run_group(group):
        entries, outs, lam_g, act_g, info = group
        with nvtx_range(range_name):
            if act_g is None:          # a low-rank factor
                kernels.smw_inv(entries[0][1], lam_g, out=outs[0], info=info)
            elif GROUPED_INVERSE:
                kernels.chol_inv_grouped([e[1] for e in entries], outs, lam_g, 1, active=act_g, active_stride=1,
                                         info=info)
            else:
                kernels.chol_inv_batched([e[1] for e in entries], outs, lam_g, 1, active=act_g, active_stride=1,
                                         info=info)

    if use_streams:
        main = torch.cuda.current_stream()
        # successive calls start on different side streams (each with its own enqueue thread and workspace), so
        # that an early batch and the remainder of one step run side by side
        global _next_side_stream
        pool = _side_streams(dev, N_SIDE_STREAMS)
        first = _next_side_stream % len(pool)
        n_used = min(len(pool), len(prepared))
        _next_side_stream += n_used
        chosen = [(first + i) % len(pool) for i in range(n_used)]
        side = [pool[i] for i in chosen]
        start = torch.cuda.Event()
        start.record(main)
        per_stream = [prepared[i::len(side)] for i in range(len(side))]

        def run_stream(st, groups_of_stream):
            with torch.cuda.device(dev), torch.cuda.stream(st):
                st.wait_event(start)
                for group in groups_of_stream:
                    run_group(group)
                done = torch.cuda.Event()
                done.record(st)
            return done

        for si, st, groups_of_stream in zip(chosen, side, per_stream):
            if defer:
                futures.append(_worker(si).submit(run_stream, st, groups_of_stream))
            else:
                events.append(run_stream(st, groups_of_stream))
    else:
        for group in prepared:
            run_group(group)
    for entries, outs, lam_g, act_g, info in prepared:
        infos.append(info)
        records.extend((e[0], e[2], e[3], out) for e, out in zip(entries, outs))
    pending = PendingInverses(records, infos, nz_flat, events, replace,
                              keep_alive=(prepared, lam, nonzero, A_list, B_list), futures=futures,
                              fresh=[fresh_of[id(r[3])] for r in records])
    if defer:
        return pending
    pending.finish()
    return None


def batched_unit_update_inv(units, damping=_default_damping, replace=False):
    """UnitWise.update_inv (asdl/symmatrix.py:687-699) for many modules: one grouped launch, then a single
    device-to-host read for all zero / singular flags instead of one per module."""
    units = [u for u in units if u is not None]
    for u in units:
        if not u.has_data:
            raise ValueError('data do not exist.')
    if not units:
        return
    invs, flags = kernels.unit_wise_inv_grouped([u.data for u in units], [float(damping)] * len(units))
    host = flags.cpu().tolist()
    for u, inv, (nonzero, bad) in zip(units, invs, host):
        if not nonzero:
            continue                       # an all-zero tensor keeps its old inverse (none)
        if bad != 0x7fffffff:
            raise torch.linalg.LinAlgError(f'unit-wise block {bad - 1} + damping is singular')
        u.inv = inv
        if replace:
            u.data = None


class Kron:
    def __init__(self, A, B, A_inv=None, B_inv=None):
        self.A: Tensor = A
        self.B: Tensor = B
        self.A_inv: Tensor = A_inv
        self.B_inv: Tensor = B_inv
        self._A_dim = self._B_dim = None

    def __add__(self, other):
        if not other.has_data:
            return self
        A = (self.A.add(other.A) if self.has_A else other.A) if other.has_A else self.A
        B = (self.B.add(other.B) if self.has_B else other.B) if other.has_B else self.B
        return Kron(A, B)

    def __iadd__(self, other):
        if not other.has_data:
            return self
        if other.has_A:
            if self.has_A:
                self.A.add_(other.A)
            else:
                self.A = other.A
        if other.has_B:
            if self.has_B:
                self.B.add_(other.B)
            else:
                self.B = other.B
        return self

    @property
    def data(self):
        return [self.A, self.B]

    @property
    def has_data(self):
        return self.has_A or self.has_B

    @property
    def has_A(self):
        return self.A is not None

    @property
    def has_B(self):
        return self.B is not None

    @property
    def has_inv(self):
        return self.A_inv is not None and self.B_inv is not None

    @property
    def A_dim(self):
        if self._A_dim is None:
            if self.A is not None:
                self._A_dim = self.A.shape[-1]
            elif self.A_inv is not None:
                self._A_dim = self.A_inv.shape[-1]
            else:
                raise ValueError('A nor A_inv has not been set.')
        return self._A_dim

    @property
    def B_dim(self):
        if self._B_dim is None:
            if self.B is not None:
                self._B_dim = self.B.shape[-1]
            elif self.B_inv is not None:
                self._B_dim = self.B_inv.shape[-1]
            else:
                raise ValueError('B nor B_inv has not been set.')
        return self._B_dim

    @property
    def A_is_square(self):
        return self.A is not None and self.A.shape[0] == self.A.shape[1]

    @property
    def B_is_square(self):
        return self.B is not None and self.B.shape[0] == self.B.shape[1]

    def mul_(self, value):
        if self.has_A:
            self.A.mul_(value)
        if self.has_B:
            self.B.mul_(value)
        return self

    def trace(self):
        return torch.diag(self.A).sum().item() * torch.diag(self.B).sum().item()

    def update_inv(self, damping=_default_damping, calc_A_inv=True, calc_B_inv=True, eps=1e-7, replace=False):
        batched_update_inv([self], damping, calc_A_inv, calc_B_inv, eps, replace)

    def mvp(self, vec_weight, vec_bias=None, use_inv=False, inplace=False):
        """B G A (or B^-1 G A^-1) on a weight gradient viewed as [B_dim, -1], and B b on the bias
        (asdl/symmatrix.py:536-548)."""
        mat_A = self.A_inv if use_inv else self.A
        mat_B = self.B_inv if use_inv else self.B
        direct = inplace and vec_weight.is_contiguous() and vec_weight.dtype == torch.float32
        w = vec_weight if direct else vec_weight.detach().to(torch.float32).contiguous().clone()
        b = None
        if vec_bias is not None:
            direct_b = inplace and vec_bias.is_contiguous() and vec_bias.dtype == torch.float32
            b = vec_bias if direct_b else vec_bias.detach().to(torch.float32).contiguous().clone()
        kernels.kron_precond(mat_B, mat_A, w.data, b.data if b is not None else None, 1.0)
        if inplace and w is not vec_weight:
            vec_weight.copy_(w)
        if vec_bias is not None:
            if inplace and b is not vec_bias:
                vec_bias.copy_(b)
            return w, b
        return w


    def save(self, root, relative_dir):
        """Writes <root>/<relative_dir>/kron/{A,B}_tril.npy and returns their relative paths under the keys
        'A_tril' / 'B_tril' (asdl/symmatrix.py:471-485)."""
        relative_paths = {}
        for name in ['A', 'B']:
            mat = getattr(self, name, None)
            if mat is None:
                continue
            tril_name = f'{name}_tril'
            relative_path = os.path.join(relative_dir, 'kron', f'{tril_name}.npy')
            _save_as_numpy(os.path.join(root, relative_path), matrix_to_tril(mat))
            relative_paths[tril_name] = relative_path
        return relative_paths

    def load(self, A_path, B_path, device=None):
        """asdl/symmatrix.py:487-491."""
        self.A = tril_to_matrix(_load_from_numpy(A_path, device))
        self.B = tril_to_matrix(_load_from_numpy(B_path, device))
        self._A_dim = self._B_dim = None


class UnitWise:
    """[f, 2, 2] blocks of a BatchNorm / LayerNorm module (asdl/symmatrix.py:617-719)."""

    def __init__(self, data=None, inv=None):
        self.data = data.contiguous() if isinstance(data, torch.Tensor) else data
        self.inv = inv

    def __add__(self, other):
        if not other.has_data:
            return self
        return UnitWise(data=self.data.add(other.data) if self.has_data else other.data)

    def __iadd__(self, other):
        if not other.has_data:
            return self
        if self.has_data:
            self.data.add_(other.data)
        else:
            self.data = other.data
        return self

    @property
    def has_data(self):
        return self.data is not None

    @property
    def has_inv(self):
        return self.inv is not None

    def mul_(self, value):
        if self.has_data:
            self.data.mul_(value)
        return self

    def trace(self):
        return float(torch.diagonal(self.data, dim1=1, dim2=2).sum())

    def save(self, root, relative_dir):
        """Writes the [f, 2, 2] blocks whole to <root>/<relative_dir>/unit_wise.npy (asdl/symmatrix.py:672-676)."""
        relative_path = os.path.join(relative_dir, 'unit_wise.npy')
        _save_as_numpy(os.path.join(root, relative_path), self.data)
        return relative_path

    def load(self, path=None, device=None):
        """asdl/symmatrix.py:678-680."""
        if path:
            self.data = _load_from_numpy(path, device).contiguous()

    def update_inv(self, damping=_default_damping, replace=False):
        """asdl/symmatrix.py:687-699: an all-zero tensor keeps its old inverse (none)."""
        batched_unit_update_inv([self], damping, replace)

    def mvp(self, vec_weight, vec_bias, use_inv=False, inplace=False):
        """asdl/symmatrix.py:701-719 for modules with one (weight, bias) pair per block."""
        mat = self.inv if use_inv else self.data
        if mat is None:
            raise ValueError('inv does not exist.' if use_inv else 'data do not exist.')
        if vec_bias is None or vec_weight.shape != vec_bias.shape or mat.ndim != 3 or mat.shape[1:] != (2, 2):
            raise NotImplementedError('unit-wise blocks larger than 2 x 2 (Linear / Conv2d) are not on this path')
        if not inplace:
            vec_weight, vec_bias = vec_weight.clone(), vec_bias.clone()
        w = vec_weight if vec_weight.is_contiguous() else vec_weight.contiguous()
        b = vec_bias if vec_bias.is_contiguous() else vec_bias.contiguous()
        kernels.unit_wise_mvp(mat, w.view(-1), b.view(-1))
        if w is not vec_weight:
            vec_weight.copy_(w)
        if b is not vec_bias:
            vec_bias.copy_(b)
        return vec_weight, vec_bias


class SymMatrix:
    def __init__(self, data=None, inv=None, kron=None, kfe=None, diag=None, unit=None,
                 kron_A=None, kron_B=None, kron_A_inv=None, kron_B_inv=None):
        self.data: Tensor = data
        self.inv: Tensor = inv
        if not _is_all_none([kron_A, kron_B, kron_A_inv, kron_B_inv]):
            self.kron = Kron(kron_A, kron_B, kron_A_inv, kron_B_inv)
        else:
            self.kron: Kron = kron
        self.kfe = kfe
        self.diag = diag
        self.unit = unit

    def __repr__(self):
        parts = []
        if self.has_kron:
            for key in ('A', 'B', 'A_inv', 'B_inv'):
                v = getattr(self.kron, key)
                if v is not None:
                    parts.append(f'kron.{key} {tuple(v.shape)}')
        if self.has_unit:
            for key in ('data', 'inv'):
                v = getattr(self.unit, key)
                if v is not None:
                    parts.append(f'unit.{key} {tuple(v.shape)}')
        return 'SymMatrix(' + ', '.join(parts) + ')'

    @property
    def has_data(self):
        return self.data is not None

    @property
    def has_kron(self):
        return self.kron is not None

    @property
    def has_kfe(self):
        return self.kfe is not None

    @property
    def has_diag(self):
        return self.diag is not None

    @property
    def has_unit(self):
        return self.unit is not None

    def _only_kron(self, what):
        if self.has_data or self.has_kfe or self.has_diag:
            raise NotImplementedError(f'{what}: only the Kronecker-factored and unit-wise shapes are on this path')

    def __iadd__(self, other):
        self._only_kron('__iadd__')
        if other.kron is not None:
            if self.kron is not None:
                self.kron += other.kron
            else:
                self.kron = other.kron
        if other.unit is not None:
            if self.unit is not None:
                self.unit += other.unit
            else:
                self.unit = other.unit
        return self

    def mul_(self, value):
        self._only_kron('mul_')
        if self.has_kron:
            self.kron.mul_(value)
        if self.has_unit:
            self.unit.mul_(value)
        return self

    def update_inv(self, damping=_default_damping, replace=False):
        self._only_kron('update_inv')
        if self.has_kron:
            self.kron.update_inv(damping, replace=replace)
        if self.has_unit:
            self.unit.update_inv(damping, replace=replace)

    def save(self, root, relative_dir):
        """Saves what the matrix holds below <root>/<relative_dir> and returns the relative paths, keyed as in
        asdl/symmatrix.py:226-244: 'tril' (full matrix, packed lower triangle), 'kron' ({'A_tril', 'B_tril'}),
        'unit_wise'.  A diagonal part is not on this path."""
        if self.has_diag:
            raise NotImplementedError('save: the diagonal shape is not on this path')
        relative_paths = {}
        if self.has_data:
            relative_path = os.path.join(relative_dir, 'tril.npy')
            _save_as_numpy(os.path.join(root, relative_path), matrix_to_tril(self.data))
            relative_paths['tril'] = relative_path
        if self.has_kron:
            relative_paths['kron'] = self.kron.save(root, relative_dir)
        if self.has_unit:
            relative_paths['unit_wise'] = self.unit.save(root, relative_dir)
        return relative_paths

    def load(self, path=None, kron_path=None, diag_path=None, unit_path=None, device=None):
        """asdl/symmatrix.py:246-269; ``device`` None is the current GPU."""
        if diag_path is not None:
            raise NotImplementedError('load: the diagonal shape is not on this path')
        if path:
            self.data = tril_to_matrix(_load_from_numpy(path, device))
        if kron_path is not None:
            if not self.has_kron:
                self.kron = Kron(A=None, B=None)
            self.kron.load(A_path=kron_path['A_tril'], B_path=kron_path['B_tril'], device=device)
        if unit_path is not None:
            if not self.has_unit:
                self.unit = UnitWise()
            self.unit.load(path=unit_path, device=device)

    def mvp(self, vectors=None, vec_weight=None, vec_bias=None, use_inv=False, inplace=False):
        raise NotImplementedError('SymMatrix.mvp with a full / layer-wise matrix is not on this path; '
                                  'use SymMatrix.kron.mvp')
