"""Test-only stand-ins for asdl_amd.kernels built on the CPU oracle, so that the host logic
(hooks, schedules, result store, batching) can be exercised without a GPU.  Installed with
pytest's monkeypatch; the product never imports this file."""
import torch

from oracle import cpu_ref as R


def syrk_tn(x, out=None, alpha=1.0, beta=0.0, round_bf16=False):
    x = x.bfloat16() if round_bf16 else x
    val = alpha * R.linear_cov_kron_A(x.float())
    if out is None:
        return val
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def conv_syrk(x, kernel_size, stride, padding, out=None, alpha=1.0, beta=0.0, round_bf16=False):
    x = x.bfloat16() if round_bf16 else x
    col = R.im2col_2d(x.float(), kernel_size, stride, padding)
    m = col.transpose(0, 1).flatten(start_dim=1)
    val = alpha * (m @ m.T)
    if out is None:
        return val
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def syrk_nt(x, out=None, alpha=1.0, beta=0.0):
    if x.ndim == 2:
        x = x.unsqueeze(0)
    m = x.float().transpose(0, 1).flatten(start_dim=1)
    val = alpha * (m @ m.T)
    if out is None:
        return val
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def kron_damping(A_list, B_list, damping, eps=1e-7, eig_scale=None):
    lam = torch.empty(len(A_list), 2)
    nz = torch.empty(len(A_list), 2, dtype=torch.int32)
    for i, (A, B) in enumerate(zip(A_list, B_list)):
        sa, sb = eig_scale[i] if eig_scale is not None else (1.0, 1.0)
        # a scale on an eigenvalue mean is a scale on the matrix (square) or on its square root (row matrix)
        As = A * sa if A.shape[0] == A.shape[1] else A * sa ** 0.5
        Bs = B * sb if B.shape[0] == B.shape[1] else B * sb ** 0.5
        lam[i, 0], lam[i, 1] = R.swift_kron_damping(As, Bs, damping, eps)
        nz[i, 0] = int(not bool(torch.all(A == 0)))
        nz[i, 1] = int(not bool(torch.all(B == 0)))
    return lam, nz


def chol_inv_batched(mats, outs, lam, lam_stride=1, active=None, active_stride=1, info=None):
    if info is None:
        info = torch.empty(len(mats), dtype=torch.int32)
    info.zero_()
    for b, (m, o) in enumerate(zip(mats, outs)):
        if active is not None and int(active[b * active_stride]) == 0:
            continue
        try:
            o.copy_(R.cholesky_inv(m, float(lam[b * lam_stride])))
        except torch.linalg.LinAlgError:
            info[b] = 1
    return info


chol_inv_grouped = chol_inv_batched    # same contract; the stand-in never needed equal sizes


def cholesky_inv(X, damping=1e-7):
    return R.cholesky_inv(X, damping)


def conv_patch_sum(x, kernel_size=(1, 1), stride=(1, 1), padding=(0, 0), out=None, alpha=1.0, beta=0.0):
    x = x.float()
    if x.ndim == 2:
        val = x
    elif x.ndim == 3:
        val = x.sum(-1)
    else:
        val = R.im2col_2d(x, kernel_size, stride, padding).sum(-1)
    val = alpha * val
    if out is None:
        return val.clone()
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def smw_inv(x, lam, out=None, info=None):
    val = R.smw_inv(x, float(lam.reshape(-1)[0]))
    if out is not None:
        out.copy_(val)
        val = out
    if info is None:
        info = torch.zeros(1, dtype=torch.int32)
    info.zero_()
    return val, info


def kron_precond(B_inv, A_inv, grad_w, grad_b=None, grad_scale=1.0):
    if grad_b is not None:
        w, b = R.kron_mvp(A_inv, B_inv, grad_w, grad_b)
        grad_b.copy_(grad_scale * b)
    else:
        w = R.kron_mvp(A_inv, B_inv, grad_w)
    grad_w.copy_(grad_scale * w)
    return grad_w, grad_b


def gemm(A, B, out=None, transA=False, transB=False, alpha=1.0, beta=0.0):
    val = alpha * ((A.T if transA else A) @ (B.T if transB else B))
    if out is None:
        return val
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def unit_wise_stats(y, g, weight, bias, out=None, alpha=1.0, beta=0.0):
    f = weight.numel()
    shape = (1, f) + (1,) * (y.ndim - 2)
    x = (y.float() - bias.view(shape)) / weight.view(shape)
    gw, gb = x * g.float(), g.float()
    if gw.ndim > 2:
        dims = tuple(range(2, gw.ndim))
        gw, gb = gw.sum(dims), gb.sum(dims)
    ww, bb, wb = (gw ** 2).sum(0), (gb ** 2).sum(0), (gw * gb).sum(0)
    val = alpha * torch.stack([ww, wb, wb, bb], dim=1).reshape(f, 2, 2)
    if out is None:
        return val
    out.copy_(val if beta == 0 else beta * out + val)
    return out


def unit_wise_inv(blocks, damping, out=None):
    flags = torch.tensor([int(bool((blocks != 0).any())), 0x7fffffff], dtype=torch.int32)
    inv = torch.inverse(blocks + damping * torch.eye(2))
    if out is not None:
        out.copy_(inv)
        inv = out
    return inv, flags


def unit_wise_inv_grouped(blocks_list, dampings, outs=None):
    invs, flags = [], []
    for i, blocks in enumerate(blocks_list):
        inv, fl = unit_wise_inv(blocks, dampings[i], out=outs[i] if outs is not None else None)
        invs.append(inv)
        flags.append(fl)
    return invs, torch.stack(flags)


def unit_wise_mvp(mat, vec_weight, vec_bias, scale=1.0):
    w, b = R.unit_wise_mvp(mat, vec_weight * scale, vec_bias * scale)
    vec_weight.copy_(w)
    vec_bias.copy_(b)
    return vec_weight, vec_bias


def identity_where_zero(outs, nonzero, flag_index):
    flags = nonzero.view(-1)
    for out, i in zip(outs, flag_index):
        if int(flags[i]) == 0:
            out.copy_(torch.eye(out.shape[0], dtype=out.dtype))


def install(monkeypatch):
    from asdl_amd import kernels
    for name in ['syrk_tn', 'conv_syrk', 'syrk_nt', 'kron_damping', 'chol_inv_batched', 'chol_inv_grouped', 'cholesky_inv',
                 'kron_precond', 'gemm', 'unit_wise_stats', 'unit_wise_inv', 'unit_wise_inv_grouped', 'unit_wise_mvp', 'conv_patch_sum', 'smw_inv', 'identity_where_zero']:
        monkeypatch.setattr(kernels, name, globals()[name])
