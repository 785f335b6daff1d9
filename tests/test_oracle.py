"""Pins the CPU oracle: closed forms, invariants, library routines, brute force, and the golden
runs written from the reference (tests/golden/make_golden.py)."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from conftest import GOLDEN
from models_small import GOLDEN_KFAC, GOLDEN_SHAMPOO, get_mlp
from oracle import cpu_ref as R


def relerr(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-300))


def grad_close(got, ref, tol):
    """Relative error below tol, or both essentially zero (a bias in front of a normalisation layer has an
    exactly zero gradient; what is left of it in fp32 is rounding noise)."""
    ref = ref.double()
    got = got.detach().double().cpu()
    if float(ref.norm()) < 1e-6:
        return float((got - ref).norm()) < 1e-5
    return float((got - ref).norm() / ref.norm()) < tol


# ----------------------------------------------------------------- factors
def test_linear_factors_closed_form():
    torch.manual_seed(0)
    a = torch.randn(3, 7, 11)
    g = torch.randn(3, 7, 5)
    A = R.linear_cov_kron_A(a)
    B = R.linear_cov_kron_B(g)
    a2 = a.reshape(-1, 11).double()
    assert A.shape == (11, 11) and B.shape == (5, 5)
    assert relerr(A, a2.T @ a2) < 1e-6
    torch.testing.assert_close(A, A.T)
    assert abs(float(A.trace()) - float((a ** 2).sum())) < 1e-3
    assert relerr(B, g.reshape(-1, 5).double().T @ g.reshape(-1, 5).double()) < 1e-6


def test_single_datum_kron_is_exact_fisher():
    # test/grad_maker/test_fisher.py:152-156: for one datum kron(B, A) equals the weight block of
    # the per-example-gradient outer product and the bias block equals B.
    torch.manual_seed(1)
    lin = nn.Linear(5, 4)
    x = torch.randn(1, 5)
    y = lin(x)
    gy = torch.randn(1, 4)
    gw, gb = torch.autograd.grad(y, [lin.weight, lin.bias], gy)
    A = R.linear_cov_kron_A(x)
    B = R.linear_cov_kron_B(gy)
    torch.testing.assert_close(torch.outer(gw.flatten(), gw.flatten()), torch.kron(B, A))
    torch.testing.assert_close(torch.outer(gb, gb), B)


def _brute_im2col(x, kh, kw, sy, sx, ph, pw):
    n, c, h, w = x.shape
    ho = (h + 2 * ph - kh) // sy + 1
    wo = (w + 2 * pw - kw) // sx + 1
    out = torch.zeros(n, c * kh * kw, ho * wo, dtype=x.dtype)
    for b in range(n):
        for ci in range(c):
            for ky in range(kh):
                for kx in range(kw):
                    for oy in range(ho):
                        for ox in range(wo):
                            iy, ix = oy * sy + ky - ph, ox * sx + kx - pw
                            if 0 <= iy < h and 0 <= ix < w:
                                out[b, (ci * kh + ky) * kw + kx, oy * wo + ox] = x[b, ci, iy, ix]
    return out


@pytest.mark.parametrize('k,s,p,hw', [((2, 2), (1, 1), (0, 0), (4, 4)), ((3, 3), (1, 1), (1, 1), (6, 5)),
                                        ((3, 3), (2, 2), (1, 1), (7, 8)), ((1, 1), (2, 2), (0, 0), (6, 6)),
                                        ((7, 7), (2, 2), (3, 3), (12, 12)), ((3, 2), (2, 1), (0, 1), (9, 6))])
def test_im2col_vs_unfold_and_brute_force(k, s, p, hw):
    torch.manual_seed(2)
    x = torch.randn(2, 3, *hw)
    col = R.im2col_2d(x, k, s, p)
    torch.testing.assert_close(col, F.unfold(x, k, padding=p, stride=s))
    torch.testing.assert_close(col, _brute_im2col(x, *k, *s, *p))
    A = R.conv_cov_kron_A(x, k, s, p)
    bf = _brute_im2col(x.double(), *k, *s, *p)
    ref = sum(bf[i] @ bf[i].T for i in range(2)) / bf.shape[-1]
    assert relerr(A, ref) < 1e-6


def test_conv_B_not_divided_by_out_size():
    torch.manual_seed(3)
    g = torch.randn(2, 4, 3, 3)
    B = R.conv_cov_kron_B(g)
    ref = torch.zeros(4, 4, dtype=torch.float64)
    for n in range(2):
        for y in range(3):
            for x in range(3):
                v = g[n, :, y, x].double()
                ref += torch.outer(v, v)
    assert relerr(B, ref) < 1e-6


def test_single_datum_conv_fisher_bias_block():
    torch.manual_seed(4)
    conv = nn.Conv2d(3, 4, 2)
    x = torch.randn(1, 3, 4, 4)
    y = conv(x)
    gy = torch.randn_like(y)
    gw, gb = torch.autograd.grad(y, [conv.weight, conv.bias], gy)
    # sum over positions of per-position outer products: dW = sum_pos g_pos x_pos^T
    col = R.im2col_2d(x, (2, 2), (1, 1), (0, 0))[0]
    torch.testing.assert_close(gw.view(4, -1), gy.flatten(2)[0] @ col.T)
    torch.testing.assert_close(gb, gy.sum(dim=(0, 2, 3)))


# ----------------------------------------------------------------- damping, inverse, mvp
def test_kron_damping_formula_and_special_cases():
    torch.manual_seed(5)
    X = torch.randn(20, 6)
    Y = torch.randn(20, 3)
    A, B = X.T @ X, Y.T @ Y
    dA, dB = R.kron_damping(A, B, 0.04)
    pi = ((A.trace() / 6) / (B.trace() / 3)) ** 0.5          # test_fisher.py:267-273
    assert abs(dA - max(0.2 * float(pi), 1e-7)) < 1e-6 and abs(dB - max(0.2 / float(pi), 1e-7)) < 1e-6
    assert abs(dA * dB - 0.04) < 1e-6
    assert R.kron_damping(A, torch.zeros(3, 3), 0.04) == (0.04, 0.04)      # pi = inf
    assert R.kron_damping(torch.zeros(6, 6), B, 0.04) == (0.04, 0.04)      # pi = 0
    dA, dB = R.kron_damping(A * 1e-20, B, 1e-12)
    assert dA == 1e-7                                                      # eps floor


def test_cholesky_inv_identity_and_input_unchanged():
    torch.manual_seed(6)
    X = torch.randn(10, 30)
    A = X @ X.T
    A0 = A.clone()
    inv = R.cholesky_inv(A, 0.5)
    torch.testing.assert_close(A, A0)
    Ad = A + 0.5 * torch.eye(10)
    torch.testing.assert_close(Ad @ inv, torch.eye(10), atol=1e-4, rtol=0)
    assert relerr(inv, torch.linalg.inv(Ad.double())) < 1e-5
    with pytest.raises(torch.linalg.LinAlgError):
        R.cholesky_inv(-torch.eye(4), 0.1)


def test_kron_update_inv_skips_zero_factor():
    A = torch.eye(3)
    Ai, Bi = R.kron_update_inv(A, torch.zeros(2, 2), 0.1)
    assert Bi is None and Ai is not None


def test_kron_mvp_is_kronecker_inverse():
    torch.manual_seed(7)
    Ai = torch.randn(5, 5)
    Ai = Ai @ Ai.T
    Bi = torch.randn(3, 3)
    Bi = Bi @ Bi.T
    G = torch.randn(3, 5)
    b = torch.randn(3)
    w, bb = R.kron_mvp(Ai, Bi, G, b)
    torch.testing.assert_close(w.flatten(), torch.kron(Bi, Ai) @ G.flatten(), atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(bb, Bi @ b)
    conv_g = torch.randn(3, 5, 1, 1)
    torch.testing.assert_close(R.kron_mvp(Ai, Bi, conv_g).flatten(), w.new_tensor(torch.kron(Bi, Ai) @ conv_g.flatten()),
                               atol=1e-4, rtol=1e-4)


# ----------------------------------------------------------------- Shampoo pieces
def test_power_iter_converges_to_lambda_max():
    torch.manual_seed(8)
    X = torch.randn(50, 12).double()
    S = X.T @ X
    lam, iters = R.power_iter(S, torch.rand(12).double() * 2 - 1, error_tolerance=1e-12, num_iters=10000)
    assert abs(float(lam) - float(torch.linalg.eigvalsh(S)[-1])) / float(lam) < 1e-6


@pytest.mark.parametrize('p', [2, 4, 8])
def test_compute_power_closed_form(p):
    torch.manual_seed(9)
    X = torch.randn(60, 10).double()
    S = X.T @ X / 60
    S0 = S.clone()
    root, iters, err = R.compute_power(S, p, torch.rand(10).double() * 2 - 1, ridge_epsilon=1e-6)
    lam = torch.linalg.eigvalsh(S0)[-1]
    # ridge stays in the statistic (shampoo.py:498-499)
    assert relerr(S, S0 + 1e-6 * lam * torch.eye(10).double()) < 1e-6
    w, V = torch.linalg.eigh(S)
    ref = V @ torch.diag(w ** (-1.0 / p)) @ V.T
    assert relerr(root, ref) < 1e-5
    assert relerr(torch.linalg.matrix_power(root, p) @ S, torch.eye(10).double()) < 1e-5
    assert 0 < iters < 100


def test_mat_power_generic_exponent():
    torch.manual_seed(10)
    M = torch.randn(4, 4).double() * 0.5
    for p in [1, 2, 3, 4, 6, 8]:
        assert relerr(R.mat_power(M, p), torch.linalg.matrix_power(M, p)) < 1e-12


def test_compute_power_matches_reference_golden():
    z = np.load(os.path.join(GOLDEN, 'power.npz'))
    names = sorted({k.split('/')[0] for k in z.files})
    assert len(names) >= 6
    for name in names:
        mat = torch.from_numpy(z[f'{name}/in']).clone()
        root, iters, err = R.compute_power(mat, int(z[f'{name}/p']), torch.from_numpy(z[f'{name}/v0']),
                                           ridge_epsilon=float(z[f'{name}/eps']))
        torch.testing.assert_close(root, torch.from_numpy(z[f'{name}/root']), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(mat, torch.from_numpy(z[f'{name}/mat_after']), rtol=1e-6, atol=1e-12)


def test_shampoo_statistics_and_precondition_closed_form():
    torch.manual_seed(11)
    G = torch.randn(4, 6)
    stats = [torch.zeros(4, 4), torch.zeros(6, 6)]
    R.shampoo_statistics(G, stats)
    torch.testing.assert_close(stats[0], G @ G.T)
    torch.testing.assert_close(stats[1], G.T @ G)
    R.shampoo_statistics(G, stats, ema_decay=0.25)
    torch.testing.assert_close(stats[0], G @ G.T)             # 0.75 S + 0.25 S
    P0, P1 = torch.randn(4, 4), torch.randn(6, 6)
    torch.testing.assert_close(R.shampoo_precondition(G, [P0, P1]), P0.T @ G @ P1)


# ----------------------------------------------------------------- golden end-to-end runs
def _load_model(factory, z):
    model = factory()
    sd = {k[len('init/'):]: torch.from_numpy(z[k]) for k in z.files if k.startswith('init/')}
    model.load_state_dict(sd)
    return model


@pytest.mark.parametrize('tag', sorted(GOLDEN_KFAC))
def test_kfac_oracle_matches_reference_golden(tag):
    factory, fisher_type, ema, damping, seed, ci, pi = GOLDEN_KFAC[tag]
    z = np.load(os.path.join(GOLDEN, f'kfac_{tag}.npz'))
    model = _load_model(factory, z)
    n_steps = len({k.split('/')[0] for k in z.files if k.startswith('step')})
    x0 = torch.from_numpy(z['step0/x'])
    orc = R.KfacOracle(model, data_size=x0.shape[0], damping=damping, ema_decay=ema, fisher_type=fisher_type,
                       seed=seed, curvature_upd_interval=ci, preconditioner_upd_interval=pi,
                       unit_wise_norm=True,        # the fixtures come from the default KfacGradientMaker
                       swift=tag.startswith('swift_'))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    for step in range(n_steps):
        opt.zero_grad(set_to_none=True)
        x = torch.from_numpy(z[f'step{step}/x'])
        t = torch.from_numpy(z[f'step{step}/t'])
        y, loss = orc.forward_and_backward(x, t)
        torch.testing.assert_close(loss, torch.from_numpy(z[f'step{step}/loss']), rtol=1e-5, atol=1e-6)
        for name, p in model.named_parameters():
            ref = torch.from_numpy(z[f'step{step}/grad/{name}'])
            assert grad_close(p.grad, ref, 2e-4), (tag, step, name, relerr(p.grad, ref))
        for key in z.files:
            if not key.startswith(f'step{step}/kron/'):
                continue
            _, _, mname, which = key.split('/')
            got = getattr(orc, which).get(mname)
            assert got is not None, key
            assert relerr(got, torch.from_numpy(z[key])) < 2e-4, (tag, key)
        for key in z.files:
            if not key.startswith(f'step{step}/unit/'):
                continue
            _, _, mname, which = key.split('/')
            got = (orc.unit if which == 'data' else orc.unit_inv).get(mname)
            assert got is not None, key
            assert relerr(got, torch.from_numpy(z[key])) < 2e-4, (tag, key, relerr(got, torch.from_numpy(z[key])))
        opt.step()


@pytest.mark.parametrize('tag', sorted(GOLDEN_SHAMPOO))
def test_shampoo_oracle_matches_reference_golden(tag):
    damping, ema, ci, pi = GOLDEN_SHAMPOO[tag]
    z = np.load(os.path.join(GOLDEN, f'shampoo_{tag}.npz'))
    model = _load_model(get_mlp, z)
    orc = R.ShampooOracle(model, damping=damping, ema_decay=ema, curvature_upd_interval=ci,
                          preconditioner_upd_interval=pi)
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    torch.manual_seed(int(z['seed']))
    n_steps = len({k.split('/')[0] for k in z.files if k.startswith('step')})
    for step in range(n_steps):
        opt.zero_grad(set_to_none=True)
        x = torch.from_numpy(z[f'step{step}/x'])
        t = torch.from_numpy(z[f'step{step}/t'])
        orc.forward_and_backward(x, t)
        for i in range(len(orc.params)):
            for j in range(2):
                torch.testing.assert_close(orc.stats[i][j], torch.from_numpy(z[f'step{step}/stat/{i}/{j}']),
                                           rtol=1e-4, atol=1e-12)
                assert relerr(orc.precs[i][j], torch.from_numpy(z[f'step{step}/prec/{i}/{j}'])) < 1e-4
        for name, p in model.named_parameters():
            assert relerr(p.grad, torch.from_numpy(z[f'step{step}/grad/{name}'])) < 1e-4, (tag, step, name)
        opt.step()


# ------------------------------------------------------------------ unit-wise blocks (BatchNorm / LayerNorm)
def _per_sample_blocks(module, x, G, sample_of_row=None):
    """Brute force: gradient of sum(y_n * G_n) with respect to (weight, bias), one sample at a time by autograd."""
    y = module(x)
    n = x.shape[0]
    f = module.weight.numel()
    blocks = torch.zeros(f, 2, 2, dtype=torch.float64)
    rows = y.reshape(n, -1) if sample_of_row is None else None
    if sample_of_row is None:
        groups = [[i] for i in range(n)]
        yr, Gr = y, G
    else:
        yr, Gr = y.reshape(-1, f), G.reshape(-1, f)
        groups = [[i] for i in range(yr.shape[0])]
    for idx in groups:
        gw, gb = torch.autograd.grad((yr[idx] * Gr[idx]).sum(), [module.weight, module.bias], retain_graph=True)
        v = torch.stack([gw.flatten().double(), gb.flatten().double()], dim=1)      # [f, 2]
        blocks += v.unsqueeze(2) * v.unsqueeze(1)
    return blocks, y.detach()


@pytest.mark.parametrize('kind', ['bn1d', 'bn2d', 'ln', 'ln_seq'])
def test_norm_cov_unit_wise_matches_per_sample_autograd(kind):
    torch.manual_seed(11)
    if kind == 'bn1d':
        m, x = nn.BatchNorm1d(5), torch.randn(7, 5)
    elif kind == 'bn2d':
        m, x = nn.BatchNorm2d(4), torch.randn(6, 4, 3, 5)
    elif kind == 'ln':
        m, x = nn.LayerNorm(6), torch.randn(9, 6)
    else:
        m, x = nn.LayerNorm(6), torch.randn(3, 4, 6)
    with torch.no_grad():
        m.weight.uniform_(0.5, 1.5)
        m.bias.uniform_(-0.5, 0.5)
    if isinstance(m, (nn.BatchNorm1d, nn.BatchNorm2d)):
        m.running_mean.normal_()
        m.running_var.uniform_(0.5, 2.0)
        m.eval()                          # samples are independent, so per-sample gradients are well defined
    x = x.double()
    m = m.double()
    G = torch.randn_like(x)
    ref, y = _per_sample_blocks(m, x, G, sample_of_row=True if kind.startswith('ln') else None)
    got = R.norm_cov_unit_wise(m, y, G)
    assert got.shape == ref.shape
    assert relerr(got, ref) < 1e-10
    assert torch.equal(got[:, 0, 1], got[:, 1, 0])


def test_unit_wise_inv_and_mvp():
    torch.manual_seed(12)
    v = torch.randn(9, 2, 3, dtype=torch.float64)
    blocks = v @ v.transpose(1, 2)
    inv = R.unit_wise_inv(blocks, 0.1)
    eye = torch.eye(2, dtype=torch.float64)
    assert relerr((blocks + 0.1 * eye) @ inv, eye.expand(9, 2, 2)) < 1e-12
    assert R.unit_wise_inv(torch.zeros(3, 2, 2), 0.1) is None
    w, b = torch.randn(9, dtype=torch.float64), torch.randn(9, dtype=torch.float64)
    dense = torch.block_diag(*inv)                                  # [18, 18], (w_f, b_f) interleaved
    ref = dense @ torch.stack([w, b], dim=1).flatten()
    mw, mb = R.unit_wise_mvp(inv, w, b)
    assert relerr(torch.stack([mw, mb], dim=1).flatten(), ref) < 1e-12


def test_tril_packing_matches_docstring_example_and_numpy():
    # the worked example of asdl/symmatrix.py:25-54
    mat = torch.tensor([[1., 9., 9.], [2., 3., 9.], [4., 5., 6.]])
    tril = R.matrix_to_tril(mat)
    assert tril.tolist() == [1., 2., 3., 4., 5., 6.]
    assert R.tril_to_matrix(tril).tolist() == [[1., 2., 4.], [2., 3., 5.], [4., 5., 6.]]
    # numpy's row-major lower-triangle indices on a larger, non-symmetric input; round trip
    g = torch.Generator().manual_seed(0)
    big = torch.randn(37, 37, generator=g)
    rows, cols = np.tril_indices(37)
    packed = R.matrix_to_tril(big)
    assert np.array_equal(packed.numpy(), big.numpy()[rows, cols])
    full = R.tril_to_matrix(packed)
    assert torch.equal(full, full.T) and torch.equal(torch.tril(full), torch.tril(big))
    assert torch.equal(R.matrix_to_tril(full), packed)


def test_smw_inv_is_the_inverse_of_the_damped_gram_form():
    # asdl/utils.py:107-115 implements (x^T x / n + damping I)^-1 through the n x n Gram matrix
    g = torch.Generator().manual_seed(3)
    for n, d, lam in [(4, 9, 1e-2), (8, 27, 0.3), (1, 5, 1e-3)]:
        x = torch.randn(n, d, generator=g, dtype=torch.float64)
        dense = torch.linalg.inv(x.T @ x / n + lam * torch.eye(d, dtype=torch.float64))
        assert relerr(R.smw_inv(x, lam), dense) < 1e-9
        assert relerr(R.smw_inv(x.float(), lam), dense) < 1e-3        # fp32: cond ~ |x|^2 / (n lam)


def test_swift_factors_are_row_sums_or_the_ordinary_factors():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(3, 4, 6, 5, generator=g)                   # n = 3 < d = 4*3*3 = 36
    got = R.conv_cov_swift_kron_A(x, (3, 3), (2, 1), (1, 0))
    want = F.unfold(x, (3, 3), padding=(1, 0), stride=(2, 1)).sum(-1)
    assert got.shape == (3, 36) and relerr(got, want) < 1e-6
    x = torch.randn(40, 4, 6, 5, generator=g)                  # n = 40 >= 36: the ordinary factor
    assert relerr(R.conv_cov_swift_kron_A(x, (3, 3), (2, 1), (1, 0)), R.conv_cov_kron_A(x, (3, 3), (2, 1), (1, 0))) == 0
    gr = torch.randn(3, 7, 4, 4, generator=g)
    assert relerr(R.conv_cov_swift_kron_B(gr), gr.sum((2, 3))) < 1e-6
    assert R.conv_cov_swift_kron_B(torch.randn(9, 7, 2, 2, generator=g)).shape == (7, 7)
    a = torch.randn(3, 8, generator=g)
    assert torch.equal(R.linear_cov_swift(a), a) and R.linear_cov_swift(torch.randn(8, 3, generator=g)).shape == (3, 3)
    # eigenvalue mean of a row matrix: trace of its Gram form over the column count
    la, lb = R.swift_kron_damping(a, torch.eye(5) * 2.0, 1e-2)
    pi = ((a ** 2).sum() / 8 / 2.0) ** 0.5
    assert abs(la - 0.1 * float(pi)) < 1e-6 and abs(lb - 0.1 / float(pi)) < 1e-6


def test_merge_small_dims_and_block_partition():
    # the worked examples of asdl/precondition/shampoo.py:370-384
    assert R.merge_small_dims([1, 2, 512, 1, 2048, 1, 3, 4], 1024) == [1024, 2048, 12]
    assert R.merge_small_dims([1, 2, 768, 1, 2048], 1024) == [2, 768, 2048]
    # the example of the class docstring (:398-404): (4096, 512) with blocks of 1024 -> four (1024, 512) tensors
    blocks = R.block_slices((4096, 512), 1024)
    assert [(b[0].stop - b[0].start, b[1].stop - b[1].start) for b in blocks] == [(1024, 512)] * 4
    # ragged last block, first axis slowest, every element in exactly one block
    blocks = R.block_slices((10, 6), 4)
    assert [(b[0].start, b[0].stop, b[1].start, b[1].stop) for b in blocks] == \
        [(0, 4, 0, 4), (0, 4, 4, 6), (4, 8, 0, 4), (4, 8, 4, 6), (8, 10, 0, 4), (8, 10, 4, 6)]
    count = torch.zeros(10, 6)
    for b in blocks:
        count[b] += 1
    assert bool((count == 1).all())
    assert R.block_slices((3, 5), -1) == [(slice(0, 3), slice(0, 5))]


@pytest.mark.parametrize('tag', ['mat_10x6_b4', 'mat_9x13_b5_ema', 'conv_5x4x3x3_b4'])
def test_partitioned_shampoo_oracle_matches_reference_golden(tag):
    z = np.load(os.path.join(GOLDEN, f'shampoo_blocks_{tag}.npz'))
    orc = R.PartitionedShampooOracle(tuple(int(v) for v in z['shape']), int(z['block_size']), bool(int(z['merge'])),
                                     float(z['damping']), float(z['ema_decay']))
    n_stats = len(orc.statistics)
    assert n_stats == len([k for k in z.files if k.startswith('step0/stat/')])
    for step in range(3):
        grad = torch.from_numpy(z[f'step{step}/grad_in'])
        orc.update_statistics(grad)
        torch.manual_seed(1000 * int(z['seed']) + step)
        orc.update_preconditioners(lambda n: torch.rand(n) * 2 - 1)
        out = orc.precondition(grad)
        for i in range(n_stats):
            torch.testing.assert_close(orc.statistics[i], torch.from_numpy(z[f'step{step}/stat/{i}']), rtol=1e-5, atol=1e-12)
            assert relerr(orc.preconditioners[i], torch.from_numpy(z[f'step{step}/prec/{i}'])) < 1e-4, (tag, step, i)
        assert relerr(out, torch.from_numpy(z[f'step{step}/grad_out'])) < 1e-4, (tag, step)
