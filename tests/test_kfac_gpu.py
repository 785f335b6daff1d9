"""End-to-end K-FAC parity on the GPU: KfacGradientMaker (HIP kernels) against the reference's
golden runs and against the CPU oracle on identical seeded inputs.

Tolerances: factors 1e-5, inverses 1e-4, preconditioned gradients 1e-3 (relative Frobenius norm); looser only
where the test says why.
"""
import copy
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from asdl_amd import PreconditioningConfig, KfacGradientMaker, FISHER_EMP, FISHER_MC, FISHER_EXACT
from conftest import GOLDEN
from models_small import GOLDEN_KFAC
from oracle import cpu_ref as R
import bench_models

pytestmark = pytest.mark.gpu
TOL_FACTOR, TOL_INV, TOL_GRAD = 1e-5, 1e-4, 1e-3


def relerr(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def grad_close(got, ref, tol):
    """Relative error below tol, or both essentially zero (a bias in front of a normalisation layer has an
    exactly zero gradient; what is left of it in fp32 is rounding noise)."""
    ref = ref.double()
    got = got.detach().double().cpu()
    if float(ref.norm()) < 1e-6:
        return float((got - ref).norm()) < 1e-5
    return float((got - ref).norm() / ref.norm()) < tol


def inverse_errors(factor, inv, lam):
    """Distances of a damped inverse from the fp64 inverse of the very factor it was computed from: (this build,
    the fp32 oracle).  The oracle is the reference's arithmetic: LAPACK's Cholesky on the CPU in fp32."""
    dim = factor.shape[0]
    W = factor.double().cuda() + lam * torch.eye(dim, dtype=torch.float64, device='cuda')
    ref = torch.linalg.inv(W)
    e_hip = relerr(inv, ref)
    e_oracle = relerr(R.cholesky_inv(factor.float().cpu(), lam), ref)
    return e_hip, e_oracle


def assert_inverse_as_good_as_oracle(label, factor, inv, lam):
    """The contract for inverses is 1e-4; where the conditioning puts that out of reach of fp32 the inverse may be
    at most twice as far from the fp64 inverse as the oracle's."""
    e_hip, e_oracle = inverse_errors(factor, inv, lam)
    print(f'  inverse {label}: d {factor.shape[0]}, lam {lam:.3e}, vs fp64: here {e_hip:.2e}, fp32 oracle {e_oracle:.2e}',
          flush=True)
    assert e_hip <= max(TOL_INV, 2 * e_oracle), (label, e_hip, e_oracle)
    return e_hip, e_oracle


@pytest.mark.parametrize('tag', sorted(GOLDEN_KFAC))
def test_kfac_gpu_matches_reference_golden(tag):
    factory, fisher_type, ema, damping, seed, ci, pi = GOLDEN_KFAC[tag]
    z = np.load(os.path.join(GOLDEN, f'kfac_{tag}.npz'))
    sd = {k[len('init/'):]: torch.from_numpy(z[k]) for k in z.files if k.startswith('init/')}
    model = factory()
    model.load_state_dict(sd)
    bs = z['step0/x'].shape[0]
    replay = None
    if fisher_type == FISHER_MC:
        # the sampled targets depend on the CPU RNG stream: draw them with the oracle and replay them
        cpu_model = copy.deepcopy(model)
        orc = R.KfacOracle(cpu_model, data_size=bs, damping=damping, ema_decay=ema, fisher_type=fisher_type, seed=seed,
                           curvature_upd_interval=ci, preconditioner_upd_interval=pi, unit_wise_norm=True,
                           swift=tag.startswith('swift_'))
        cpu_opt = torch.optim.SGD(cpu_model.parameters(), lr=0.05)
        replay = []
    model = model.cuda()
    config = PreconditioningConfig(data_size=bs, damping=damping, ema_decay=ema, curvature_upd_interval=ci,
                                   preconditioner_upd_interval=pi)
    gm = KfacGradientMaker(model, config, fisher_type=fisher_type, seed=seed, swift=tag.startswith('swift_'))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    n_steps = len({k.split('/')[0] for k in z.files if k.startswith('step')})
    worst = {}
    for step in range(n_steps):
        x, t = torch.from_numpy(z[f'step{step}/x']), torch.from_numpy(z[f'step{step}/t'])
        if replay is not None:
            cpu_opt.zero_grad(set_to_none=True)
            orc.forward_and_backward(x, t)
            cpu_opt.step()
            targets = orc.last_mc_targets.cuda()
            gm.fisher_maker.sample_targets = lambda dist, i, _t=targets: _t
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(model, x.cuda())
        gm.setup_loss_call(F.cross_entropy, dummy_y, t.cuda())
        print(f'golden {tag} step {step}', flush=True)
        y, loss = gm.forward_and_backward()
        torch.testing.assert_close(loss.cpu(), torch.from_numpy(z[f'step{step}/loss']), rtol=1e-4, atol=1e-5)
        for key in z.files:
            if key.startswith(f'step{step}/kron/'):
                _, _, mname, which = key.split('/')
                got = getattr(model.get_submodule(mname).fisher.kron, which)
                assert got is not None, key
                e = relerr(got, torch.from_numpy(z[key]))
                tol = TOL_INV if which.endswith('_inv') else TOL_FACTOR
                worst[which] = max(worst.get(which, 0.0), e)
                assert e < tol, (key, e)
            if key.startswith(f'step{step}/unit/'):
                _, _, mname, which = key.split('/')
                got = getattr(model.get_submodule(mname).fisher.unit, which)
                assert got is not None, key
                e = relerr(got, torch.from_numpy(z[key]))
                tol = TOL_INV if which == 'inv' else TOL_FACTOR
                worst['unit.' + which] = max(worst.get('unit.' + which, 0.0), e)
                assert e < tol, (key, e)
        for name, p in model.named_parameters():
            assert grad_close(p.grad, torch.from_numpy(z[f'step{step}/grad/{name}']), TOL_GRAD), (tag, step, name)
        opt.step()
    print(f'golden {tag}: worst relative errors ' + ', '.join(f'{k} {v:.1e}' for k, v in sorted(worst.items())), flush=True)


def _run_pair(model_cpu, x, t, damping, ema=-1, steps=1, autocast=False, fisher_type=FISHER_EMP, tol_grad=TOL_GRAD,
              tol_inv=TOL_INV, check_inv=True, inv_vs_fp64=False):
    """Runs the product on the GPU and the oracle on the CPU on identical inputs; returns max errors.
    ``inv_vs_fp64`` (factors not accumulated): every inverse is judged on the factor the GPU itself formed (the
    per-module scratch buffer), against the fp64 inverse of that factor and the oracle's fp32 inverse of it, by the
    rule of assert_inverse_as_good_as_oracle; for ill-conditioned factors, where the two fp32 inverses of slightly
    different factors cannot agree to 1e-4."""
    bs = x.shape[0]
    model_gpu = copy.deepcopy(model_cpu).cuda()
    ignore = [nn.BatchNorm2d, nn.BatchNorm1d, nn.LayerNorm]
    config = PreconditioningConfig(data_size=bs, damping=damping, ema_decay=ema, ignore_modules=ignore)
    gm = KfacGradientMaker(model_gpu, config, fisher_type=fisher_type)
    orc = R.KfacOracle(model_cpu, data_size=bs, damping=damping, ema_decay=ema, fisher_type=fisher_type,
                       factor_dtype=torch.float32)
    worst_g = worst_i = 0.0
    for step in range(steps):
        model_cpu.zero_grad(set_to_none=True)
        model_gpu.zero_grad(set_to_none=True)
        if autocast:
            def fwd_cpu(inp):
                with torch.autocast('cpu', dtype=torch.bfloat16):
                    return model_cpu(inp).float()

            def fwd_gpu(inp):
                with torch.autocast('cuda', dtype=torch.bfloat16):
                    return model_gpu(inp).float()
        else:
            fwd_cpu, fwd_gpu = model_cpu, model_gpu
        y_ref, loss_ref = _oracle_step(orc, fwd_cpu, x, t)
        dummy_y = gm.setup_model_call(fwd_gpu, x.cuda())
        gm.setup_loss_call(F.cross_entropy, dummy_y, t.cuda())
        y, loss = gm.forward_and_backward()
        assert abs(float(loss) - float(loss_ref)) < 1e-3 * max(1.0, abs(float(loss_ref)))
        for (name, m_cpu), (_, m_gpu) in zip(model_cpu.named_modules(), model_gpu.named_modules()):
            if not isinstance(m_cpu, (nn.Linear, nn.Conv2d)):
                continue
            if check_inv:
                for which, store in (('A_inv', orc.A_inv), ('B_inv', orc.B_inv)):
                    e = relerr(getattr(m_gpu.fisher.kron, which), store[name])
                    worst_i = max(worst_i, e)
                    assert e < tol_inv, (name, which, e)
            if inv_vs_fp64:
                cache = getattr(m_gpu, '_asdl_amd_factor_cache')
                A, B = cache['A'], cache['B']
                pi = ((float(A.diagonal().sum().double()) / A.shape[0]) / (float(B.diagonal().sum().double()) / B.shape[0])) ** 0.5
                assert_inverse_as_good_as_oracle(f'{name} A', A, m_gpu.fisher.kron.A_inv, max(damping ** 0.5 * pi, 1e-7))
                assert_inverse_as_good_as_oracle(f'{name} B', B, m_gpu.fisher.kron.B_inv, max(damping ** 0.5 / pi, 1e-7))
            for pn, p_cpu in m_cpu.named_parameters(recurse=False):
                e = relerr(getattr(m_gpu, pn).grad, p_cpu.grad)
                worst_g = max(worst_g, e)
                assert e < tol_grad, (name, pn, e)
    return worst_g, worst_i


class _CallableModel:
    """Lets KfacOracle call an autocast wrapper while still iterating the module's parameters."""

    def __init__(self, module, fn):
        self._module, self._fn = module, fn

    def __call__(self, x):
        return self._fn(x)

    def parameters(self):
        return self._module.parameters()


def _oracle_step(orc, fwd, x, t):
    module = orc.model
    orc.model = _CallableModel(module, fwd)
    try:
        return orc.forward_and_backward(x, t)
    finally:
        orc.model = module


def test_config1_mlp_784_512_512_10_batch128():
    torch.manual_seed(0)
    model = bench_models.mlp()
    x, t = torch.randn(128, 784), torch.randint(0, 10, (128,))
    g, i = _run_pair(model, x, t, damping=0.01)
    print(f'C1 MLP: worst grad err {g:.2e}, worst inverse err {i:.2e}', flush=True)


def test_config1_mlp_ema_three_steps():
    torch.manual_seed(1)
    model = bench_models.mlp()
    x, t = torch.randn(128, 784), torch.randint(0, 10, (128,))
    _run_pair(model, x, t, damping=0.01, ema=0.05, steps=3)


def test_resnet18_cifar_fp32_small_batch():
    # config 3 geometry (3x3 convs up to d = 4608, stride-2 and 1x1 shortcuts) at batch 8.
    # layer4 factors are rank deficient (M = 8*16 < d = 4608), cond(A + lam I) ~ 1e3..1e4: the fp32 inverses of
    # the CPU's and the GPU's factors (which differ by 1e-7) agree to 1.6e-4 only (bar 5e-4), so every inverse is also judged on the
    # GPU's own factor against fp64 and the oracle's inverse of that factor.
    torch.manual_seed(2)
    model = bench_models.resnet18_cifar()
    x, t = torch.randn(8, 3, 32, 32), torch.randint(0, 10, (8,))
    g, i = _run_pair(model, x, t, damping=1e-3, tol_inv=5e-4, tol_grad=5e-3, inv_vs_fp64=True)
    print(f'ResNet-18: worst grad err {g:.2e}, worst inverse err {i:.2e}', flush=True)


@pytest.mark.parametrize('channels_last', [False, True])
def test_small_cnn_bf16_autocast(channels_last):
    # bf16 forward/backward through autocast, fp32 factors accumulated from the bf16 activations.  CPU and GPU
    # bf16 convolutions round differently, so the oracle is fed the very activations / output gradients the GPU
    # run produced (captured with extra hooks) and the GPU's raw gradients: same inputs, same formulas.
    torch.manual_seed(3)
    model = nn.Sequential(nn.Conv2d(3, 16, 3, 1, 1), nn.ReLU(), nn.Conv2d(16, 32, 3, 2, 1), nn.ReLU(),
                          nn.Conv2d(32, 32, 1), nn.ReLU(), nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10)).cuda()
    bs, damping = 16, 1e-2
    x, t = torch.randn(bs, 3, 16, 16).cuda(), torch.randint(0, 10, (bs,)).cuda()
    if channels_last:
        # NHWC activations: conv factors are gathered in place (16 and 32 channels), output gradients stay 4-D
        model = model.to(memory_format=torch.channels_last)
        x = x.contiguous(memory_format=torch.channels_last)

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    layers = [(n, m) for n, m in model.named_modules() if isinstance(m, (nn.Linear, nn.Conv2d))]
    ins, gouts, raw, handles = {}, {}, {}, []
    for name, m in layers:
        def fhook(mod, inp, out, name=name):
            ins[name] = inp[0].detach()
            out.register_hook(lambda g, name=name: gouts.__setitem__(name, g.detach()))
        handles.append(m.register_forward_hook(fhook))
        for pn, p in m.named_parameters(recurse=False):
            handles.append(p.register_hook(lambda g, key=f'{name}.{pn}': raw.__setitem__(key, g.detach().clone())))

    # the capture hooks stay on during the maker's own pass: the oracle gets the very tensors the kernels read
    gm = KfacGradientMaker(model, PreconditioningConfig(data_size=bs, damping=damping), fisher_type=FISHER_EMP)
    model.zero_grad(set_to_none=True)
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
    gm.forward_and_backward()
    for h in handles:
        h.remove()
    assert any(v.dtype == torch.bfloat16 for v in ins.values()), 'autocast should hand bf16 activations to the hooks'
    if channels_last:
        assert any(v.ndim == 4 and not v.is_contiguous() and v.is_contiguous(memory_format=torch.channels_last)
                   for v in ins.values()), 'the hooks should see channels-last activations'
    worst = {}
    for name, m in layers:
        # forward hooks run inside the autocast region: an fp32 input (the first layer's) enters its factor rounded
        # to bf16, as it enters the reference's torch.matmul there and the layer's own convolution
        a = ins[name].bfloat16().float().cpu()
        g = gouts[name].float().cpu()                 # the maker back-propagates the summed loss
        if isinstance(m, nn.Conv2d):
            A = R.conv_cov_kron_A(a, m.kernel_size, m.stride, m.padding) / bs
            B = R.conv_cov_kron_B(g) / bs
        else:
            A, B = R.linear_cov_kron_A(a) / bs, R.linear_cov_kron_B(g) / bs
        A_inv, B_inv = R.kron_update_inv(A, B, damping)
        w, b = R.kron_mvp(A_inv, B_inv, raw[name + '.weight'].float().cpu() / bs, raw[name + '.bias'].float().cpu() / bs)
        errs = dict(A_inv=relerr(m.fisher.kron.A_inv, A_inv), B_inv=relerr(m.fisher.kron.B_inv, B_inv),
                    weight=relerr(m.weight.grad, w), bias=relerr(m.bias.grad, b))
        for k, v in errs.items():
            worst[k] = max(worst.get(k, 0.0), v)
        assert errs['A_inv'] < TOL_INV and errs['B_inv'] < TOL_INV, (name, errs)
        assert errs['weight'] < TOL_GRAD and errs['bias'] < TOL_GRAD, (name, errs)
    print('bf16 autocast cnn: worst relative errors ' + ', '.join(f'{k} {v:.1e}' for k, v in worst.items()), flush=True)


def test_config2_linear_4096_batch8192_bf16_ema():
    """The large single-layer configuration at full size: Linear(4096, 4096) with bias, 8192 rows of bf16 activations
    and output gradients, fp32 factors, damping 1e-3, EMA decay 0.95, two steps (the second one runs the
    beta != 0 accumulate path of the factor kernels at 4096 x 4096).  Everything is judged against fp64 arithmetic on
    the tensors the kernels read (captured by extra hooks during the maker's own pass): A and B against the fp64
    running averages of the fp64 products, the inverses against fp64 inverses of those references and through
    (F + lam I) F_inv = I, the preconditioned gradient against B_inv G A_inv in fp64 on the raw gradient."""
    torch.manual_seed(5)
    M, d, damping, ema = 8192, 4096, 1e-3, 0.95
    lin = nn.Linear(d, d).cuda()
    model = nn.Sequential(lin)
    config = PreconditioningConfig(data_size=M, damping=damping, ema_decay=ema)
    gm = KfacGradientMaker(model, config, fisher_type=FISHER_EMP, loss_type='mse')

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp)                      # bf16 output: the output gradient reaches the hook in bf16

    def mse_fp32(y, target, reduction='mean'):
        return F.mse_loss(y.float(), target.float(), reduction=reduction)

    cap, handles = {}, []

    def fhook(mod, inp, out):
        cap['a'] = inp[0].detach()
        out.register_hook(lambda g: cap.__setitem__('g', g.detach()))
    handles.append(lin.register_forward_hook(fhook))
    handles.append(lin.weight.register_hook(lambda g: cap.__setitem__('gw', g.detach().clone())))
    handles.append(lin.bias.register_hook(lambda g: cap.__setitem__('gb', g.detach().clone())))
    eye = torch.eye(d, dtype=torch.float64, device='cuda')
    A_ref = B_ref = None
    for step in range(2):
        a = torch.randn(M, d).to(torch.bfloat16).cuda()
        t = (torch.randn(M, d) * 0.01).to(torch.bfloat16).cuda()
        model.zero_grad(set_to_none=True)
        gm.setup_loss_call(mse_fp32, gm.setup_model_call(fwd, a), t)
        print(f'config 2 step {step}', flush=True)
        gm.forward_and_backward()
        assert cap['a'].dtype == torch.bfloat16 and cap['g'].dtype == torch.bfloat16
        a64, g64 = cap['a'].double(), cap['g'].double()
        SA, SB = a64.T @ a64 / M, g64.T @ g64 / M
        A_ref = ema * SA if A_ref is None else (1 - ema) * A_ref + ema * SA
        B_ref = ema * SB if B_ref is None else (1 - ema) * B_ref + ema * SB
        kron = lin.fisher.kron
        errs = dict(A=relerr(kron.A, A_ref), B=relerr(kron.B, B_ref))
        assert errs['A'] < TOL_FACTOR and errs['B'] < TOL_FACTOR, (step, errs)
        assert torch.equal(kron.A, kron.A.T) and torch.equal(kron.B, kron.B.T)
        pi = (float(A_ref.trace()) / float(B_ref.trace())) ** 0.5           # dA == dB
        for which, ref, lam in (('A', A_ref, damping ** 0.5 * pi), ('B', B_ref, damping ** 0.5 / pi)):
            lam = max(lam, 1e-7)
            inv = getattr(kron, which + '_inv')
            assert torch.equal(inv, inv.T)
            errs[which + '_inv'] = relerr(inv, torch.linalg.inv(ref + lam * eye))
            resid = (getattr(kron, which).double() + lam * eye) @ inv.double() - eye
            errs[which + '_resid'] = float(resid.norm()) / d ** 0.5
            assert errs[which + '_inv'] < TOL_INV and errs[which + '_resid'] < TOL_INV, (step, which, errs)
        G = cap['gw'].double() / M
        w_ref = kron.B_inv.double() @ G @ kron.A_inv.double()
        b_ref = kron.B_inv.double() @ (cap['gb'].double() / M)
        errs['weight'], errs['bias'] = relerr(lin.weight.grad, w_ref), relerr(lin.bias.grad, b_ref)
        assert errs['weight'] < TOL_GRAD and errs['bias'] < TOL_GRAD, (step, errs)
        print(f'config 2 step {step}: ' + ', '.join(f'{k} {v:.1e}' for k, v in errs.items()), flush=True)
    for h in handles:
        h.remove()


@pytest.mark.parametrize('rounds', [True, False])
def test_fp32_inputs_of_a_bf16_autocast_region_enter_the_A_factor_rounded(rounds, monkeypatch):
    """The reference forms the A factor with torch.matmul inside its forward hook (asdl/operations/linear.py:75-77,
    conv.py:80-88), i.e. inside the caller's autocast region, where an fp32 operand is cast to bf16.
    operations.AUTOCAST_ROUNDS_FP32_OPERANDS does the same to an fp32 module input (first layers): the factor is the
    fp32 sum over the bf16-rounded input, 1e-5 from the oracle on the rounded values and clearly away from the one on
    the unrounded values; switched off, or outside an autocast region, the fp32 values are used as they are."""
    import asdl_amd.operations as ops_mod
    monkeypatch.setattr(ops_mod, 'AUTOCAST_ROUNDS_FP32_OPERANDS', rounds)
    torch.manual_seed(17)
    bs = 4
    conv = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(8, 8)).cuda()
    mlp = nn.Sequential(nn.Linear(24, 16), nn.ReLU(), nn.Linear(16, 8)).cuda()
    for model, x in ((conv, torch.randn(bs, 3, 6, 6).cuda()), (mlp, torch.randn(bs, 24).cuda())):
        t = torch.randint(8, (bs,)).cuda()
        for autocast in (True, False):
            def fwd(inp):
                with torch.autocast('cuda', dtype=torch.bfloat16, enabled=autocast):
                    return model(inp).float()
            ema = 0.5                         # with a moving average the factors are kept beside their inverses
            for m in model.modules():         # a fresh average for every run
                if hasattr(m, 'fisher'):
                    delattr(m, 'fisher')
            gm = KfacGradientMaker(model, PreconditioningConfig(data_size=bs, damping=1e-2, ema_decay=ema),
                                   fisher_type=FISHER_EMP)
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
            gm.forward_and_backward()
            first = model[0]
            stat = {}
            for key, seen in (('rounded', x.bfloat16().double().cpu()), ('plain', x.double().cpu())):
                if isinstance(first, nn.Conv2d):
                    stat[key] = ema * R.conv_cov_kron_A(seen, first.kernel_size, first.stride, first.padding) / bs
                else:
                    stat[key] = ema * R.linear_cov_kron_A(seen) / bs
            want, other = ('rounded', 'plain') if rounds and autocast else ('plain', 'rounded')
            A = first.fisher.kron.A
            assert relerr(A, stat[want]) < 1e-5, (type(first).__name__, autocast, relerr(A, stat[want]))
            assert relerr(A, stat[other]) > 1e-4, (type(first).__name__, autocast, relerr(A, stat[other]))


def test_resnet50_batch64_channels_last_properties():
    """The benchmark configuration (ResNet-50, batch 64) at full size, checked through properties that do not need a CPU run of
    the model: every conv A factor against an fp64 product of the unfolded input the GPU produced, every inverse
    through its defining identity, and the preconditioned gradients against B_inv G A_inv recomputed in fp64 from
    the stored inverses (sampled layers, to keep the host time down)."""
    torch.manual_seed(6)
    bs, damping, ema = 64, 1e-3, 0.5
    model = bench_models.resnet50().cuda().to(memory_format=torch.channels_last)
    x = torch.randn(bs, 3, 224, 224).cuda().contiguous(memory_format=torch.channels_last)
    t = torch.randint(0, 1000, (bs,)).cuda()

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    picks = ['conv1', 'layer1.0.conv2', 'layer2.0.conv2', 'layer3.1.conv1', 'layer3.0.conv2', 'layer4.0.downsample.0', 'layer4.2.conv2', 'fc']
    mods = dict(model.named_modules())
    ins, gouts, handles = {}, {}, []
    for name in picks:
        def fhook(mod, inp, out, name=name):
            ins[name] = inp[0].detach()
            out.register_hook(lambda g, name=name: gouts.__setitem__(name, g.detach()))
        handles.append(mods[name].register_forward_hook(fhook))
    raw = {}
    handles.append(mods['layer4.2.conv2'].weight.register_hook(lambda g: raw.__setitem__('g', g.detach().clone())))
    config = PreconditioningConfig(data_size=bs, damping=damping, ema_decay=ema, ignore_modules=[nn.BatchNorm2d])
    gm = KfacGradientMaker(model, config, fisher_type=FISHER_EMP)
    model.zero_grad(set_to_none=True)
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
    gm.forward_and_backward()
    for h in handles:
        h.remove()
    for name in picks:
        m = mods[name]
        kron = m.fisher.kron
        a = ins[name].bfloat16().float()     # conv1's fp32 images enter its factor rounded to bf16 (autocast region)
        g = gouts[name].float()              # summed loss inside the maker: these are the K-FAC out-grads
        if isinstance(m, nn.Conv2d):
            u = F.unfold(a.contiguous().double(), m.kernel_size, padding=m.padding, stride=m.stride)   # [n, d, hw]
            hw = u.shape[-1]
            U = u.permute(1, 0, 2).reshape(u.shape[1], -1)
            A_ref = ema * (U @ U.T) / hw / bs
            del u, U
            g2 = g.permute(0, 2, 3, 1).reshape(-1, g.shape[1]).double()
        else:
            A_ref = ema * a.double().T @ a.double() / bs
            g2 = g.double()
        B_ref = ema * g2.T @ g2 / bs
        assert relerr(kron.A, A_ref) < 1e-5, (name, 'A', relerr(kron.A, A_ref))
        assert relerr(kron.B, B_ref) < 1e-5, (name, 'B', relerr(kron.B, B_ref))
        assert torch.equal(kron.A, kron.A.T) and torch.equal(kron.B, kron.B.T)
        dA, dB = kron.A.shape[0], kron.B.shape[0]
        trA, trB = float(kron.A.diagonal().sum().double()), float(kron.B.diagonal().sum().double())
        pi = ((trA / dA) / (trB / dB)) ** 0.5
        for which, lam, dim in (('A', max(damping ** 0.5 * pi, 1e-7), dA), ('B', max(damping ** 0.5 / pi, 1e-7), dB)):
            assert_inverse_as_good_as_oracle(f'{name} {which}', getattr(kron, which), getattr(kron, which + '_inv'), lam)
    # preconditioned gradient of a large layer: B_inv G A_inv in fp64 on the raw gradient of the same backward pass
    m = mods['layer4.2.conv2']
    G = raw['g'].double().reshape(m.weight.shape[0], -1) / bs
    ref = m.fisher.kron.B_inv.double() @ G @ m.fisher.kron.A_inv.double()
    got = m.weight.grad.detach().double().reshape(m.weight.shape[0], -1)
    assert relerr(got, ref) < 1e-3, relerr(got, ref)


@pytest.mark.parametrize('early_batch,late_flags', [(False, False), (True, False), (False, True)])
def test_benchmark_path_resnet50_batch64_against_a_sequential_replay(early_batch, late_flags, monkeypatch):
    """The very code path bench.py times, at its size: ResNet-50, batch 64, channels-last, bf16 autocast, sampled
    (MC) Fisher without EMA, the grouped inverse on a side stream fed by a worker thread beside the loss backward pass
    (and, with ``early_batch``, a first batch started from inside the hooks of the sampled pass:
    fisher.EAGER_INVERSE_SAMPLED), the grouped preconditioning plan prepared before the flags are read.  On the
    third step (the eager path needs the cost of an earlier step) extra hooks capture, for every Conv2d / Linear,
    the activation and the output gradient the factor kernels read, and the raw gradient of the loss.  Afterwards
    the same tensors go through the same operations one module after the other on the current stream, with one
    batched inverse at the end and nothing running beside it, and through the per-module Kron.mvp.  The kernels
    are deterministic, so an inverse that differs from its replay by more than rounding was computed from a factor
    that was not final (or was overwritten) when its inverse ran."""
    import asdl_amd.fisher as fisher_mod
    import asdl_amd.natural_gradient as ng_mod
    from asdl_amd.core import no_centered_cov
    from asdl_amd.matrices import SHAPE_KRON
    assert fisher_mod.EAGER_INVERSE and ng_mod.GROUPED_PRECONDITION and ng_mod.PREPARE_PRECONDITION_EARLY
    monkeypatch.setattr(fisher_mod, 'EAGER_INVERSE_SAMPLED', early_batch)
    torch.manual_seed(12)
    bs, damping = 64, 1e-3
    model = bench_models.resnet50().cuda().to(memory_format=torch.channels_last)
    x = torch.randn(bs, 3, 224, 224).cuda().contiguous(memory_format=torch.channels_last)
    t = torch.randint(0, 1000, (bs,)).cuda()

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    config = PreconditioningConfig(data_size=bs, damping=damping, ignore_modules=[nn.BatchNorm2d])
    gm = KfacGradientMaker(model, config, fisher_type=FISHER_MC)
    gm.late_inverse_flags = late_flags      # bench.py's setting: the host reads the flags of a step one step late
    layers = [(n, m) for n, m in model.named_modules() if isinstance(m, (nn.Linear, nn.Conv2d))]
    ins, gouts, raw, handles = {}, {}, {}, []
    benchmark_flag = torch.backends.cudnn.benchmark
    torch.backends.cudnn.benchmark = True
    try:
        for step in range(3):
            if step == 2:
                for name, m in layers:
                    def fhook(mod, inp, out, name=name):
                        ins[name] = inp[0].detach()
                        # the sampled pass comes first; the loss backward pass fires the hook a second time
                        out.register_hook(lambda g, name=name: gouts.setdefault(name, g.detach()))
                    handles.append(m.register_forward_hook(fhook))
                    for pn, p in m.named_parameters(recurse=False):
                        handles.append(p.register_hook(
                            lambda g, key=(name, pn): raw.__setitem__(key, g.detach().clone())))
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
            print(f'benchmark path step {step}', flush=True)
            gm.forward_and_backward()
    finally:
        torch.backends.cudnn.benchmark = benchmark_flag
        for h in handles:
            h.remove()
    gm.check_late_flags()
    torch.cuda.synchronize()
    got = {name: (m.fisher.kron.A_inv.clone(), m.fisher.kron.B_inv.clone(),
                  {pn: p.grad.detach().clone() for pn, p in m.named_parameters(recurse=False)}) for name, m in layers}
    assert len(ins) == len(gouts) == len(layers) == 54

    # sequential replay of the captured tensors
    replay = {}
    with no_centered_cov(model, [SHAPE_KRON], ignore_modules=[nn.BatchNorm2d], calc_inv=True) as cxt:
        cxt.set_damping(damping)
        cxt.set_cov_scale(1.0 / bs)
        for name, m in layers:
            with torch.autocast('cuda', dtype=torch.bfloat16):      # as the forward hooks of the run
                cxt.call_operations_in_forward(m, ins[name], None)
            cxt.call_operations_in_backward(m, gouts[name])
        torch.cuda.synchronize()
        cxt.flush_inverses()
        for name, m in layers:
            replay[name] = cxt.cov_symmatrix(m, pop=True).kron
    torch.cuda.synchronize()
    worst = dict(A_inv=0.0, B_inv=0.0, weight=0.0, bias=0.0)
    for name, m in layers:
        kron = replay[name]
        eA, eB = relerr(got[name][0], kron.A_inv), relerr(got[name][1], kron.B_inv)
        worst['A_inv'], worst['B_inv'] = max(worst['A_inv'], eA), max(worst['B_inv'], eB)
        # the run sums the rows of a factor in the grouped launch's order, the replay in the single launch's: the
        # factors differ by ~1e-7 and the inverses by that times the condition number; 1e-4 is the bar for inverses
        assert eA < 1e-4 and eB < 1e-4, (name, eA, eB)
        g_w = raw[(name, 'weight')] / bs
        g_b = raw[(name, 'bias')] / bs if m.bias is not None else None
        exact = kron.B_inv.double() @ g_w.double().reshape(kron.B_inv.shape[0], -1) @ kron.A_inv.double()
        kron.mvp(vec_weight=g_w, vec_bias=g_b, use_inv=True, inplace=True)
        e = relerr(got[name][2]['weight'], g_w)
        worst['weight'] = max(worst['weight'], e)
        # The grouped path multiplies two fp16 pieces per element (22 bits), the per-module path three bf16 pieces
        # (24 bits); the sums cancel (entries of the inverses reach 1 / damping), most in the classifier, whose A factor
        # has rank 64 of 2048: both are compared with the fp64 product of the very same inverses as well.
        e_grouped = relerr(got[name][2]['weight'].reshape(exact.shape), exact)
        e_single = relerr(g_w.reshape(exact.shape), exact)
        worst['weight vs fp64 (grouped)'] = max(worst.get('weight vs fp64 (grouped)', 0.0), e_grouped)
        worst['weight vs fp64 (per module)'] = max(worst.get('weight vs fp64 (per module)', 0.0), e_single)
        assert e < 1e-4 and e_grouped < 1e-4 and e_single < 1e-4, (name, 'weight', e, e_grouped, e_single)
        if g_b is not None:
            e = relerr(got[name][2]['bias'], g_b)
            worst['bias'] = max(worst['bias'], e)
            assert e < 1e-5, (name, 'bias', e)
    # The replay above is a self-comparison (it proves the ordering of the streams).  The inverses of this route
    # (sampled Fisher, no EMA, flags possibly read late) are also held against the fp32 oracle and fp64, on factors
    # formed in fp64 from the very tensors the factor kernels read: the widest layer of each stage and the classifier.
    mods = dict(layers)
    for name in ('layer1.0.conv2', 'layer2.3.conv2', 'layer3.5.conv2', 'layer4.2.conv2', 'layer4.0.downsample.0', 'fc'):
        m = mods[name]
        a, g = ins[name].bfloat16().double(), gouts[name].double()
        if isinstance(m, nn.Conv2d):
            u = F.unfold(a.contiguous(), m.kernel_size, padding=m.padding, stride=m.stride)
            U = u.permute(1, 0, 2).reshape(u.shape[1], -1)
            A64 = (U @ U.T) / u.shape[-1] / bs
            del u, U
            g2 = g.permute(0, 2, 3, 1).reshape(-1, g.shape[1])
        else:
            A64, g2 = a.T @ a / bs, g
        B64 = g2.T @ g2 / bs
        dA, dB = A64.shape[0], B64.shape[0]
        pi = ((float(A64.diagonal().sum()) / dA) / (float(B64.diagonal().sum()) / dB)) ** 0.5
        assert_inverse_as_good_as_oracle(f'{name} A', A64, got[name][0], max(damping ** 0.5 * pi, 1e-7))
        assert_inverse_as_good_as_oracle(f'{name} B', B64, got[name][1], max(damping ** 0.5 / pi, 1e-7))
    print('benchmark path vs sequential replay: worst relative differences ' +
          ', '.join(f'{k} {v:.1e}' for k, v in worst.items()), flush=True)


def test_resnet18_cifar_batch128_fp32_properties():
    """The ResNet-18 configuration at full size (fp32, NCHW, batch 128, Conv2d factors up to 4608 x 4608), checked
    through the same size-independent properties as the ResNet-50 test."""
    torch.manual_seed(8)
    bs, damping, ema = 128, 1e-3, 0.5
    model = bench_models.resnet18_cifar().cuda()
    x, t = torch.randn(bs, 3, 32, 32).cuda(), torch.randint(0, 10, (bs,)).cuda()
    picks = ['conv1', 'layer1.0.conv2', 'layer2.0.conv1', 'layer3.0.shortcut.0', 'layer4.1.conv2', 'linear']
    mods = dict(model.named_modules())
    ins, gouts, handles = {}, {}, []
    for name in picks:
        def fhook(mod, inp, out, name=name):
            ins[name] = inp[0].detach()
            out.register_hook(lambda g, name=name: gouts.__setitem__(name, g.detach()))
        handles.append(mods[name].register_forward_hook(fhook))
    raw = {}
    handles.append(mods['layer4.1.conv2'].weight.register_hook(lambda g: raw.__setitem__('g', g.detach().clone())))
    config = PreconditioningConfig(data_size=bs, damping=damping, ema_decay=ema,
                                   ignore_modules=[nn.BatchNorm2d, nn.BatchNorm1d])
    gm = KfacGradientMaker(model, config, fisher_type=FISHER_EMP)
    model.zero_grad(set_to_none=True)
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
    gm.forward_and_backward()
    for h in handles:
        h.remove()
    for name in picks:
        m = mods[name]
        kron = m.fisher.kron
        a, g = ins[name].double(), gouts[name].double()
        if isinstance(m, nn.Conv2d):
            u = F.unfold(a, m.kernel_size, padding=m.padding, stride=m.stride)
            U = u.permute(1, 0, 2).reshape(u.shape[1], -1)
            A_ref = ema * (U @ U.T) / u.shape[-1] / bs
            del u, U
            g2 = g.permute(0, 2, 3, 1).reshape(-1, g.shape[1])
        else:
            A_ref, g2 = ema * a.T @ a / bs, g
        B_ref = ema * g2.T @ g2 / bs
        assert relerr(kron.A, A_ref) < 1e-5, (name, 'A', relerr(kron.A, A_ref))
        assert relerr(kron.B, B_ref) < 1e-5, (name, 'B', relerr(kron.B, B_ref))
        assert torch.equal(kron.A, kron.A.T) and torch.equal(kron.B, kron.B.T)
        dA, dB = kron.A.shape[0], kron.B.shape[0]
        pi = ((float(kron.A.diagonal().sum().double()) / dA) / (float(kron.B.diagonal().sum().double()) / dB)) ** 0.5
        for which, lam, dim in (('A', max(damping ** 0.5 * pi, 1e-7), dA), ('B', max(damping ** 0.5 / pi, 1e-7), dB)):
            assert_inverse_as_good_as_oracle(f'{name} {which}', getattr(kron, which), getattr(kron, which + '_inv'), lam)
    m = mods['layer4.1.conv2']
    G = raw['g'].double().reshape(m.weight.shape[0], -1) / bs
    ref = m.fisher.kron.B_inv.double() @ G @ m.fisher.kron.A_inv.double()
    assert relerr(m.weight.grad.detach().double().reshape(m.weight.shape[0], -1), ref) < 1e-3


@pytest.mark.parametrize('network', ['mlp', 'resnet18'])
def test_early_start_of_inverses_gives_the_same_result(network, monkeypatch):
    """fisher.EAGER_INVERSE starts the inverse of the layers whose factors are final while the backward pass still
    runs (from the second step on, when the total cost is known); the results must be those of the single batch
    after the pass: bit for bit on an MLP, whose kernels are deterministic, and up to the step-to-step differences of
    the library's convolution backward kernels on a ResNet."""
    import asdl_amd.fisher as fisher_mod
    import asdl_amd.operations as ops_mod
    monkeypatch.setattr(ops_mod, 'EAGER_COST_FRACTION', 0.3)

    def run(eager):
        monkeypatch.setattr(fisher_mod, 'EAGER_INVERSE', eager)
        torch.manual_seed(7)
        if network == 'mlp':
            model = bench_models.mlp().cuda()
            x, t = torch.randn(32, 784).cuda(), torch.randint(0, 10, (32,)).cuda()
        else:
            model = bench_models.resnet18_cifar().cuda()
            x, t = torch.randn(4, 3, 32, 32).cuda(), torch.randint(0, 10, (4,)).cuda()
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=x.shape[0], damping=1e-2), fisher_type='fisher_emp')
        out = {}
        for step in range(3):
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
            gm.forward_and_backward()
            for name, m in model.named_modules():
                if isinstance(m, (nn.Linear, nn.Conv2d)):
                    out[(step, name, 'A_inv')] = m.fisher.kron.A_inv.clone()
                    out[(step, name, 'B_inv')] = m.fisher.kron.B_inv.clone()
                    out[(step, name, 'grad')] = m.weight.grad.clone()
        return out

    lazy, eager = run(False), run(True)
    assert lazy.keys() == eager.keys()
    for key in lazy:
        if network == 'mlp':
            assert torch.equal(eager[key], lazy[key]), key
        else:
            # MIOpen picks between backward solvers of different accuracy from step to step (the raw gradients of
            # one and the same input differ by up to 6e-3 between steps of one run), so this is a coarse check
            assert relerr(eager[key], lazy[key]) < 3e-2, key


def test_grouped_precondition_and_its_early_preparation_give_the_per_module_result(monkeypatch):
    """natural_gradient.GROUPED_PRECONDITION preconditions all modules in a handful of launches and
    PREPARE_PRECONDITION_EARLY builds that plan before the inverses' flags are read.  A layer whose A factor is
    all zero (no bias, zero input) gets no inverse: the plan prepared early must be dropped then, the gradient of
    that layer stays raw, the others match the per-module path; a gradient replaced by the user between
    update_curvature() and precondition() must be the one that is preconditioned."""
    import asdl_amd.natural_gradient as ng_mod

    def run(grouped, early, zero_input, replace_grad=False):
        monkeypatch.setattr(ng_mod, 'GROUPED_PRECONDITION', grouped)
        monkeypatch.setattr(ng_mod, 'PREPARE_PRECONDITION_EARLY', early)
        torch.manual_seed(11)
        class Gate(nn.Module):
            def forward(self, x):
                return x * 0 if zero_input else x

        model = nn.Sequential(nn.Linear(8, 16), Gate(), nn.Linear(16, 12, bias=False), nn.Tanh(),
                              nn.Linear(12, 8), nn.ReLU(), nn.Linear(8, 4)).cuda()
        with torch.no_grad():
            model[4].bias.fill_(0.5)
        x = torch.randn(32, 8).cuda()
        t = torch.randint(0, 4, (32,)).cuda()
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=32, damping=1e-2), fisher_type='fisher_emp')
        grads = {}
        for step in range(2):
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
            if replace_grad:
                gm.update_curvature()
                model[4].weight.grad = torch.ones_like(model[4].weight.grad)
                gm.precondition()
            else:
                gm.forward_and_backward()
            for name, p in model.named_parameters():
                grads[(step, name)] = p.grad.detach().cpu().clone()
        return grads, model

    for zero_input in (False, True):
        ref, model = run(False, False, zero_input)
        if zero_input:
            assert model[2].fisher.kron.A_inv is None          # all-zero factor: never inverted
        for grouped, early in ((True, False), (True, True)):
            got, _ = run(grouped, early, zero_input)
            for key in ref:
                assert grad_close(got[key], ref[key], 1e-5), (zero_input, grouped, early, key)
    ref, _ = run(False, False, False, replace_grad=True)
    got, _ = run(True, True, False, replace_grad=True)
    for key in ref:
        assert grad_close(got[key], ref[key], 1e-5), key


def test_identity_where_zero_touches_only_the_flagged_matrices():
    from asdl_amd import kernels as K
    outs = [torch.full((d, d), 7.0, device='cuda') for d in (5, 130, 64)]
    flags = torch.tensor([1, 1, 9, 0, 0, 3], dtype=torch.int32, device='cuda')
    K.identity_where_zero(outs, flags, [0, 3, 5])
    torch.cuda.synchronize()
    assert torch.all(outs[0] == 7.0) and torch.all(outs[2] == 7.0)
    assert torch.equal(outs[1], torch.eye(130, device='cuda'))


def test_late_flags_of_a_batched_inverse():
    """PendingInverses.finish_late(): no host synchronisation; a factor that is not positive definite raises when the
    flags are read (strictly: at once), an all-zero factor's fresh inverse buffer holds the identity until then and
    the factor has no inverse afterwards (as with finish()), the inverses of the others are those of finish()."""
    from asdl_amd.symmatrix import Kron, batched_update_inv
    g = torch.Generator().manual_seed(9)

    def spd(d):
        X = torch.randn(3 * d, d, generator=g)
        return (X.T @ X / (3 * d)).cuda()

    mats = [(spd(24), spd(40)), (torch.zeros(16, 16).cuda(), spd(8)), (spd(130), spd(12))]
    strict = [Kron(A.clone(), B.clone()) for A, B in mats]
    batched_update_inv(strict, damping=1e-2)
    late = [Kron(A.clone(), B.clone()) for A, B in mats]
    flags = batched_update_inv(late, damping=1e-2, defer=True).finish_late()
    assert strict[1].A_inv is None and torch.equal(late[1].A_inv, torch.eye(16, device='cuda'))
    zero = flags.check()                            # nothing to raise; the all-zero factor is reported ...
    assert zero == [(late[1], 'A')] and late[1].A_inv is None        # ... and loses the identity it had meanwhile
    assert flags.check() == []                      # a second call is a no-op
    for a, b in zip(strict, late):
        assert torch.equal(a.B_inv, b.B_inv)
        assert a.A_inv is None or torch.equal(a.A_inv, b.A_inv)
    bad = [Kron(spd(24), -torch.eye(8).cuda()), Kron(spd(12), spd(12))]
    with pytest.raises(torch.linalg.LinAlgError):
        batched_update_inv([Kron(k.A.clone(), k.B.clone()) for k in bad], damping=1e-2)
    flags = batched_update_inv(bad, damping=1e-2, defer=True).finish_late()     # enqueued, inverses stored, no error yet
    assert bad[1].A_inv is not None and bad[0].B_inv is not None
    with pytest.raises(torch.linalg.LinAlgError, match='reported late'):
        flags.check()


@pytest.mark.parametrize('fisher_type', [FISHER_MC, FISHER_EMP])
def test_late_inverse_flags_give_the_same_steps(fisher_type, monkeypatch):
    """FisherMaker.late_inverse_flags (fisher.LATE_INVERSE_FLAGS, off by default, on in bench.py): the flags of an
    update are read when the next update reaches the same point, so the host never waits for the device inside a
    step.  Same kernels in the same order: every inverse of three steps is bit for bit the one of the strict order, every
    preconditioned gradient within 1e-4; each step checks the flags of the one before, check_late_flags() those of
    the last."""
    import asdl_amd.symmatrix as sm_mod
    import asdl_amd.natural_gradient as ng_mod
    checks = []
    plain_check = sm_mod.LateFlags.check
    monkeypatch.setattr(sm_mod.LateFlags, 'check', lambda self, *a, **k: (checks.append(self), plain_check(self, *a, **k))[1])
    xs = [torch.randn(8, 16, 12, 12, generator=torch.Generator().manual_seed(50 + i)).cuda()
          .contiguous(memory_format=torch.channels_last) for i in range(3)]
    ts = [torch.randint(10, (8,), generator=torch.Generator().manual_seed(60 + i)).cuda() for i in range(3)]

    def run(late, after=False):
        monkeypatch.setattr(ng_mod, 'FLAGS_AFTER_PRECONDITION', after)
        torch.manual_seed(33)
        model = nn.Sequential(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(), nn.Conv2d(32, 32, 1), nn.ReLU(),
                              nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10)).cuda()
        model = model.to(memory_format=torch.channels_last)
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=8, damping=1e-2), fisher_type=fisher_type, seed=5)
        gm.late_inverse_flags = late
        assert gm.fisher_maker.late_inverse_flags == late

        fwd = model                 # fp32: the framework's bf16 convolution kernels vary too much from call to call
        out = {}
        for step, (x, t) in enumerate(zip(xs, ts)):
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
            gm.forward_and_backward()
            for name, m in model.named_modules():
                if hasattr(m, 'fisher'):
                    out[(step, name, 'A_inv')] = m.fisher.kron.A_inv.clone()
                    out[(step, name, 'B_inv')] = m.fisher.kron.B_inv.clone()
                    out[(step, name, 'grad')] = m.weight.grad.clone()
        n_pending = len(gm.fisher_maker._late_flags)
        gm.state_dict()                     # a checkpoint reads what is still unread
        assert not gm.fisher_maker._late_flags
        gm.check_late_flags()               # nothing left: a no-op
        return out, n_pending

    ref, n = run(False)
    assert n == 0 and not checks
    got, n = run(True)
    # fisher_emp computes its inverses inside the one backward pass it has: no loss backward pass follows, nothing is
    # deferred and the flags are read at once as before
    expect_late = fisher_type == FISHER_MC
    assert (n > 0 and len(checks) == 3 * n) if expect_late else (n == 0 and not checks), (n, len(checks))   # 2 by the next steps, 1 by the checkpoint
    assert got.keys() == ref.keys() and len(ref) == 27
    for key in ref:
        # the raw weight gradients come from the framework's convolution kernels, which do not sum in a fixed order
        assert relerr(got[key], ref[key]) < 1e-4 if key[2] == 'grad' else torch.equal(got[key], ref[key]), key
    # the library's default (natural_gradient.FLAGS_AFTER_PRECONDITION): read in the step's own call, once its
    # preconditioning is enqueued; nothing is left for the next step or the checkpoint
    del checks[:]
    got, n = run(False, after=True)
    assert n == 0 and len(checks) == 3, (n, len(checks))      # also with the single pass of the empirical Fisher
    for key in ref:
        assert relerr(got[key], ref[key]) < 1e-4 if key[2] == 'grad' else torch.equal(got[key], ref[key]), key


def test_flags_read_after_the_preconditioning_leave_raw_gradients_when_they_raise(monkeypatch):
    """natural_gradient.FLAGS_AFTER_PRECONDITION: forward_and_backward() enqueues the preconditioning before it reads
    the flags of the step's inverses.  A factor that is not positive definite (here: every damping value replaced by
    a large negative one) has to raise torch.linalg.LinAlgError from that very call and leave in .grad what the
    backward pass wrote there, exactly what the strict order (flags first) leaves; the next step with sound factors
    works as if nothing had happened."""
    import asdl_amd.natural_gradient as ng_mod
    import asdl_amd.symmatrix as sm_mod
    from asdl_amd import kernels
    plain_damping = kernels.kron_damping
    broken = [False]

    def damping(*args, **kwargs):
        lam, nonzero = plain_damping(*args, **kwargs)
        return (lam * -1e6 if broken[0] else lam), nonzero
    monkeypatch.setattr(sm_mod.kernels, 'kron_damping', damping)
    x = torch.randn(8, 16, 12, 12, generator=torch.Generator().manual_seed(70)).cuda().contiguous(memory_format=torch.channels_last)
    t = torch.randint(10, (8,), generator=torch.Generator().manual_seed(71)).cuda()

    def run(after):
        monkeypatch.setattr(ng_mod, 'FLAGS_AFTER_PRECONDITION', after)
        torch.manual_seed(34)
        model = nn.Sequential(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(), nn.Conv2d(32, 32, 1), nn.ReLU(),
                              nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10)).cuda()
        model = model.to(memory_format=torch.channels_last)
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=8, damping=1e-2), fisher_type=FISHER_MC, seed=5)
        out = {}
        for step, bad in enumerate((False, True, False)):
            broken[0] = bad
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
            if bad:
                with pytest.raises(torch.linalg.LinAlgError, match='positive-definite'):
                    gm.forward_and_backward()
            else:
                gm.forward_and_backward()
            assert gm.fisher_maker.take_caller_flags() is None
            for name, p in model.named_parameters():
                out[(step, name)] = p.grad.clone()
        return out

    strict, after = run(False), run(True)
    # the raw gradients of the step that raised: the loss gradient divided by the data size
    torch.manual_seed(34)
    model = nn.Sequential(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(), nn.Conv2d(32, 32, 1), nn.ReLU(),
                          nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10)).cuda()
    model = model.to(memory_format=torch.channels_last)
    F.cross_entropy(model(x), t, reduction='sum').div(8).backward()
    raw = {name: p.grad for name, p in model.named_parameters()}
    for (step, name), g in strict.items():
        assert relerr(after[(step, name)], g) < 1e-4, (step, name)
        if step == 1:
            assert relerr(after[(step, name)], raw[name]) < 1e-4 and relerr(g, raw[name]) < 1e-4, name
        else:
            assert relerr(g, raw[name]) > 1e-2, name              # preconditioned


@pytest.mark.parametrize('pi', [1, 2])
def test_overlapped_inverse_update_in_ema_mode_gives_the_same_result(pi, monkeypatch):
    """natural_gradient.OVERLAP_INVERSE_UPDATE: with accumulated factors and a sampled Fisher, the inverses of
    update_preconditioner() are enqueued beside the loss backward pass when that step follows in the same call.
    Same kernels on the same factors: bit for bit the result of the sequential order, also when the inverses are
    only due every second step."""
    import asdl_amd.natural_gradient as ng_mod

    def run(overlap):
        monkeypatch.setattr(ng_mod, 'OVERLAP_INVERSE_UPDATE', overlap)
        torch.manual_seed(3)
        model = bench_models.mlp().cuda()
        x, t = torch.randn(32, 784).cuda(), torch.randint(0, 10, (32,)).cuda()
        config = PreconditioningConfig(data_size=32, damping=1e-2, ema_decay=0.5, curvature_upd_interval=1,
                                       preconditioner_upd_interval=pi)
        gm = KfacGradientMaker(model, config, fisher_type='fisher_mc', seed=5)
        out = {}
        for step in range(4):
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
            gm.forward_and_backward()
            for name, m in model.named_modules():
                if isinstance(m, nn.Linear):
                    out[(step, name, 'A')] = m.fisher.kron.A.clone()
                    out[(step, name, 'A_inv')] = m.fisher.kron.A_inv.clone()
                    out[(step, name, 'B_inv')] = m.fisher.kron.B_inv.clone()
                    out[(step, name, 'grad')] = m.weight.grad.clone()
        return out

    seq, ovl = run(False), run(True)
    assert seq.keys() == ovl.keys()
    for key in seq:
        assert torch.equal(seq[key], ovl[key]), key


@pytest.mark.parametrize('tag', ['cnn2_fisher_emp_ema0.5_int2', 'cnn_fisher_mc_ema-1', 'cnnbn_fisher_emp_ema-1'])
def test_factor_side_stream_gives_the_golden_results(tag, monkeypatch):
    """fisher.FACTOR_SIDE_STREAM (off by default: ordering the side stream costs more host time per hook than the
    overlap gains on this runtime) runs the statistics kernels of the hooks on a side stream."""
    import asdl_amd.fisher as fisher_mod
    monkeypatch.setattr(fisher_mod, 'FACTOR_SIDE_STREAM', True)
    test_kfac_gpu_matches_reference_golden(tag)


@pytest.mark.parametrize('ema,fisher_type,n_mc', [(-1, FISHER_EMP, 1), (0.3, FISHER_EMP, 1), (0.3, FISHER_MC, 2), (-1, FISHER_EXACT, 1)])
def test_grouped_factor_launches_give_the_single_launch_factors(ema, fisher_type, n_mc, monkeypatch):
    """fisher.GROUPED_FACTORS collects the bf16 Kronecker-factor statistics of a pass and launches them together
    (kernels.FactorGroup), at the end of the pass or every few hooks, all or only the plain ones of the forward pass
    (fisher.GROUP_FLUSH_EVERY).  On a channels-last
    CNN under bf16 autocast (3x3, strided 1x1 and plain 1x1 convolutions, a Linear head; two steps, so that with EMA
    the second one accumulates) every setting has to give the factors of the one-launch-per-factor path up to the
    summation order (2e-6), inverses within 1e-4 and the same preconditioned gradients (1e-4).  With two Monte-Carlo
    samples or the exact Fisher (one backward pass per class) a factor receives several contributions per step: the
    group has to launch before it takes the second one."""
    import asdl_amd.fisher as fisher_mod
    torch.manual_seed(31)
    xs = [torch.randn(8, 16, 12, 12).cuda().contiguous(memory_format=torch.channels_last) for _ in range(2)]
    ts = [torch.randint(10, (8,)).cuda() for _ in range(2)]

    def run(grouped, every):
        monkeypatch.setattr(fisher_mod, 'GROUPED_FACTORS', grouped)
        monkeypatch.setattr(fisher_mod, 'GROUP_FLUSH_EVERY', every)
        torch.manual_seed(32)
        model = nn.Sequential(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU(), nn.Conv2d(32, 64, 1, stride=2), nn.ReLU(),
                              nn.Conv2d(64, 64, 1), nn.ReLU(), nn.Conv2d(64, 32, 3, padding=1), nn.ReLU(),
                              nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10)).cuda()
        model = model.to(memory_format=torch.channels_last)
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=8, damping=1e-2, ema_decay=ema),
                               fisher_type=fisher_type, n_mc_samples=n_mc, seed=7)

        def fwd(inp):
            with torch.autocast('cuda', dtype=torch.bfloat16):
                return model(inp).float()
        for x, t in zip(xs, ts):
            model.zero_grad(set_to_none=True)
            gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(fwd, x), t)
            gm.forward_and_backward()
        torch.cuda.synchronize()
        out = {}
        for name, m in model.named_modules():
            if hasattr(m, 'fisher'):
                kron = m.fisher.kron
                for key in ('A', 'B', 'A_inv', 'B_inv'):
                    if getattr(kron, key) is not None:
                        out[f'{name}.{key}'] = getattr(kron, key).clone()
                out[f'{name}.grad'] = m.weight.grad.clone()
        return out

    from asdl_amd import kernels
    taken = []
    plain_add = kernels.FactorGroup.add
    monkeypatch.setattr(kernels.FactorGroup, 'add', lambda self, row, *a: (taken.append(row[0]), plain_add(self, row, *a))[1])
    ref = run(False, (0, 0))
    assert not taken
    assert any(k.endswith('A_inv') for k in ref) and (ema == -1 or any(k.endswith('.A') for k in ref))
    plain_forward = None
    for every in [(0, 0), (-1, 0), (-2, 0), (2, 3), (-2, 2), (1, 1)]:
        del taken[:]
        got = run(True, every)
        # per step: B of the four convolutions once per backward pass (the Linear layer's 10 columns are not a
        # multiple of 8), and with forward grouping A of the three layers that are neither the few-channel stem nor
        # the 64-channel 3x3 layer (whose factor comes from shifted correlations of its input, launched at once);
        # with -2 only those of them that are plain X^T X products (kind 0, like every B)
        passes = {FISHER_EMP: 1, FISHER_MC: n_mc, FISHER_EXACT: 10}[fisher_type]
        if plain_forward is None:
            plain_forward = taken.count(0) - 2 * 4 * passes
            assert 0 < plain_forward < 2 * 3
        forward = {-1: 0, -2: plain_forward}.get(every[0], 2 * 3)
        assert len(taken) == 2 * 4 * passes + forward and (every[0] < 0 or 1 in taken), (every, taken)
        assert every[0] != -2 or 1 not in taken
        assert got.keys() == ref.keys()
        for key in ref:
            tol = 2e-6 if key.endswith(('.A', '.B')) else 1e-4
            assert relerr(got[key], ref[key]) < tol, (every, key, relerr(got[key], ref[key]))


def test_grouped_factors_are_dropped_when_the_pass_raises():
    """Factor calls recorded by the hooks of a pass that ends in an exception are not launched later on (their
    tensors belong to a step that never finished); the maker works as before on the next call."""
    torch.manual_seed(41)
    model = nn.Sequential(nn.Conv2d(16, 32, 1), nn.ReLU(), nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 16)).cuda()
    model = model.to(memory_format=torch.channels_last)
    gm = KfacGradientMaker(model, PreconditioningConfig(data_size=4, damping=1e-2), fisher_type=FISHER_EMP)
    x = torch.randn(4, 16, 6, 6).cuda().contiguous(memory_format=torch.channels_last)
    t = torch.randint(16, (4,)).cuda()
    state = {'fail': True}

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    def loss_fn(y, target, reduction='mean'):
        if state['fail']:
            raise RuntimeError('boom')
        return F.cross_entropy(y, target, reduction=reduction)

    gm.setup_loss_call(loss_fn, gm.setup_model_call(fwd, x), t)
    import asdl_amd.fisher as fisher_mod
    saved = fisher_mod.GROUP_FLUSH_EVERY
    fisher_mod.GROUP_FLUSH_EVERY = (0, 0)          # the forward hooks record too
    try:
        with pytest.raises(RuntimeError, match='boom'):
            gm.forward_and_backward()
        group = gm.fisher_maker._factor_stream_obj.group
        assert len(group) == 0
        state['fail'] = False
        gm.forward_and_backward()
        assert len(group) == 0
    finally:
        fisher_mod.GROUP_FLUSH_EVERY = saved
    torch.cuda.synchronize()
    assert model[0].fisher.kron.A_inv is not None and torch.isfinite(model[0].weight.grad).all()


def test_fisher_attributes_and_steps_without_curvature_update():
    torch.manual_seed(4)
    model = bench_models.mlp(20, 16, 5).cuda()
    config = PreconditioningConfig(data_size=8, damping=1e-2, preconditioner_upd_interval=2)
    gm = KfacGradientMaker(model, config, fisher_type=FISHER_EMP)
    x, t = torch.randn(8, 20).cuda(), torch.randint(0, 5, (8,)).cuda()
    invs = []
    for step in range(3):
        model.zero_grad(set_to_none=True)
        gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
        y, loss = gm.forward_and_backward()
        kron = model[0].fisher.kron
        assert kron.A is None and kron.B is None and kron.has_inv
        assert kron.A_inv.shape == (20, 20) and kron.B_inv.shape == (16, 16) and kron.A_inv.is_cuda
        invs.append(kron.A_inv.clone())
    assert torch.equal(invs[0], invs[1])            # step 1 reuses the stale inverse
    assert gm.state_dict()['step'] == 3


@pytest.mark.parametrize('ema,ci,pi', [(-1, 3, 3), (0.4, 1, 3)])
def test_state_dict_resume_continues_the_run(ema, ci, pi):
    """Save after two of four steps (state_dict: step + Kronecker factors / inverses + unit-wise blocks), load into a
    fresh maker on a fresh copy of the model (through torch.save / torch.load, as a checkpoint would), continue:
    with update intervals of 3 the third step preconditions with inverses from before the save, and with EMA the
    running averages carry on.  The empirical Fisher on an MLP with BatchNorm1d / LayerNorm (unit-wise blocks) is
    deterministic, so the continued run has to equal the uninterrupted one bit for bit."""
    import io
    torch.manual_seed(21)
    data = [(torch.randn(16, 12).cuda(), torch.randint(5, (16,)).cuda()) for _ in range(4)]

    def net():
        torch.manual_seed(22)
        return nn.Sequential(nn.Linear(12, 16), nn.BatchNorm1d(16), nn.ReLU(), nn.Linear(16, 10), nn.LayerNorm(10),
                             nn.Linear(10, 5)).cuda()

    def make(model):
        config = PreconditioningConfig(data_size=16, damping=1e-2, ema_decay=ema, curvature_upd_interval=ci,
                                       preconditioner_upd_interval=pi)
        return KfacGradientMaker(model, config, fisher_type=FISHER_EMP), torch.optim.SGD(model.parameters(), lr=0.05)

    def step(model, gm, opt, x, t):
        opt.zero_grad(set_to_none=True)
        gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
        gm.forward_and_backward()
        grads = [p.grad.clone() for p in model.parameters()]
        opt.step()
        return grads

    model = net()
    gm, opt = make(model)
    straight = [step(model, gm, opt, x, t) for x, t in data]
    model = net()
    gm, opt = make(model)
    resumed = [step(model, gm, opt, x, t) for x, t in data[:2]]
    buf = io.BytesIO()
    torch.save({'model': model.state_dict(), 'kfac': gm.state_dict()}, buf)
    entry = gm.state_dict()['curvature']
    assert {'kron.A_inv', 'kron.B_inv'} <= set(entry['0']) and 'unit.inv' in entry['1'] and 'unit.inv' in entry['4']
    assert ('kron.A' in entry['0']) == (ema != -1) and ('unit.data' in entry['1']) == (ema != -1)
    del model, gm, opt
    buf.seek(0)
    ckpt = torch.load(buf, weights_only=True)
    model = net()
    model.load_state_dict(ckpt['model'])
    gm, opt = make(model)
    gm.load_state_dict(ckpt['kfac'])
    assert gm.state['step'] == 2
    resumed += [step(model, gm, opt, x, t) for x, t in data[2:]]
    for k, (a, b) in enumerate(zip(straight, resumed)):
        for ga, gb in zip(a, b):
            assert torch.equal(ga, gb), f'step {k}'
