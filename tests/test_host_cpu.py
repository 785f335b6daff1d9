"""Host logic on the CPU: the GradientMaker API, schedules, the hook engine and the K-FAC
orchestration, with the kernel entry points replaced by oracle-backed stand-ins
(tests/cpu_backend.py).  Also checks that the C-ABI library loads and exports every declared symbol
and that the product refuses CPU tensors."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import asdl_amd
from asdl_amd import (PreconditioningConfig, KfacGradientMaker, GradientMaker, FisherConfig, get_fisher_maker,
                      get_update_schedule, SHAPE_KRON, FISHER_EMP, FISHER_MC, FISHER_EXACT, LOSS_CROSS_ENTROPY, LOSS_MSE)
from conftest import GOLDEN
from models_small import GOLDEN_KFAC, get_mlp, get_cnn
import cpu_backend


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


# ------------------------------------------------------------------ library / boundary
def test_library_loads_and_exports_every_declared_symbol():
    from asdl_amd import _lib
    lib = _lib.load()
    declared = _lib.declared_symbols()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f'{name} is declared in include/asdl_amd.h but not exported'
        assert name in _lib._SIGNATURES, f'{name} has no ctypes signature'
    assert lib.ak_version() >= 100
    assert b'workspace' in lib.ak_error_string(-2)


def test_no_hot_kernel_spills_registers():
    """asdl_amd.build writes the compiler's resource figures of every kernel next to the library.  The matrix-core
    kernels keep their accumulators in registers for the whole k-loop: scratch memory (a spill) in one of them costs
    a factor of two and more (it happened to the 256-wide gathered SYRK tile after an epilogue change), so none is
    allowed outside the short list of kernels that have always had a few bytes."""
    report = os.path.join(os.path.dirname(asdl_amd.__file__), 'lib', 'kernel_resources.txt')
    if not os.path.exists(report):
        pytest.skip('no kernel_resources.txt: the library was not built by asdl_amd.build in this tree')
    allowed = {'conv_patch_syrk_kernel': 16, 'conv_syrk_kernel': 96}        # bytes per lane
    rows = [l.split() for l in open(report) if l.strip() and not l.startswith('#')]
    assert len(rows) > 100
    spilled = []
    for src, name, vgprs, agprs, scratch, occupancy, lds in rows:
        limit = max([v for k, v in allowed.items() if k in name] or [0])
        if int(scratch) > limit:
            spilled.append((src, name, int(scratch)))
    assert not spilled, spilled


def test_product_refuses_cpu_tensors():
    from asdl_amd import kernels
    with pytest.raises(RuntimeError, match='ROCm device'):
        kernels.syrk_tn(torch.randn(4, 4))
    with pytest.raises(RuntimeError, match='ROCm device'):
        kernels.conv_syrk(torch.randn(1, 2, 4, 4), (3, 3), (1, 1), (1, 1))
    with pytest.raises(RuntimeError, match='ROCm device'):
        asdl_amd.cholesky_inv(torch.eye(3), 0.1)
    model = get_mlp()
    gm = KfacGradientMaker(model, PreconditioningConfig(data_size=2, damping=1e-2), fisher_type=FISHER_EMP)
    x, t = torch.randn(2, 5), torch.randint(4, (2,))
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
    with pytest.raises(RuntimeError, match='ROCm device'):
        gm.forward_and_backward()


# ------------------------------------------------------------------ GradientMaker API (test/grad_maker/test_grad_maker.py)
class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.model = get_mlp()

    def forward(self, inputs, targets=None, flip=False):
        logits = self.model(inputs)
        if targets is not None:
            loss = F.cross_entropy(logits, targets)
            return (loss, logits) if flip else (logits, loss)
        return logits


def _vanilla(model, x, t):
    model.zero_grad(set_to_none=True)
    loss = F.cross_entropy(model(x), t)
    loss.backward()
    return loss, [p.grad.clone() for p in model.parameters()]


def test_grad_maker_matches_vanilla_autograd_for_every_calling_style():
    torch.manual_seed(0)
    model = _Net()
    x, t = torch.randn(4, 5), torch.randint(4, (4,))
    ref_loss, ref_grads = _vanilla(model, x, t)
    gm = GradientMaker(model)

    def check(loss):
        torch.testing.assert_close(loss, ref_loss)
        for p, g in zip(model.parameters(), ref_grads):
            torch.testing.assert_close(p.grad, g)

    model.zero_grad(set_to_none=True)
    dummy_y = gm.setup_model_call(model, x)
    gm.setup_loss_call(F.cross_entropy, dummy_y, t)
    y, loss = gm.forward_and_backward()
    check(loss)
    torch.testing.assert_close(y, model(x))

    for flip, idx in [(False, 1), (True, 0)]:
        model.zero_grad(set_to_none=True)
        gm_repr = GradientMaker(model)
        dummy_y = gm_repr.setup_model_call(model, x, targets=t, flip=flip)
        gm_repr.setup_loss_repr(dummy_y[idx])
        y, loss = gm_repr.forward_and_backward()
        check(loss)
        # a registered loss function wins over a loss expression (asdl/grad_maker.py:272-281)
        gm_repr.setup_loss_call(lambda out: out[idx] * 2, dummy_y)
        assert torch.allclose(gm_repr.forward_and_backward()[1], ref_loss * 2)

    # delegation: the other maker runs what was registered here, results land in both
    model.zero_grad(set_to_none=True)
    other = GradientMaker(model)
    y, loss = gm.delegate_forward_and_backward(other)
    check(loss)
    assert other.loss is gm.loss and other.model_output is gm.model_output

    with pytest.raises(TypeError):
        gm.setup_loss_repr('not a dummy')
    with pytest.raises(ValueError):
        GradientMaker(model).forward_and_backward()


def test_dummy_object_replays_attribute_item_and_call():
    lin = nn.Linear(5, 3)
    assert asdl_amd.DummyObject().weight[0].numel().eval(lin) == 5
    d = asdl_amd.DummyObject()
    assert d['a'][1].eval({'a': [1, 2]}) == 2
    # placeholders among the arguments of a recorded call are evaluated on the same base value
    base = {'f': lambda a, b=0: 10 * a + b, 'x': 3, 'y': 4}
    assert d['f'](d['x'], b=d['y']).eval(base) == 34
    assert d['a'].eval({'a': 1}) == 1 and d.eval(7) == 7        # d itself was not changed by the longer paths


def test_loss_reduction_override_for_functions_and_modules():
    """A maker that names a reduction passes it as a keyword to loss functions and sets (then restores) the
    attribute of loss modules; a loss without the option is refused (asdl/grad_maker.py:283-300)."""
    class Summed(GradientMaker):
        _loss_reduction = 'sum'

    torch.manual_seed(0)
    model = _Net()
    x, t = torch.randn(4, 5), torch.randint(4, (4,))
    expected = F.cross_entropy(model(x), t, reduction='sum')
    gm = Summed(model)
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t, reduction='mean')
    torch.testing.assert_close(gm.forward_and_backward()[1], expected)
    crit = nn.CrossEntropyLoss()
    gm.setup_loss_call(crit, gm.setup_model_call(model, x), t)
    torch.testing.assert_close(gm.forward_and_backward()[1], expected)
    assert crit.reduction == 'mean'
    gm.setup_loss_call(lambda y, t: F.cross_entropy(y, t), gm.setup_model_call(model, x), t)
    with pytest.raises(AttributeError):
        gm.forward_and_backward()


# ------------------------------------------------------------------ schedules
def test_update_schedule_and_intervals():
    s = get_update_schedule(10, update_ratio=0.5)
    assert len(s) == 10 and sum(s) == 5 and s[0]
    s = get_update_schedule(10, update_ratio=0.5, warmup_ratio=0.2)
    assert s[:2] == [True, True] and sum(s) == 5
    assert get_update_schedule(4, 1.0) == [True] * 4
    assert get_update_schedule(6, 0.5, interval_type='step') == [True] * 3 + [False] * 3
    # vectors worked out by hand from asdl/precondition/prec_grad_maker.py:204-254
    T_, F_ = True, False
    assert get_update_schedule(10, 0.5) == [T_, F_] * 5
    assert get_update_schedule(10, 0.3) == [T_, F_, F_, T_, F_, F_, T_, F_, F_, F_]      # the 4th multiple of 3 is over budget
    assert get_update_schedule(10, 0.5, 0.2) == [T_, T_, T_, F_, T_, F_, T_, F_, F_, F_]
    assert get_update_schedule(10, 0.5, 0.2, reverse=True) == [T_, T_, T_, F_, T_, F_, T_, F_, F_, F_][::-1]
    linear = get_update_schedule(20, 0.25, interval_type='linear')         # gaps 0, 2, 4, 6
    assert [i for i, f in enumerate(linear) if f] == [0, 1, 4, 9, 16] and len(linear) == 20
    with pytest.raises(ValueError):
        get_update_schedule(10, 0.5, interval_type='linear')               # gaps 0, 1, 2, 3 end at step 11 of 10
    with pytest.raises(ZeroDivisionError):
        get_update_schedule(10, 0.2, interval_type='linear')               # two updates: n (n - 1) = 0
    with pytest.raises(ValueError):
        get_update_schedule(10, 0.2, warmup_ratio=0.5)
    with pytest.raises(ValueError):
        get_update_schedule(10, 0.5, interval_type='quadratic')
    with pytest.raises(ValueError):
        get_update_schedule(0)
    with pytest.raises(ValueError):
        get_update_schedule(10, 1.5)
    gm = KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1, preconditioner_upd_interval=3,
                                                            curvature_upd_interval=2, ema_decay=0.1))
    assert [gm.do_update_preconditioner(s) for s in range(6)] == [True, False, False, True, False, False]
    assert [gm.do_update_curvature(s) for s in range(4)] == [True, False, True, False]
    assert gm.state_dict() == {'step': 0, 'curvature': {}}
    gm.load_state_dict({'step': 5})
    assert gm.state['step'] == 5
    gm2 = KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1, num_total_steps=4,
                                                             preconditioner_upd_ratio=0.5))
    with pytest.warns(UserWarning):
        assert gm2.do_update_preconditioner(10) is False
    assert gm2.preconditioner_upd_schedule == [True, False, True, False] and gm2.curvature_upd_schedule is None
    assert [gm2.do_update_curvature(s) for s in range(4)] == [True, False, True, False]      # follows the preconditioner
    with pytest.warns(UserWarning):                      # a known horizon overrides the interval
        gm3 = KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1, num_total_steps=4, ema_decay=0.1,
                                                                 preconditioner_upd_interval=2, curvature_upd_ratio=1.,
                                                                 preconditioner_upd_ratio=0.5))
    assert gm3.curvature_upd_schedule == [True] * 4 and gm3.do_update_curvature(1) and not gm3.do_update_preconditioner(1)
    gm4 = KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1, preconditioner_upd_interval=4,
                                                             preconditioner_warmup_steps=3))
    assert [gm4.do_update_preconditioner(s) for s in range(9)] == [True] * 4 + [False] * 3 + [True, False]


def test_update_schedules_are_assignable_like_the_reference_attributes():
    """asdl/precondition/prec_grad_maker.py:85-99, 174-195: the schedules are plain attributes there; an assigned
    list decides step by step, None hands the decision back to the intervals."""
    model = get_mlp()
    gm = KfacGradientMaker(model, PreconditioningConfig(data_size=4, preconditioner_upd_interval=3))
    assert gm.preconditioner_upd_schedule is None and gm.curvature_upd_schedule is None
    assert [gm.do_update_preconditioner(s) for s in range(4)] == [True, False, False, True]
    gm.preconditioner_upd_schedule = [False, True, True, False]
    assert [gm.do_update_preconditioner(s) for s in range(4)] == [False, True, True, False]
    assert [gm.do_update_curvature(s) for s in range(4)] == [False, True, True, False]      # follows the preconditioner
    gm.curvature_upd_schedule = [True, True, False, False]
    assert [gm.do_update_curvature(s) for s in range(4)] == [True, True, False, False]
    gm.curvature_upd_schedule = None
    assert [gm.do_update_curvature(s) for s in range(4)] == [False, True, True, False]
    gm.preconditioner_upd_schedule = None
    assert [gm.do_update_preconditioner(s) for s in range(4)] == [True, False, False, True]


def test_module_selection_by_ignore_list_and_trainability():
    model = nn.Sequential(nn.Linear(3, 3), nn.ReLU(), nn.Linear(3, 3), nn.Sequential(nn.Linear(3, 2)), nn.Linear(2, 2))
    for p in model[4].parameters():
        p.requires_grad_(False)
    keys = lambda **kw: list(KfacGradientMaker(model, PreconditioningConfig(data_size=1, **kw)).module_dict.keys())
    assert keys() == ['0', '2', '3/0']                           # leaves with trainable parameters, '/' for '.'
    assert keys(ignore_modules=[model[0]]) == ['2', '3/0']
    assert keys(ignore_modules=['3.']) == ['0', '2']
    model_c = nn.Sequential(nn.Linear(3, 3), nn.Conv1d(3, 3, 1))
    with pytest.warns(UserWarning):
        assert list(KfacGradientMaker(model_c, PreconditioningConfig(data_size=1)).module_dict.keys()) == ['0']


def test_hooked_modules_follow_the_model_between_steps():
    """The list of hooked modules is kept between calls of no_centered_cov() and rebuilt when the module tree, a
    parameter object or a requires_grad flag has changed (the reference walks the modules at every call)."""
    from asdl_amd.core import no_centered_cov
    model = nn.Sequential(nn.Linear(3, 3), nn.ReLU(), nn.Linear(3, 3), nn.BatchNorm1d(3))

    def hooked(**kw):
        with no_centered_cov(model, ['kron'], **kw) as cxt:
            return [m for m in model.modules() if cxt.is_operation_registered(m) and m is not model]

    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [model[0], model[2]]
    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [model[0], model[2]]            # from the kept list
    assert len(model.__dict__['_asdl_amd_assignment_plans']) == 1
    for p in model[0].parameters():
        p.requires_grad_(False)
    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [model[2]]                      # a frozen layer drops out
    model[0].weight.requires_grad_(True)
    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [model[0], model[2]]
    new = nn.Linear(3, 3)
    model[2] = new                                                                    # a replaced module is picked up
    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [model[0], new]
    model[0].weight = nn.Parameter(torch.zeros(3, 3), requires_grad=False)            # a replaced parameter too
    model[0].bias.requires_grad_(False)
    assert hooked(ignore_modules=[nn.BatchNorm1d]) == [new]
    assert hooked(ignore_modules=[new, nn.BatchNorm1d]) == []                         # other arguments, other list
    assert len(model.__dict__['_asdl_amd_assignment_plans']) == 2


def test_config_defaults_match_reference():
    c = PreconditioningConfig()
    assert (c.num_total_steps, c.preconditioner_upd_interval, c.preconditioner_warmup_steps) == (None, 1, 0)
    assert (c.curvature_upd_interval, c.curvature_upd_ratio, c.data_size, c.damping, c.ema_decay) == (None, None, -1, 1e-7, -1)
    assert c.ignore_modules is None and c.preconditioner_interval_type == 'constant'


def test_constructor_errors():
    from torch.nn.parallel import DistributedDataParallel
    model = nn.Sequential(nn.Embedding(4, 3), nn.Linear(3, 3), nn.BatchNorm1d(3))
    with pytest.raises(NotImplementedError, match='ignore_modules'):
        KfacGradientMaker(model, PreconditioningConfig(data_size=1))
    gm_bn = KfacGradientMaker(model, PreconditioningConfig(data_size=1, ignore_modules=[nn.Embedding]))
    assert gm_bn.shape_for[model[2]] == 'unit_wise' and gm_bn.shape_for[model[1]] == 'kron'
    with pytest.raises(NotImplementedError, match='unit-wise'):      # unit-wise blocks of a Linear layer are not built
        from asdl_amd.natural_gradient import NaturalGradientMaker
        NaturalGradientMaker(nn.Sequential(nn.Linear(3, 3)), PreconditioningConfig(data_size=1), fisher_shape='unit_wise')
    with pytest.raises(ValueError):
        KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1, curvature_upd_ratio=0.5, num_total_steps=10))
    gm = KfacGradientMaker(get_mlp(), PreconditioningConfig())
    gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(gm.model, torch.randn(2, 5)), torch.zeros(2, dtype=torch.long))
    with pytest.raises(ValueError, match='data_size'):
        gm.forward_and_backward()


# ------------------------------------------------------------------ K-FAC orchestration vs the reference's golden runs
@pytest.mark.parametrize('tag', sorted(GOLDEN_KFAC))
def test_kfac_host_logic_matches_reference_golden(tag, monkeypatch):
    cpu_backend.install(monkeypatch)
    factory, fisher_type, ema, damping, seed, ci, pi = GOLDEN_KFAC[tag]
    z = np.load(os.path.join(GOLDEN, f'kfac_{tag}.npz'))
    model = factory()
    model.load_state_dict({k[len('init/'):]: torch.from_numpy(z[k]) for k in z.files if k.startswith('init/')})
    bs = z['step0/x'].shape[0]
    config = PreconditioningConfig(data_size=bs, damping=damping, ema_decay=ema, curvature_upd_interval=ci,
                                   preconditioner_upd_interval=pi)
    gm = KfacGradientMaker(model, config, fisher_type=fisher_type, seed=seed, swift=tag.startswith('swift_'))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    n_steps = len({k.split('/')[0] for k in z.files if k.startswith('step')})
    for step in range(n_steps):
        opt.zero_grad(set_to_none=True)
        x, t = torch.from_numpy(z[f'step{step}/x']), torch.from_numpy(z[f'step{step}/t'])
        dummy_y = gm.setup_model_call(model, x)
        gm.setup_loss_call(F.cross_entropy, dummy_y, t)
        y, loss = gm.forward_and_backward()
        torch.testing.assert_close(loss, torch.from_numpy(z[f'step{step}/loss']), rtol=1e-5, atol=1e-6)
        for name, p in model.named_parameters():
            assert grad_close(p.grad, torch.from_numpy(z[f'step{step}/grad/{name}']), 2e-4), (tag, step, name)
        for key in z.files:
            if key.startswith(f'step{step}/kron/'):
                _, _, mname, which = key.split('/')
                got = getattr(model.get_submodule(mname).fisher.kron, which)
                assert got is not None, key
                assert relerr(got, torch.from_numpy(z[key])) < 2e-4, key
            if key.startswith(f'step{step}/unit/'):
                _, _, mname, which = key.split('/')
                got = getattr(model.get_submodule(mname).fisher.unit, which)
                assert got is not None, key
                assert relerr(got, torch.from_numpy(z[key])) < 2e-4, key
        for name, m in model.named_modules():
            if isinstance(m, (nn.BatchNorm1d, nn.BatchNorm2d, nn.LayerNorm)) and ema == -1:
                assert m.fisher.unit.data is None and m.fisher.unit.has_inv
            if isinstance(m, (nn.Linear, nn.Conv2d)) and ema == -1:
                assert m.fisher.kron.A is None and m.fisher.kron.B is None    # only inverses are kept
        opt.step()
    assert gm.state_dict()['step'] == n_steps


def _resume_run(monkeypatch, ema, ci, pi, fisher_type, n_steps=4, stop=2):
    """Gradients of an uninterrupted run and of one that is saved after ``stop`` steps and continued by a fresh
    maker on a fresh copy of the model."""
    cpu_backend.install(monkeypatch)
    torch.manual_seed(3)
    data = [(torch.randn(8, 5), torch.randint(4, (8,))) for _ in range(n_steps)]
    init = get_mlp().state_dict()

    def make():
        model = get_mlp()
        model.load_state_dict(init)
        config = PreconditioningConfig(data_size=8, damping=1e-2, ema_decay=ema, curvature_upd_interval=ci,
                                       preconditioner_upd_interval=pi)
        return model, KfacGradientMaker(model, config, fisher_type=fisher_type, seed=1), \
            torch.optim.SGD(model.parameters(), lr=0.05)

    def step(model, gm, opt, x, t):
        opt.zero_grad(set_to_none=True)
        gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
        gm.forward_and_backward()
        grads = [p.grad.clone() for p in model.parameters()]
        opt.step()
        return grads

    model, gm, opt = make()
    straight = [step(model, gm, opt, x, t) for x, t in data]
    model, gm, opt = make()
    resumed = [step(model, gm, opt, x, t) for x, t in data[:stop]]
    saved = gm.state_dict()
    weights = {k: v.clone() for k, v in model.state_dict().items()}
    for m in model.modules():                   # poison the live state: the clone in `saved` must not alias it
        fisher = getattr(m, 'fisher', None)
        if fisher is not None and fisher.has_kron:
            for attr in ('A', 'B', 'A_inv', 'B_inv'):
                if getattr(fisher.kron, attr) is not None:
                    getattr(fisher.kron, attr).fill_(float('nan'))
    model, gm, opt = make()
    model.load_state_dict(weights)
    gm.load_state_dict(saved)
    assert gm.state['step'] == stop
    resumed += [step(model, gm, opt, x, t) for x, t in data[stop:]]
    return straight, resumed, saved


@pytest.mark.parametrize('ema,ci,pi,fisher_type', [(-1, 3, 3, FISHER_EMP), (0.3, 1, 3, FISHER_EMP), (0.5, 2, 2, FISHER_MC)])
def test_state_dict_carries_the_curvature_through_a_resume(ema, ci, pi, fisher_type, monkeypatch):
    """Stop after step 2 of 4 with update intervals that make steps 2 and 3 depend on curvature computed earlier
    (stale inverses without EMA; running-average factors with EMA): the continued run has to reproduce the
    uninterrupted one bit for bit."""
    straight, resumed, saved = _resume_run(monkeypatch, ema, ci, pi, fisher_type)
    entry = saved['curvature']['0']
    assert {'kron.A_inv', 'kron.B_inv'} <= set(entry)
    assert ('kron.A' in entry) == (ema != -1)
    for a, b in zip(straight, resumed):
        for ga, gb in zip(a, b):
            assert torch.equal(ga, gb)


def test_load_state_dict_accepts_the_reference_form_and_rejects_unknown_modules():
    gm = KfacGradientMaker(get_mlp(), PreconditioningConfig(data_size=1))
    gm.load_state_dict({'step': 7})
    assert gm.state_dict() == {'step': 7, 'curvature': {}}
    with pytest.raises(KeyError, match='nosuch'):
        gm.load_state_dict({'step': 1, 'curvature': {'nosuch': {'kron.A': torch.eye(2)}}})


@pytest.mark.parametrize('per_call', [True, False])
def test_module_called_twice_in_one_forward(per_call, monkeypatch):
    """A module that is called twice per forward pass (shared weights), without EMA.  Default (the reference,
    asdl/operations/operation.py:225-233, 265-279, pinned by the golden runs 'shared_*'): every backward call inverts
    the pair (A of the LAST forward call, B of its own output gradient) with the pi-damping of that pair, and the
    inverses are added.  With operations.PER_CALL_INVERSES = False the contributions are summed and inverted once,
    (A1 + A2 + lam I)^-1."""
    import oracle.cpu_ref as R
    from asdl_amd import operations
    cpu_backend.install(monkeypatch)
    monkeypatch.setattr(operations, 'PER_CALL_INVERSES', per_call)
    torch.manual_seed(5)

    class Twice(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(6, 6)
            self.head = nn.Linear(6, 3)

        def forward(self, x):
            return self.head(torch.tanh(self.lin(torch.tanh(self.lin(x)))))

    model = Twice()
    x, t = torch.randn(10, 6), torch.randint(3, (10,))
    ins, gouts = [], []
    def capture(m, i, o):
        ins.append(i[0].detach())
        o.register_hook(lambda g: gouts.append(g.detach()))
    handle = model.lin.register_forward_hook(capture)
    gm = KfacGradientMaker(model, PreconditioningConfig(data_size=10, damping=1e-2), fisher_type=FISHER_EMP)
    for _ in range(2):        # the second step reuses the per-call scratch buffers
        ins.clear(), gouts.clear()
        model.zero_grad(set_to_none=True)
        gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
        gm.forward_and_backward()
        assert len(ins) == 2 and len(gouts) == 2
        if per_call:
            A = R.linear_cov_kron_A(ins[-1]) / 10
            pairs = [R.kron_update_inv(A, R.linear_cov_kron_B(g) / 10, 1e-2) for g in gouts]
            A_inv, B_inv = sum(p[0] for p in pairs), sum(p[1] for p in pairs)
        else:
            A = sum(R.linear_cov_kron_A(a) for a in ins) / 10
            B = sum(R.linear_cov_kron_B(g) for g in gouts) / 10
            A_inv, B_inv = R.kron_update_inv(A, B, 1e-2)
        assert relerr(model.lin.fisher.kron.A_inv, A_inv) < 1e-5
        assert relerr(model.lin.fisher.kron.B_inv, B_inv) < 1e-5
    handle.remove()


# ------------------------------------------------------------------ FisherMaker invariants (test/grad_maker/test_fisher.py)
@pytest.mark.parametrize('network', ['mlp', 'cnn'])
@pytest.mark.parametrize('fisher_type', [FISHER_EMP, FISHER_MC, FISHER_EXACT])
@pytest.mark.parametrize('loss_type', [LOSS_CROSS_ENTROPY, LOSS_MSE])
def test_fisher_maker_invariants(network, fisher_type, loss_type, monkeypatch):
    cpu_backend.install(monkeypatch)
    torch.manual_seed(0)
    model = get_mlp() if network == 'mlp' else get_cnn()
    bs = 4
    x = torch.randn(bs, 5) if network == 'mlp' else torch.randn(bs, 5, 4, 4)
    t = torch.randint(4, (bs,)) if loss_type == LOSS_CROSS_ENTROPY else torch.randn(bs, 4)
    loss_fn = F.cross_entropy if loss_type == LOSS_CROSS_ENTROPY else F.mse_loss
    fm = get_fisher_maker(model, FisherConfig(fisher_type=fisher_type, fisher_shapes=[SHAPE_KRON], data_size=1,
                                              loss_type=loss_type, seed=1))
    fm.setup_loss_call(loss_fn, fm.setup_model_call(model, x), t)
    mods = [m for m in model.modules() if isinstance(m, (nn.Linear, nn.Conv2d))]

    def snap():
        return [(m.fisher.kron.A.clone(), m.fisher.kron.B.clone()) for m in mods]

    fm.forward_and_backward()
    first = snap()
    for m, (A, B) in zip(mods, first):
        in_dim = m.in_features if isinstance(m, nn.Linear) else m.in_channels * 4
        out_dim = m.out_features if isinstance(m, nn.Linear) else m.out_channels
        assert A.shape == (in_dim, in_dim) and B.shape == (out_dim, out_dim)
        torch.testing.assert_close(A, A.T)
        torch.testing.assert_close(B, B.T)
    for k in [2, 3]:                                     # test_accumulate
        fm.forward_and_backward(accumulate=True)
        for (A, B), (A1, B1) in zip(snap(), first):
            torch.testing.assert_close(A, A1 * k)
            torch.testing.assert_close(B, B1 * k)
    fm.forward_and_backward(scale=0.1)                   # test_scale
    for (A, B), (A1, B1) in zip(snap(), first):
        torch.testing.assert_close(A, A1 * 0.1)
    fm.forward_and_backward(data_size=32)                # test_data_size
    for (A, B), (A1, B1) in zip(snap(), first):
        torch.testing.assert_close(B, B1 / 32)
    damping = 1.0                                        # test_inv
    fm.forward_and_backward(calc_inv=True, damping=damping)
    for m, (A, B) in zip(mods, first):
        kron = m.fisher.kron
        assert kron.A is None and kron.B is None and kron.A_inv is not None and kron.B_inv is not None
        pi = torch.sqrt((A.trace() / A.shape[0]) / (B.trace() / B.shape[0]))
        dA, dB = max(damping ** 0.5 * pi, 1e-7), max(damping ** 0.5 / pi, 1e-7)
        torch.testing.assert_close(torch.eye(A.shape[0]), (A + dA * torch.eye(A.shape[0])) @ kron.A_inv)
        torch.testing.assert_close(torch.eye(B.shape[0]), (B + dB * torch.eye(B.shape[0])) @ kron.B_inv)
    N, damping = 10, 10.0                                # test_inv_data_size
    fm.forward_and_backward(calc_inv=True, damping=damping * N * N)
    inv1 = [(m.fisher.kron.A_inv.clone(), m.fisher.kron.B_inv.clone()) for m in mods]
    fm.forward_and_backward(data_size=N, calc_inv=True, damping=damping)
    for m, (Ai, Bi) in zip(mods, inv1):
        torch.testing.assert_close(m.fisher.kron.A_inv, Ai * N)
        torch.testing.assert_close(m.fisher.kron.B_inv, Bi * N)


@pytest.mark.parametrize('fisher_type', [FISHER_MC, FISHER_EXACT])
def test_pruned_fisher_backward_equals_full_backward(fisher_type, monkeypatch):
    """The sampled / exact passes differentiate with respect to the hooked module outputs only; every hook must
    still fire and see the same gradients, also when the first trainable module is a BatchNorm whose output an
    in-place ReLU overwrites, and the loss gradient that follows must be untouched."""
    import asdl_amd.fisher as fisher_mod
    cpu_backend.install(monkeypatch)

    def run(pruned):
        monkeypatch.setattr(fisher_mod, 'PRUNED_FISHER_BACKWARD', pruned)
        torch.manual_seed(3)
        model = nn.Sequential(nn.BatchNorm2d(5), nn.ReLU(inplace=True), nn.Conv2d(5, 6, 3, padding=1, bias=False),
                              nn.BatchNorm2d(6), nn.ReLU(inplace=True), nn.Conv2d(6, 4, 2), nn.Flatten(),
                              nn.Linear(4 * 3 * 3, 4))
        x, t = torch.randn(6, 5, 4, 4), torch.randint(4, (6,))
        gm = KfacGradientMaker(model, PreconditioningConfig(data_size=6, damping=1e-2, ema_decay=0.5),
                               fisher_type=fisher_type, seed=11)
        gm.setup_loss_call(F.cross_entropy, gm.setup_model_call(model, x), t)
        gm.forward_and_backward()
        out = {}
        for name, m in model.named_modules():
            f = getattr(m, 'fisher', None)
            if f is None:
                continue
            if f.has_kron:
                out[name + '.A'], out[name + '.B'] = f.kron.A.clone(), f.kron.B.clone()
            if f.has_unit:
                out[name + '.unit'] = f.unit.data.clone()
        for name, p in model.named_parameters():
            out['grad.' + name] = p.grad.clone()
        return out

    full, pruned = run(False), run(True)
    assert full.keys() == pruned.keys() and any(k.endswith('.unit') for k in full)
    for key in full:
        assert torch.equal(full[key], pruned[key]), key
