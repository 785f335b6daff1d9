"""Writes tests/golden/*.npz from the reference implementation (CPU, this container only).

Run once as ``python tests/golden/make_golden.py`` with the reference checkout at
/root/reference.  It covers only what closed forms cannot pin:

  * kfac_*.npz     multi-step KfacGradientMaker runs (orchestration, EMA state, MC sampling
                   under a fixed seed) on the tiny MLP / CNN of the reference's test/conftest.py and
                   on a CNN with BatchNorm / LayerNorm (unit-wise blocks of the default K-FAC)
  * shampoo_*.npz  multi-step ShampooGradientMaker run (in-place ridge accumulation,
                   power-iteration start vectors under a fixed seed)
  * power_*.npz    ComputePower outputs for well- and ill-conditioned inputs

The fixtures hold inputs and expected outputs only.
"""
import os
import sys

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

sys.path.insert(0, '/root/reference')
import asdl  # noqa: E402
from asdl.precondition import PreconditioningConfig, KfacGradientMaker, ShampooGradientMaker  # noqa: E402
from asdl.precondition.shampoo import ComputePower  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def get_mlp(in_dim=5, hid=4, out=4):
    return nn.Sequential(nn.Linear(in_dim, hid), nn.ReLU(), nn.Linear(hid, hid), nn.ReLU(), nn.Linear(hid, out))


def get_cnn(in_dim=5, hid=4, out=4):
    return nn.Sequential(nn.Conv2d(in_dim, hid, kernel_size=2), nn.ReLU(), nn.Conv2d(hid, hid, kernel_size=2),
                         nn.ReLU(), nn.Flatten(), nn.Linear(hid * 2 * 2, out))


def get_cnn2(in_dim=3, hid=6, out=5):
    # padded / strided convolutions with bias, 8x8 inputs
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.ReLU(), nn.Conv2d(hid, hid, 3, 2, 1), nn.ReLU(),
                         nn.Conv2d(hid, 8, 1, 2, 0, bias=False), nn.ReLU(), nn.Flatten(), nn.Linear(8 * 2 * 2, out))


def get_cnn_bn(in_dim=3, hid=8, out=5):
    # BatchNorm2d behind an in-place ReLU, BatchNorm1d and LayerNorm: unit-wise shapes of the default K-FAC
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.BatchNorm2d(hid), nn.ReLU(inplace=True),
                         nn.Conv2d(hid, hid, 3, 2, 1), nn.BatchNorm2d(hid), nn.ReLU(), nn.Flatten(),
                         nn.Linear(hid * 4 * 4, 12), nn.BatchNorm1d(12), nn.ReLU(), nn.Linear(12, 10),
                         nn.LayerNorm(10), nn.Linear(10, out))


def state_arrays(model, prefix):
    return {f'{prefix}{k}': v.detach().numpy().copy() for k, v in model.state_dict().items()}


def run_kfac(tag, model, xs, ts, fisher_type, ema_decay, damping, seed=None, curv_interval=None, prec_interval=1,
             swift=False):
    out = {}
    out.update(state_arrays(model, 'init/'))
    config = PreconditioningConfig(data_size=xs[0].shape[0], damping=damping, ema_decay=ema_decay,
                                   curvature_upd_interval=curv_interval, preconditioner_upd_interval=prec_interval)
    gm = KfacGradientMaker(model, config, fisher_type=fisher_type, seed=seed, swift=swift)
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    for step, (x, t) in enumerate(zip(xs, ts)):
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(model, x)
        gm.setup_loss_call(F.cross_entropy, dummy_y, t)
        y, loss = gm.forward_and_backward()
        out[f'step{step}/x'] = x.numpy()
        out[f'step{step}/t'] = t.numpy()
        out[f'step{step}/loss'] = loss.detach().numpy()
        out[f'step{step}/y'] = y.detach().numpy()
        for name, p in model.named_parameters():
            out[f'step{step}/grad/{name}'] = p.grad.detach().numpy().copy()
        for name, m in model.named_modules():
            fisher = getattr(m, 'fisher', None)
            if fisher is None or fisher.kron is None:
                continue
            for key in ['A', 'B', 'A_inv', 'B_inv']:
                v = getattr(fisher.kron, key)
                if v is not None:
                    out[f'step{step}/kron/{name}/{key}'] = v.detach().numpy().copy()
        for name, m in model.named_modules():
            fisher = getattr(m, 'fisher', None)
            if fisher is None or fisher.unit is None:
                continue
            for key in ['data', 'inv']:
                v = getattr(fisher.unit, key)
                if v is not None:
                    out[f'step{step}/unit/{name}/{key}'] = v.detach().numpy().copy()
        opt.step()
    np.savez_compressed(os.path.join(HERE, f'kfac_{tag}.npz'), **out)
    print('wrote', tag, len(out))


def run_shampoo(tag, model, xs, ts, damping, ema_decay, curv_interval, prec_interval, seed):
    out = {}
    out.update(state_arrays(model, 'init/'))
    config = PreconditioningConfig(damping=damping, ema_decay=ema_decay, curvature_upd_interval=curv_interval,
                                   preconditioner_upd_interval=prec_interval)
    gm = ShampooGradientMaker(model, config)
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    torch.manual_seed(seed)
    for step, (x, t) in enumerate(zip(xs, ts)):
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(model, x)
        gm.setup_loss_call(F.cross_entropy, dummy_y, t)
        y, loss = gm.forward_and_backward()
        out[f'step{step}/x'] = x.numpy()
        out[f'step{step}/t'] = t.numpy()
        out[f'step{step}/loss'] = loss.detach().numpy()
        for name, p in model.named_parameters():
            out[f'step{step}/grad/{name}'] = p.grad.detach().numpy().copy()
        for i, prec in enumerate(gm.preconditioners):
            for j, (s, pm) in enumerate(zip(prec.statistics, prec.preconditioners)):
                out[f'step{step}/stat/{i}/{j}'] = s.numpy().copy()
                out[f'step{step}/prec/{i}/{j}'] = pm.numpy().copy()
        opt.step()
    out['seed'] = np.array(seed)
    np.savez_compressed(os.path.join(HERE, f'shampoo_{tag}.npz'), **out)
    print('wrote shampoo', tag, len(out))


def run_power():
    out = {}
    g = torch.Generator().manual_seed(7)
    cases = {}
    X = torch.randn(64, 24, generator=g)
    cases['wellcond_p4'] = (X.T @ X / 64, 4, 1e-6)
    X = torch.randn(6, 24, generator=g)
    cases['rankdef_p4'] = (X.T @ X / 6, 4, 1e-6)
    cases['rankdef_p4_eps12'] = (X.T @ X / 6, 4, 1e-12)
    X = torch.randn(40, 16, generator=g)
    cases['wellcond_p2'] = (X.T @ X, 2, 1e-4)
    cases['wellcond_p8'] = (X.T @ X, 8, 1e-6)
    cases['tiny_init'] = (1e-12 * torch.eye(12) + 1e-3 * torch.diag(torch.rand(12, generator=g)), 4, 1e-6)
    for seed, (name, (mat, p, eps)) in enumerate(cases.items()):
        torch.manual_seed(100 + seed)
        v0 = torch.rand(mat.shape[0]) * 2 - 1          # the draw PowerIter makes first
        torch.manual_seed(100 + seed)
        m = mat.clone()
        root = ComputePower(m, p, ridge_epsilon=eps)
        out[f'{name}/in'] = mat.numpy()
        out[f'{name}/p'] = np.array(p)
        out[f'{name}/eps'] = np.array(eps)
        out[f'{name}/v0'] = v0.numpy()
        out[f'{name}/root'] = root.numpy()
        out[f'{name}/mat_after'] = m.numpy()
    np.savez_compressed(os.path.join(HERE, 'power.npz'), **out)
    print('wrote power', len(out))


def main_bn():
    torch.manual_seed(5)
    bs = 8
    xs = [torch.randn(bs, 3, 8, 8) for _ in range(3)]
    ts = [torch.randint(5, (bs,)) for _ in range(3)]
    torch.manual_seed(17)
    run_kfac('cnnbn_fisher_emp_ema-1', get_cnn_bn(), xs, ts, 'fisher_emp', -1, 1e-2)
    torch.manual_seed(18)
    run_kfac('cnnbn_fisher_emp_ema0.4', get_cnn_bn(), xs, ts, 'fisher_emp', 0.4, 1e-2)
    torch.manual_seed(19)
    run_kfac('cnnbn_fisher_mc_ema-1', get_cnn_bn(), xs, ts, 'fisher_mc', -1, 1e-2, seed=3)


def get_mlp_wide():
    # more columns than samples (batch 8) in the first two layers, on both sides
    return get_mlp(in_dim=12, hid=10, out=4)


def get_cnn3(in_dim=3, hid=6, out=5):
    # convolutions with more patch elements than samples, a Linear layer with fewer
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.ReLU(), nn.Conv2d(hid, hid, 3, 2, 1), nn.ReLU(),
                         nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(hid, out))


def main_swift():
    # KfacGradientMaker(swift=True): factors of layers with fewer samples than columns stay n x d row matrices
    bs = 8
    torch.manual_seed(23)
    xs = [torch.randn(bs, 3, 8, 8) for _ in range(3)]
    ts = [torch.randint(5, (bs,)) for _ in range(3)]
    torch.manual_seed(24)
    run_kfac('swift_cnn2_fisher_emp_ema-1', get_cnn2(), xs, ts, 'fisher_emp', -1, 1e-2, swift=True)
    torch.manual_seed(25)
    run_kfac('swift_cnn2_fisher_mc_ema-1', get_cnn2(), xs, ts, 'fisher_mc', -1, 1e-3, seed=4, swift=True)
    # accumulation (EMA) of row matrices: only for layers whose row matrix is a fresh tensor (convolutions); for a
    # Linear layer the reference scales the live activation in place in this mode
    torch.manual_seed(26)
    run_kfac('swift_cnn3_fisher_emp_ema0.5', get_cnn3(), xs, ts, 'fisher_emp', 0.5, 1e-2, swift=True)
    xs = [torch.randn(bs, 12) for _ in range(3)]
    ts = [torch.randint(4, (bs,)) for _ in range(3)]
    torch.manual_seed(27)
    run_kfac('swift_mlpw_fisher_emp_ema-1', get_mlp_wide(), xs, ts, 'fisher_emp', -1, 1e-2, swift=True)


class SharedNet(nn.Module):
    """One Conv2d and one Linear that are each called twice per forward pass (shared weights)."""

    def __init__(self, ch=4, hid=6, out=5):
        super().__init__()
        self.stem = nn.Conv2d(3, ch, 3, 1, 1)
        self.conv = nn.Conv2d(ch, ch, 3, 1, 1)
        self.fc_in = nn.Linear(ch * 4 * 4, hid)
        self.fc = nn.Linear(hid, hid)
        self.head = nn.Linear(hid, out)

    def forward(self, x):
        x = F.relu(self.stem(x))
        x = F.relu(self.conv(x))
        x = F.max_pool2d(F.relu(self.conv(x)), 2)
        x = F.relu(self.fc_in(x.flatten(1)))
        x = torch.tanh(self.fc(x))
        x = F.relu(self.fc(x))
        return self.head(x)


def main_shared():
    # modules called twice per forward pass: without EMA the reference inverts inside every backward hook call and
    # adds the inverses up (asdl/operations/operation.py:267-279); with EMA the factors of the calls are summed
    bs = 8
    torch.manual_seed(41)
    xs = [torch.randn(bs, 3, 8, 8) for _ in range(3)]
    ts = [torch.randint(5, (bs,)) for _ in range(3)]
    torch.manual_seed(42)
    run_kfac('shared_fisher_emp_ema-1', SharedNet(), xs, ts, 'fisher_emp', -1, 1e-2)
    torch.manual_seed(43)
    run_kfac('shared_fisher_mc_ema-1', SharedNet(), xs, ts, 'fisher_mc', -1, 1e-2, seed=5)
    torch.manual_seed(44)
    run_kfac('shared_fisher_emp_ema0.5', SharedNet(), xs, ts, 'fisher_emp', 0.5, 1e-2)
    torch.manual_seed(45)
    run_kfac('shared_fisher_mc_ema0.5', SharedNet(), xs, ts, 'fisher_mc', 0.5, 1e-2, seed=6)


def run_partitioned(tag, shape, block_size, merge, damping, ema_decay, seed):
    """The reference's Preconditioner driven directly (ShampooGradientMaker never passes it a block size)."""
    from asdl.precondition.shampoo import Preconditioner
    out = {}
    g = torch.Generator().manual_seed(seed)
    param = torch.nn.Parameter(torch.randn(*shape, generator=g))
    config = PreconditioningConfig(damping=damping, ema_decay=ema_decay)
    prec = Preconditioner(param, config, block_size=block_size, best_effort_shape_interpretation=merge)
    out['shape'] = np.array(shape)
    out['block_size'] = np.array(block_size)
    out['merge'] = np.array(int(merge))
    out['damping'] = np.array(damping)
    out['ema_decay'] = np.array(ema_decay)
    out['seed'] = np.array(seed)
    for step in range(3):
        grad = torch.randn(*shape, generator=g)
        param.grad = grad.clone()
        out[f'step{step}/grad_in'] = grad.numpy().copy()
        prec.update_statistics()
        torch.manual_seed(1000 * seed + step)          # the start vectors of the power iterations
        prec.update_preconditioners()
        prec.precondition()
        out[f'step{step}/grad_out'] = param.grad.detach().numpy().copy()
        for i, (st, pm) in enumerate(zip(prec.statistics, prec.preconditioners)):
            out[f'step{step}/stat/{i}'] = st.numpy().copy()
            out[f'step{step}/prec/{i}'] = pm.numpy().copy()
    np.savez_compressed(os.path.join(HERE, f'shampoo_blocks_{tag}.npz'), **out)
    print('wrote shampoo blocks', tag, len(out))


def main_blocks():
    run_partitioned('mat_10x6_b4', (10, 6), 4, False, 1e-6, -1, 31)
    # best_effort_shape_interpretation=True cannot be recorded: the reference compares torch.Size with the merged
    # list in BlockPartitioner.partition and raises ValueError for every input
    run_partitioned('mat_9x13_b5_ema', (9, 13), 5, False, 1e-5, 0.2, 32)
    run_partitioned('conv_5x4x3x3_b4', (5, 4, 3, 3), 4, False, 1e-6, -1, 33)


def main():
    if len(sys.argv) > 1 and sys.argv[1] == 'blocks':
        return main_blocks()
    if len(sys.argv) > 1 and sys.argv[1] == 'bn':
        return main_bn()
    if len(sys.argv) > 1 and sys.argv[1] == 'swift':
        return main_swift()
    if len(sys.argv) > 1 and sys.argv[1] == 'shared':
        return main_shared()
    main_bn()
    main_swift()
    main_blocks()
    main_shared()
    torch.manual_seed(0)
    bs = 8
    xs = [torch.randn(bs, 5) for _ in range(3)]
    ts = [torch.randint(4, (bs,)) for _ in range(3)]
    for fisher_type, seed in [('fisher_emp', None), ('fisher_mc', 1)]:
        for ema in [-1, 0.3]:
            torch.manual_seed(11)
            run_kfac(f'mlp_{fisher_type}_ema{ema}', get_mlp(), xs, ts, fisher_type, ema, 1e-2, seed=seed)
    xs = [torch.randn(bs, 5, 4, 4) for _ in range(3)]
    for fisher_type, seed in [('fisher_emp', None), ('fisher_mc', 1)]:
        torch.manual_seed(12)
        run_kfac(f'cnn_{fisher_type}_ema-1', get_cnn(), xs, ts, fisher_type, -1, 1e-2, seed=seed)
    xs = [torch.randn(bs, 3, 8, 8) for _ in range(4)]
    ts = [torch.randint(5, (bs,)) for _ in range(4)]
    torch.manual_seed(13)
    run_kfac('cnn2_fisher_emp_ema0.5_int2', get_cnn2(), xs, ts, 'fisher_emp', 0.5, 1e-3, curv_interval=1, prec_interval=2)
    torch.manual_seed(14)
    run_kfac('cnn2_fisher_emp_ema-1_int2', get_cnn2(), xs, ts, 'fisher_emp', -1, 1e-3, prec_interval=2)

    xs = [torch.randn(bs, 5) for _ in range(4)]
    ts = [torch.randint(4, (bs,)) for _ in range(4)]
    torch.manual_seed(15)
    run_shampoo('mlp', get_mlp(), xs, ts, damping=1e-6, ema_decay=-1, curv_interval=1, prec_interval=2, seed=21)
    torch.manual_seed(16)
    run_shampoo('mlp_ema', get_mlp(), xs, ts, damping=1e-4, ema_decay=0.1, curv_interval=None, prec_interval=1, seed=22)
    run_power()


if __name__ == '__main__':
    main()
