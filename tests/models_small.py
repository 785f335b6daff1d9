"""Tiny models shared by the oracle tests and the GPU end-to-end tests (the same shapes as
the fixtures of the reference's test/conftest.py:11-25, plus a padded / strided CNN)."""
import torch
import torch.nn as nn
import torch.nn.functional as F


def get_mlp(in_dim=5, hid=4, out=4):
    return nn.Sequential(nn.Linear(in_dim, hid), nn.ReLU(), nn.Linear(hid, hid), nn.ReLU(), nn.Linear(hid, out))


def get_cnn(in_dim=5, hid=4, out=4):
    return nn.Sequential(nn.Conv2d(in_dim, hid, kernel_size=2), nn.ReLU(), nn.Conv2d(hid, hid, kernel_size=2),
                         nn.ReLU(), nn.Flatten(), nn.Linear(hid * 2 * 2, out))


def get_cnn2(in_dim=3, hid=6, out=5):
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.ReLU(), nn.Conv2d(hid, hid, 3, 2, 1), nn.ReLU(),
                         nn.Conv2d(hid, 8, 1, 2, 0, bias=False), nn.ReLU(), nn.Flatten(), nn.Linear(8 * 2 * 2, out))


def get_cnn_bn(in_dim=3, hid=8, out=5):
    # BatchNorm2d behind an in-place ReLU, BatchNorm1d and LayerNorm: unit-wise shapes of the default K-FAC
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.BatchNorm2d(hid), nn.ReLU(inplace=True),
                         nn.Conv2d(hid, hid, 3, 2, 1), nn.BatchNorm2d(hid), nn.ReLU(), nn.Flatten(),
                         nn.Linear(hid * 4 * 4, 12), nn.BatchNorm1d(12), nn.ReLU(), nn.Linear(12, 10),
                         nn.LayerNorm(10), nn.Linear(10, out))


def get_mlp_wide():
    # more columns than samples (batch 8) in the first two layers, on both sides
    return get_mlp(in_dim=12, hid=10, out=4)


def get_cnn3(in_dim=3, hid=6, out=5):
    # convolutions with more patch elements than samples, a Linear layer with fewer
    return nn.Sequential(nn.Conv2d(in_dim, hid, 3, 1, 1), nn.ReLU(), nn.Conv2d(hid, hid, 3, 2, 1), nn.ReLU(),
                         nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(hid, out))


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


GOLDEN_KFAC = {
    # tag: (model factory, fisher_type, ema_decay, damping, seed, curvature interval, preconditioner interval)
    'mlp_fisher_emp_ema-1': (get_mlp, 'fisher_emp', -1, 1e-2, None, None, 1),
    'mlp_fisher_emp_ema0.3': (get_mlp, 'fisher_emp', 0.3, 1e-2, None, None, 1),
    'mlp_fisher_mc_ema-1': (get_mlp, 'fisher_mc', -1, 1e-2, 1, None, 1),
    'mlp_fisher_mc_ema0.3': (get_mlp, 'fisher_mc', 0.3, 1e-2, 1, None, 1),
    'cnn_fisher_emp_ema-1': (get_cnn, 'fisher_emp', -1, 1e-2, None, None, 1),
    'cnn_fisher_mc_ema-1': (get_cnn, 'fisher_mc', -1, 1e-2, 1, None, 1),
    'cnn2_fisher_emp_ema0.5_int2': (get_cnn2, 'fisher_emp', 0.5, 1e-3, None, 1, 2),
    'cnn2_fisher_emp_ema-1_int2': (get_cnn2, 'fisher_emp', -1, 1e-3, None, None, 2),
    'cnnbn_fisher_emp_ema-1': (get_cnn_bn, 'fisher_emp', -1, 1e-2, None, None, 1),
    'cnnbn_fisher_emp_ema0.4': (get_cnn_bn, 'fisher_emp', 0.4, 1e-2, None, None, 1),
    'cnnbn_fisher_mc_ema-1': (get_cnn_bn, 'fisher_mc', -1, 1e-2, 3, None, 1),
    # modules called twice per forward pass
    'shared_fisher_emp_ema-1': (SharedNet, 'fisher_emp', -1, 1e-2, None, None, 1),
    'shared_fisher_mc_ema-1': (SharedNet, 'fisher_mc', -1, 1e-2, 5, None, 1),
    'shared_fisher_emp_ema0.5': (SharedNet, 'fisher_emp', 0.5, 1e-2, None, None, 1),
    'shared_fisher_mc_ema0.5': (SharedNet, 'fisher_mc', 0.5, 1e-2, 6, None, 1),
    # tags that start with 'swift_': KfacGradientMaker(swift=True)
    'swift_cnn2_fisher_emp_ema-1': (get_cnn2, 'fisher_emp', -1, 1e-2, None, None, 1),
    'swift_cnn2_fisher_mc_ema-1': (get_cnn2, 'fisher_mc', -1, 1e-3, 4, None, 1),
    'swift_cnn3_fisher_emp_ema0.5': (get_cnn3, 'fisher_emp', 0.5, 1e-2, None, None, 1),
    'swift_mlpw_fisher_emp_ema-1': (get_mlp_wide, 'fisher_emp', -1, 1e-2, None, None, 1),
}

GOLDEN_SHAMPOO = {
    # tag: (damping, ema_decay, curvature interval, preconditioner interval)
    'mlp': (1e-6, -1, 1, 2),
    'mlp_ema': (1e-4, 0.1, None, 1),
}
