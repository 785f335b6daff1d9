"""Synthetic model definitions used by bench.py and the end-to-end tests.

Random-init architectures only (no checkpoints, no datasets):

* ``mlp``            784-512-512-10 ReLU MLP.
* ``resnet18_cifar`` ResNet-18 with a CIFAR stem (3x3 conv, no max-pool), the
  layout of the reference's examples/arxiv_results/models/resnet.py:66-100.
* ``resnet50``       ResNet-50 v1.5 (stride on the 3x3 conv of each bottleneck).
* ``gpt2_small``     12-layer decoder, d=768, 12 heads, MLP 3072, vocab 50257;
  the token embedding and the output head are frozen so that every trainable
  2-D parameter is at most 3072 wide.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def mlp(in_dim=784, hid=512, out_dim=10):
    return nn.Sequential(nn.Linear(in_dim, hid), nn.ReLU(),
                         nn.Linear(hid, hid), nn.ReLU(),
                         nn.Linear(hid, out_dim))


class BasicBlock(nn.Module):
    expansion = 1

    def __init__(self, in_planes, planes, stride=1):
        super().__init__()
        self.conv1 = nn.Conv2d(in_planes, planes, 3, stride, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(planes)
        self.conv2 = nn.Conv2d(planes, planes, 3, 1, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(planes)
        self.shortcut = nn.Sequential()
        if stride != 1 or in_planes != planes:
            self.shortcut = nn.Sequential(
                nn.Conv2d(in_planes, planes, 1, stride, bias=False),
                nn.BatchNorm2d(planes))

    def forward(self, x):
        out = F.relu(self.bn1(self.conv1(x)))
        out = self.bn2(self.conv2(out))
        return F.relu(out + self.shortcut(x))


class ResNetCifar(nn.Module):
    def __init__(self, num_blocks=(2, 2, 2, 2), num_classes=10):
        super().__init__()
        self.in_planes = 64
        self.conv1 = nn.Conv2d(3, 64, 3, 1, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        self.layer1 = self._make(64, num_blocks[0], 1)
        self.layer2 = self._make(128, num_blocks[1], 2)
        self.layer3 = self._make(256, num_blocks[2], 2)
        self.layer4 = self._make(512, num_blocks[3], 2)
        self.linear = nn.Linear(512, num_classes)

    def _make(self, planes, n, stride):
        layers = []
        for s in [stride] + [1] * (n - 1):
            layers.append(BasicBlock(self.in_planes, planes, s))
            self.in_planes = planes
        return nn.Sequential(*layers)

    def forward(self, x):
        out = F.relu(self.bn1(self.conv1(x)))
        out = self.layer4(self.layer3(self.layer2(self.layer1(out))))
        out = F.adaptive_avg_pool2d(out, 1).flatten(1)
        return self.linear(out)


def resnet18_cifar(num_classes=10):
    return ResNetCifar((2, 2, 2, 2), num_classes)


class Bottleneck(nn.Module):
    expansion = 4

    def __init__(self, in_planes, planes, stride=1):
        super().__init__()
        out_planes = planes * 4
        self.conv1 = nn.Conv2d(in_planes, planes, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(planes)
        self.conv2 = nn.Conv2d(planes, planes, 3, stride, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(planes)
        self.conv3 = nn.Conv2d(planes, out_planes, 1, bias=False)
        self.bn3 = nn.BatchNorm2d(out_planes)
        self.downsample = None
        if stride != 1 or in_planes != out_planes:
            self.downsample = nn.Sequential(
                nn.Conv2d(in_planes, out_planes, 1, stride, bias=False),
                nn.BatchNorm2d(out_planes))

    def forward(self, x):
        idt = x if self.downsample is None else self.downsample(x)
        out = F.relu(self.bn1(self.conv1(x)))
        out = F.relu(self.bn2(self.conv2(out)))
        out = self.bn3(self.conv3(out))
        return F.relu(out + idt)


class ResNet50(nn.Module):
    def __init__(self, num_classes=1000):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 64, 7, 2, 3, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        self.in_planes = 64
        self.layer1 = self._make(64, 3, 1)
        self.layer2 = self._make(128, 4, 2)
        self.layer3 = self._make(256, 6, 2)
        self.layer4 = self._make(512, 3, 2)
        self.fc = nn.Linear(2048, num_classes)

    def _make(self, planes, n, stride):
        layers = []
        for s in [stride] + [1] * (n - 1):
            layers.append(Bottleneck(self.in_planes, planes, s))
            self.in_planes = planes * 4
        return nn.Sequential(*layers)

    def forward(self, x):
        x = F.relu(self.bn1(self.conv1(x)))
        x = F.max_pool2d(x, 3, 2, 1)
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        x = F.adaptive_avg_pool2d(x, 1).flatten(1)
        return self.fc(x)


def resnet50(num_classes=1000):
    return ResNet50(num_classes)


class GPT2Block(nn.Module):
    def __init__(self, d, n_head):
        super().__init__()
        self.n_head = n_head
        self.ln_1 = nn.LayerNorm(d)
        self.c_attn = nn.Linear(d, 3 * d)
        self.c_proj = nn.Linear(d, d)
        self.ln_2 = nn.LayerNorm(d)
        self.c_fc = nn.Linear(d, 4 * d)
        self.c_proj2 = nn.Linear(4 * d, d)

    def forward(self, x):
        b, t, d = x.shape
        q, k, v = self.c_attn(self.ln_1(x)).split(d, dim=2)
        q, k, v = (z.view(b, t, self.n_head, d // self.n_head).transpose(1, 2) for z in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.c_proj(y.transpose(1, 2).reshape(b, t, d))
        return x + self.c_proj2(F.gelu(self.c_fc(self.ln_2(x))))


class GPT2Small(nn.Module):
    def __init__(self, vocab=50257, d=768, n_layer=12, n_head=12, n_ctx=1024):
        super().__init__()
        self.wte = nn.Embedding(vocab, d)
        self.wpe = nn.Embedding(n_ctx, d)
        self.h = nn.ModuleList(GPT2Block(d, n_head) for _ in range(n_layer))
        self.ln_f = nn.LayerNorm(d)
        self.lm_head = nn.Linear(d, vocab, bias=False)
        for m in self.modules():
            if isinstance(m, (nn.Linear, nn.Embedding)):
                nn.init.normal_(m.weight, std=0.02)
        # frozen: a 50257-wide statistic would be 50257 x 50257
        self.wte.weight.requires_grad_(False)
        self.lm_head.weight.requires_grad_(False)

    def forward(self, idx):
        t = idx.shape[1]
        x = self.wte(idx) + self.wpe(torch.arange(t, device=idx.device))
        for blk in self.h:
            x = blk(x)
        return self.lm_head(self.ln_f(x))


def gpt2_small(**kw):
    return GPT2Small(**kw)
