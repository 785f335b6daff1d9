"""Parity of every HIP kernel (through the C ABI) with the CPU oracle on identical seeded inputs.

Tolerances (relative Frobenius error): Kronecker factors 1e-5 for fp32 inputs, 5e-3 for bf16 inputs
(the oracle is fed the same bf16-rounded values upcast to fp32; fp32 accumulation leaves only
summation-order differences, so the bf16 cases are in fact held to 1e-5 as well); damped inverses
1e-4 against the fp32 oracle where the matrix is well conditioned, otherwise both are compared with
an fp64 inverse; preconditioned gradients 1e-3.
"""
import time

import numpy as np

import pytest
import torch
import torch.nn as nn

from oracle import cpu_ref as R

pytestmark = pytest.mark.gpu

TOL_FACTOR_F32 = 1e-5
TOL_FACTOR_BF16 = 5e-3
TOL_INV = 1e-4
TOL_PRECOND = 1e-3


def relerr(a, b):
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


@pytest.fixture(scope='module')
def K():
    from asdl_amd import kernels
    return kernels


def _inputs(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    if dtype == torch.bfloat16:
        x = x.to(torch.bfloat16)
    return x


# ------------------------------------------------------------------ syrk_tn (Linear A / B, Shampoo G^T G)
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('M,d', [(128, 784), (128, 512), (128, 10), (1, 5), (37, 129), (1000, 300), (4096, 64),
                                 (70000, 40), (513, 1024)])
def test_syrk_tn_matches_oracle(K, dtype, M, d):
    x = _inputs((M, d), dtype, seed=M * 7 + d)
    ref = R.linear_cov_kron_A(x.float().double())
    print(f'syrk_tn dtype={dtype} M={M} d={d}', flush=True)
    out = K.syrk_tn(x.cuda())
    torch.cuda.synchronize()
    tol = TOL_FACTOR_F32 if dtype == torch.float32 else TOL_FACTOR_BF16
    assert relerr(out, ref) < min(tol, 1e-5)
    assert torch.equal(out, out.T)


def test_syrk_tn_alpha_beta_ema_and_strided_rows(K):
    x = _inputs((300, 200), torch.float32, 3)
    xs = x[:, :150]                                    # ldx = 200 > d = 150
    C0 = _inputs((150, 150), torch.float32, 4)
    C0 = C0 + C0.T
    ref = 0.7 * C0.double() + 0.3 / 64 * R.linear_cov_kron_A(xs.double())
    out = C0.cuda().clone()
    K.syrk_tn(x.cuda()[:, :150], out=out, alpha=0.3 / 64, beta=0.7)
    assert relerr(out, ref) < TOL_FACTOR_F32
    # beta == 0 must not read the destination
    out = torch.full((150, 150), float('nan'), device='cuda')
    K.syrk_tn(x.cuda()[:, :150], out=out, alpha=1.0, beta=0.0)
    assert relerr(out, R.linear_cov_kron_A(xs.double())) < TOL_FACTOR_F32


def test_syrk_tn_3d_input_rows_flatten(K):
    x = _inputs((4, 9, 33), torch.bfloat16, 5)
    ref = R.linear_cov_kron_A(x.float().double())
    out = K.syrk_tn(x.cuda().flatten(end_dim=1))
    assert relerr(out, ref) < 1e-5


def test_cpu_tensor_is_refused(K):
    with pytest.raises(RuntimeError):
        K.syrk_tn(torch.randn(4, 4))


# ------------------------------------------------------------------ conv_syrk (fused unfold)
CONV_CASES = [
    # N, C, H, W, k, s, p
    (2, 5, 4, 4, (2, 2), (1, 1), (0, 0)),          # the reference's test CNN
    (3, 4, 4, 3, (2, 2), (1, 1), (0, 0)),
    (4, 3, 32, 32, (3, 3), (1, 1), (1, 1)),        # CIFAR stem
    (2, 16, 16, 16, (3, 3), (2, 2), (1, 1)),
    (2, 3, 30, 30, (7, 7), (2, 2), (3, 3)),        # ImageNet stem geometry
    (3, 64, 7, 7, (3, 3), (1, 1), (1, 1)),         # 7x7 maps, ragged rows
    (2, 32, 14, 14, (1, 1), (1, 1), (0, 0)),       # 1x1 conv: flattened
    (2, 32, 14, 14, (1, 1), (2, 2), (0, 0)),       # 1x1 stride 2 (downsample)
    (2, 6, 9, 6, (3, 2), (2, 1), (0, 1)),          # asymmetric everything
    (1, 150, 8, 8, (3, 3), (1, 1), (1, 1)),        # d = 1350: many tiles
    (2, 20, 5, 70, (3, 3), (1, 1), (1, 1)),        # W_out > 64: column chunks
    (2, 4, 10, 10, (3, 3), (3, 3), (0, 0)),        # stride 3: generic gather path
]


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('case', CONV_CASES, ids=[str(c) for c in CONV_CASES])
def test_conv_syrk_matches_oracle(K, dtype, case):
    N, C, H, W, k, s, p = case
    x = _inputs((N, C, H, W), dtype, seed=N + 10 * C + H)
    ref = R.conv_cov_kron_A(x.float().double(), k, s, p)
    out_size = ((H + 2 * p[0] - k[0]) // s[0] + 1) * ((W + 2 * p[1] - k[1]) // s[1] + 1)
    print(f'conv_syrk dtype={dtype} case={case}', flush=True)
    out = K.conv_syrk(x.cuda(), k, s, p, alpha=1.0 / out_size)
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5
    assert torch.equal(out, out.T)


WINDOW_CASES = [
    # N, C, H, W, kernel, stride, padding: layers with C*kh*kw <= 160, taken by the LDS-window kernel
    (2, 3, 64, 64, (7, 7), (2, 2), (3, 3)),        # ImageNet stem geometry, d = 147 (15 tiles, two per wave)
    (3, 3, 37, 29, (7, 7), (2, 2), (3, 3)),        # odd sizes: last strip shorter than the others
    (2, 40, 9, 9, (2, 2), (1, 1), (0, 0)),         # d = 160: the largest it takes
    (2, 1, 28, 28, (5, 5), (1, 1), (2, 2)),        # one channel, d = 25: one tile, eight position slices
    (2, 7, 12, 10, (3, 3), (1, 1), (1, 1)),        # d = 63: three tiles, two position slices
    (2, 10, 12, 10, (3, 3), (2, 1), (1, 0)),       # d = 90: six tiles
    (2, 13, 8, 8, (3, 3), (1, 1), (1, 1)),         # d = 117: ten tiles, idle waves
    (700, 3, 6, 6, (3, 3), (1, 1), (1, 1)),        # more strips than work groups
    (2, 3, 8, 40, (3, 5), (1, 8), (1, 2)),         # stride wider than the kernel, few output columns
    (1, 2, 5, 3, (5, 3), (1, 1), (0, 0)),          # a single output position
    (2, 3, 224, 224, (7, 7), (2, 2), (3, 3)),      # the ImageNet stem at its size: 112 positions per output row
    (2, 4, 20, 45, (3, 3), (3, 3), (0, 0)),        # stride 3, 15 positions per row: a full and a ragged group of 8
]


@pytest.mark.parametrize('layout', ['nchw', 'channels_last'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, 'f32_as_bf16'])
@pytest.mark.parametrize('case', WINDOW_CASES, ids=[str(c) for c in WINDOW_CASES])
def test_conv_syrk_window_kernel_matches_oracle(K, dtype, layout, case):
    """fp32 input: fp32 matrix instructions; bf16 input, and fp32 input that the kernel rounds to bf16 as it reads
    it (round_bf16: what the reference's matmul does to it inside a bf16 autocast region), the bf16 ones.  The
    oracle gets the rounded values: the sums are fp32 in every case."""
    N, C, H, W, k, s, p = case
    rounded = dtype == 'f32_as_bf16'
    x = _inputs((N, C, H, W), torch.float32 if rounded else dtype, seed=N + 10 * C + H)
    out_size = ((H + 2 * p[0] - k[0]) // s[0] + 1) * ((W + 2 * p[1] - k[1]) // s[1] + 1)
    seen = x.bfloat16() if rounded else x
    ref = R.conv_cov_kron_A(seen.float().double(), k, s, p) * out_size      # the plain sum over positions
    print(f'conv_syrk window dtype={dtype} layout={layout} case={case}', flush=True)
    xg = x.cuda()
    if layout == 'channels_last':
        xg = xg.contiguous(memory_format=torch.channels_last)
    out = K.conv_syrk(xg, k, s, p, alpha=0.5, round_bf16=rounded)
    torch.cuda.synchronize()
    assert relerr(out, 0.5 * ref) < 1e-5
    assert torch.equal(out, out.T)
    if rounded and N * out_size <= 4096:     # not the statistic of the unrounded input: the rounding is really applied
        assert relerr(out, 0.5 * R.conv_cov_kron_A(x.double(), k, s, p) * out_size) > 1e-5
    # accumulation: out <- beta * out + alpha * stat
    K.conv_syrk(xg, k, s, p, out=out, alpha=0.25, beta=2.0, round_bf16=rounded)
    torch.cuda.synchronize()
    assert relerr(out, 1.25 * ref) < 1e-5
    assert torch.equal(out, out.T)


NHWC_CASES = [
    # N, C, H, W, kernel, stride, padding
    (2, 8, 6, 6, (3, 3), (1, 1), (1, 1)),          # smallest channel count the gather path takes
    (2, 64, 12, 12, (3, 3), (1, 1), (1, 1)),       # d = 576
    (3, 64, 7, 7, (3, 3), (1, 1), (1, 1)),         # 7x7 maps: k-tiles straddle rows and images
    (2, 128, 14, 14, (3, 3), (2, 2), (1, 1)),      # stride 2
    (2, 32, 14, 14, (1, 1), (1, 1), (0, 0)),       # 1x1 conv: plain rows
    (2, 32, 14, 14, (1, 1), (2, 2), (0, 0)),       # 1x1 stride 2 (downsample)
    (2, 16, 9, 6, (3, 2), (2, 1), (0, 1)),         # asymmetric everything
    (1, 152, 8, 8, (3, 3), (1, 1), (1, 1)),        # d = 1368: edge tiles, C not a power of two
    (2, 24, 5, 70, (5, 5), (1, 1), (2, 2)),        # 25 taps
    (5, 40, 33, 35, (3, 3), (1, 1), (1, 1)),       # M = 5775: split-K with a ragged last split
    (2, 176, 12, 12, (3, 3), (1, 1), (1, 1)),      # d = 1584: 256-wide tiles with an edge tile
    (2, 12, 6, 6, (3, 3), (1, 1), (1, 1)),         # C % 8 != 0: falls back to the NCHW kernel
]


@pytest.mark.parametrize('case', NHWC_CASES, ids=[str(c) for c in NHWC_CASES])
def test_conv_syrk_channels_last_matches_oracle(K, case):
    N, C, H, W, k, s, p = case
    x = _inputs((N, C, H, W), torch.bfloat16, seed=N + 10 * C + H)
    ref = R.conv_cov_kron_A(x.float().double(), k, s, p)
    out_size = ((H + 2 * p[0] - k[0]) // s[0] + 1) * ((W + 2 * p[1] - k[1]) // s[1] + 1)
    print(f'conv_syrk channels_last case={case}', flush=True)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    out = K.conv_syrk(xg, k, s, p, alpha=1.0 / out_size)
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5
    assert torch.equal(out, out.T)
    # same bits as the NCHW kernel is not required, same statistic is
    out2 = K.conv_syrk(x.cuda(), k, s, p, alpha=1.0 / out_size)
    assert relerr(out, out2.double()) < 1e-5


CORR_CASES = [
    # N, C, H, W: 3 x 3 windows, stride 1, padding 1, a multiple of 64 channels: the shifted-correlation form
    (2, 64, 5, 7),          # 64-wide tiles, one tile per shift
    (3, 128, 8, 8),         # 128-wide tiles
    (2, 256, 4, 6),         # two row tiles of 128
    (2, 512, 7, 7),         # 256-wide tiles of 8 waves
    (1, 64, 1, 1),          # a single pixel: only the centre tap sees it
    (2, 64, 2, 3),          # the first and the last image row are neighbours
    (2, 64, 1, 9),          # one image row: both row corrections remove the same pixels
    (3, 192, 6, 5),         # 64-wide tiles, three per shift
    (16, 64, 28, 28),       # 12544 pixels: row splits; image rows of 14 ... 64 pixels: the main product on windows
    (5, 128, 33, 35),       # windows of 48 + 16 pixels, ragged last split
    (4, 64, 14, 14),        # three image rows per pipeline stage
    (2, 128, 56, 56),       # windows of 64 + 16 pixels
    (3, 64, 3, 16),         # W a multiple of 16: no padding pixels; three image rows per sample
    (1, 192, 17, 64),       # the widest image row the windows take
    (2, 256, 14, 14),       # 32 units of (row channels, column channels)
    (5, 64, 20, 30),        # 100 image rows: splits of unequal length
    (7, 64, 5, 65),         # one pixel too wide for the windows: tiles again
]


@pytest.mark.parametrize('case', CORR_CASES, ids=[str(c) for c in CORR_CASES])
def test_conv_syrk_shifted_correlations_match_oracle(K, case):
    """3 x 3 / stride 1 / padding 1 factors of channels-last bf16 inputs are assembled from 13 shifted correlations of
    the input and 16 border corrections (csrc/conv_corr.hip) instead of the unfolded matrix: same statistic
    (asdl/operations/conv.py:80-88), checked against the oracle's unfolded product in fp64, exact symmetry, and
    accumulation into an existing factor."""
    N, C, H, W = case
    from asdl_amd import _lib
    assert _lib.load().ak_conv_syrk_nhwc_ws_bytes(N, C, H, W, 3, 3, 1, 1, 1, 1) > 0
    x = _inputs((N, C, H, W), torch.bfloat16, seed=N + 10 * C + H)
    ref = R.conv_cov_kron_A(x.float().double(), (3, 3), (1, 1), (1, 1))
    print(f'conv_syrk shifted correlations case={case}', flush=True)
    xg = x.cuda().contiguous(memory_format=torch.channels_last)
    out = K.conv_syrk(xg, (3, 3), (1, 1), (1, 1), alpha=1.0 / (H * W))
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5, relerr(out, ref)
    assert torch.equal(out, out.T)
    # every 9C x 9C block against its own norm: a wrong correction of one border block must not hide in the total
    blocks = (out.double().cpu() - ref).reshape(C, 9, C, 9).permute(1, 3, 0, 2)
    ref_blocks = ref.reshape(C, 9, C, 9).permute(1, 3, 0, 2)
    for t1 in range(9):
        for t2 in range(9):
            if float(ref_blocks[t1, t2].norm()) > 0:
                assert float(blocks[t1, t2].norm() / ref_blocks[t1, t2].norm()) < 1e-5, (t1, t2)
            else:
                assert float(blocks[t1, t2].abs().max()) < 1e-6 * float(ref.abs().max()), (t1, t2)
    K.conv_syrk(xg, (3, 3), (1, 1), (1, 1), out=out, alpha=0.25 / (H * W), beta=2.0)
    torch.cuda.synchronize()
    assert relerr(out, 2.25 * ref) < 1e-5
    assert torch.equal(out, out.T)


CORR_F32_CASES = [(2, 64, 5, 7), (3, 128, 8, 8), (2, 256, 4, 6), (1, 512, 7, 7), (4, 64, 16, 16), (2, 192, 6, 5),
                  (8, 64, 32, 32)]


@pytest.mark.parametrize('case', CORR_F32_CASES, ids=[str(c) for c in CORR_F32_CASES])
def test_conv_syrk_fp32_nchw_shifted_correlations_match_oracle(K, case):
    """fp32 NCHW inputs of 3 x 3 / stride 1 / padding 1 layers: the input is split exactly into three bf16 planes
    (channels-last, 3 C channels), the shifted correlations run on the bf16 matrix cores, and the plane pairs are
    folded before the assembly.  The result has to be the fp32 statistic (asdl/operations/conv.py:80-88) to 1e-5,
    not a bf16-rounded one: inputs with a wide dynamic range inside every patch."""
    N, C, H, W = case
    g = torch.Generator().manual_seed(7 * N + C + H)
    x = torch.randn(N, C, H, W, generator=g) * torch.exp(2 * torch.randn(N, C, H, W, generator=g))
    ref = R.conv_cov_kron_A(x.double(), (3, 3), (1, 1), (1, 1))
    print(f'conv_syrk fp32 nchw shifted correlations case={case}', flush=True)
    xg = x.cuda()
    out = K.conv_syrk(xg, (3, 3), (1, 1), (1, 1), alpha=1.0 / (H * W))
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5, relerr(out, ref)
    assert torch.equal(out, out.T)
    # not the statistic of the bf16-rounded input
    assert relerr(out, R.conv_cov_kron_A(x.bfloat16().double(), (3, 3), (1, 1), (1, 1))) > 1e-4
    K.conv_syrk(xg, (3, 3), (1, 1), (1, 1), out=out, alpha=0.25 / (H * W), beta=2.0)
    torch.cuda.synchronize()
    assert relerr(out, 2.25 * ref) < 1e-5
    assert torch.equal(out, out.T)


@pytest.mark.parametrize('layout', ['nchw', 'channels_last'])
def test_round_bf16_outside_the_window_kernel_is_a_cast(K, layout):
    """round_bf16 for operands the window kernel does not take (many channels, 1x1 windows, plain rows): the wrappers
    cast to bf16 and use the bf16 kernels; the C entry points answer AK_ERR_UNSUPPORTED to AK_F32_AS_BF16 there."""
    import ctypes
    from asdl_amd import _lib
    x = _inputs((2, 32, 10, 10), torch.float32, seed=5)
    xg = x.cuda().contiguous(memory_format=torch.channels_last) if layout == 'channels_last' else x.cuda()
    for k, s, p in (((3, 3), (1, 1), (1, 1)), ((1, 1), (1, 1), (0, 0))):
        ref = R.conv_cov_kron_A(x.bfloat16().double(), k, s, p)
        out_size = ((10 + 2 * p[0] - k[0]) // s[0] + 1) ** 2
        out = K.conv_syrk(xg, k, s, p, alpha=1.0 / out_size, round_bf16=True)
        assert relerr(out, ref) < 1e-5
        assert relerr(out, R.conv_cov_kron_A(x.double(), k, s, p)) > 1e-5
    rows = _inputs((300, 48), torch.float32, seed=6)
    out = K.syrk_tn(rows.cuda(), round_bf16=True)
    assert relerr(out, R.linear_cov_kron_A(rows.bfloat16().double())) < 1e-5
    assert relerr(out, R.linear_cov_kron_A(rows.double())) > 1e-5
    # the C ABI itself: the third dtype code is the window kernel's only
    A = torch.empty(288, 288, device='cuda')
    lib = _lib.load()
    args = (ctypes.c_void_p(xg.data_ptr()), K.AK_F32_AS_BF16, 2, 32, 10, 10, 3, 3, 1, 1, 1, 1, 1.0, 0.0,
            ctypes.c_void_p(A.data_ptr()), 288, ctypes.c_void_p(0), 0, ctypes.c_void_p(0))
    fn = lib.ak_conv_syrk_nhwc if layout == 'channels_last' else lib.ak_conv_syrk
    assert fn(*args) == K.AK_ERR_UNSUPPORTED
    torch.cuda.synchronize()


def test_conv_syrk_channels_last_ema_accumulate(K):
    x = _inputs((4, 16, 10, 10), torch.bfloat16, 1)
    x2 = _inputs((4, 16, 10, 10), torch.bfloat16, 2)
    A0 = R.conv_cov_kron_A(x.float(), (3, 3), (1, 1), (1, 1))
    ref = 0.9 * A0.double() + 0.1 * R.conv_cov_kron_A(x2.float().double(), (3, 3), (1, 1), (1, 1))
    out = A0.cuda().clone()
    K.conv_syrk(x2.cuda().contiguous(memory_format=torch.channels_last), (3, 3), (1, 1), (1, 1), out=out,
                alpha=0.1 / 100, beta=0.9)
    assert relerr(out, ref) < TOL_FACTOR_F32


@pytest.mark.parametrize('C,H', [(64, 14), (16, 12)])     # shifted correlations; the gathered kernel
def test_remembered_direct_launch_repeats_the_factor_call(K, C, H):
    """kernels.DirectCall: a hook remembers the library call its factor function made and repeats it on the tensor
    of the next pass (another address, other values) without going through conv_syrk(): the same factor as a fresh
    call bit for bit, and no launch at all for a tensor that would not give the same call."""
    xs = [_inputs((4, C, H, H), torch.bfloat16, seed).cuda().contiguous(memory_format=torch.channels_last) for seed in (3, 4)]
    out = torch.empty(9 * C, 9 * C, device='cuda')
    K.GroupedCall.begin()
    K.conv_syrk(xs[0], (3, 3), (1, 1), (1, 1), out=out, alpha=0.25, beta=0.0)
    assert K.DirectCall.remember(xs[0].clone(), out, 'same') is None         # not the tensor the call read
    K.GroupedCall.begin()
    K.conv_syrk(xs[0], (3, 3), (1, 1), (1, 1), out=out, alpha=0.25, beta=0.0)
    assert K.DirectCall.remember(xs[0], torch.empty_like(out), 'same') is None      # not the buffer it wrote
    K.GroupedCall.begin()
    K.conv_syrk(xs[0], (3, 3), (1, 1), (1, 1), out=out, alpha=0.25, beta=0.0)
    rec = K.DirectCall.remember(xs[0], out, 'same')
    assert rec is not None and K.DirectCall.remember(xs[0], out, 'same') is None    # a note is taken once
    first = out.clone()
    assert rec.again(xs[1], 'same')
    fresh = K.conv_syrk(xs[1], (3, 3), (1, 1), (1, 1), alpha=0.25)
    assert torch.equal(out, fresh) and not torch.equal(out, first)
    out.fill_(-1.0)
    assert not rec.again(xs[1], 'other')                                       # the caller's own state differs
    assert not rec.again(xs[1][:2], 'same')                                    # another shape
    assert not rec.again(xs[1].float(), 'same')                                # another type
    assert not rec.again(xs[1].contiguous(), 'same')                           # other strides (NCHW)
    assert float(out.min()) == -1.0 and float(out.max()) == -1.0               # none of them launched anything
    assert rec.again(xs[0], 'same') and torch.equal(out, first)


@pytest.mark.parametrize('M,d,ld', [(4096, 64, 64), (20000, 64, 64), (3000, 1000, 1000), (777, 256, 320),
                                    (100000, 128, 128), (33, 2048, 2048), (3000, 1600, 1600), (1500, 2560, 2568)])
def test_syrk_tn_bf16_split_k_and_strided(K, M, d, ld):
    """Shapes that exercise split-K, ragged last splits, edge tiles and a row stride larger than d."""
    x = _inputs((M, ld), torch.bfloat16, seed=M % 97)
    ref = x[:, :d].float().double().T @ x[:, :d].float().double()
    print(f'syrk_tn bf16 M={M} d={d} ld={ld}', flush=True)
    out = K.syrk_tn(x.cuda()[:, :d])
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5
    assert torch.equal(out, out.T)


@pytest.mark.parametrize('N,C,H,k,s,p', [(8, 64, 28, 3, 1, 1),      # G = 32, 9 taps
                                         (8, 24, 28, 3, 1, 1),      # G = C = 24 (not a multiple of 32)
                                         (8, 32, 20, 5, 1, 2),      # 25 taps: four channels per column block
                                         (8, 40, 24, 2, 2, 0),      # 4 taps, G = 40
                                         (16, 8, 40, 5, 1, 2),      # G = 8 (few channels, but more than 160 columns)
                                         (64, 256, 14, 3, 1, 1)])   # 8 channel groups: blocks right of the diagonal
def test_gathered_factor_reduction_pass_variants(K, N, C, H, k, s, p):
    """Split gathered factors end in a reduction pass that permutes the working column order (c/G, tap, c%G) into
    the result order (c, tap), staged through the LDS in blocks of a few channels.  Shapes with different group
    sizes G, tap counts and block counts, all of them split along the rows (their workspace query is non-zero),
    against the fp64 product of the unfolded input; alpha and beta (the EMA form) included."""
    import torch.nn.functional as F
    from asdl_amd import _lib
    assert _lib.load().ak_conv_syrk_nhwc_ws_bytes(N, C, H, H, k, k, s, s, p, p) > 0, 'this case should be split'
    torch.manual_seed(C + k)
    x = torch.randn(N, C, H, H, device='cuda').to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
    d = C * k * k
    u = F.unfold(x.double(), k, padding=p, stride=s).transpose(1, 2).reshape(-1, d)
    old = torch.randn(d, d, device='cuda')
    old = old + old.T
    ref = 0.25 * (u.T @ u) + 0.5 * old.double()
    out = old.clone()
    print(f'gathered reduction N={N} C={C} H={H} k={k} s={s} p={p}', flush=True)
    K.conv_syrk(x, (k, k), (s, s), (p, p), out=out, alpha=0.25, beta=0.5)
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5
    assert torch.equal(out, out.T)


def _group_cases():
    """(kind, args): plain [M, d] operands (with a row stride, ragged sizes, a result with a wide row stride) and
    channels-last convolution inputs (3x3, strided 1x1, 5x5 with padding), small and at the benchmark's sizes."""
    plain = [(64, 128, 128), (777, 264, 264), (333, 1000, 1000), (3000, 64, 64), (4096, 512, 520), (12544, 1024, 1024),
             (3136, 2048, 2048), (50176, 256, 256), (100, 136, 136), (1500, 1600, 1608)]
    conv = [(2, 32, 9, 9, 3, 1, 1), (4, 64, 14, 14, 3, 2, 1), (3, 24, 11, 11, 3, 1, 0), (8, 128, 28, 28, 3, 1, 1),
            (2, 16, 13, 13, 5, 2, 2), (16, 64, 56, 56, 3, 1, 1), (4, 256, 14, 14, 1, 2, 0), (8, 256, 14, 14, 3, 1, 1)]
    return plain, conv


def test_factor_group_matches_the_single_launches_and_fp64(K):
    """kernels.FactorGroup: the factors of many layers in one grouped launch per tile class.  Every result has to
    agree with the fp64 product of the rounded operand to 1e-5 and to be exactly symmetric; alpha / beta (the EMA
    form) and a second contribution to the same result (which forces a flush in between) are covered.  The layers
    that the library computes from shifted correlations are launched at once and checked with the others."""
    import torch.nn.functional as F
    plain, conv = _group_cases()
    torch.manual_seed(3)
    xs, outs, refs = [], [], []
    grp = K.FactorGroup(torch.device('cuda'))
    K._group.active = grp
    try:
        for i, (M, d, ld) in enumerate(plain):
            x = torch.randn(M, ld, device='cuda').to(torch.bfloat16)[:, :d]
            alpha, beta = (0.5, 0.0) if i % 3 else (0.25, 0.75)
            out = torch.full((d, d + 8), 2.0, device='cuda')[:, :d] if i % 4 == 0 else torch.full((d, d), 2.0, device='cuda')
            ref = alpha * (x.double().T @ x.double()) + beta * out.double()
            r = K.syrk_tn(x, out=out, alpha=alpha, beta=beta)
            assert r is out
            xs.append(x); outs.append(out); refs.append(ref)
        for (N, C, H, W, k, s, p) in conv:
            x = torch.randn(N, C, H, W, device='cuda').to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
            d = C * k * k
            u = F.unfold(x.double(), k, padding=p, stride=s).transpose(1, 2).reshape(-1, d)
            out = torch.zeros(d, d, device='cuda')
            K.conv_syrk(x, (k, k), (s, s), (p, p), out=out, alpha=2.0)
            xs.append(x); outs.append(out); refs.append(2.0 * (u.T @ u))
        # 3x3 stride-1 padding-1 layers of whole 64-channel tiles run at once as shifted correlations of the input
        at_once = [c for c in conv if c[4:] == (3, 1, 1) and c[1] % 64 == 0]
        assert len(at_once) == 3
        assert len(grp) == len(plain) + len(conv) - len(at_once), 'every other case should have been taken by the group'
        assert float(outs[1].abs().max()) == 2.0, 'nothing may be written before the flush'
        # a second contribution to the first result: the group has to flush before it takes it
        M, d, _ = plain[0]
        x2 = torch.randn(M, d, device='cuda').to(torch.bfloat16)
        refs[0] = refs[0] + (x2.double().T @ x2.double())
        K.syrk_tn(x2, out=outs[0], alpha=1.0, beta=1.0)
        assert len(grp) == 1
        grp.flush()
        assert len(grp) == 0
    finally:
        K._group.active = None
    torch.cuda.synchronize()
    for i, (out, ref) in enumerate(zip(outs, refs)):
        assert relerr(out, ref) < 1e-5, (i, relerr(out, ref))
        assert torch.equal(out, out.T), i
    # the same calls one by one give the same factors up to the summation order
    for i, (M, d, ld) in enumerate(plain[:4]):
        single = K.syrk_tn(xs[i], alpha=1.0)
        assert single.shape == (d, d)


def test_factor_group_leaves_ineligible_calls_alone(K):
    """fp32 operands, rows that are not 16-byte aligned, the few-channel stem and factors of 3456 columns and more are
    launched at once even while a group is active."""
    grp = K.FactorGroup(torch.device('cuda'))
    K._group.active = grp
    try:
        x = torch.randn(300, 40, device='cuda')
        out = K.syrk_tn(x)
        assert len(grp) == 0 and relerr(out, x.double().T @ x.double()) < 1e-5
        xb = torch.randn(300, 44, device='cuda').to(torch.bfloat16)        # 88-byte rows
        out = K.syrk_tn(xb)
        assert len(grp) == 0 and relerr(out, xb.double().T @ xb.double()) < 1e-5
        stem = torch.randn(2, 3, 32, 32, device='cuda').to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        K.conv_syrk(stem, (7, 7), (2, 2), (3, 3))
        assert len(grp) == 0
        wide = torch.randn(1, 512, 7, 7, device='cuda').to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        K.conv_syrk(wide, (3, 3), (1, 1), (1, 1))
        assert len(grp) == 0
    finally:
        K._group.active = None


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('N,C,hw', [(2, 4, (3, 3)), (8, 64, (7, 7)), (4, 130, (14, 14)), (2, 1000, (1, 1)),
                                    (3, 17, (28, 28)), (1, 257, (5, 9))])
def test_conv_B_factor_matches_oracle(K, dtype, N, C, hw):
    g = _inputs((N, C, *hw), dtype, seed=C)
    ref = R.conv_cov_kron_B(g.float().double())
    print(f'conv B dtype={dtype} N={N} C={C} hw={hw}', flush=True)
    out = K.syrk_nt(g.cuda().flatten(start_dim=2))
    torch.cuda.synchronize()
    assert relerr(out, ref) < 1e-5


def test_conv_syrk_ema_accumulate(K):
    x = _inputs((2, 8, 6, 6), torch.float32, 1)
    A0 = R.conv_cov_kron_A(x, (3, 3), (1, 1), (1, 1))
    x2 = _inputs((2, 8, 6, 6), torch.float32, 2)
    ref = 0.9 * A0.double() + 0.1 * R.conv_cov_kron_A(x2.double(), (3, 3), (1, 1), (1, 1))
    out = A0.cuda().clone()
    K.conv_syrk(x2.cuda(), (3, 3), (1, 1), (1, 1), out=out, alpha=0.1 / 36, beta=0.9)
    assert relerr(out, ref) < TOL_FACTOR_F32


# ------------------------------------------------------------------ damping
def test_kron_damping_matches_oracle(K):
    torch.manual_seed(0)
    pairs = []
    for dA, dB in [(6, 3), (200, 17), (5, 5), (4, 4), (3, 2), (1000, 64)]:
        X = torch.randn(2 * dA, dA)
        Y = torch.randn(2 * dB, dB) * 0.1
        pairs.append((X.T @ X, Y.T @ Y))
    pairs[2] = (pairs[2][0], torch.zeros(5, 5))                      # pi = inf
    pairs[3] = (torch.zeros(4, 4), pairs[3][1])                      # pi = 0
    offdiag = torch.zeros(3, 3)
    offdiag[0, 2] = offdiag[2, 0] = 1.0                              # zero diagonal, non-zero matrix
    pairs[4] = (offdiag, pairs[4][1])
    lam, nz = K.kron_damping([a.cuda() for a, _ in pairs], [b.cuda() for _, b in pairs], 1e-3)
    lam, nz = lam.cpu(), nz.cpu()
    for i, (A, B) in enumerate(pairs):
        ra, rb = R.kron_damping(A, B, 1e-3)
        assert abs(float(lam[i, 0]) - ra) <= 1e-5 * abs(ra), (i, lam[i], ra)
        assert abs(float(lam[i, 1]) - rb) <= 1e-5 * abs(rb), (i, lam[i], rb)
        assert bool(nz[i, 0]) == (not bool(torch.all(A == 0)))
        assert bool(nz[i, 1]) == (not bool(torch.all(B == 0)))


# ------------------------------------------------------------------ damped inverse
@pytest.mark.parametrize('d', [1, 2, 10, 63, 64, 65, 128, 147, 200, 512, 576, 1000, 1152])
def test_chol_inv_matches_oracle(K, d):
    g = torch.Generator().manual_seed(d)
    X = torch.randn(2 * d + 3, d, generator=g)
    A = X.T @ X / (2 * d + 3)
    lam = 0.05
    ref32 = R.cholesky_inv(A, lam)
    ref64 = torch.linalg.inv(A.double() + lam * torch.eye(d, dtype=torch.float64))
    print(f'chol_inv d={d}', flush=True)
    Ag = A.cuda()
    out = K.cholesky_inv(Ag, lam)
    torch.cuda.synchronize()
    assert torch.equal(Ag.cpu(), A), 'input must be left unchanged'
    assert relerr(out, ref32) < TOL_INV
    assert relerr(out, ref64) < TOL_INV
    resid = (A.double() + lam * torch.eye(d, dtype=torch.float64)) @ out.double().cpu() - torch.eye(d, dtype=torch.float64)
    assert float(resid.abs().max()) < 1e-4
    assert torch.equal(out, out.T)


def test_chol_inv_rank_deficient_vs_fp64(K):
    # d > M: conditioning, not the algorithm, limits accuracy; both fp32 results are judged against fp64
    g = torch.Generator().manual_seed(11)
    d, M = 384, 96
    X = torch.randn(M, d, generator=g)
    A = X.T @ X / M
    lam = 1e-3
    ref64 = torch.linalg.inv(A.double() + lam * torch.eye(d, dtype=torch.float64))
    e_ref = relerr(R.cholesky_inv(A, lam), ref64)
    e_hip = relerr(K.cholesky_inv(A.cuda(), lam), ref64)
    print(f'rank deficient: oracle fp32 err {e_ref:.3e}, hip err {e_hip:.3e}', flush=True)
    # cond(A + lam I) ~ 1e4: eps * cond ~ 1e-3 is the fp32 floor for any algorithm
    assert e_hip < max(8 * e_ref, 1e-4)


def test_chol_inv_batched_skip_and_info(K):
    g = torch.Generator().manual_seed(5)
    d = 96
    mats = []
    for _ in range(4):
        X = torch.randn(200, d, generator=g)
        mats.append((X.T @ X / 200).cuda())
    mats[2] = -torch.eye(d).cuda()                                   # not positive definite
    lam = torch.tensor([0.1, 0.2, 0.3, 0.4], device='cuda')
    active = torch.tensor([1, 0, 1, 1], dtype=torch.int32, device='cuda')
    outs = [torch.full((d, d), 7.0, device='cuda') for _ in range(4)]
    info = K.chol_inv_batched(mats, outs, lam, active=active).cpu()
    assert info[0] == 0 and info[3] == 0
    assert info[2] == 1                                              # first leading minor fails
    assert torch.all(outs[1] == 7.0)                                 # skipped: untouched
    for b in (0, 3):
        assert relerr(outs[b], R.cholesky_inv(mats[b].cpu(), float(lam[b]))) < TOL_INV
    with pytest.raises(torch.linalg.LinAlgError):
        K.cholesky_inv(mats[2], 0.5)
    # failure in a later block is reported with its global index
    A = torch.eye(100)
    A[70, 70] = -5.0
    info = K.chol_inv_batched([A.cuda()], [torch.empty(100, 100, device='cuda')], torch.zeros(1, device='cuda')).cpu()
    assert int(info[0]) == 71


def _spd(d, seed, rows=None):
    g = torch.Generator().manual_seed(seed)
    rows = 2 * d + 3 if rows is None else rows
    X = torch.randn(rows, d, generator=g)
    return X.T @ X / rows


def test_chol_inv_grouped_mixed_sizes_match_oracle(K):
    # one call for matrices of many sizes (ragged, not multiples of 4, single-leaf and multi-level ones)
    dims = [1, 2, 10, 63, 64, 65, 128, 147, 200, 256, 384, 512, 576, 640, 1000, 1152, 129, 64, 256, 512]
    mats = [_spd(d, 100 + i) for i, d in enumerate(dims)]
    lams = [0.05 + 0.01 * (i % 5) for i in range(len(dims))]
    print(f'chol_inv_grouped dims={dims}', flush=True)
    dev = [m.cuda() for m in mats]
    outs = [torch.full_like(m, 7.0) for m in dev]
    info = K.chol_inv_grouped(dev, outs, torch.tensor(lams, device='cuda'))
    torch.cuda.synchronize()
    assert torch.all(info == 0)
    for A, Ag, out, lam, d in zip(mats, dev, outs, lams, dims):
        assert torch.equal(Ag.cpu(), A), 'input must be left unchanged'
        ref64 = torch.linalg.inv(A.double() + lam * torch.eye(d, dtype=torch.float64))
        assert relerr(out, R.cholesky_inv(A, lam)) < TOL_INV, d
        assert relerr(out, ref64) < TOL_INV, d
        assert torch.equal(out, out.T), d


def test_chol_inv_grouped_reads_the_lower_triangle_only(K):
    d = 300
    A = _spd(d, 7)
    junk = A.clone()
    junk[torch.triu(torch.ones(d, d, dtype=torch.bool), diagonal=1)] = float('nan')
    out = torch.empty(d, d, device='cuda')
    info = K.chol_inv_grouped([junk.cuda()], [out], torch.tensor([0.1], device='cuda'))
    assert int(info.cpu()[0]) == 0
    assert relerr(out, R.cholesky_inv(A, 0.1)) < TOL_INV


def test_chol_inv_grouped_skip_and_info(K):
    dims = [96, 300, 96, 140, 520]
    mats = [_spd(d, 40 + i).cuda() for i, d in enumerate(dims)]
    mats[2] = -torch.eye(96).cuda()                                  # not positive definite at the first pivot
    bad = torch.eye(520)
    bad[400, 400] = -5.0                                             # fails in a later diagonal block
    mats[4] = bad.cuda()
    lam = torch.tensor([0.1, 0.2, 0.3, 0.4, 0.0], device='cuda')
    active = torch.tensor([1, 0, 1, 1, 1], dtype=torch.int32, device='cuda')
    outs = [torch.full_like(m, 7.0) for m in mats]
    info = K.chol_inv_grouped(mats, outs, lam, active=active).cpu()
    assert info[0] == 0 and info[3] == 0
    assert info[2] == 1 and info[4] == 401
    assert torch.all(outs[1] == 7.0)                                 # skipped: untouched
    for b in (0, 3):
        assert relerr(outs[b], R.cholesky_inv(mats[b].cpu(), float(lam[b]))) < TOL_INV
    # strided lam / flags, and the same call twice (the plan and the workspace are reused)
    lam2 = torch.zeros(5, 2, device='cuda')
    lam2[:, 1] = lam
    info = K.chol_inv_grouped(mats[:2], outs[:2], lam2[:, 1], lam_stride=2).cpu()
    assert info[0] == 0 and info[1] == 0
    assert relerr(outs[1], R.cholesky_inv(mats[1].cpu(), 0.2)) < TOL_INV


@pytest.mark.parametrize('scale,lam_rel', [(1e-8, 1e-2), (1e6, 1e-2), (1.0, 1e-4), (1e-3, 3e-5), (1.0, 1e-6), (3e-5, 1e-8), (1.0, 1e-12), (1e4, 0.0)])
def test_chol_inv_grouped_operand_scaling(K, scale, lam_rel):
    """The products of the grouped inverse run on fp16 pieces of operands scaled by powers of two that come from the
    diagonal maximum and the damping; matrices whose bound a / lam exceeds 2^16 (or lam = 0) keep the bf16 three-piece
    products.  Factors of very different magnitudes (1e-8 ... 1e6) and dampings from 1e-2 down to 1e-12 of the diagonal,
    full-rank and rank-deficient, against fp64: the error has to stay at the level conditioning allows in fp32
    (a few eps * cond), and nothing may overflow."""
    d = 640
    mats, lams = [], []
    for rows, seed in ((2 * d, 1), (d // 4, 2)):                 # full rank; rank 160 of 640
        A = _spd(d, 400 + seed, rows=rows) * scale
        mats.append(A.cuda())
        lams.append(lam_rel * float(A.diagonal().max()))
    lam = torch.tensor(lams, device='cuda')
    outs = [torch.empty_like(m) for m in mats]
    print(f'chol_inv_grouped scaling scale={scale} lam_rel={lam_rel}', flush=True)
    info = K.chol_inv_grouped(mats, outs, lam).cpu()
    eye = torch.eye(d, dtype=torch.float64, device='cuda')
    for i, (A, o) in enumerate(zip(mats, outs)):
        W = A.double() + lams[i] * eye
        ref = torch.linalg.inv(W)
        cond = float(torch.linalg.cond(W))
        try:                                  # what the reference's fp32 Cholesky makes of the same matrix
            e_ref = relerr(R.cholesky_inv(A.cpu(), lams[i]), ref)
        except torch.linalg.LinAlgError:
            e_ref = None
        if e_ref is None or not np.isfinite(e_ref) or e_ref > 1e-2:
            # eps * cond >= 1: beyond what fp32 can factor; LAPACK's unblocked potrf may get through with a result
            # that is wrong in the first digit where the blocked recursion here reports the lost definiteness
            print(f'  matrix {i}: cond {cond:.1e} is out of reach of fp32 (oracle: {e_ref}; info here {int(info[i])})',
                  flush=True)
            continue
        assert int(info[i]) == 0, (i, cond, int(info[i]), e_ref)
        assert torch.isfinite(o).all()
        e = relerr(o, ref)
        print(f'  matrix {i}: cond {cond:.1e}, relative error {e:.1e} (fp32 oracle {e_ref:.1e})', flush=True)
        # Explicit inverses are taken of the 128 x 128 diagonal blocks only (LAPACK solves with the factor itself):
        # measured 1.4-1.7 times the error of potrf + potri on the rank-deficient matrices, 1.3-1.6 on the full-rank
        # ones.  The contract for inverses is 1e-4; beyond the conditioning that allows it, at most twice the oracle.
        assert e < max(1e-4, 2 * e_ref), (i, cond, e, e_ref)


@pytest.mark.parametrize('d', [2048, 2304, 4096, 4608])
def test_chol_inv_large_matches_fp32_oracle_and_fp64(K, d):
    # the sizes of the largest ResNet factors: deepest recursion, every level on the split-bf16 tile kernel
    A = _spd(d, d, rows=2 * d)
    lam = 0.05
    eye = torch.eye(d, dtype=torch.float64)
    ref64 = torch.linalg.inv(A.double() + lam * eye)
    ref32 = R.cholesky_inv(A, lam)
    print(f'chol_inv large d={d}', flush=True)
    out_g = torch.empty(d, d, device='cuda')
    info = K.chol_inv_grouped([A.cuda()], [out_g], torch.tensor([lam], device='cuda'))
    out_b = K.cholesky_inv(A.cuda(), lam)
    torch.cuda.synchronize()
    assert int(info.cpu()[0]) == 0
    for name, out in (('grouped', out_g), ('batched', out_b)):
        e32, e64 = relerr(out, ref32), relerr(out, ref64)
        print(f'  {name}: vs fp32 oracle {e32:.2e}, vs fp64 {e64:.2e} (oracle vs fp64 {relerr(ref32, ref64):.2e})', flush=True)
        assert e32 < TOL_INV and e64 < TOL_INV
        assert torch.equal(out, out.T)


# ------------------------------------------------------------------ products
@pytest.mark.parametrize('tA', [False, True])
@pytest.mark.parametrize('tB', [False, True])
@pytest.mark.parametrize('M,N,K_', [(5, 7, 3), (130, 257, 65), (512, 384, 1000)])
def test_gemm_matches_fp64(K, tA, tB, M, N, K_):
    g = torch.Generator().manual_seed(M + N)
    A = torch.randn((K_, M) if tA else (M, K_), generator=g)
    B = torch.randn((N, K_) if tB else (K_, N), generator=g)
    C0 = torch.randn(M, N, generator=g)
    ref = 0.5 * (A.double().T if tA else A.double()) @ (B.double().T if tB else B.double()) - 2.0 * C0.double()
    out = C0.cuda().clone()
    K.gemm(A.cuda(), B.cuda(), out=out, transA=tA, transB=tB, alpha=0.5, beta=-2.0)
    assert relerr(out, ref) < 1e-5


@pytest.mark.parametrize('pieces,tol', [(3, 2e-6), (2, 3e-5)])
@pytest.mark.parametrize('tA', [False, True])
@pytest.mark.parametrize('tB', [False, True])
@pytest.mark.parametrize('M,N,K_', [(256, 256, 128), (384, 640, 1000), (1100, 520, 516)])
def test_gemm_split_matches_fp64(K, pieces, tol, tA, tB, M, N, K_):
    """fp32 product on the bf16 matrix cores: 3 pieces have to be as good as the fp32 MFMA kernel."""
    torch.manual_seed(M + N)
    A = torch.randn((K_, M) if tA else (M, K_)) * torch.logspace(-3, 3, K_ if not tA else M)[None, :]
    B = torch.randn((N, K_) if tB else (K_, N))
    ref = (A.T if tA else A).double() @ (B.T if tB else B).double()
    print(f'gemm split pieces={pieces} tA={tA} tB={tB} M={M} N={N} K={K_}', flush=True)
    out = K.gemm(A.cuda(), B.cuda(), transA=tA, transB=tB, pieces=pieces)
    out32 = K.gemm(A.cuda(), B.cuda(), transA=tA, transB=tB)
    torch.cuda.synchronize()
    e, e32 = relerr(out, ref), relerr(out32, ref)
    assert e < tol, (e, e32)
    if pieces == 3:
        assert e < 4 * e32 + 1e-7, (e, e32)
    # accumulate form
    C0 = torch.randn(M, N)
    out2 = K.gemm(A.cuda(), B.cuda(), out=C0.cuda().clone(), transA=tA, transB=tB, alpha=0.5, beta=-2.0, pieces=pieces)
    assert relerr(out2, 0.5 * ref - 2.0 * C0.double()) < tol


def test_unit_wise_grouped_kernels_match_the_single_ones(K):
    """Grouped inverse and grouped block-vector product of many modules against the per-module kernels (bit for
    bit: same arithmetic per feature), including an all-zero module and a singular block."""
    torch.manual_seed(9)
    sizes = [64, 256, 300, 1, 2048, 512]
    blocks = []
    for F_ in sizes:
        g = torch.randn(F_, 2, 2, device='cuda')
        blocks.append((g @ g.transpose(1, 2)).contiguous())
    blocks[3].zero_()                                   # all-zero module: flag 0
    blocks[2][7] = torch.tensor([[-0.5, 0.0], [0.0, -0.5]], device='cuda')      # + damping 0.5 -> singular
    dampings = [0.5] * len(sizes)
    invs, flags = K.unit_wise_inv_grouped(blocks, dampings)
    flags = flags.cpu().tolist()
    for b, inv, fl in zip(blocks, invs, flags):
        ref_inv, ref_fl = K.unit_wise_inv(b, 0.5)
        assert fl == ref_fl.cpu().tolist()
        assert torch.equal(torch.nan_to_num(inv, posinf=7.0, neginf=-7.0), torch.nan_to_num(ref_inv, posinf=7.0, neginf=-7.0))
    assert flags[3][0] == 0 and flags[2][1] == 8 and flags[0] == [1, 0x7fffffff]
    # grouped product through the plan
    ws = [torch.randn(F_, device='cuda') for F_ in sizes]
    bs = [torch.randn(F_, device='cuda') for F_ in sizes]
    refs = []
    for inv, w, b in zip(invs, ws, bs):
        rw, rb = w.clone(), b.clone()
        K.unit_wise_mvp(inv, rw, rb, 0.25)
        refs.append((rw, rb))
    K.KronPrecondPlan([], 0.25, unit_items=list(zip(invs, ws, bs))).launch()
    torch.cuda.synchronize()
    for i, ((rw, rb), w, b) in enumerate(zip(refs, ws, bs)):
        if i == 2:
            continue        # holds the singular block (inf / nan entries)
        assert torch.equal(w, rw) and torch.equal(b, rb)


def test_gemm_grouped_matches_fp64(K):
    """Products of very different sizes in one launch, each against its fp64 product; edge tiles, transposes,
    strided rows, a scale per product."""
    torch.manual_seed(5)
    shapes = [(64, 576, 64, False, False), (512, 4608, 512, False, False), (512, 4608, 4608, False, True),
              (1000, 2048, 1000, False, False), (132, 260, 516, True, False), (256, 64, 2048, True, True),
              (4, 8, 12, False, False)]
    for pieces, tol in [(3, 2e-6), (2, 3e-5)]:
        problems, refs = [], []
        for i, (M, N, K_, tA, tB) in enumerate(shapes):
            A = torch.randn((K_, M) if tA else (M, K_), device='cuda')
            B = torch.randn(N, K_ + 8, device='cuda')[:, :K_] if tB else torch.randn(K_, N, device='cuda')   # strided rows
            C = torch.full((M, N), float('nan'), device='cuda')
            alpha = 0.25 * (i + 1)
            problems.append((A, B, C, tA, tB, alpha))
            refs.append(alpha * (A.T if tA else A).double() @ (B.T if tB else B).double())
        print(f'grouped gemm pieces={pieces}', flush=True)
        K.gemm_grouped(problems, pieces=pieces)
        torch.cuda.synchronize()
        for (A, B, C, tA, tB, alpha), ref in zip(problems, refs):
            assert relerr(C, ref) < tol, (tuple(C.shape), A.shape, relerr(C, ref))
    # accumulate form and symmetric products (lower tiles, mirrored) through the raw table
    for pieces in (3, 0):          # 0: the grouped kernel with true fp32 products
        G = torch.randn(260, 516, device='cuda')
        S0 = torch.randn(260, 260, device='cuda'); S0 = S0 + S0.T
        S1 = torch.randn(516, 516, device='cuda'); S1 = S1 + S1.T
        r0 = 0.3 * G.double() @ G.double().T + 0.7 * S0.double()
        r1 = 0.3 * G.double().T @ G.double() + 0.7 * S1.double()
        g = G.data_ptr()
        K.gemm_grouped_raw([(g, 516, g, 516, S0.data_ptr(), 260, 260, 260, 516, 0, 1, 0.3, 0.7, True),
                            (g, 516, g, 516, S1.data_ptr(), 516, 516, 516, 260, 1, 0, 0.3, 0.7, True)], G.device,
                           pieces=pieces)
        torch.cuda.synchronize()
        assert relerr(S0, r0) < 2e-6 and relerr(S1, r1) < 2e-6, pieces
        assert torch.equal(S0, S0.T) and torch.equal(S1, S1.T), pieces
    with pytest.raises(ValueError):
        K.gemm_grouped([(torch.randn(6, 6, device='cuda'), torch.randn(6, 6, device='cuda'),
                         torch.empty(6, 6, device='cuda'), False, False, 1.0)])       # extents not multiples of 4


def test_kron_precond_grouped_matches_fp64(K):
    """All modules in three launches: against B_inv G A_inv and B_inv b in fp64, and against the per-module kernel."""
    torch.manual_seed(6)
    dims = [(64, 576, False), (512, 4608, False), (1000, 2048, True), (64, 64, True), (256, 1152, False),
            (128, 128, True), (2048, 512, False), (8, 12, True), (64, 576, 'cl'), (128, 1152, 'cl'), (16, 100, 'cl5')]
    items, refs, singles = [], [], []
    for dB, dA, bias in dims:
        Bi = torch.randn(dB, dB, device='cuda'); Bi = Bi @ Bi.T / dB
        Ai = torch.randn(dA, dA, device='cuda'); Ai = Ai @ Ai.T / dA
        G = torch.randn(dB, dA, device='cuda')
        if isinstance(bias, str):          # a convolution gradient in the channels-last layout (3x3 or 5x5 window)
            k = 5 if bias == 'cl5' else 3
            G = G.view(dB, dA // (k * k), k, k).contiguous(memory_format=torch.channels_last)
            assert not G.is_contiguous()
            bias = False
        b = torch.randn(dB, device='cuda') if bias else None
        assert K.kron_precond_groupable(Bi, Ai, G, b)
        refs.append((0.5 * Bi.double() @ G.double().reshape(dB, dA) @ Ai.double(),
                     0.5 * Bi.double() @ b.double() if bias else None))
        Gs, bs = G.contiguous().clone(), (b.clone() if bias else None)
        K.kron_precond(Bi, Ai, Gs, bs, grad_scale=0.5)
        singles.append((Gs, bs))
        items.append((Bi, Ai, G, b))
    print('grouped precondition', flush=True)
    K.kron_precond_grouped(items, grad_scale=0.5)
    torch.cuda.synchronize()
    for (Bi, Ai, G, b), (rw, rb), (Gs, bs) in zip(items, refs, singles):
        assert relerr(G.reshape(rw.shape), rw) < 5e-6, (tuple(G.shape), relerr(G.reshape(rw.shape), rw))
        assert relerr(G.reshape(rw.shape), Gs.double().reshape(rw.shape)) < 5e-6
        if b is not None:
            assert relerr(b, rb) < 1e-5
    assert not K.kron_precond_groupable(torch.eye(6, device='cuda'), torch.eye(8, device='cuda'),
                                        torch.zeros(6, 8, device='cuda'))
    assert not K.kron_precond_groupable(torch.eye(8, device='cuda'), torch.eye(8, device='cuda'),
                                        torch.zeros(8, 8, device='cuda', dtype=torch.float64))


@pytest.mark.parametrize('dB,dA,bias', [(4, 5, True), (10, 784, True), (512, 512, True), (64, 147, False),
                                        (300, 1152, False)])
def test_kron_precond_matches_oracle(K, dB, dA, bias):
    g = torch.Generator().manual_seed(dB * 3 + dA)
    Bi = torch.randn(dB, dB, generator=g)
    Bi = Bi @ Bi.T / dB
    Ai = torch.randn(dA, dA, generator=g)
    Ai = Ai @ Ai.T / dA
    G = torch.randn(dB, dA, generator=g)
    b = torch.randn(dB, generator=g) if bias else None
    if bias:
        rw, rb = R.kron_mvp(Ai.double(), Bi.double(), G.double(), b.double())
    else:
        rw, rb = R.kron_mvp(Ai.double(), Bi.double(), G.double()), None
    Gg = G.cuda()
    bg = b.cuda() if bias else None
    K.kron_precond(Bi.cuda(), Ai.cuda(), Gg, bg, grad_scale=1.0)
    assert relerr(Gg, rw) < TOL_PRECOND
    assert relerr(Gg, rw) < 1e-5
    if bias:
        assert relerr(bg, rb) < 1e-5
    # conv-shaped gradient and grad_scale
    if dA % 9 == 0:
        G4 = G.view(dB, dA // 9, 3, 3).contiguous().cuda()
        K.kron_precond(Bi.cuda(), Ai.cuda(), G4, None, grad_scale=0.5)
        assert relerr(G4.view(dB, dA), 0.5 * rw) < 1e-5


# ------------------------------------------------------------------ unit-wise blocks (BatchNorm / LayerNorm)
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('kind,shape', [('bn2d', (6, 16, 7, 5)), ('bn2d_cl', (6, 16, 7, 5)), ('bn2d', (3, 70, 14, 14)),
                                        ('bn2d_cl', (3, 70, 14, 14)), ('bn2d_cl', (2, 8, 33, 40)), ('bn1d', (300, 12)),
                                        ('ln', (5, 37, 48)), ('ln', (200, 768))])
def test_unit_wise_stats_matches_oracle(K, dtype, kind, shape):
    torch.manual_seed(len(shape) + shape[1])
    if kind.startswith('bn2d'):
        m = nn.BatchNorm2d(shape[1])
    elif kind == 'bn1d':
        m = nn.BatchNorm1d(shape[1])
    else:
        m = nn.LayerNorm(shape[-1])
    with torch.no_grad():
        m.weight.uniform_(0.5, 1.5)
        m.bias.uniform_(-0.5, 0.5)
    y = _inputs(shape, dtype, seed=1)
    g = _inputs(shape, dtype, seed=2) * 0.1
    ref = R.norm_cov_unit_wise(m.double(), y.float().double(), g.float().double())
    yg, gg = y.cuda(), g.cuda()
    if kind == 'bn2d_cl':
        yg = yg.contiguous(memory_format=torch.channels_last)
        gg = gg.contiguous(memory_format=torch.channels_last)
    if kind == 'ln':
        yg, gg = yg.reshape(-1, shape[-1]), gg.reshape(-1, shape[-1])
    print(f'unit_wise_stats {kind} {shape} {dtype}', flush=True)
    w, b = m.weight.detach().float().cuda(), m.bias.detach().float().cuda()
    out = K.unit_wise_stats(yg, gg, w, b, alpha=0.25)
    torch.cuda.synchronize()
    assert relerr(out, 0.25 * ref) < 1e-5
    # accumulate form
    out2 = K.unit_wise_stats(yg, gg, w, b, out=out.clone(), alpha=0.5, beta=2.0)
    assert relerr(out2, 1.0 * ref) < 1e-5


def test_unit_wise_inv_and_mvp_match_oracle(K):
    torch.manual_seed(3)
    v = torch.randn(1000, 2, 3)
    blocks = v @ v.transpose(1, 2)
    inv, flags = K.unit_wise_inv(blocks.cuda(), 0.05)
    ref = R.unit_wise_inv(blocks.double(), 0.05)
    assert relerr(inv, ref) < 1e-5
    assert flags.cpu().tolist() == [1, 0x7fffffff]
    _, flags0 = K.unit_wise_inv(torch.zeros(5, 2, 2).cuda(), 0.05)
    assert flags0.cpu().tolist()[0] == 0
    _, flags_bad = K.unit_wise_inv(torch.zeros(5, 2, 2).cuda(), 0.0)
    assert flags_bad.cpu().tolist()[1] == 1                           # first singular block, 1-based
    w, b = torch.randn(1000), torch.randn(1000)
    rw, rb = R.unit_wise_mvp(ref, w.double(), b.double())
    gw, gb = K.unit_wise_mvp(inv, w.cuda(), b.cuda(), scale=2.0)
    assert relerr(gw, 2 * rw) < 1e-5 and relerr(gb, 2 * rb) < 1e-5


# ------------------------------------------------------------------------------ saved factors (bit-exact)
@pytest.mark.parametrize('d', [1, 3, 64, 257, 1000, 4608])
def test_tril_pack_unpack_bit_exact(K, d):
    import numpy as np
    g = torch.Generator().manual_seed(d)
    mat = torch.randn(d, d, generator=g)
    packed = K.tril_pack(mat.cuda())
    rows, cols = np.tril_indices(d)
    assert np.array_equal(packed.cpu().numpy(), mat.numpy()[rows, cols])
    if d <= 257:
        assert torch.equal(packed.cpu(), R.matrix_to_tril(mat))
        assert torch.equal(K.tril_unpack(packed, d).cpu(), R.tril_to_matrix(R.matrix_to_tril(mat)))
    full = K.tril_unpack(packed, d).cpu()
    assert torch.equal(full, full.T) and torch.equal(torch.tril(full), torch.tril(mat))
    # a row stride larger than d (a view of a wider buffer)
    wide = torch.zeros(d, d + 5)
    wide[:, :d] = mat
    assert torch.equal(K.tril_pack(wide.cuda()[:, :d]), packed)


def test_symmatrix_save_load_files(K, tmp_path):
    """File names, dictionary keys and contents as written by asdl/symmatrix.py:226-269, 471-491, 672-680: float32
    .npy, Kronecker factors as packed lower triangles, unit-wise blocks whole."""
    import numpy as np
    from asdl_amd.symmatrix import Kron, SymMatrix, UnitWise, matrix_to_tril, tril_to_matrix
    g = torch.Generator().manual_seed(5)
    a = torch.randn(40, 23, generator=g)
    b = torch.randn(40, 7, generator=g)
    A, B = a.T @ a, b.T @ b
    A, B = (A + A.T) / 2, (B + B.T) / 2     # bit-exact symmetry, so that equality below is exact
    unit = torch.randn(9, 2, 2, generator=g)
    full = torch.randn(11, 11, generator=g)
    full = full + full.T
    sm = SymMatrix(data=full.cuda(), kron=Kron(A.cuda(), B.cuda()), unit=UnitWise(data=unit.cuda()))
    paths = sm.save(str(tmp_path), 'fisher_emp/layer1')
    assert paths == {'tril': 'fisher_emp/layer1/tril.npy',
                     'kron': {'A_tril': 'fisher_emp/layer1/kron/A_tril.npy',
                              'B_tril': 'fisher_emp/layer1/kron/B_tril.npy'},
                     'unit_wise': 'fisher_emp/layer1/unit_wise.npy'}
    on_disk = np.load(tmp_path / paths['kron']['A_tril'])
    assert on_disk.dtype == np.float32 and on_disk.ndim == 1
    assert np.array_equal(on_disk, A.numpy()[np.tril_indices(23)])
    assert np.array_equal(np.load(tmp_path / paths['unit_wise']), unit.numpy())
    assert np.array_equal(np.load(tmp_path / paths['tril']), R.matrix_to_tril(full).numpy())

    back = SymMatrix()
    back.load(path=str(tmp_path / paths['tril']),
              kron_path={k: str(tmp_path / v) for k, v in paths['kron'].items()},
              unit_path=str(tmp_path / paths['unit_wise']))
    assert back.kron.A.is_cuda and torch.equal(back.kron.A.cpu(), A) and torch.equal(back.kron.B.cpu(), B)
    assert torch.equal(back.unit.data.cpu(), unit) and torch.equal(back.data.cpu(), full)
    assert back.kron.A_dim == 23 and back.kron.B_dim == 7

    # a file written the reference's way (numpy only) loads to the same factor
    ref_file = tmp_path / 'ref_A_tril.npy'
    np.save(ref_file, R.matrix_to_tril(A).numpy().astype('float32'))
    k2 = Kron(None, None)
    k2.load(str(ref_file), str(ref_file))
    assert torch.equal(k2.A.cpu(), A)
    assert torch.equal(tril_to_matrix(matrix_to_tril(B.cuda())).cpu(), B)
    with pytest.raises(RuntimeError):
        k2.load(str(ref_file), str(ref_file), device='cpu')
    with pytest.raises(ValueError):
        matrix_to_tril(torch.zeros(3, device='cuda'))


# ------------------------------------------------------------------------------ low-rank (swift) factors
@pytest.mark.parametrize('layout', ['nchw', 'channels_last'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('case', [(3, 4, 6, 5, (3, 3), (2, 1), (1, 0)), (5, 70, 9, 9, (3, 3), (1, 1), (1, 1)),
                                  (2, 3, 20, 20, (7, 7), (2, 2), (3, 3)), (4, 130, 7, 7, (1, 1), (1, 1), (0, 0))])
def test_conv_patch_sum_matches_oracle(K, dtype, layout, case):
    N, C, H, W, k, s, p = case
    x = _inputs((N, C, H, W), dtype, seed=N + C)
    want = torch.nn.functional.unfold(x.double(), k, padding=p, stride=s).sum(-1)
    xg = x.cuda()
    if layout == 'channels_last':
        xg = xg.contiguous(memory_format=torch.channels_last)
    print(f'conv_patch_sum dtype={dtype} layout={layout} case={case}', flush=True)
    out = K.conv_patch_sum(xg, k, s, p, alpha=0.5)
    torch.cuda.synchronize()
    assert out.shape == (N, C * k[0] * k[1]) and relerr(out, 0.5 * want) < 1e-5
    K.conv_patch_sum(xg, k, s, p, out=out, alpha=0.25, beta=2.0)
    assert relerr(out, 1.25 * want) < 1e-5


def test_patch_sum_of_rows_and_positions(K):
    g = torch.Generator().manual_seed(2)
    a = torch.randn(7, 300, generator=g).to(torch.bfloat16)
    assert torch.equal(K.conv_patch_sum(a.cuda(), alpha=1.0).cpu(), a.float())          # Linear: a float32 copy
    gr = torch.randn(5, 33, 49, generator=g)                                              # [n, c, positions]
    assert relerr(K.conv_patch_sum(gr.cuda()), gr.double().sum(-1)) < 1e-6


@pytest.mark.parametrize('n,d,lam', [(8, 27, 1e-2), (64, 576, 3e-2), (3, 300, 0.5), (16, 1100, 1e-1)])
def test_smw_inv_matches_oracle(K, n, d, lam):
    g = torch.Generator().manual_seed(n + d)
    x = torch.randn(n, d, generator=g)
    dense = torch.linalg.inv(x.double().T @ x.double() / n + lam * torch.eye(d, dtype=torch.float64))
    out, info = K.smw_inv(x.cuda(), torch.tensor([lam], device='cuda'))
    assert int(info[0]) == 0
    assert relerr(out, dense) < TOL_INV and relerr(out, R.smw_inv(x, lam)) < TOL_INV


def test_kron_damping_with_row_matrices(K):
    g = torch.Generator().manual_seed(9)
    a_rows, b_sq = torch.randn(6, 40, generator=g), torch.randn(30, 12, generator=g)
    b_sq = b_sq.T @ b_sq
    a_sq = torch.randn(50, 9, generator=g)
    a_sq = a_sq.T @ a_sq
    b_rows = torch.randn(4, 21, generator=g)
    zero = torch.zeros(3, 17)
    pairs = [(a_rows, b_sq), (a_sq, b_rows), (a_rows, b_rows), (zero, b_sq)]
    lam, nz = K.kron_damping([p[0].cuda() for p in pairs], [p[1].cuda() for p in pairs], 1e-2,
                             eig_scale=[(1.0, 4.0), (0.25, 1.0), (1.0, 1.0), (1.0, 1.0)])
    lam, nz = lam.cpu(), nz.cpu()
    for i, ((A, B), (sa, sb)) in enumerate(zip(pairs, [(1.0, 4.0), (0.25, 1.0), (1.0, 1.0), (1.0, 1.0)])):
        want = R.swift_kron_damping(A * (sa if A.shape[0] == A.shape[1] else sa ** 0.5),
                                    B * (sb if B.shape[0] == B.shape[1] else sb ** 0.5), 1e-2)
        assert abs(float(lam[i, 0]) - want[0]) < 1e-5 * want[0] and abs(float(lam[i, 1]) - want[1]) < 1e-5 * want[1]
    assert nz.tolist() == [[1, 1], [1, 1], [1, 1], [0, 1]]
