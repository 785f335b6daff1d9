"""Achieved HBM bandwidth of the memory-bound kernels of the K-FAC path at the shapes of the ResNet-50 / batch 64 step.

`python bench_hbm.py` (or `python bench.py --workload hbm_kernels`) prints ONE JSON line: per case the algorithmic
bytes (every operand read once, every result written once), the time per call (HIP events on the launching stream
around `--reps` back-to-back calls) and bytes / time against the 8 TB/s of an MI355X.  A case whose call is more than
one kernel (SYRK main kernel + split-K sum / EMA pass, the grouped inverse) is timed as a whole here; the per-kernel
durations of the same command come from `rocprofv3 --kernel-trace`, whose kernel names are given in `kernels`.

The first case is the yardstick: a plain copy kernel of 1 GiB.
"""
import argparse
import ctypes
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument('--reps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=3)
    return ap.parse_args(argv)


def main(argv=None):
    args = parse(argv)
    import torch
    from asdl_amd import kernels as K, _lib
    from asdl_amd.symmatrix import matrix_to_tril, tril_to_matrix
    if not torch.cuda.is_available():
        print('bench_hbm.py needs a ROCm GPU.', file=sys.stderr)
        sys.exit(2)
    dev = torch.device('cuda:0')
    torch.manual_seed(0)
    lib = _lib.load()
    cases = []

    def timed(name, kernels, nbytes, fn, note=None):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(args.reps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        us = start.elapsed_time(stop) * 1e3 / args.reps
        gbs = nbytes / us * 1e-3
        case = {'case': name, 'kernels': kernels, 'bytes': int(nbytes), 'us': round(us, 2), 'GB/s': round(gbs, 1),
                'frac': round(gbs / HBM_PEAK_GBS, 4)}
        if note:
            case['note'] = note
        cases.append(case)
        print(f'{name}: {us:.1f} us, {gbs:.0f} GB/s', file=sys.stderr, flush=True)

    def nhwc(n, c, h, w, dtype=torch.bfloat16):
        return torch.randn(n, c, h, w, device=dev).to(dtype).contiguous(memory_format=torch.channels_last)

    # yardstick
    n = 1 << 30
    src, dst = torch.ones(n // 4, device=dev), torch.empty(n // 4, device=dev)
    timed('plain copy, 1 GiB', ['ak::copy_bytes_kernel'], 2 * n,
          lambda: _lib.check(lib.ak_copy_bytes(src.data_ptr(), dst.data_ptr(), n, K._stream()), 'ak_copy_bytes'))
    del src, dst

    # unfold of the 3-channel stem fused into its factor kernel (fp32 images, 7x7 window, stride 2, pad 3), as the
    # benchmark step runs it: inside a bf16 autocast region the fp32 images are rounded to bf16 while they are read
    # and the 17.5 GFLOP run on the bf16 matrix cores; the input is read once
    x = nhwc(64, 3, 224, 224, torch.float32)
    out = torch.empty(147, 147, device=dev)
    timed('stem unfold + A factor, [64,3,224,224] fp32 rounded to bf16, 7x7/2',
          ['ak::conv_patch_bf16_kernel', 'ak::conv_patch_bf16_reduce_kernel'],
          x.numel() * 4 + 147 * 147 * 4, lambda: K.conv_syrk(x, (7, 7), (2, 2), (3, 3), out=out, round_bf16=True),
          note='bound by the window staging and the LDS gathers of its single wave per SIMD, not by memory')
    timed('stem unfold + A factor, [64,3,224,224] fp32 kept fp32, 7x7/2',
          ['ak::conv_patch_syrk_kernel', 'ak::conv_patch_reduce_kernel'],
          x.numel() * 4 + 147 * 147 * 4, lambda: K.conv_syrk(x, (7, 7), (2, 2), (3, 3), out=out),
          note='fp32 MFMA bound (17.5 GFLOP: 0.11 ms at 157.3 TFLOP/s), listed for its unfold traffic')

    # a 3x3 stride-1 convolution's A factor from shifted correlations of its input, d = 576 (layer1): 13 shifts of a
    # [C, C] correlation instead of the [9C, 9C] product of the unfolded input, the input read from the L2 / MALL
    x = nhwc(64, 64, 56, 56)
    out = torch.empty(576, 576, device=dev)
    timed('3x3 A factor by shifted correlations, [64,64,56,56] bf16, d=576',
          ['ak::corr_products_kernel', 'ak::corr_reduce_kernel', 'ak::corr_assemble_kernel'],
          x.numel() * 2 + 576 * 576 * 4, lambda: K.conv_syrk(x, (3, 3), (1, 1), (1, 1), out=out))

    # the unfold of a strided 3x3 convolution fused into the gathered bf16 factor kernel, d = 1152 (layer2.0)
    x = nhwc(64, 128, 56, 56)
    out = torch.empty(1152, 1152, device=dev)
    timed('3x3/2 unfold + A factor, [64,128,56,56] bf16, d=1152',
          ['ak::syrk_dtl_kernel<..., true>', 'ak::syrk_dtl_finalize_blk_kernel'],
          x.numel() * 2 + 1152 * 1152 * 4, lambda: K.conv_syrk(x, (3, 3), (2, 2), (1, 1), out=out),
          note='MFMA bound (33 GFLOP by the SYRK count: 13 us at the bf16 peak), listed for its gather traffic')

    # plain factors of 1x1 convolutions with few channels: (d + 1) / 2 FLOP per byte, memory bound for d <= 512
    for c, hw in ((64, 56), (256, 56), (512, 28)):
        g = nhwc(64, c, hw, hw).permute(0, 2, 3, 1).reshape(-1, c)
        out = torch.empty(c, c, device=dev)
        timed(f'factor x^T x, [{g.shape[0]},{c}] bf16', ['ak::syrk_dtl_kernel<..., false>', 'ak::syrk_dtl_finalize_kernel'],
              g.numel() * 2 + c * c * 4, lambda g=g, out=out: K.syrk_tn(g, out=out))
        timed(f'factor x^T x with EMA (beta = 0.05), [{g.shape[0]},{c}] bf16',
              ['ak::syrk_dtl_kernel<..., false>', 'ak::syrk_dtl_finalize_kernel'],
              g.numel() * 2 + 2 * c * c * 4, lambda g=g, out=out: K.syrk_tn(g, out=out, alpha=0.95, beta=0.05))

    # the widest factor of the step with EMA (d = 4608, 3136 rows): the assembly of the shifted correlations reads the
    # old factor and writes the new one
    x = nhwc(64, 512, 7, 7)
    out = torch.zeros(4608, 4608, device=dev)
    timed('3x3 A factor by shifted correlations with EMA, [64,512,7,7] bf16, d=4608',
          ['ak::corr_products_kernel', 'ak::corr_reduce_kernel', 'ak::corr_assemble_kernel'],
          x.numel() * 2 + 2 * 4608 * 4608 * 4, lambda: K.conv_syrk(x, (3, 3), (1, 1), (1, 1), out=out, alpha=0.95, beta=0.05),
          note='result-bound: 85 MB read and 85 MB written for 1.6 MB of input')

    # unit-wise statistics of a BatchNorm layer (output and output gradient read once)
    y, g = nhwc(64, 256, 56, 56), nhwc(64, 256, 56, 56)
    w, b = torch.rand(256, device=dev) + 0.5, torch.randn(256, device=dev)
    out = torch.empty(256, 2, 2, device=dev)
    timed('unit-wise statistics, [64,256,56,56] bf16 x 2', ['ak::uw_cols_vec_kernel', 'ak::uw_finalize_kernel'],
          2 * y.numel() * 2, lambda: K.unit_wise_stats(y, g, w, b, out=out))

    # SKFAC row matrix: per-sample sums over the positions
    x = nhwc(64, 256, 56, 56)
    timed('per-sample position sums (SKFAC), [64,256,56,56] bf16', ['ak::patch_sum_chan_kernel'],
          x.numel() * 2 + 64 * 256 * 4, lambda: K.conv_patch_sum(x))

    # pi-damping of all 54 layers of ResNet-50: one launch that reads the diagonals
    dims = resnet50_factor_dims()
    A_list = [torch.rand(a, a, device=dev) for a, _ in dims]
    B_list = [torch.rand(b, b, device=dev) for _, b in dims]
    timed('pi-damping of 54 layers (diagonals only)', ['ak::damping_trace_kernel', 'ak::damping_scan_kernel'],
          sum(a + b for a, b in dims) * 4, lambda: K.kron_damping(A_list, B_list, 1e-3),
          note='latency bound: 0.4 MB in one launch')

    # copy-in of the grouped inverse: lower triangles of all 108 factors + damping into the work matrices; timed
    # with the rest of the inverse here, its own duration (ak::cg_copy_in_kernel) is in the kernel trace
    mats = A_list + B_list
    for m in mats:
        m.copy_(torch.eye(m.shape[0], device=dev))
    outs = [torch.empty_like(m) for m in mats]
    lam = torch.full((len(mats),), 1e-3, device=dev)
    tri_bytes = sum(m.shape[0] * (m.shape[0] + 1) // 2 for m in mats) * 4
    timed('grouped inverse of 108 factors (whole call; copy-in = ak::cg_copy_in_kernel in the trace)',
          ['ak::cg_copy_in_kernel', 'ak::cg_leaf_kernel', 'ak::cg_prod_kernel'], 2 * tri_bytes,
          lambda: K.chol_inv_grouped(mats, outs, lam),
          note=f'copy-in alone moves {2 * tri_bytes} bytes (lower triangles read and written); the call is MFMA bound')
    del mats, outs, A_list, B_list

    # packed lower triangle of a saved factor and back
    m = torch.randn(4608, 4608, device=dev)
    m = m + m.T
    tril = matrix_to_tril(m)
    timed('tril pack, d=4608', ['ak::tril_pack_kernel'], tril.numel() * 8, lambda: matrix_to_tril(m))
    timed('tril unpack, d=4608', ['ak::tril_unpack_kernel'], tril.numel() * 4 + m.numel() * 4, lambda: tril_to_matrix(tril))

    print(json.dumps({'metric': 'achieved HBM bandwidth of the memory-bound kernels', 'unit': 'GB/s', 'peak': HBM_PEAK_GBS,
                      'reps': args.reps, 'cases': cases}))


def resnet50_factor_dims():
    """(A size, B size) of the 54 Conv2d / Linear layers of ResNet-50 (A: in_channels * kh * kw, + 1 for the bias of
    the classifier; B: out_channels)."""
    dims = [(147, 64)]
    inplanes = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            dims += [(inplanes, planes), (planes * 9, planes), (planes, planes * 4)]
            if b == 0:
                dims.append((inplanes, planes * 4))
            inplanes = planes * 4
    dims.append((2049, 1000))
    return dims


if __name__ == '__main__':
    main()
