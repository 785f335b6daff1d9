"""Headline benchmark: full K-FAC steps per second on ResNet-50, batch 64, one MI355X.

A step = optimizer.zero_grad(); setup_model_call; setup_loss_call; KfacGradientMaker
.forward_and_backward() (forward, Monte-Carlo Fisher backward with the factor kernels in its hooks,
pi-damped inverses of all 54 layers, loss backward, preconditioning of every gradient);
optimizer.step().  bf16 autocast forward/backward, fp32 factors and inverses, factors refreshed every
step, BatchNorm excluded (Conv2d + Linear only).  Inputs are synthetic N(0,1) images resident in HBM.

Prints ONE JSON line; see --help for the knobs.  The `roofline` object is for the dominant kernel
family (the factor-statistics SYRK kernels): algorithmic FLOP M*d*(d+1) per launch summed over the
108 launches of a step, divided by their summed durations measured with events on the launching
stream inside the timed region (on every fourth step, to keep the instrumentation's own cost small).  `cpu_baseline` times the CPU oracle's K-FAC step (same formulas in
PyTorch CPU ops) on the host cores of the same box.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

BF16_MFMA_PEAK_TFLOPS = 2500.0
FACTOR_TIMING_EVERY = 4     # steps between two steps whose factor launches are timed with events
# Device-memory bytes per factor call (fetched + written, average over the 108 calls of a step) of the default
# workload, from two `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE) of this script scaled by a plain copy kernel of
# known size (--traffic-calibration-mib); counters cannot be read from inside the timed run, so the figure is recorded
# here, reported only for the configuration it was measured on and marked as such (`traffic_source`).  Algorithmic
# bytes of the same calls: 31.7e6.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 71.1e6    # FETCH_SIZE + WRITE_SIZE of the factor kernels per step / 108 factors (see profiles/)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--batch', type=int, default=64)
    ap.add_argument('--fisher', default='fisher_mc', choices=['fisher_mc', 'fisher_emp'])
    ap.add_argument('--damping', type=float, default=1e-3)
    ap.add_argument('--memory-format', default='channels_last', choices=['channels_last', 'contiguous'],
                    help='layout of activations and conv weights; the K-FAC step is the same either way')
    ap.add_argument('--with-batchnorm', action='store_true',
                    help='do not ignore BatchNorm2d: the 53 BN layers get the unit-wise 2x2 blocks of the default K-FAC '
                         '(the headline configuration ignores them, as the reference training script does)')
    ap.add_argument('--workload', default='resnet50', choices=['resnet50', 'linear4096', 'shampoo_gpt2', 'hbm_kernels'],
                    help="resnet50: the headline benchmark.  linear4096: the large single-layer configuration, a single "
                         'Linear 4096x4096 with bias on 8192 bf16 rows, EMA 0.95 (factor + inverse + precondition of one '
                         'large layer; its own metric name, not the headline).  shampoo_gpt2: ShampooGradientMaker '
                         'on a 12-layer GPT-2-small-shaped decoder, 8 x 1024 random tokens, bf16 autocast, statistics and '
                         'preconditioning every step, inverse 4th roots every 10 steps, epsilon 1e-6 (own metric name).  '
                         'hbm_kernels: achieved HBM bandwidth of the memory-bound kernels (bench_hbm.py, own JSON line)')
    ap.add_argument('--swift', action='store_true',
                    help='KfacGradientMaker(swift=True): factors of layers with fewer samples than columns are kept as '
                         'row matrices (SKFAC); not the headline configuration')
    ap.add_argument('--no-conv-autotune', action='store_true',
                    help='leave torch.backends.cudnn.benchmark off (it is on by default, as in the reference training '
                         'script examples/arxiv_results/train.py:227: MIOpen then times its convolution kernels once '
                         'per layer shape during the warm-up and keeps the fastest)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--cpu-batch', type=int, default=0,
                    help='batch of the CPU baseline sample; 0 (default): the full batch of the workload, nothing scaled')
    ap.add_argument('--phase-steps', type=int, default=5,
                    help='steps run after the timed region with phase marks on (events at the phase boundaries of the '
                         'main stream): the per-phase breakdown in the `phases` object; 0 switches it off')
    ap.add_argument('--ranges', action='store_true',
                    help='emit roctx ranges with the reference\'s range names (cov_kron_A, cov_kron_B, inv_kron_A_B, '
                         'fwd, bwd, upd_curv, upd_inv, precond) for `rocprofv3 --marker-trace`')
    ap.add_argument('--no-factor-timing', action='store_true')
    ap.add_argument('--factor-launches', choices=['default', 'single', 'grouped'], default='default',
                    help='single: one launch per Kronecker factor; grouped: the factors of a pass in one grouped launch '
                         '(asdl_amd.fisher.GROUPED_FACTORS); default: the library\'s own setting')
    ap.add_argument('--inverse-flags', choices=['late', 'now'], default='late',
                    help='K-FAC workloads: when the host reads the zero / not-positive-definite flags of a step\'s '
                         'inverses.  now: before it enqueues the preconditioning, as the reference\'s '
                         'torch.linalg.cholesky does (the library\'s default); late: when the next step gets there '
                         '(FisherMaker.late_inverse_flags; the last step\'s flags are read inside the timed region), '
                         'so that the host prepares the next step while the device finishes this one.  Same kernels, '
                         'same results; an error would be raised one step later')
    ap.add_argument('--traffic-calibration-mib', type=int, default=0,
                    help='before the warm-up, launch one plain copy kernel (ak::copy_bytes_kernel) of this many MiB: '
                         'the known traffic against which a `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` run of this '
                         'command is scaled')
    return ap.parse_args()


def cpu_baseline(args):
    """One K-FAC step of the CPU oracle on a bounded sample; returns the cpu_baseline object."""
    import torch
    import torch.nn as nn
    import torch.nn.functional as F
    import bench_models
    from oracle import cpu_ref
    # a one-GPU box gives a job 16 host cores whatever os.cpu_count() shows
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    model = bench_models.resnet50()
    bs = args.cpu_batch or args.batch
    x = torch.randn(bs, 3, 224, 224)
    t = torch.randint(0, 1000, (bs,))

    def fwd(inp):
        with torch.autocast('cpu', dtype=torch.bfloat16):
            return model(inp).float()

    class Wrapped:
        def __call__(self, inp):
            return fwd(inp)

        def parameters(self):
            return model.parameters()

    orc = cpu_ref.KfacOracle(model, data_size=bs, damping=args.damping, fisher_type=args.fisher,
                             factor_dtype=torch.float32)
    orc.model = Wrapped()
    t0 = time.time()
    orc.forward_and_backward(x, t)
    dt = time.time() - t0
    # forward/backward and factor statistics scale with the batch, inverses and preconditioning do not: a sample at
    # a smaller batch, scaled linearly, over-estimates the CPU time of a full step
    scaled = dt * args.batch / bs
    sample = f'one K-FAC step of the CPU oracle (PyTorch CPU ops, {cores} threads) on ResNet-50 at batch {bs} took {dt:.1f} s'
    if bs != args.batch:
        sample += f'; value = 1 / (that time x {args.batch}/{bs})'
    return {'value': 1.0 / scaled, 'unit': 'steps/s', 'cores': cores, 'kind': 'port', 'sample': sample}


def cpu_baseline_linear4096(args):
    """One K-FAC step of the CPU oracle on the single Linear 4096 x 4096 at its full size (8192 bf16 rows, EMA 0.95)."""
    import torch
    import torch.nn as nn
    from oracle import cpu_ref
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(4096, 4096, bias=True))
    x = torch.randn(8192, 4096).to(torch.bfloat16)
    t = torch.randint(0, 4096, (8192,))

    class Wrapped:
        def __call__(self, inp):
            with torch.autocast('cpu', dtype=torch.bfloat16):
                return model(inp).float()

        def parameters(self):
            return model.parameters()

    orc = cpu_ref.KfacOracle(model, data_size=8192, damping=args.damping, ema_decay=0.95, fisher_type=args.fisher,
                             factor_dtype=torch.float32)
    orc.model = Wrapped()
    t0 = time.time()
    orc.forward_and_backward(x, t)
    dt = time.time() - t0
    return {'value': 1.0 / dt, 'unit': 'steps/s', 'cores': cores, 'kind': 'port',
            'sample': f'one K-FAC step of the CPU oracle (PyTorch CPU ops, {cores} threads) on the full workload took {dt:.1f} s'}


def cpu_baseline_shampoo(args, root_interval=10):
    """Shampoo step of the CPU oracle on a bounded sample: one step without a root update at 2 x 1024 tokens (a
    quarter of the batch; forward, backward, statistics, preconditioning), and the inverse 4th root of one statistic
    of each size (768, 1024, 2304, 3072) taken from that step, scaled by how many statistics of that size the model
    has and spread over the root interval."""
    import torch
    import torch.nn.functional as F
    import bench_models
    from oracle import cpu_ref
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    model = bench_models.gpt2_small()
    frac = 4
    x = torch.randint(0, 50257, (8 // frac, 1024))
    t = torch.randint(0, 50257, (8 // frac * 1024,))

    class Wrapped:
        def __call__(self, inp):
            with torch.autocast('cpu', dtype=torch.bfloat16):
                return model(inp).float()

        def parameters(self):
            return model.parameters()

    orc = cpu_ref.ShampooOracle(model, damping=1e-6, curvature_upd_interval=1, preconditioner_upd_interval=10 ** 9)
    orc.model = Wrapped()
    orc.step = 1                                   # not a root step
    t0 = time.time()
    orc.forward_and_backward(x, t, loss_fn=lambda y, tt: F.cross_entropy(y.reshape(-1, y.shape[-1]), tt))
    t_step = time.time() - t0
    counts, sample_stat = {}, {}
    for stats in orc.stats:
        for st in stats:
            n = st.shape[0]
            counts[n] = counts.get(n, 0) + 1
            sample_stat.setdefault(n, st)
    t_roots, parts = 0.0, []
    for n in sorted(counts):
        t0 = time.time()
        _, iters, _ = cpu_ref.compute_power(sample_stat[n].clone(), 4, torch.rand(n) * 2 - 1, ridge_epsilon=1e-6)
        dt = time.time() - t0
        t_roots += dt * counts[n]
        parts.append(f'n={n}: {dt:.1f} s ({iters} iterations) x {counts[n]}')
    per_step = t_step * frac + t_roots / root_interval
    return {'value': 1.0 / per_step, 'unit': 'steps/s', 'cores': cores, 'kind': 'port',
            'sample': f'CPU oracle (PyTorch CPU ops, {cores} threads): one step without roots at 2 x 1024 tokens took '
                      f'{t_step:.1f} s (x {frac} for the full batch); one inverse 4th root per statistic size: '
                      + '; '.join(parts) + f'; value = 1 / (step + all roots / {root_interval})'}


def main():
    args = parse()
    if args.gpus != 1:
        print(f'bench.py measures one GPU: this build has no multi-GPU path (got --gpus {args.gpus}).',
              file=sys.stderr)
        sys.exit(2)
    if args.workload == 'hbm_kernels':
        import bench_hbm          # achieved bandwidth of the memory-bound kernels: its own JSON line
        bench_hbm.main([])
        return
    import torch
    import torch.nn as nn
    import torch.nn.functional as F
    import bench_models
    from asdl_amd import PreconditioningConfig, KfacGradientMaker, kernels
    if args.factor_launches != 'default':
        from asdl_amd import fisher as fisher_mod
        fisher_mod.GROUPED_FACTORS = args.factor_launches == 'grouped'

    if not torch.cuda.is_available():
        print('bench.py needs a ROCm GPU.', file=sys.stderr)
        sys.exit(2)
    dev = torch.device('cuda:0')
    # MIOpen's search over NCHW bf16 solvers takes many minutes on a fresh machine: only the default layout is tuned
    autotune = not args.no_conv_autotune and args.memory_format == 'channels_last'
    torch.backends.cudnn.benchmark = autotune
    torch.manual_seed(0)
    if args.workload == 'shampoo_gpt2':
        pass                                             # built below, with its own gradient maker
    elif args.workload == 'linear4096':
        model = nn.Sequential(nn.Linear(4096, 4096, bias=True)).to(dev)
        bs = 8192
        x = torch.randn(bs, 4096).to(dev).to(torch.bfloat16)
        t = torch.randint(0, 4096, (bs,)).to(dev)
        config = PreconditioningConfig(data_size=bs, damping=args.damping, ema_decay=0.95)
    else:
        model = bench_models.resnet50().to(dev)
        bs = args.batch
        x = torch.randn(bs, 3, 224, 224).to(dev)
        if args.memory_format == 'channels_last':
            model = model.to(memory_format=torch.channels_last)
            x = x.contiguous(memory_format=torch.channels_last)
        t = torch.randint(0, 1000, (bs,)).to(dev)
        ignore = [] if args.with_batchnorm else [nn.BatchNorm2d]
        config = PreconditioningConfig(data_size=bs, damping=args.damping, ignore_modules=ignore)
    if args.workload == 'shampoo_gpt2':
        from asdl_amd import ShampooGradientMaker
        model = bench_models.gpt2_small().to(dev)       # token embedding and output head frozen (50257-wide)
        bs = 8
        x = torch.randint(0, 50257, (bs, 1024)).to(dev)
        t = torch.randint(0, 50257, (bs * 1024,)).to(dev)
        config = PreconditioningConfig(damping=1e-6, curvature_upd_interval=1, preconditioner_upd_interval=10)
        gm = ShampooGradientMaker(model, config)
        args.no_factor_timing = True
        # the dominant kernels of this workload are the products of the coupled Newton iteration: events around every
        # root update of the timed region, FLOP from the iteration counts the update reports (8 n^3 per iteration)
        root_records = []
        plain_update = gm.update_preconditioner

        def timed_update():
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            plain_update()
            stop.record()
            root_records.append((start, stop, {key: st for key, st in gm.last_root_stats.items()}))
        gm.update_preconditioner = timed_update
    else:
        gm = KfacGradientMaker(model, config, fisher_type=args.fisher, swift=args.swift)
        gm.late_inverse_flags = args.inverse_flags == 'late'
    late_flags = getattr(gm, 'late_inverse_flags', False)
    opt = torch.optim.SGD([p for p in model.parameters() if p.requires_grad], lr=1e-4)

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    def token_loss(y, target):
        return F.cross_entropy(y.reshape(-1, y.shape[-1]), target)

    # the K-FAC makers call the loss with reduction='sum' themselves (as the reference's do) and need its keyword
    loss_fn = token_loss if args.workload == 'shampoo_gpt2' else F.cross_entropy

    def step():
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(fwd, x)
        gm.setup_loss_call(loss_fn, dummy_y, t)
        gm.forward_and_backward()
        opt.step()

    if args.traffic_calibration_mib > 0:
        import ctypes
        from asdl_amd import _lib
        n = args.traffic_calibration_mib << 20
        src = torch.ones(n // 4, device=dev)
        dst = torch.empty_like(src)
        lib = _lib.load()
        torch.cuda.synchronize()
        _lib.check(lib.ak_copy_bytes(src.data_ptr(), dst.data_ptr(), n, None), 'ak_copy_bytes')
        torch.cuda.synchronize()
        del src, dst

    if args.ranges:
        from asdl_amd import profiling
        profiling.enable_ranges(True)
    for i in range(args.warmup):
        step()
        if i == 0:
            torch.cuda.synchronize()
            print('bench.py: first warm-up step done (kernel selection, workspaces)', file=sys.stderr, flush=True)
    if args.workload == 'shampoo_gpt2':
        del root_records[:]
    sink = None if args.no_factor_timing else []
    kernels.set_timing_sink(sink, n_events=2 * 110 * args.steps)     # two events per factor call, made up front
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        # the factor launches of every fourth step are bracketed by events (each pair costs a few microseconds of
        # host time and a marker in the queue: 216 pairs per step would slow the measured step by 5 %)
        kernels.enable_timing(i % FACTOR_TIMING_EVERY == 0)
        step()
    if late_flags:
        gm.check_late_flags()         # the flags of the last step's inverses
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernels.enable_timing(True)
    kernels.set_timing_sink(None)

    ms_per_step = elapsed / args.steps * 1e3

    phases = None
    if args.phase_steps > 0:
        # Separate, untimed steps: an event at every phase boundary of the main stream.  The phases are those of the
        # reference's profiling example (examples/prof/time_step.py: fwd_bwd_upd_curv, upd_inv, precond, upd_param),
        # with the curvature update split into its three passes.  Work on side streams (the inverses) shows up in the
        # phase it runs beside; `upd_inv` is what is left of it after the loss backward pass.
        from asdl_amd import profiling
        marks = []
        profiling.set_phase_sink(marks)
        for _ in range(args.phase_steps):
            profiling.phase_mark('begin')
            step()
            profiling.phase_mark('upd_param')
        torch.cuda.synchronize()
        profiling.set_phase_sink(None)
        sums, host = {}, {}
        for (_, e0, h0), (name, e1, h1) in zip(marks, marks[1:]):
            if name != 'begin':
                sums[name] = sums.get(name, 0.0) + e0.elapsed_time(e1)
                host[name] = host.get(name, 0.0) + (h1 - h0) * 1e3
        # `ms`: between the events on the device; `host_ms`: between the moments the host enqueued them (a phase
        # whose host time is close to its device time is bound by the host's launch rate)
        phases = {'steps': args.phase_steps, 'unit': 'ms per step',
                  'ms': {k: round(v / args.phase_steps, 4) for k, v in sums.items()},
                  'host_ms': {k: round(v / args.phase_steps, 4) for k, v in host.items()},
                  'sum_ms': round(sum(sums.values()) / args.phase_steps, 4)}
    out = {
        'metric': 'K-FAC steps/s ResNet-50 bs64',
        'value': args.steps / elapsed,
        'unit': 'steps/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': ms_per_step,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': f'K-FAC step (factors + pi-damped Cholesky inverses + precondition every step, '
                               f'{args.fisher}) on ResNet-50, batch {bs}, 3x224x224 N(0,1) images, 1000 classes, '
                               f'bf16 autocast forward/backward, fp32 factors/inverses, damping {args.damping}, '
                               f'BatchNorm {"unit-wise" if args.with_batchnorm else "ignored"}, {args.memory_format} activations and weights, '
                               f'cudnn.benchmark {"on" if autotune else "off"}' + (', swift (SKFAC) factors' if args.swift else '')
                               + (', flags of a step\'s inverses read by the host one step late' if late_flags else ''),
                   'batch': bs},
    }
    if sink:
        timed_steps = len(range(0, args.steps, FACTOR_TIMING_EVERY))
        flops = sum(s[1] for s in sink)
        secs = sum(s[2].elapsed_time(s[3]) for s in sink) * 1e-3
        achieved = flops / secs / 1e12
        default_workload = (bs == 64 and args.fisher == 'fisher_mc' and args.memory_format == 'channels_last'
                            and not args.with_batchnorm and not args.swift)
        traffic = MEASURED_TRAFFIC_BYTES_PER_LAUNCH if default_workload else None
        out['roofline'] = {'bound': 'mfma', 'achieved': achieved, 'peak': BF16_MFMA_PEAK_TFLOPS, 'unit': 'TFLOP/s',
                           'frac': achieved / BF16_MFMA_PEAK_TFLOPS, 'traffic': traffic,
                           'traffic_source': None if traffic is None else
                           'not measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command '
                           '(profiles/factor_kernels_resnet50_bs64_hbm_traffic.txt), bytes per factor call',
                           'floor_ms_per_step': 0.908 if default_workload else None,
                           'kernel': 'factor statistics (syrk_dtl_kernel, single and grouped; conv_patch_bf16_kernel for the 3-channel '
                                     'stem), SYRK FLOP M*d*(d+1)',
                           'launches_per_step': sum(s[4] for s in sink) // timed_steps,
                           'timed_regions_per_step': len(sink) // timed_steps,
                           'factor_ms_per_step': secs / timed_steps * 1e3,
                           'timed_steps': timed_steps,
                           'gemm_equiv_tflops': 2 * achieved}
    if args.workload == 'linear4096':
        out['metric'] = 'K-FAC steps/s Linear 4096x4096, 8192 rows'
        out['config'] = {'workload': f'K-FAC step (factors with EMA 0.95 + pi-damped Cholesky inverses + precondition every '
                                     f'step, {args.fisher}) on one Linear 4096x4096 with bias, 8192 N(0,1) rows, bf16 '
                                     f'autocast, fp32 factors/inverses, damping {args.damping}', 'batch': bs}
        if 'roofline' in out:
            out['roofline']['traffic'] = None
            out['roofline']['kernel'] = 'factor statistics (syrk_dtl_kernel, 8192 x 4096 bf16 operands), SYRK FLOP M*d*(d+1)'
    elif args.workload == 'shampoo_gpt2':
        out['metric'] = 'Shampoo steps/s GPT-2-small decoder, 8x1024 tokens'
        out['config'] = {'workload': 'Shampoo step (L/R statistics and preconditioning of the 49 trainable weight matrices '
                                     'every step, inverse 4th roots every 10 steps, epsilon 1e-6) on a 12-layer '
                                     'GPT-2-small-shaped decoder (d 768, 12 heads, MLP 3072; token embedding and output '
                                     'head frozen), 8 x 1024 uniform random tokens, bf16 autocast forward/backward, '
                                     'fp32 statistics and roots', 'batch': bs}
        if root_records:
            secs = sum(a.elapsed_time(b) for a, b, _ in root_records) * 1e-3
            flops, executed_flops, iters = 0.0, 0.0, []
            for _, _, stats in root_records:
                for (n, exp), st in stats.items():
                    it = st[:, 2].double().cpu()
                    products = 2 + (exp - 1).bit_length()      # root T, T^p by squaring (p a power of two), T^p M
                    f = float(it.sum()) * products * 2.0 * n ** 3
                    flops += f
                    # every fp32 product runs as 6 bf16 piece products; matrices of 512 and up are known to be
                    # symmetric and only their T (T + 1) / 2 tiles of 128 on and below the diagonal are computed
                    tiles = -(-n // 128)
                    executed_flops += 6.0 * f * ((tiles + 1) / (2.0 * tiles) if n >= 512 else 1.0)
                    iters.append(int(it.max()))
            executed = executed_flops / secs / 1e12
            out['roofline'] = {'bound': 'mfma', 'achieved': executed, 'peak': BF16_MFMA_PEAK_TFLOPS, 'unit': 'TFLOP/s',
                               'frac': executed / BF16_MFMA_PEAK_TFLOPS, 'traffic': None,
                               'kernel': 'products of the coupled Newton iteration (gemm_x3_kernel); `achieved` counts the '
                                         'bf16 MFMA work executed: 6 piece products per fp32 product, lower tiles only '
                                         'for the symmetric results; algorithmic_fp32_tflops counts the 2 n^3 per '
                                         'product of the reference',
                               'algorithmic_fp32_tflops': flops / secs / 1e12,
                               'root_updates_timed': len(root_records),
                               'ms_per_root_update': secs / len(root_records) * 1e3,
                               'newton_iterations_max': max(iters)}
    if not args.no_cpu_baseline:
        if args.workload == 'linear4096':
            out['cpu_baseline'] = cpu_baseline_linear4096(args)
        elif args.workload == 'shampoo_gpt2':
            out['cpu_baseline'] = cpu_baseline_shampoo(args)
        else:
            out['cpu_baseline'] = cpu_baseline(args)
    if phases is not None:
        out['phases'] = phases
    print(json.dumps(out))


if __name__ == '__main__':
    main()
