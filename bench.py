"""Headline benchmark: full K-FAC steps per second on ResNet-50, batch 64, one MI355X.

A step = optimizer.zero_grad(); setup_model_call; setup_loss_call; KfacGradientMaker
.forward_and_backward() (forward, Monte-Carlo Fisher backward with the factor kernels in its hooks,
pi-damped inverses of all 54 layers, loss backward, preconditioning of every gradient);
optimizer.step().  bf16 autocast forward/backward, fp32 factors and inverses, factors refreshed every
step, BatchNorm excluded (Conv2d + Linear only).  Inputs are synthetic N(0,1) images resident in HBM.

Prints ONE JSON line; see --help for the knobs.  The headline (`value`, `ms_per_step`) is measured with the library's
defaults (the flags of a step's inverses are read in the step's own call, once its preconditioning is enqueued); the
same steps with the flags read one step late are reported beside it (`late_inverse_flags`).  The `roofline` object is for the dominant kernel family (the factor-statistics kernels):
algorithmic FLOP M*d*(d+1) per launch summed over the 108 factors of a step, divided by their summed durations
measured with events on the launching stream inside the timed region (on every fourth step, to keep the
instrumentation's own cost small); `floor_ms_per_step` is the sum of the per-launch roofline floors of the same
launches.  `roofline_inverse` times the damped Cholesky inverses of the step's factors stand-alone.  `secondary`
holds brief runs of the single-layer (linear4096), the fp32 ResNet-18 (resnet18_cifar) and the Shampoo (shampoo_gpt2)
configurations.
`cpu_baseline` times the CPU oracle's K-FAC step (same formulas in PyTorch CPU ops) on the host cores of the same box.
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
FP32_MFMA_PEAK_TFLOPS = 157.3
FACTOR_TIMING_EVERY = 4     # steps between two steps whose factor launches are timed with events


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
    ap.add_argument('--workload', default='resnet50', choices=['resnet50', 'linear4096', 'resnet18_cifar', 'shampoo_gpt2', 'hbm_kernels'],
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
    ap.add_argument('--no-secondary', action='store_true',
                    help='default workload only: skip the second measurement with the other setting of --inverse-flags '
                         'and the brief runs of the linear4096, resnet18_cifar and shampoo_gpt2 workloads (the `secondary` object)')
    ap.add_argument('--no-inverse-roofline', action='store_true',
                    help='skip the stand-alone timing of the damped inverses (the `roofline_inverse` object)')
    ap.add_argument('--factor-launches', choices=['default', 'single', 'grouped'], default='default',
                    help='single: one launch per Kronecker factor; grouped: the factors of a pass in one grouped launch '
                         '(asdl_amd.fisher.GROUPED_FACTORS); default: the library\'s own setting')
    ap.add_argument('--inverse-flags', choices=['late', 'now', 'before'], default='now',
                    help='K-FAC workloads: when the host reads the zero / not-positive-definite flags of a step\'s '
                         'inverses in the headline measurement.  now (default, the library\'s default): in the same '
                         'forward_and_backward() call, once the preconditioning has been enqueued (a bad factor raises '
                         'from that call with the gradients put back as the backward pass left them, as the '
                         'reference\'s torch.linalg.cholesky would leave them); before: before the preconditioning is '
                         'enqueued (asdl_amd.natural_gradient.FLAGS_AFTER_PRECONDITION = False); late: when the next '
                         'step gets there (FisherMaker.late_inverse_flags; the last step\'s flags are read inside the '
                         'timed region), an error would be raised one step later.  Same kernels, same results')
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


def build_workload(args, name, dev):
    """Model, synthetic batch (resident in HBM), K-FAC configuration and forward function of one K-FAC workload."""
    import torch
    import torch.nn as nn
    import bench_models
    from asdl_amd import PreconditioningConfig
    w = {'name': name, 'autocast': True, 'peak': BF16_MFMA_PEAK_TFLOPS, 'dtype': 'bf16', 'autotune': False}
    if name == 'linear4096':
        model = nn.Sequential(nn.Linear(4096, 4096, bias=True)).to(dev)
        bs = 8192
        x = torch.randn(bs, 4096).to(dev).to(torch.bfloat16)
        t = torch.randint(0, 4096, (bs,)).to(dev)
        config = PreconditioningConfig(data_size=bs, damping=args.damping, ema_decay=0.95)
    elif name == 'resnet18_cifar':
        # fp32 end to end, NCHW: the reference's own CIFAR-10 training configuration (examples/arxiv_results)
        model = bench_models.resnet18_cifar().to(dev)
        bs = 128
        x = torch.randn(bs, 3, 32, 32).to(dev)
        t = torch.randint(0, 10, (bs,)).to(dev)
        config = PreconditioningConfig(data_size=bs, damping=args.damping, ignore_modules=[nn.BatchNorm2d])
        w.update(autocast=False, peak=FP32_MFMA_PEAK_TFLOPS, dtype='f32')
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
        # MIOpen's search over NCHW bf16 solvers takes many minutes on a fresh machine: only the default layout is tuned
        w['autotune'] = not args.no_conv_autotune and args.memory_format == 'channels_last'
    autocast = w['autocast']

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16, enabled=autocast):
            return model(inp).float()

    w.update(model=model, x=x, t=t, bs=bs, config=config, fwd=fwd)
    return w


def measure_kfac(w, args, steps, warmup, flags_mode, factor_timing, phase_steps):
    """Warm-up, then `steps` timed K-FAC steps of workload `w`; returns the wall time per step, the factor launches
    recorded with events inside the timed region, and the per-phase breakdown of extra steps after it."""
    import torch
    import torch.nn.functional as F
    from asdl_amd import KfacGradientMaker, kernels
    torch.backends.cudnn.benchmark = w['autotune']
    model, x, t = w['model'], w['x'], w['t']
    for m in model.modules():                      # a fresh maker starts from fresh curvature
        if hasattr(m, 'fisher'):
            delattr(m, 'fisher')
    gm = KfacGradientMaker(model, w['config'], fisher_type=args.fisher, swift=args.swift)
    import asdl_amd.natural_gradient as ng_mod
    late_flags = flags_mode == 'late'
    gm.late_inverse_flags = late_flags
    ng_mod.FLAGS_AFTER_PRECONDITION = flags_mode != 'before'
    opt = torch.optim.SGD([p for p in model.parameters() if p.requires_grad], lr=1e-4)

    def step():
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(w['fwd'], x)
        gm.setup_loss_call(F.cross_entropy, dummy_y, t)      # the maker calls it with reduction='sum', as the reference's does
        gm.forward_and_backward()
        opt.step()

    for i in range(warmup):
        step()
        if i == 0:
            torch.cuda.synchronize()
            print(f'bench.py: first warm-up step of {w["name"]} done (kernel selection, workspaces)', file=sys.stderr,
                  flush=True)
    sink = [] if factor_timing else None
    kernels.set_timing_sink(sink, n_events=2 * 110 * steps)     # two events per factor call, made up front
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
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
    res = {'ms_per_step': elapsed / steps * 1e3, 'value': steps / elapsed, 'gm': gm, 'step': step}
    if sink:
        timed_steps = len(range(0, steps, FACTOR_TIMING_EVERY))
        flops = sum(s[1] for s in sink)
        secs = sum(s[2].elapsed_time(s[3]) for s in sink) * 1e-3
        achieved = flops / secs / 1e12
        res['roofline'] = {'bound': 'mfma', 'achieved': achieved, 'peak': w['peak'], 'unit': 'TFLOP/s',
                           'frac': achieved / w['peak'], 'traffic': None,
                           # per launch max(FLOP / matrix peak, algorithmic bytes / 8 TB/s), summed over the launches of a step
                           'floor_ms_per_step': sum(s[5] for s in sink) / timed_steps * 1e3,
                           'launches_per_step': sum(s[4] for s in sink) // timed_steps,
                           'timed_regions_per_step': len(sink) // timed_steps,
                           'factor_ms_per_step': secs / timed_steps * 1e3,
                           'flop_per_step': flops / timed_steps,
                           'timed_steps': timed_steps,
                           'gemm_equiv_tflops': 2 * achieved}
    if phase_steps > 0:
        # Separate, untimed steps: an event at every phase boundary of the main stream.  The phases are those of the
        # reference's profiling example (examples/prof/time_step.py: fwd_bwd_upd_curv, upd_inv, precond, upd_param),
        # with the curvature update split into its three passes.  Work on side streams (the inverses) shows up in the
        # phase it runs beside; `upd_inv` is what is left of it after the loss backward pass.
        from asdl_amd import profiling
        marks = []
        profiling.set_phase_sink(marks)
        for _ in range(phase_steps):
            profiling.phase_mark('begin')
            step()
            profiling.phase_mark('upd_param')
        if late_flags:
            gm.check_late_flags()
        torch.cuda.synchronize()
        profiling.set_phase_sink(None)
        sums, host = {}, {}
        for (_, e0, h0), (name, e1, h1) in zip(marks, marks[1:]):
            if name != 'begin':
                sums[name] = sums.get(name, 0.0) + e0.elapsed_time(e1)
                host[name] = host.get(name, 0.0) + (h1 - h0) * 1e3
        # `ms`: between the events on the device; `host_ms`: between the moments the host enqueued them (a phase
        # whose host time is close to its device time is bound by the host's launch rate)
        res['phases'] = {'steps': phase_steps, 'unit': 'ms per step',
                         'ms': {k: round(v / phase_steps, 4) for k, v in sums.items()},
                         'host_ms': {k: round(v / phase_steps, 4) for k, v in host.items()},
                         'sum_ms': round(sum(sums.values()) / phase_steps, 4)}
    return res


def inverse_roofline(w, damping, reps=5):
    """The pi-damped Cholesky inverses of all Kronecker factors of the workload, stand-alone: the factors the last
    step left on the modules go through the same damping launch and grouped inverse as in the step, with nothing
    running beside them.  FLOP: d^3 per factor (factorization, triangular inverse and M^T M together: what POTRF +
    POTRI cost), priced at the fp32 matrix peak the reference's arithmetic would run at; `executed_fp16_frac` prices
    the three fp16 piece products that each fp32 product is executed as against the fp16 peak."""
    import torch
    from asdl_amd.symmatrix import Kron, batched_update_inv
    krons = []
    for m in w['model'].modules():
        cache = getattr(m, '_asdl_amd_factor_cache', None)
        fisher = getattr(m, 'fisher', None)
        A = B = None
        if fisher is not None and fisher.kron is not None and fisher.kron.A is not None:
            A, B = fisher.kron.A, fisher.kron.B                  # accumulated factors (EMA)
        elif cache is not None and 'A' in cache and 'B' in cache:
            A, B = cache['A'], cache['B']                        # per-step factors: scratch buffers reused every step
        if A is not None and B is not None and A.shape[0] == A.shape[1] and B.shape[0] == B.shape[1]:
            krons.append(Kron(A, B))
    if not krons:
        return None
    flop = float(sum(k.A.shape[0] ** 3 + k.B.shape[0] ** 3 for k in krons))
    batched_update_inv(krons, damping=damping)                   # plan, workspaces, output buffers
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        batched_update_inv(krons, damping=damping)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    achieved = flop / (ms * 1e-3) / 1e12
    return {'bound': 'mfma', 'achieved': achieved, 'peak': FP32_MFMA_PEAK_TFLOPS, 'unit': 'TFLOP/s',
            'frac': achieved / FP32_MFMA_PEAK_TFLOPS, 'executed_fp16_frac': 3 * achieved / BF16_MFMA_PEAK_TFLOPS,
            'flop_per_step': flop, 'matrices': 2 * len(krons), 'standalone_ms': ms,
            'kernel': 'damped Cholesky inverses of all Kronecker factors of a step (cg_leaf_kernel, cg_prod_kernel, '
                      'cg_copy_in_kernel, damping kernels), one grouped call with its flag read, nothing beside it; in '
                      'the step the same call runs on a side stream beside the loss backward pass'}


def read_measured_traffic():
    """Bytes per factor call (fetched + written) of the default workload, from the committed summary of the counter
    runs (profiles/factor_kernels_resnet50_bs64_hbm_traffic.txt): counters cannot be read from inside the timed run."""
    path = os.path.join(ROOT, 'profiles', 'factor_kernels_resnet50_bs64_hbm_traffic.txt')
    try:
        import re
        m = re.search(r'per factor call \(\d+\): [0-9.]+ MiB = (\d+) bytes', open(path).read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


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
    if args.factor_launches != 'default':
        from asdl_amd import fisher as fisher_mod
        fisher_mod.GROUPED_FACTORS = args.factor_launches == 'grouped'
    if not torch.cuda.is_available():
        print('bench.py needs a ROCm GPU.', file=sys.stderr)
        sys.exit(2)
    dev = torch.device('cuda:0')
    torch.manual_seed(0)
    if args.workload == 'shampoo_gpt2':
        return main_shampoo(args, dev)

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

    w = build_workload(args, args.workload, dev)
    bs = w['bs']
    late = args.inverse_flags == 'late'
    res = measure_kfac(w, args, args.steps, args.warmup, args.inverse_flags, not args.no_factor_timing, args.phase_steps)
    out = {
        'metric': 'K-FAC steps/s ResNet-50 bs64',
        'value': res['value'],
        'unit': 'steps/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': res['ms_per_step'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': w['dtype'],
        'data': 'synthetic',
        'config': {'workload': f'K-FAC step (factors + pi-damped Cholesky inverses + precondition every step, '
                               f'{args.fisher}) on ResNet-50, batch {bs}, 3x224x224 N(0,1) images, 1000 classes, '
                               f'bf16 autocast forward/backward, fp32 factors/inverses, damping {args.damping}, '
                               f'BatchNorm {"unit-wise" if args.with_batchnorm else "ignored"}, {args.memory_format} activations and weights, '
                               f'cudnn.benchmark {"on" if w["autotune"] else "off"}' + (', swift (SKFAC) factors' if args.swift else '')
                               + {'late': ', flags of a step\'s inverses read by the host one step late',
                                  'before': ', flags of a step\'s inverses read before its preconditioning is enqueued',
                                  'now': ', the library\'s defaults (a factor that is not positive definite raises '
                                         'from the step\'s own call and leaves the raw gradients, as the reference\'s '
                                         'Cholesky does; the host reads the flags once the preconditioning is enqueued)'
                                  }[args.inverse_flags],
                   'batch': bs},
    }
    default_workload = (args.workload == 'resnet50' and bs == 64 and args.fisher == 'fisher_mc'
                        and args.memory_format == 'channels_last' and not args.with_batchnorm and not args.swift)
    if 'roofline' in res:
        out['roofline'] = res['roofline']
        out['roofline']['kernel'] = ('factor statistics (syrk_dtl_kernel, single and grouped; corr_products_kernel + '
                                     'corr_reduce_kernel + corr_assemble_kernel for the 3x3 stride-1 layers; '
                                     'conv_patch_bf16_kernel for the 3-channel stem), SYRK FLOP M*d*(d+1)')
        if default_workload:
            traffic = read_measured_traffic()
            out['roofline']['traffic'] = traffic
            out['roofline']['traffic_source'] = None if traffic is None else (
                'not measured by this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, read from '
                'profiles/factor_kernels_resnet50_bs64_hbm_traffic.txt, bytes per factor call')
    if args.workload == 'linear4096':
        out['metric'] = 'K-FAC steps/s Linear 4096x4096, 8192 rows'
        out['config'] = {'workload': f'K-FAC step (factors with EMA 0.95 + pi-damped Cholesky inverses + precondition every '
                                     f'step, {args.fisher}) on one Linear 4096x4096 with bias, 8192 N(0,1) rows, bf16 '
                                     f'autocast, fp32 factors/inverses, damping {args.damping}', 'batch': bs}
        if 'roofline' in out:
            out['roofline']['kernel'] = 'factor statistics (syrk_dtl_kernel, 8192 x 4096 bf16 operands), SYRK FLOP M*d*(d+1)'
    elif args.workload == 'resnet18_cifar':
        out['metric'] = 'K-FAC steps/s ResNet-18 (CIFAR stem) bs128 fp32'
        out['config'] = {'workload': f'K-FAC step (factors + pi-damped Cholesky inverses + precondition every step, '
                                     f'{args.fisher}) on ResNet-18 with the CIFAR stem (3x3, no max-pool), batch 128, '
                                     f'3x32x32 N(0,1) images, 10 classes, fp32 and NCHW end to end, Conv2d factors up to '
                                     f'4608 x 4608, damping {args.damping}, BatchNorm ignored, cudnn.benchmark off',
                         'batch': bs}
        if 'roofline' in out:
            out['roofline']['kernel'] = ('factor statistics of fp32 NCHW operands: the 3x3 stride-1 layers as shifted '
                                         'correlations of three bf16 planes of the input (corr_split_nchw_kernel, '
                                         'corr_products_kernel, corr_fold_kernel, corr_assemble_kernel: bf16 matrix '
                                         'cores, fp32 accuracy), the others on conv_syrk_kernel<float>, '
                                         'conv_patch_syrk_kernel<float>, syrk_tn_kernel<float> (v_mfma_f32_32x32x2_f32); '
                                         'SYRK FLOP M*d*(d+1) against the fp32 matrix peak, the rate the reference\'s '
                                         'fp32 arithmetic is priced at')
    inv = inverse_roofline(w, args.damping) if not args.no_inverse_roofline else None
    if inv is not None:
        out['roofline_inverse'] = inv
    if 'phases' in res:
        out['phases'] = res['phases']
    other = None
    if default_workload and not args.no_secondary:
        # the same steps with the flags of a step's inverses read one step late (FisherMaker.late_inverse_flags): the
        # host then runs ahead of the device; same kernels, same results, errors raised one update late
        other = measure_kfac(w, args, args.steps, 2, 'now' if late else 'late', False, args.phase_steps)
        key = 'late_inverse_flags' if not late else 'default_inverse_flags'
        out[key] = {'ms_per_step': other['ms_per_step'], 'value': other['value'], 'unit': 'steps/s',
                    'note': 'same process, same model; flags of a step\'s inverses read '
                            + ('one step late (not the library\'s default: a factor that is not positive definite '
                               'raises one update late)' if not late else 'in the same call, after its preconditioning is enqueued'),
                    'phases': other.get('phases')}
    if not args.no_cpu_baseline:
        if args.workload == 'linear4096':
            out['cpu_baseline'] = cpu_baseline_linear4096(args)
        elif args.workload == 'resnet18_cifar':
            out['cpu_baseline'] = cpu_baseline_resnet18(args)
        else:
            out['cpu_baseline'] = cpu_baseline(args)
    res = other = None
    if default_workload and not args.no_secondary:
        # the other K-FAC configurations, briefly and without their CPU legs (each has a workload of its own:
        # --workload linear4096 / resnet18_cifar)
        w.clear()
        torch.cuda.empty_cache()
        secondary = {}
        for name, metric in (('linear4096', 'K-FAC steps/s Linear 4096x4096, 8192 rows'),
                             ('resnet18_cifar', 'K-FAC steps/s ResNet-18 (CIFAR stem) bs128 fp32')):
            w2 = build_workload(args, name, dev)
            r2 = measure_kfac(w2, args, 10, 3, False, True, 0)
            entry = {'metric': metric, 'value': r2['value'], 'unit': 'steps/s', 'ms_per_step': r2['ms_per_step'],
                     'steps': 10, 'warmup': 3, 'dtype': w2['dtype'], 'roofline': r2.get('roofline')}
            inv2 = inverse_roofline(w2, args.damping, reps=3)
            if inv2 is not None:
                entry['roofline_inverse'] = {k: inv2[k] for k in ('achieved', 'peak', 'frac', 'standalone_ms', 'flop_per_step', 'matrices')}
            secondary[name] = entry
            w2.clear()
            del r2
            torch.cuda.empty_cache()
        # the Shampoo configuration: ten steps, one of them with a root update (every tenth step has one)
        sh = main_shampoo(args, dev, steps=10, warmup=2, emit=False)
        secondary['shampoo_gpt2'] = {k: sh[k] for k in ('metric', 'value', 'unit', 'ms_per_step', 'steps', 'warmup', 'dtype',
                                                        'roofline') if k in sh}
        del sh
        torch.cuda.empty_cache()
        out['secondary'] = secondary
    print(json.dumps(out))


def cpu_baseline_resnet18(args):
    """One K-FAC step of the CPU oracle on ResNet-18 (CIFAR stem), batch 128, fp32."""
    import torch
    import bench_models
    from oracle import cpu_ref
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    model = bench_models.resnet18_cifar()
    x, t = torch.randn(128, 3, 32, 32), torch.randint(0, 10, (128,))
    orc = cpu_ref.KfacOracle(model, data_size=128, damping=args.damping, fisher_type=args.fisher,
                             factor_dtype=torch.float32)
    t0 = time.time()
    orc.forward_and_backward(x, t)
    dt = time.time() - t0
    return {'value': 1.0 / dt, 'unit': 'steps/s', 'cores': cores, 'kind': 'port',
            'sample': f'one K-FAC step of the CPU oracle (PyTorch CPU ops, {cores} threads) on the full workload took {dt:.1f} s'}


def main_shampoo(args, dev, steps=None, warmup=None, emit=True):
    """The Shampoo workload; emit=False: a brief run for the `secondary` object of the default line (no CPU leg),
    returned instead of printed."""
    import torch
    import torch.nn.functional as F
    import bench_models
    from asdl_amd import PreconditioningConfig, ShampooGradientMaker
    torch.backends.cudnn.benchmark = False
    model = bench_models.gpt2_small().to(dev)       # token embedding and output head frozen (50257-wide)
    bs = 8
    x = torch.randint(0, 50257, (bs, 1024)).to(dev)
    t = torch.randint(0, 50257, (bs * 1024,)).to(dev)
    config = PreconditioningConfig(damping=1e-6, curvature_upd_interval=1, preconditioner_upd_interval=10)
    gm = ShampooGradientMaker(model, config)
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
    opt = torch.optim.SGD([p for p in model.parameters() if p.requires_grad], lr=1e-4)

    def fwd(inp):
        with torch.autocast('cuda', dtype=torch.bfloat16):
            return model(inp).float()

    def token_loss(y, target):
        return F.cross_entropy(y.reshape(-1, y.shape[-1]), target)

    def step():
        opt.zero_grad(set_to_none=True)
        dummy_y = gm.setup_model_call(fwd, x)
        gm.setup_loss_call(token_loss, dummy_y, t)
        gm.forward_and_backward()
        opt.step()

    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    for i in range(warmup):
        step()
    del root_records[:]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    out = {
        'metric': 'Shampoo steps/s GPT-2-small decoder, 8x1024 tokens',
        'value': steps / elapsed, 'unit': 'steps/s', 'n_gpus': 1, 'steps': steps, 'warmup': warmup,
        'ms_per_step': elapsed / steps * 1e3, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': 'Shampoo step (L/R statistics and preconditioning of the 49 trainable weight matrices '
                               'every step, inverse 4th roots every 10 steps, epsilon 1e-6) on a 12-layer '
                               'GPT-2-small-shaped decoder (d 768, 12 heads, MLP 3072; token embedding and output '
                               'head frozen), 8 x 1024 uniform random tokens, bf16 autocast forward/backward, '
                               'fp32 statistics and roots', 'batch': bs}}
    if root_records:
        from asdl_amd import _lib

        def plane_format(n, exp):
            return int(_lib.load().ak_inv_root_plane_format(n, exp, config.damping))

        secs = sum(a.elapsed_time(b) for a, b, _ in root_records) * 1e-3
        flops, executed_flops, iters = 0.0, 0.0, []
        for _, _, stats in root_records:
            for (n, exp), st in stats.items():
                it = st[:, 2].double().cpu()
                products = 2 + (exp - 1).bit_length()      # root T, T^p by squaring (p a power of two), T^p M
                f = float(it.sum()) * products * 2.0 * n ** 3
                flops += f
                # matrices of 512 and up are known to be symmetric: only the T (T + 1) / 2 tiles of 192 on and above
                # the diagonal of the matrix padded to a multiple of 192 are computed (the planes kernel), as 3 fp16
                # piece products per fp32-grade product where the ridge bounds the root (2 planes), else 6 bf16 ones
                if n >= 512:
                    tiles = -(-n // 192)
                    pieces = 3.0 if plane_format(n, exp) == 2 else 6.0
                    executed_flops += float(it.sum()) * products * pieces * 2.0 * (tiles * (tiles + 1) / 2) * 192.0 ** 2 * (192.0 * tiles)
                else:
                    executed_flops += 6.0 * f
                iters.append(int(it.max()))
        algorithmic = flops / secs / 1e12
        # `achieved` is the ALGORITHMIC rate: 2 n^3 per fp32-grade product of the reference's iteration, against the
        # bf16 matrix peak the products are executed on; the executed piece products are the labelled extra
        out['roofline'] = {'bound': 'mfma', 'achieved': algorithmic, 'peak': BF16_MFMA_PEAK_TFLOPS, 'unit': 'TFLOP/s',
                           'frac': algorithmic / BF16_MFMA_PEAK_TFLOPS, 'traffic': None,
                           'kernel': 'products of the coupled Newton iteration (plane_gemm_kernel: matrices kept as two '
                                     'fp16 planes where the ridge bounds the root, else three bf16 planes; gemm_x3_kernel / '
                                     'gemm_f32_kernel below 512 columns): 2 n^3 FLOP per product of the reference; '
                                     'executed_bf16_tflops counts the 16-bit MFMA work actually run (3 fp16 or 6 bf16 piece '
                                     'products per fp32 product, the tiles on and above the diagonal only)',
                           'executed_bf16_tflops': executed_flops / secs / 1e12,
                           'executed_bf16_frac': executed_flops / secs / 1e12 / BF16_MFMA_PEAK_TFLOPS,
                           'fp32_peak_frac': algorithmic / FP32_MFMA_PEAK_TFLOPS,
                           'root_updates_timed': len(root_records),
                           'ms_per_root_update': secs / len(root_records) * 1e3,
                           'newton_iterations_max': max(iters)}
    if not emit:
        return out
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline_shampoo(args)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
