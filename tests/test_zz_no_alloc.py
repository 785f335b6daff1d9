"""ak_kron_precond_static (the entry point that brings its own scratch memory and allocates nothing) against
ak_kron_precond (caller's workspace), both through the C ABI: same kernels, so the results have to be bit-identical.
Two calls in a row on one GPU, the second with a smaller input, share the library's scratch array; the oracle's
B_inv G A_inv is checked as well (1e-3, the bar for preconditioned gradients)."""
import ctypes

import pytest
import torch

from oracle import cpu_ref as R

pytestmark = pytest.mark.gpu


def _case(dB, dA, seed, bias):
    g = torch.Generator().manual_seed(seed)

    def spd(n):
        q = torch.randn(n, n + 8, generator=g)
        return (q @ q.T / (n + 8) + 0.5 * torch.eye(n)).contiguous()

    return spd(dB), spd(dA), torch.randn(dB, dA, generator=g), (torch.randn(dB, generator=g) if bias else None)


def _relerr(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm())


def test_static_entry_point_rejects_sizes_beyond_its_array():
    from asdl_amd import _lib
    lib = _lib.load()
    cap = lib.ak_kron_precond_static_max_floats()
    assert cap == 4 << 20
    x = torch.zeros(16, device='cuda')
    p = ctypes.c_void_p(x.data_ptr())
    rc = lib.ak_kron_precond_static(p, p, p, 2048, 2048, None, 1.0, None)       # 2048*2048 + 2048 > 4 Mi
    assert rc == -5 and b'maximum' in lib.ak_error_string(rc)
    assert lib.ak_kron_precond_static(p, p, p, 0, 4, None, 1.0, None) == -1


def test_static_entry_point_matches_workspace_entry_point_twice_in_a_row():
    from asdl_amd import kernels as K
    # the second case is smaller, so it finds the first one's intermediate in the shared array
    for call, (dB, dA, seed, bias) in enumerate([(512, 4608, 1, True), (200, 136, 2, True), (64, 64, 3, False)]):
        Binv, Ainv, G, b = _case(dB, dA, seed, bias)
        print(f'kron_precond_static dB={dB} dA={dA} bias={bias}', flush=True)
        dev = [t.cuda() if t is not None else None for t in (Binv, Ainv, G, b)]
        G_ws, b_ws = dev[2].clone(), (dev[3].clone() if bias else None)
        G_st, b_st = dev[2].clone(), (dev[3].clone() if bias else None)
        K.kron_precond(dev[0], dev[1], G_ws, b_ws, grad_scale=0.5)
        torch.cuda.synchronize()
        # the property the entry point exists for: the device's free memory and torch's allocator counters do not
        # move across the call.  Checked from the second call on: the first call on a device looks up the array's
        # address (hipGetSymbolAddress), which may load the library's code object; callers that capture a stream make
        # that first call before the capture.
        free_before, _ = torch.cuda.mem_get_info()
        stats_before = torch.cuda.memory_stats()
        K.kron_precond_static(dev[0], dev[1], G_st, b_st, grad_scale=0.5)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        stats_after = torch.cuda.memory_stats()
        if call > 0:
            assert free_after == free_before, (free_before, free_after)
            for key in ('allocation.all.allocated', 'segment.all.allocated', 'reserved_bytes.all.current'):
                assert stats_after[key] == stats_before[key], key
        assert torch.equal(G_st, G_ws)
        ref = R.kron_mvp(Ainv.double(), Binv.double(), (0.5 * G).double(), (0.5 * b).double() if bias else None)
        ref_w, ref_b = ref if bias else (ref, None)
        assert _relerr(G_st, ref_w) < 1e-3
        if bias:
            assert torch.equal(b_st, b_ws)
            assert _relerr(b_st, ref_b) < 1e-3
