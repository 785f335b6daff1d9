"""torch.Tensor front ends of the C ABI (include/asdl_amd.h).

Every function takes tensors that live on a ROCm device, passes raw device pointers and the
calling thread's current HIP stream to libasdl_amd.so, and returns without synchronising.
There is no CPU path: a CPU tensor raises.
"""
import contextlib
import ctypes
import struct
import threading

import torch

from . import _lib

AK_F32, AK_BF16, AK_F32_AS_BF16 = 0, 1, 2

_ws_lock = threading.Lock()
_workspaces = {}
_ptr_cache = {}
_timing_sink = None      # when set to a list, factor launches append (name, flops, start event, end event)


_event_pool = []         # pre-created timing events: creating one costs more host time than recording it


class _RawEvent:
    """Timing event of the HIP runtime recorded on an explicit stream handle (torch.cuda.Event only sees torch's
    current stream, not the side stream a FactorStream launches on)."""

    def __init__(self):
        handle = ctypes.c_void_p()
        _lib.check(_lib.load().ak_event_create(ctypes.byref(handle), 1), 'ak_event_create')
        self.handle = handle

    def record(self):
        _lib.check(_lib.load().ak_event_record(self.handle, _stream()), 'ak_event_record')

    def elapsed_time(self, other):
        ms = ctypes.c_float()
        _lib.check(_lib.load().ak_event_elapsed_ms(self.handle, other.handle, ctypes.byref(ms)), 'ak_event_elapsed_ms')
        return ms.value

    def __del__(self):
        try:
            _lib.load().ak_event_destroy(self.handle)
        except Exception:
            pass


def set_timing_sink(sink, n_events=0):
    """Benchmark instrumentation: with a list as sink every factor-statistics launch is bracketed by
    two events on the launching stream and recorded with its algorithmic FLOP count M*d*(d+1).
    ``n_events`` events are created up front so that the timed region only records them."""
    global _timing_sink
    _timing_sink = sink
    del _event_pool[:]
    if sink is not None:
        _event_pool.extend(_RawEvent() for _ in range(n_events))


def enable_timing(flag):
    """Switches the recording into the sink set by set_timing_sink() on or off (to sample a subset of steps)."""
    global _timing_on
    _timing_on = bool(flag)


_timing_on = True


def _timing_event():
    return _event_pool.pop() if _event_pool else _RawEvent()


MFMA_PEAK_FLOPS = {torch.bfloat16: 2.5e15, torch.float32: 157.3e12}      # dense matrix-core peaks of an MI355X
HBM_PEAK_BYTES = 8.0e12


def factor_floor_seconds(flops, dtype, in_bytes, d, beta):
    """Roofline floor of one factor statistic: its FLOP at the matrix-core peak of the operand type, or its
    algorithmic bytes (the operand once, the factor written once, and read once when it is accumulated into) at the
    memory peak, whichever takes longer."""
    out_bytes = d * d * 4 * (2 if beta != 0.0 else 1)
    return max(flops / MFMA_PEAK_FLOPS.get(dtype, 157.3e12), (in_bytes + out_bytes) / HBM_PEAK_BYTES)


class _Timed:
    def __init__(self, name, flops, calls=1, floor=0.0):
        # calls: factors covered by the timed region; floor: the sum of their roofline floors in seconds
        self.name, self.flops, self.calls, self.floor = name, flops, calls, floor

    def __enter__(self):
        self.timed = _timing_sink is not None and _timing_on
        if self.timed:
            self.start = _timing_event()
            self.start.record()
        return self

    def __exit__(self, *exc):
        if self.timed:
            end = _timing_event()
            end.record()
            _timing_sink.append((self.name, self.flops, self.start, end, self.calls, self.floor))
        return False


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError('asdl_amd kernels run on a ROCm device only; got a tensor on '
                               f'{t.device}. There is no CPU fallback.')


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


_override = threading.local()      # .handle: stream the calling thread's kernel launches go to instead of the current one


def _stream_handle(device=None):
    """The calling thread's current HIP stream on ``device`` as an integer handle (or the side stream a
    FactorStream has switched this thread to)."""
    forced = getattr(_override, 'handle', None)
    if forced is not None:
        return forced
    if _raw_stream is not None:
        idx = device.index if device is not None and device.index is not None else torch.cuda.current_device()
        return _raw_stream(idx)
    return torch.cuda.current_stream(device).cuda_stream


def _stream(device=None):
    return ctypes.c_void_p(_stream_handle(device))


_size_cache = {}


def _ws_need(fn_name, *args):
    """Cached ak_*_ws_bytes query (pure functions of the shape)."""
    key = (fn_name, args)
    need = _size_cache.get(key)
    if need is None:
        need = getattr(_lib.load(), fn_name)(*args)
        if len(_size_cache) > 8192:
            _size_cache.clear()
        _size_cache[key] = need
    return need


def _dtype_code(t):
    if t.dtype == torch.float32:
        return AK_F32
    if t.dtype == torch.bfloat16:
        return AK_BF16
    raise TypeError(f'unsupported dtype {t.dtype}: the kernels take float32 or bfloat16 inputs')


def workspace(nbytes, device):
    """A cached scratch buffer per (device, stream); grows geometrically, never shrinks.
    Kernels on one stream run in order, so consecutive calls may share it."""
    if nbytes <= 0:
        return None, 0
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream_handle(device))
    with _ws_lock:
        buf = _workspaces.get(key)
        if buf is None or buf.numel() < nbytes:
            size = max(nbytes, 1 << 20)
            if buf is not None:
                size = max(size, int(buf.numel() * 1.5))
            buf = torch.empty(size, dtype=torch.uint8, device=device)
            _workspaces[key] = buf
    return buf, buf.numel()


def _ws_args(nbytes, device):
    buf, size = workspace(nbytes, device)
    if buf is None:
        return ctypes.c_void_p(0), 0, None
    return ctypes.c_void_p(buf.data_ptr()), size, buf


def device_ptr_array(tensors):
    """int64 device tensor holding the data pointers of ``tensors`` (cached by pointer tuple)."""
    ptrs = tuple(t.data_ptr() for t in tensors)
    dev = tensors[0].device
    key = (dev.index, ptrs)
    arr = _ptr_cache.get(key)
    if arr is None:
        if len(_ptr_cache) > 4096:
            _ptr_cache.clear()
        # staged through pinned memory and copied asynchronously on the launch stream, like device_table(): a
        # pageable copy would block the caller behind everything that stream has queued
        host = torch.tensor(ptrs, dtype=torch.int64).pin_memory()
        with _on_launch_stream():
            arr = host.to(dev, non_blocking=True)
        _ptr_cache[key] = arr
    return arr


_int_cache = {}


def device_ints(values, device, dtype=torch.int64):
    """Device tensor holding a small tuple of Python ints (nested tuples give a 2-D tensor).  Cached: the
    same index sets recur every step, and building them anew costs a synchronous host-to-device copy that
    stalls the host behind everything already enqueued."""
    dev = torch.device(device)
    key = (dev.index, dtype, values)
    t = _int_cache.get(key)
    if t is None:
        if len(_int_cache) > 8192:
            _int_cache.clear()
        t = torch.tensor(values, dtype=dtype).to(dev)
        _int_cache[key] = t
    return t


def device_table(rows, device):
    """device_ints for tables that hold addresses, which may change from call to call: a miss is staged through
    pinned memory and copied asynchronously on the launch stream, so the host never waits for the device."""
    dev = torch.device(device)
    key = (dev.index, 'table', rows)
    t = _int_cache.get(key)
    if t is None:
        if len(_int_cache) > 8192:
            _int_cache.clear()
        host = torch.tensor(rows, dtype=torch.int64).pin_memory()
        with _on_launch_stream():
            t = host.to(dev, non_blocking=True)
        _int_cache[key] = t
    return t


class main_stream_launches:
    """Context: inside FactorStream.run(), kernel launches of this thread go to its current stream again."""

    def __enter__(self):
        self._saved = (getattr(_override, 'handle', None), getattr(_override, 'stream', None))
        _override.handle = _override.stream = None

    def __exit__(self, *exc):
        _override.handle, _override.stream = self._saved
        return False


def _on_launch_stream():
    """Context for the few framework ops (copies to a contiguous layout, casts) that feed a kernel: they have to run
    on the stream the kernel is launched on."""
    st = getattr(_override, 'stream', None)
    return torch.cuda.stream(st) if st is not None else contextlib.nullcontext()


def _contiguous(x):
    if x.is_contiguous():
        return x
    with _on_launch_stream():
        return x.contiguous()


FACTOR_STREAM_BATCH = 16      # hook calls per ordering of the factor stream after the main stream


class FactorStream:
    """A side stream (default priority) for the statistics kernels of the hooks.  ``run(fn, *tensors)`` orders the
    side stream after everything the calling thread's current stream holds, runs ``fn`` with this thread's kernel
    launches redirected to the side stream, and keeps ``tensors`` alive until ``join()`` makes the current stream
    wait for the side stream (the caching allocator would otherwise hand a freed gradient buffer to the next kernel
    of the main stream while the side stream still reads it)."""

    def __init__(self, device):
        self.device = torch.device(device)
        self.stream = torch.cuda.Stream(device=self.device)
        self.handle = self.stream.cuda_stream
        lib = _lib.load()
        self._events = []
        for _ in range(8):
            ev = ctypes.c_void_p()
            _lib.check(lib.ak_event_create(ctypes.byref(ev), 0), 'ak_event_create')
            self._events.append(ev)
        self._next = 0
        self._keep = []
        self._pending = []
        self._flushing = False

    def _event(self):
        ev = self._events[self._next]
        self._next = (self._next + 1) % len(self._events)
        return ev

    def run(self, fn, *tensors, backward=False):
        """Queues ``fn``; every ``batch`` queued calls are run together behind one ordering of the side stream
        after the caller's stream (that ordering costs tens of microseconds of host time, more than a hook has to
        spare).  ``fn`` must not depend on anything but its arguments; its results are only valid after join()."""
        self._pending.append(fn)
        self._keep.append(tensors)
        if len(self._pending) >= FACTOR_STREAM_BATCH:
            self._flush()

    def _flush(self):
        if self._flushing or not self._pending:
            return
        self._flushing = True
        saved = (getattr(_override, 'handle', None), getattr(_override, 'stream', None))
        try:
            main = _stream_handle(self.device)
            _lib.check(_lib.load().ak_stream_order(ctypes.c_void_p(main), ctypes.c_void_p(self.handle), self._event()),
                       'ak_stream_order')
            fns, self._pending = self._pending, []
            _override.handle, _override.stream = self.handle, self.stream
            for fn in fns:
                fn()
        finally:
            _override.handle, _override.stream = saved
            self._flushing = False

    def join(self):
        """Runs what is still queued and makes the caller's stream wait for the side stream.  Called from inside a
        queued call (a hook that starts the early inverses), it covers the calls that have run so far."""
        self._flush()
        saved = (getattr(_override, 'handle', None), getattr(_override, 'stream', None))
        _override.handle = _override.stream = None
        try:
            main = _stream_handle(self.device)
        finally:
            _override.handle, _override.stream = saved
        _lib.check(_lib.load().ak_stream_order(ctypes.c_void_p(self.handle), ctypes.c_void_p(main), self._event()),
                   'ak_stream_order')
        keep, self._keep = self._keep, []
        return keep          # the caller may drop these once work enqueued after the join has been issued

    def __del__(self):
        try:
            for ev in self._events:
                _lib.load().ak_event_destroy(ev)
        except Exception:
            pass


# ------------------------------------------------------------------------------ factors of many layers in one launch
_group = threading.local()         # .active: the FactorGroup that collects this thread's factor calls, or None
GROUP_SPEC_INTS = 16
_group_eligible = {}


def _float_bits(v):
    return struct.unpack('<I', struct.pack('<f', float(v)))[0]


class FactorGroup:
    """Collects the factor statistics that syrk_tn() / conv_syrk() are asked for while it is the calling thread's
    active group and launches them together in flush(): the factors of a whole forward or backward pass are a few
    tiles each, and one at a time each of them pays a launch ramp, a tail, its split-K partial tiles and a reduction
    launch.  The operands and results are kept alive until flush().  A call whose result tensor is already in the
    group flushes first (a second contribution to the same factor has to come after the first)."""
    SLOTS = 4

    def __init__(self, device):
        self.device = torch.device(device)
        self._rows, self._keep, self._outs, self._flops = [], [], set(), 0
        self._versions, self._floor = [], 0.0
        self._sizes = {}
        self.plain_only = False      # take X^T X calls only: unfolded inputs are launched at once
        self._slots = [dict(host=None, dev=None, event=None) for _ in range(self.SLOTS)]
        self._next = 0

    def __len__(self):
        return len(self._rows)

    @staticmethod
    def eligible(row, align_key):
        """Can the single-factor call described by ``row`` join a group?  (A pure function of the shape, the
        alignment of the operand and the kind of call: cached.)"""
        key = (tuple(row[:1] + row[3:4] + row[5:]), align_key)
        ok = _group_eligible.get(key)
        if ok is None:
            arr = (ctypes.c_int64 * GROUP_SPEC_INTS)(*row)
            ok = bool(_lib.load().ak_syrk_group_eligible(ctypes.cast(arr, ctypes.c_void_p)))
            if len(_group_eligible) > 4096:
                _group_eligible.clear()
            _group_eligible[key] = ok
        return ok

    def add(self, row, flops, floor, *tensors):
        if row[2] in self._outs:
            self.flush()
        self._rows.append(row)
        self._outs.add(row[2])
        self._keep.append(tensors)
        self._versions.append(tensors[0]._version)       # the operand must still hold these values at flush()
        self._flops += flops
        self._floor += floor

    def discard(self):
        """Forgets what has been collected without launching it (a pass that ended in an exception)."""
        self._rows, self._keep, self._outs, self._flops = [], [], set(), 0
        self._versions, self._floor = [], 0.0

    def flush(self):
        """Launches what has been collected on the calling thread's launch stream."""
        if not self._rows:
            return
        rows, self._rows, keep, self._keep = self._rows, [], self._keep, []
        flops, self._flops, self._outs = self._flops, 0, set()
        versions, self._versions = self._versions, []
        floor, self._floor = self._floor, 0.0
        for tensors, version in zip(keep, versions):
            # the reference forms a factor inside the hook; here the operand is read later, by address
            if tensors[0]._version != version:
                raise RuntimeError('an activation or output gradient was modified in place between the hook that '
                                   'recorded its factor statistic and the grouped launch of the pass; set '
                                   'asdl_amd.fisher.GROUPED_FACTORS = False for this model')
        if len(rows) == 1:
            # nothing to share a launch with: the single-factor entry points, whose plan search knows more tile
            # sizes and a two-stage reduction
            saved = getattr(_group, 'active', None)
            _group.active = None
            try:
                x, out = keep[0][0], keep[0][1]
                alpha = struct.unpack('<f', struct.pack('<I', rows[0][4] & 0xffffffff))[0]
                beta = struct.unpack('<f', struct.pack('<I', rows[0][4] >> 32))[0]
                if rows[0][0] == 0:
                    if x.ndim != 2:      # kept as the hook saw it: the [M, d] rows the row describes
                        x = torch.as_strided(x, (rows[0][5], rows[0][6]), (rows[0][7], 1))
                    syrk_tn(x, out=out, alpha=alpha, beta=beta)
                else:
                    r = rows[0]
                    conv_syrk(x, (r[9], r[10]), (r[11], r[12]), (r[13], r[14]), out=out, alpha=alpha, beta=beta)
            finally:
                _group.active = saved
            return
        lib = _lib.load()
        import numpy as np
        specs = np.ascontiguousarray(np.array(rows, dtype=np.int64))
        specs_ptr = ctypes.c_void_p(specs.ctypes.data)
        sig = tuple((r[0], r[3]) + tuple(r[5:]) + (r[1] & 15,) for r in rows)
        sizes = self._sizes.get(sig)
        if sizes is None:
            tb, wb = ctypes.c_size_t(0), ctypes.c_size_t(0)
            _lib.check(lib.ak_syrk_group_sizes(specs_ptr, len(rows), ctypes.byref(tb), ctypes.byref(wb)),
                       'ak_syrk_group_sizes')
            if len(self._sizes) > 64:
                self._sizes.clear()
            sizes = self._sizes[sig] = (tb.value, wb.value)
        table_bytes, ws_bytes = sizes
        slot = self._slots[self._next]
        self._next = (self._next + 1) % self.SLOTS
        if slot['event'] is not None:
            slot['event'].synchronize()          # the copy that last read this slot's host memory has long run
        if slot['host'] is None or slot['host'].numel() < table_bytes:
            slot['host'] = torch.empty(max(table_bytes, 1 << 16), dtype=torch.uint8).pin_memory()
            slot['dev'] = torch.empty(slot['host'].numel(), dtype=torch.uint8, device=self.device)
            slot['event'] = torch.cuda.Event()
        ws, ws_size, ws_keep = _ws_args(ws_bytes, self.device)
        with _Timed('syrk_group', flops, calls=len(rows), floor=floor):
            rc = lib.ak_syrk_group_launch(specs_ptr, len(rows), ctypes.c_void_p(slot['host'].data_ptr()),
                                          ctypes.c_void_p(slot['dev'].data_ptr()), slot['host'].numel(),
                                          ws, ws_size, _stream(self.device))
        _lib.check(rc, 'ak_syrk_group_launch')
        st = getattr(_override, 'stream', None)
        slot['event'].record(st if st is not None else torch.cuda.current_stream(self.device))
        del keep


class DeferredFactors:
    """Stands where a FactorStream stands (OperationContext.factor_stream): the hook operations run at once, on the
    caller's stream, but the factor statistics they ask for are collected in a FactorGroup; join() launches what is
    left of them.  ``every`` = (forward, backward): the group is also launched after that many hook calls of the
    pass (0: only at join(); -1: the hooks of that pass launch their factors one by one, as without a group; -2: only
    the plain X^T X factors of that pass are collected, until join(), the unfolded ones are launched at once)."""

    def __init__(self, device, every=(0, 0)):
        self.device = torch.device(device)
        self.group = FactorGroup(self.device)
        self.every = tuple(every)
        self._count = 0

    def run(self, fn, *tensors, backward=False):
        every = self.every[1 if backward else 0]
        if every == -1:
            self.group.flush()
            fn()
            return
        saved = getattr(_group, 'active', None), self.group.plain_only
        _group.active = self.group
        self.group.plain_only = every == -2
        try:
            fn()
        finally:
            _group.active, self.group.plain_only = saved
        self._count += 1
        if every > 0 and self._count >= every:
            self._count = 0
            self.group.flush()

    def join(self):
        self._count = 0
        self.group.flush()
        return []

    def discard(self):
        self._count = 0
        self.group.discard()


def _group_take(row, flops, floor, align_key, *tensors):
    """True when the calling thread has an active group and it has taken the call."""
    grp = getattr(_group, 'active', None)
    if grp is None or (grp.plain_only and row[0] != 0) or not FactorGroup.eligible(row, align_key):
        return False
    grp.add(row, flops, floor, *tensors)
    _group.last = (row, flops, floor)
    return True


class GroupedCall:
    """A factor call that the active FactorGroup took, remembered by its caller (one per hooked module and factor):
    operand geometry, the group's row, the result buffer, FLOP count and floor.  On the next pass the caller's hook
    sees a tensor of the same shape, strides, type and alignment, for which syrk_tn() / conv_syrk() would derive the
    very same row; again() appends it to the group without going through them."""
    __slots__ = ('shape', 'stride', 'dtype', 'device', 'align', 'row', 'out', 'flops', 'floor', 'timed', 'extra')

    @staticmethod
    def begin():
        """Call before the factor call that is to be remembered."""
        _group.last = None
        _group.last_direct = None

    @classmethod
    def remember(cls, x, out, extra=None):
        """After the factor call on the hook's tensor ``x`` with result ``out``: the record, or None when the call
        was launched at once, or read a converted or rearranged copy of ``x`` (whose address the next pass cannot
        know)."""
        last = getattr(_group, 'last', None)
        _group.last = None
        if last is None:
            return None
        row, flops, floor = last
        if row[1] != x.data_ptr() or row[2] != out.data_ptr():
            return None
        rec = cls()
        rec.shape, rec.stride, rec.dtype, rec.device = x.shape, x.stride(), x.dtype, x.device
        rec.align = row[1] & 15
        rec.row, rec.out, rec.flops, rec.floor = list(row), out, flops, floor
        rec.timed = _timing_sink is not None
        rec.extra = extra
        return rec

    def again(self, x, extra=None):
        """Appends the remembered call, on ``x``, to the active group.  False (nothing done) when ``x`` or the state
        of the calling thread differs from what the record was made under."""
        grp = getattr(_group, 'active', None)
        if grp is None or (grp.plain_only and self.row[0] != 0):
            return False
        if x.dtype is not self.dtype or x.shape != self.shape or x.stride() != self.stride or x.device != self.device \
                or extra != self.extra or (_timing_sink is not None) != self.timed:
            return False
        ptr = x.data_ptr()
        if ptr & 15 != self.align:
            return False
        row = list(self.row)
        row[1] = ptr
        grp.add(row, self.flops, self.floor, x, self.out)
        return True


class DirectCall:
    """A factor call that was launched at once (no group took it), remembered by its caller like a GroupedCall: the
    library function and its argument list, the workspace it needs, FLOP count and floor.  again() launches it on a
    tensor of the same shape, strides, type and alignment without going through conv_syrk() again."""
    __slots__ = ('shape', 'stride', 'dtype', 'device', 'align', 'name', 'fn', 'args', 'need', 'out', 'flops', 'floor',
                 'timed', 'extra')

    @staticmethod
    def note(name, fn, args, need, x, out, flops, floor):
        """Called by the factor function right before its launch: args[0] is x's address, args[-3:] are the
        workspace, its size and the stream."""
        _group.last_direct = (name, fn, args, need, x.data_ptr(), out, flops, floor)

    @classmethod
    def remember(cls, x, out, extra=None):
        last = getattr(_group, 'last_direct', None)
        _group.last_direct = None
        if last is None:
            return None
        name, fn, args, need, ptr, out_used, flops, floor = last
        if ptr != x.data_ptr() or out_used is not out:
            return None          # the call read a converted or rearranged copy of x
        rec = cls()
        rec.shape, rec.stride, rec.dtype, rec.device = x.shape, x.stride(), x.dtype, x.device
        rec.align = ptr & 15
        rec.name, rec.fn, rec.args, rec.need, rec.out, rec.flops, rec.floor = name, fn, list(args), need, out, flops, floor
        rec.timed = _timing_sink is not None
        rec.extra = extra
        return rec

    def again(self, x, extra=None):
        grp = getattr(_group, 'active', None)
        if grp is not None and not grp.plain_only:
            return False         # a group that takes every kind of row is open: the factor function decides
        if x.dtype is not self.dtype or x.shape != self.shape or x.stride() != self.stride or x.device != self.device \
                or extra != self.extra or (_timing_sink is not None) != self.timed:
            return False
        ptr = x.data_ptr()
        if ptr & 15 != self.align:
            return False
        args = self.args
        args[0] = ctypes.c_void_p(ptr)
        args[-3], args[-2], keep = _ws_args(self.need, x.device)
        args[-1] = _stream()
        with _Timed(self.name, self.flops, floor=self.floor):
            rc = self.fn(*args)
        _lib.check(rc, self.name)
        return True


# ------------------------------------------------------------------------------ factors
def _as_bf16(x):
    with _on_launch_stream():
        return x.to(torch.bfloat16)


def syrk_tn(x, out=None, alpha=1.0, beta=0.0, round_bf16=False):
    """out <- beta*out + alpha * x^T x for x = [M, d] (rows may be strided, columns contiguous).  round_bf16: an
    fp32 x is rounded to bf16 first (what a matmul does to it inside a bf16 autocast region)."""
    _require_gpu(x, out)
    if x.ndim != 2:
        raise ValueError(f'x.ndim has to be 2. Got {x.ndim}.')
    if round_bf16 and x.dtype == torch.float32:
        x = _as_bf16(x)
    if x.stride(1) != 1 and x.shape[1] > 1:
        x = _contiguous(x)
    M, d = x.shape
    ldx = x.stride(0) if M > 1 else max(d, x.stride(0))
    if ldx < d:
        x = _contiguous(x)
        ldx = d
    if out is None:
        out = torch.empty(d, d, dtype=torch.float32, device=x.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (d, d) or out.stride(1) != 1:
        raise ValueError('out has to be a float32 [d, d] tensor with contiguous rows')
    flops = M * d * (d + 1)
    floor = factor_floor_seconds(flops, x.dtype, M * d * x.element_size(), d, beta) if _timing_sink is not None else 0.0
    if x.dtype == torch.bfloat16 and getattr(_group, 'active', None) is not None:
        row = [0, x.data_ptr(), out.data_ptr(), out.stride(0), _float_bits(alpha) | (_float_bits(beta) << 32),
               M, d, ldx] + [0] * 8
        if _group_take(row, flops, floor, x.data_ptr() & 15, x, out):
            return out
    lib = _lib.load()
    need = _ws_need('ak_syrk_tn_ws_bytes', M, d)
    ws, ws_bytes, keep = _ws_args(need, x.device)
    with _Timed('syrk_tn', flops, floor=floor):
        rc = lib.ak_syrk_tn(ctypes.c_void_p(x.data_ptr()), _dtype_code(x), M, d, ldx, alpha, beta,
                            ctypes.c_void_p(out.data_ptr()), out.stride(0), ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_syrk_tn')
    return out


AK_ERR_UNSUPPORTED = -3
NCHW_VIA_CHANNELS_LAST = True     # bf16 NCHW activations: transpose once, then the channels-last kernels


def _is_channels_last(x):
    return (x.ndim == 4 and x.shape[1] > 1 and x.is_contiguous(memory_format=torch.channels_last)
            and not x.is_contiguous())


def conv_syrk(x, kernel_size, stride, padding, out=None, alpha=1.0, beta=0.0, round_bf16=False):
    """out <- beta*out + alpha * sum_{n,pos} patch patch^T for x = [N, C, H, W], patches ordered (c, ky, kx);
    no division by the output size (fold it into alpha).  A channels-last bf16 x is read in place
    (rows gathered from the NHWC memory); anything else goes through the NCHW kernel.  round_bf16: an fp32 x is
    rounded to bf16 (what a matmul does to it inside a bf16 autocast region): while it is read, by the window
    kernel of the few-channel layers, else by a cast beforehand."""
    _require_gpu(x, out)
    if x.ndim != 4:
        raise ValueError(f'x.ndim has to be 4. Got {x.ndim}.')
    N, C, H, W = x.shape
    kh, kw = kernel_size
    sh, sw = stride
    ph, pw = padding
    d = C * kh * kw
    if out is None:
        out = torch.empty(d, d, dtype=torch.float32, device=x.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (d, d) or out.stride(1) != 1:
        raise ValueError('out has to be a float32 [d, d] tensor with contiguous rows')
    lib = _lib.load()
    h_out, w_out = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    few_channels = d <= 160 and kh * kw > 1 and x.dtype in (torch.bfloat16, torch.float32)   # the LDS-window kernel
    code = None
    if round_bf16 and x.dtype == torch.float32:
        if few_channels:
            code = AK_F32_AS_BF16
        else:
            x = _as_bf16(x)
    if code is None:
        code = _dtype_code(x)
    flops = N * h_out * w_out * d * (d + 1)
    floor = 0.0
    if _timing_sink is not None:
        # a rounded fp32 input is read as fp32 and multiplied as bf16
        floor = factor_floor_seconds(flops, torch.float32 if code == AK_F32 else torch.bfloat16,
                                     N * C * H * W * x.element_size(), d, beta)
    if NCHW_VIA_CHANNELS_LAST and x.dtype == torch.bfloat16 and C % 8 == 0 and not few_channels \
            and x.is_contiguous() and C > 1 and N * C * H * W >= (1 << 16):
        # one transposing copy (memory-bound, a few microseconds) buys the direct-to-LDS kernels, which read rows of
        # 8 channels as 16-byte chunks; the NCHW kernel stages every operand through registers
        with _on_launch_stream():
            x = x.contiguous(memory_format=torch.channels_last)
    if _is_channels_last(x) and ((x.dtype == torch.bfloat16 and C % 8 == 0) or few_channels):
        if (kh, kw, sh, sw, ph, pw) == (1, 1, 1, 1, 0, 0):
            return syrk_tn(x.permute(0, 2, 3, 1).reshape(N * H * W, C), out=out, alpha=alpha, beta=beta)
        if x.dtype == torch.bfloat16 and getattr(_group, 'active', None) is not None:
            row = [1, x.data_ptr(), out.data_ptr(), out.stride(0), _float_bits(alpha) | (_float_bits(beta) << 32),
                   N, C, H, W, kh, kw, sh, sw, ph, pw, 0]
            if _group_take(row, flops, floor, x.data_ptr() & 15, x, out):
                return out
        need = _ws_need('ak_conv_syrk_nhwc_ws_bytes', N, C, H, W, kh, kw, sh, sw, ph, pw)
        ws, ws_bytes, keep = _ws_args(need, x.device)
        args = [ctypes.c_void_p(x.data_ptr()), code, N, C, H, W, kh, kw, sh, sw, ph, pw, alpha, beta,
                ctypes.c_void_p(out.data_ptr()), out.stride(0), ws, ws_bytes, _stream()]
        with _Timed('conv_syrk', flops, floor=floor):
            rc = lib.ak_conv_syrk_nhwc(*args)
        if rc != AK_ERR_UNSUPPORTED:
            _lib.check(rc, 'ak_conv_syrk_nhwc')
            DirectCall.note('conv_syrk', lib.ak_conv_syrk_nhwc, args, need, x, out, flops, floor)
            return out
    x = _contiguous(x)
    need = _ws_need('ak_conv_syrk_ws_bytes', N, C, H, W, kh, kw, sh, sw, ph, pw)
    ws, ws_bytes, keep = _ws_args(need, x.device)
    with _Timed('conv_syrk', flops, floor=floor):
        rc = lib.ak_conv_syrk(ctypes.c_void_p(x.data_ptr()), code, N, C, H, W, kh, kw, sh, sw, ph, pw,
                              alpha, beta, ctypes.c_void_p(out.data_ptr()), out.stride(0), ws, ws_bytes, _stream())
    if rc == AK_ERR_UNSUPPORTED and code == AK_F32_AS_BF16:     # a window too large for the LDS: cast, then the bf16 kernels
        return conv_syrk(_as_bf16(x), kernel_size, stride, padding, out=out, alpha=alpha, beta=beta)
    _lib.check(rc, 'ak_conv_syrk')
    return out


def syrk_nt(x, out=None, alpha=1.0, beta=0.0):
    """out <- beta*out + alpha * sum_n x_n x_n^T for x = [d, K] or [N, d, K] (K contiguous)."""
    if x.ndim == 2:
        x = x.unsqueeze(0)
    if x.ndim != 3:
        raise ValueError(f'x.ndim has to be 2 or 3. Got {x.ndim}.')
    return conv_syrk(x.unsqueeze(2), (1, 1), (1, 1), (0, 0), out=out, alpha=alpha, beta=beta)


# ------------------------------------------------------------------------------ unit-wise blocks
def unit_wise_stats(y, g, weight, bias, out=None, alpha=1.0, beta=0.0):
    """out[f] <- beta*out[f] + alpha * sum_n [[gw^2, gw*gb], [gw*gb, gb^2]] with the per-sample gradients
    gw = sum_s (y - bias)/weight * g, gb = sum_s g.  y, g: [n, f], [n, f, *spatial] (any strides, e.g. channels
    last) or [rows, *normalized_shape] for LayerNorm (pass them flattened to [rows, f])."""
    _require_gpu(y, g, weight, bias, out)
    if y.shape != g.shape:
        raise ValueError(f'shapes differ: {tuple(y.shape)} vs {tuple(g.shape)}')
    N, F = y.shape[0], y.shape[1]

    def strides(t):
        if t.ndim == 2:
            return t.stride(0), t.stride(1), 1, 1
        sp = t.shape[2:]
        S = 1
        for d in sp:
            S *= d
        # the positions have to be addressable with one stride
        st = t.stride(-1)
        expect = st
        for d, s_ in zip(reversed(sp), reversed(t.stride()[2:])):
            if d != 1 and s_ != expect:
                return None
            expect *= d
        return t.stride(0), t.stride(1), st, S

    sy, sg = strides(y), strides(g)
    if sy is None:
        y = _contiguous(y)
        sy = strides(y)
    if sg is None:
        g = _contiguous(g)
        sg = strides(g)
    S = sy[3]
    with _on_launch_stream():
        weight = weight.detach().float().contiguous()
        bias = bias.detach().float().contiguous()
    if out is None:
        out = torch.empty(F, 2, 2, dtype=torch.float32, device=y.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (F, 2, 2) or not out.is_contiguous():
        raise ValueError('out has to be a contiguous float32 [f, 2, 2] tensor')
    need = _ws_need('ak_unit_wise_ws_bytes', N, F, S)
    ws, ws_bytes, keep = _ws_args(need, y.device)
    rc = _lib.load().ak_unit_wise_stats(ctypes.c_void_p(y.data_ptr()), _dtype_code(y), sy[0], sy[1], sy[2],
                                        ctypes.c_void_p(g.data_ptr()), _dtype_code(g), sg[0], sg[1], sg[2],
                                        ctypes.c_void_p(weight.data_ptr()), ctypes.c_void_p(bias.data_ptr()), N, F, S,
                                        alpha, beta, ctypes.c_void_p(out.data_ptr()), ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_unit_wise_stats')
    return out


def unit_wise_inv(blocks, damping, out=None):
    """(out, flags): out[f] = (blocks[f] + damping I)^-1; flags is a device int32[2] = (any non-zero entry,
    1-based index of the first singular block or 0x7fffffff)."""
    _require_gpu(blocks, out)
    if blocks.dtype != torch.float32 or blocks.ndim != 3 or blocks.shape[1:] != (2, 2) or not blocks.is_contiguous():
        raise ValueError('blocks has to be a contiguous float32 [f, 2, 2] tensor')
    if out is None:
        out = torch.empty_like(blocks)
    flags = torch.empty(2, dtype=torch.int32, device=blocks.device)
    rc = _lib.load().ak_unit_wise_inv(ctypes.c_void_p(blocks.data_ptr()), blocks.shape[0], float(damping),
                                      ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(flags.data_ptr()), _stream())
    _lib.check(rc, 'ak_unit_wise_inv')
    return out, flags


def unit_wise_inv_grouped(blocks_list, dampings, outs=None):
    """unit_wise_inv for many modules in two launches.  Returns (list of inverses, flags [count, 2] int32 on the
    device, one (non-zero, first singular block) pair per module).  outs: optional list of output tensors or None."""
    _require_gpu(*blocks_list)
    count = len(blocks_list)
    dev = blocks_list[0].device
    invs = []
    for i, blocks in enumerate(blocks_list):
        if blocks.dtype != torch.float32 or blocks.ndim != 3 or blocks.shape[1:] != (2, 2) or not blocks.is_contiguous():
            raise ValueError('blocks has to be a contiguous float32 [f, 2, 2] tensor')
        out = outs[i] if outs is not None else None
        invs.append(out if out is not None else torch.empty_like(blocks))
    with _on_launch_stream():
        flags = device_ints(((0, 0x7fffffff),) * count, dev, dtype=torch.int32).clone()
    rows, first = [], 0
    for i, (blocks, inv) in enumerate(zip(blocks_list, invs)):
        F = blocks.shape[0]
        rows.append((blocks.data_ptr(), inv.data_ptr(), flags.data_ptr() + 8 * i, F, first, _float_bits(dampings[i])))
        first += (F + 255) // 256
    table = device_table(tuple(rows), dev)
    rc = _lib.load().ak_unit_wise_inv_grouped(ctypes.c_void_p(table.data_ptr()), count, first, _stream())
    _lib.check(rc, 'ak_unit_wise_inv_grouped')
    return invs, flags


def unit_wise_mvp(mat, vec_weight, vec_bias, scale=1.0):
    """[vec_weight, vec_bias][f] <- mat[f] @ (scale * [vec_weight, vec_bias][f]) in place."""
    _require_gpu(mat, vec_weight, vec_bias)
    F = mat.shape[0]
    for v in (vec_weight, vec_bias):
        if v.dtype != torch.float32 or v.numel() != F or not v.is_contiguous():
            raise ValueError('vectors have to be contiguous float32 tensors with one entry per block')
    rc = _lib.load().ak_unit_wise_mvp(ctypes.c_void_p(mat.data_ptr()), F, ctypes.c_void_p(vec_weight.data_ptr()),
                                      ctypes.c_void_p(vec_bias.data_ptr()), float(scale), _stream())
    _lib.check(rc, 'ak_unit_wise_mvp')
    return vec_weight, vec_bias


# ------------------------------------------------------------------------------ saved factors
def tril_pack(mat):
    """1-D lower triangle (row direction) of a float32 square matrix with contiguous rows."""
    _require_gpu(mat)
    if mat.ndim != 2:
        raise ValueError(f'mat.ndim has to be 2. Got {mat.ndim}.')
    if mat.shape[0] != mat.shape[1] or mat.dtype != torch.float32 or mat.stride(1) != 1:
        raise ValueError('mat has to be a square float32 matrix with contiguous rows')
    d = mat.shape[0]
    out = torch.empty(d * (d + 1) // 2, dtype=torch.float32, device=mat.device)
    rc = _lib.load().ak_tril_pack(ctypes.c_void_p(mat.data_ptr()), d, mat.stride(0), ctypes.c_void_p(out.data_ptr()),
                                  _stream())
    _lib.check(rc, 'ak_tril_pack')
    return out


def tril_unpack(tril, n_cols):
    """Full symmetric [n_cols, n_cols] matrix from its packed lower triangle."""
    _require_gpu(tril)
    if tril.ndim != 1:
        raise ValueError(f'tril.ndim has to be 1. Got {tril.ndim}.')
    if tril.dtype != torch.float32 or tril.numel() != n_cols * (n_cols + 1) // 2:
        raise ValueError('tril has to hold n_cols*(n_cols+1)/2 float32 values')
    tril = tril.contiguous()
    out = torch.empty(n_cols, n_cols, dtype=torch.float32, device=tril.device)
    rc = _lib.load().ak_tril_unpack(ctypes.c_void_p(tril.data_ptr()), n_cols, ctypes.c_void_p(out.data_ptr()), n_cols,
                                    _stream())
    _lib.check(rc, 'ak_tril_unpack')
    return out


# ------------------------------------------------------------------------------ damping / inverse
def identity_where_zero(outs, nonzero, flag_index):
    """outs[m] <- identity where nonzero.view(-1)[flag_index[m]] == 0 (an all-zero factor, whose inverse was
    skipped); the other matrices are left alone.  No host synchronisation."""
    if not outs:
        return
    _require_gpu(*outs, nonzero)
    dev = outs[0].device
    for o in outs:
        if o.dtype != torch.float32 or o.ndim != 2 or o.shape[0] != o.shape[1] or not o.is_contiguous():
            raise ValueError('outs have to be contiguous square float32 matrices')
    ptrs = device_ptr_array(outs)
    dims = device_ints(tuple(int(o.shape[0]) for o in outs), dev)
    index = device_ints(tuple(int(i) for i in flag_index), dev)
    rc = _lib.load().ak_identity_where_zero(ctypes.c_void_p(ptrs.data_ptr()), ctypes.c_void_p(dims.data_ptr()),
                                            ctypes.c_void_p(nonzero.data_ptr()), ctypes.c_void_p(index.data_ptr()),
                                            len(outs), _stream())
    _lib.check(rc, 'ak_identity_where_zero')


def kron_damping(A_list, B_list, damping, eps=1e-7, eig_scale=None):
    """Returns (lam [batch, 2] float32, nonzero [batch, 2] int32), both on the device.  A factor is a square
    [d, d] matrix or, for the low-rank (swift) factors, an [n, d] matrix with n < d rows; ``eig_scale``: optional
    per-pair (sA, sB) multiplied into the eigenvalue means before the pi split."""
    _require_gpu(*A_list, *B_list)
    dev = A_list[0].device
    batch = len(A_list)
    swift = eig_scale is not None
    for t in list(A_list) + list(B_list):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.ndim != 2:
            raise ValueError('factors have to be contiguous float32 matrices')
        if t.shape[0] > t.shape[1]:
            raise ValueError('a factor has to be square or have fewer rows than columns')
        swift = swift or t.shape[0] != t.shape[1]
    lam = torch.empty(batch, 2, dtype=torch.float32, device=dev)
    nonzero = torch.empty(batch, 2, dtype=torch.int32, device=dev)
    pa, pb = device_ptr_array(A_list), device_ptr_array(B_list)
    if not swift:
        dims = device_ints(tuple((a.shape[0], b.shape[0]) for a, b in zip(A_list, B_list)), dev)
        rc = _lib.load().ak_kron_damping(ctypes.c_void_p(pa.data_ptr()), ctypes.c_void_p(pb.data_ptr()),
                                         ctypes.c_void_p(dims.data_ptr()), batch, damping, eps,
                                         ctypes.c_void_p(lam.data_ptr()), ctypes.c_void_p(nonzero.data_ptr()), _stream())
        _lib.check(rc, 'ak_kron_damping')
        return lam, nonzero

    def rows(t):
        return 0 if t.shape[0] == t.shape[1] else t.shape[0]
    dims = device_ints(tuple((rows(a), a.shape[1], rows(b), b.shape[1]) for a, b in zip(A_list, B_list)), dev)
    scale = None
    if eig_scale is not None:
        scale = device_ints(tuple((float(sa), float(sb)) for sa, sb in eig_scale), dev, dtype=torch.float32)
    rc = _lib.load().ak_kron_damping_swift(ctypes.c_void_p(pa.data_ptr()), ctypes.c_void_p(pb.data_ptr()),
                                           ctypes.c_void_p(dims.data_ptr()),
                                           ctypes.c_void_p(scale.data_ptr()) if scale is not None else ctypes.c_void_p(0),
                                           batch, damping, eps, ctypes.c_void_p(lam.data_ptr()),
                                           ctypes.c_void_p(nonzero.data_ptr()), _stream())
    _lib.check(rc, 'ak_kron_damping_swift')
    return lam, nonzero


# ------------------------------------------------------------------------------ low-rank (swift) factors
def conv_patch_sum(x, kernel_size=(1, 1), stride=(1, 1), padding=(0, 0), out=None, alpha=1.0, beta=0.0):
    """out[n, (c, ky, kx)] <- beta*out + alpha * sum over output positions of the patch element, for x = [N, C, H, W]
    in any memory format ([N, C, L] and [N, C] are taken as W = L, H = 1 and H = W = 1): the [n, d] matrix the swift
    factors keep.  kernel 1x1: the sum over positions; [N, C]: a scaled float32 copy."""
    _require_gpu(x, out)
    if x.ndim == 2:
        x = x[:, :, None, None]
    elif x.ndim == 3:
        x = x[:, :, None, :]
    if x.ndim != 4:
        raise ValueError(f'x.ndim has to be 2, 3 or 4. Got {x.ndim}.')
    if x.dtype not in (torch.float32, torch.bfloat16):
        with _on_launch_stream():
            x = x.float()
    N, C, H, W = x.shape
    kh, kw = kernel_size
    sh, sw = stride
    ph, pw = padding
    d = C * kh * kw
    if out is None:
        out = torch.empty(N, d, dtype=torch.float32, device=x.device)
        beta = 0.0
    if out.dtype != torch.float32 or out.shape != (N, d) or out.stride(1) != 1:
        raise ValueError('out has to be a float32 [N, C*kh*kw] tensor with contiguous rows')
    sn, sc, sy, sx = x.stride()
    rc = _lib.load().ak_conv_patch_sum(ctypes.c_void_p(x.data_ptr()), _dtype_code(x), sn, sc, sy, sx, N, C, H, W,
                                       kh, kw, sh, sw, ph, pw, alpha, beta, ctypes.c_void_p(out.data_ptr()),
                                       out.stride(0), _stream())
    _lib.check(rc, 'ak_conv_patch_sum')
    return out


def smw_inv(x, lam, out=None, info=None):
    """(x^T x / n + lam I)^-1 for an [n, d] float32 matrix with n < d through the n x n Gram matrix
    (Sherman-Morrison-Woodbury): (I - x^T (x x^T + n lam I)^-1 x) / lam.  ``lam``: one-element float32 device tensor.
    Returns (inverse [d, d], info) with the Cholesky info word of the Gram matrix."""
    _require_gpu(x, lam, out)
    if x.ndim != 2 or x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError('x has to be a contiguous float32 matrix')
    n, d = x.shape
    lam = lam.reshape(1)
    if out is None:
        out = torch.empty(d, d, dtype=torch.float32, device=x.device)
    if out.dtype != torch.float32 or out.shape != (d, d) or out.stride(1) != 1:
        raise ValueError('out has to be a float32 [d, d] tensor with contiguous rows')
    if info is None:
        info = torch.empty(1, dtype=torch.int32, device=x.device)
    ws, ws_bytes, keep = _ws_args(_ws_need('ak_smw_inv_ws_bytes', n, d), x.device)
    rc = _lib.load().ak_smw_inv(ctypes.c_void_p(x.data_ptr()), n, d, ctypes.c_void_p(lam.data_ptr()),
                                ctypes.c_void_p(out.data_ptr()), out.stride(0), ctypes.c_void_p(info.data_ptr()),
                                ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_smw_inv')
    z = out
    return z, info


def chol_inv_batched(mats, outs, lam, lam_stride=1, active=None, active_stride=1, info=None):
    """outs[b] <- (mats[b] + lam[b*lam_stride] I)^-1 for same-size matrices; returns the device
    ``info`` tensor (int32 [batch], 0 = ok, k > 0 = leading minor k not positive definite)."""
    _require_gpu(*mats, *outs, lam, active)
    d = mats[0].shape[0]
    batch = len(mats)
    dev = mats[0].device
    for t in list(mats) + list(outs):
        if t.dtype != torch.float32 or t.shape != (d, d) or not t.is_contiguous():
            raise ValueError('matrices have to be contiguous float32 [d, d] tensors of one size')
    if info is None:
        info = torch.empty(batch, dtype=torch.int32, device=dev)
    lib = _lib.load()
    need = _ws_need('ak_chol_inv_ws_bytes', d, batch)
    ws, ws_bytes, keep = _ws_args(need, dev)
    pa, po = device_ptr_array(mats), device_ptr_array(outs)
    rc = lib.ak_chol_inv_batched(ctypes.c_void_p(pa.data_ptr()), ctypes.c_void_p(po.data_ptr()), d, batch,
                                 ctypes.c_void_p(lam.data_ptr()), lam_stride,
                                 ctypes.c_void_p(active.data_ptr()) if active is not None else ctypes.c_void_p(0),
                                 active_stride, ctypes.c_void_p(info.data_ptr()), ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_chol_inv_batched')
    return info


_chol_plans = {}


class CholGroupPlan:
    """Launch plan of ak_chol_inv_grouped for one tuple of matrix sizes: built on the host by the library, kept in
    pinned memory (the library reads the launch sequence from it on every call) with a copy on the device (the
    kernels read their descriptors from it)."""

    def __init__(self, dims, device):
        lib = _lib.load()
        self.dims = tuple(int(d) for d in dims)
        arr = (ctypes.c_int64 * len(self.dims))(*self.dims)
        nbytes = lib.ak_chol_group_plan_bytes(arr, len(self.dims))
        if nbytes == 0:
            raise ValueError(f'no grouped Cholesky plan for sizes {self.dims}')
        self.ws_bytes = lib.ak_chol_group_ws_bytes(arr, len(self.dims))
        self.host = torch.empty(nbytes, dtype=torch.uint8).pin_memory()
        _lib.check(lib.ak_chol_group_plan(arr, len(self.dims), ctypes.c_void_p(self.host.data_ptr()), nbytes),
                   'ak_chol_group_plan')
        self.launches = lib.ak_chol_group_plan_launches(ctypes.c_void_p(self.host.data_ptr()))
        with _on_launch_stream():
            self.dev = self.host.to(device, non_blocking=True)


def chol_group_plan(dims, device):
    dev = torch.device(device)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), tuple(int(d) for d in dims))
    plan = _chol_plans.get(key)
    if plan is None:
        if len(_chol_plans) > 64:
            _chol_plans.clear()
        plan = _chol_plans[key] = CholGroupPlan(dims, dev)
    return plan


def chol_inv_grouped(mats, outs, lam, lam_stride=1, active=None, active_stride=1, info=None):
    """outs[m] <- (mats[m] + lam[m*lam_stride] I)^-1 for square matrices of any mix of sizes, all in one call:
    the steps of all matrices are merged into one sequence of grouped launches (csrc/chol_group.hip).  Returns the
    device ``info`` tensor (int32 [len(mats)], 0 = ok, k > 0 = leading minor k not positive definite)."""
    _require_gpu(*mats, *outs, lam, active)
    dev = mats[0].device
    for a, o in zip(mats, outs):
        if a.dtype != torch.float32 or a.ndim != 2 or a.shape[0] != a.shape[1] or not a.is_contiguous():
            raise ValueError('matrices have to be contiguous square float32 tensors')
        if o.dtype != torch.float32 or o.shape != a.shape or not o.is_contiguous():
            raise ValueError('every output has to be a contiguous float32 tensor of its matrix\'s shape')
    if len(outs) != len(mats):
        raise ValueError('one output per matrix')
    if info is None:
        info = torch.empty(len(mats), dtype=torch.int32, device=dev)
    plan = chol_group_plan([m.shape[0] for m in mats], dev)
    ws, ws_bytes, keep = _ws_args(plan.ws_bytes, dev)
    pa, po = device_ptr_array(mats), device_ptr_array(outs)
    rc = _lib.load().ak_chol_inv_grouped(
        ctypes.c_void_p(plan.host.data_ptr()), ctypes.c_void_p(plan.dev.data_ptr()), ctypes.c_void_p(pa.data_ptr()),
        ctypes.c_void_p(po.data_ptr()), ctypes.c_void_p(lam.data_ptr()), lam_stride,
        ctypes.c_void_p(active.data_ptr()) if active is not None else ctypes.c_void_p(0), active_stride,
        ctypes.c_void_p(info.data_ptr()), ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_chol_inv_grouped')
    return info


def cholesky_inv(X, damping=1e-7):
    """(X + damping I)^-1; raises torch.linalg.LinAlgError when X + damping I is not positive
    definite (reads the device info word, i.e. synchronises)."""
    _require_gpu(X)
    lam = torch.full((1,), float(damping), dtype=torch.float32, device=X.device)
    out = torch.empty_like(X)
    info = chol_inv_batched([X.contiguous()], [out], lam)
    k = int(info.item())
    if k != 0:
        raise torch.linalg.LinAlgError(
            f'cholesky_inv: the leading minor of order {k} is not positive-definite')
    return out


# ------------------------------------------------------------------------------ products
def gemm(A, B, out=None, transA=False, transB=False, alpha=1.0, beta=0.0, pieces=0):
    """out <- alpha * op(A) op(B) + beta * out for float32 matrices with contiguous rows.  pieces = 3 / 2:
    on the bf16 matrix cores after an exact 3- / 2-way split of the operands (0: fp32 MFMA)."""
    _require_gpu(A, B, out)
    for t in (A, B):
        if t.dtype != torch.float32 or t.ndim != 2 or t.stride(1) != 1:
            raise ValueError('gemm operands have to be float32 matrices with contiguous rows')
    M = A.shape[1] if transA else A.shape[0]
    K = A.shape[0] if transA else A.shape[1]
    K2 = B.shape[1] if transB else B.shape[0]
    N = B.shape[0] if transB else B.shape[1]
    if K != K2:
        raise ValueError(f'inner dimensions differ: {K} vs {K2}')
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=A.device)
        beta = 0.0
    if out.data_ptr() in (A.data_ptr(), B.data_ptr()):
        raise ValueError('gemm cannot run in place')
    rc = _lib.load().ak_gemm_f32_split(int(pieces), int(transA), int(transB), M, N, K, alpha,
                                       ctypes.c_void_p(A.data_ptr()), max(A.stride(0), A.shape[1]),
                                       ctypes.c_void_p(B.data_ptr()), max(B.stride(0), B.shape[1]), beta,
                                       ctypes.c_void_p(out.data_ptr()), max(out.stride(0), N), 1, 0, 0, 0, _stream())
    _lib.check(rc, 'ak_gemm_f32_split')
    return out


def kron_precond(B_inv, A_inv, grad_w, grad_b=None, grad_scale=1.0):
    """grad_w <- grad_scale * B_inv @ view(grad_w, [dB, dA]) @ A_inv, grad_b <- grad_scale * B_inv @ grad_b,
    both in place."""
    _require_gpu(B_inv, A_inv, grad_w, grad_b)
    dB, dA = B_inv.shape[0], A_inv.shape[0]
    if grad_w.numel() != dB * dA or not grad_w.is_contiguous() or grad_w.dtype != torch.float32:
        raise ValueError('grad_w has to be a contiguous float32 tensor with dB * dA elements')
    if grad_b is not None and (grad_b.numel() != dB or not grad_b.is_contiguous() or grad_b.dtype != torch.float32):
        raise ValueError('grad_b has to be a contiguous float32 vector with dB elements')
    lib = _lib.load()
    ws, ws_bytes, keep = _ws_args(_ws_need('ak_kron_precond_ws_bytes', dB, dA), grad_w.device)
    rc = lib.ak_kron_precond(ctypes.c_void_p(B_inv.data_ptr()), ctypes.c_void_p(A_inv.data_ptr()),
                             ctypes.c_void_p(grad_w.data_ptr()), dB, dA,
                             ctypes.c_void_p(grad_b.data_ptr()) if grad_b is not None else ctypes.c_void_p(0),
                             grad_scale, ws, ws_bytes, _stream())
    _lib.check(rc, 'ak_kron_precond')
    return grad_w, grad_b


def kron_precond_static(B_inv, A_inv, grad_w, grad_b=None, grad_scale=1.0):
    """kron_precond through the entry point that brings its own scratch memory (a fixed array inside the library's
    device image, no workspace, no allocation): for callers that must not allocate.  Raises KernelError when
    dB * dA + dB exceeds the array; calls that overlap on one GPU race."""
    _require_gpu(B_inv, A_inv, grad_w, grad_b)
    dB, dA = B_inv.shape[0], A_inv.shape[0]
    if grad_w.numel() != dB * dA or not grad_w.is_contiguous() or grad_w.dtype != torch.float32:
        raise ValueError('grad_w has to be a contiguous float32 tensor with dB * dA elements')
    if grad_b is not None and (grad_b.numel() != dB or not grad_b.is_contiguous() or grad_b.dtype != torch.float32):
        raise ValueError('grad_b has to be a contiguous float32 vector with dB elements')
    rc = _lib.load().ak_kron_precond_static(ctypes.c_void_p(B_inv.data_ptr()), ctypes.c_void_p(A_inv.data_ptr()),
                                            ctypes.c_void_p(grad_w.data_ptr()), dB, dA,
                                            ctypes.c_void_p(grad_b.data_ptr()) if grad_b is not None
                                            else ctypes.c_void_p(0), grad_scale, _stream())
    _lib.check(rc, 'ak_kron_precond_static')
    return grad_w, grad_b


def _float_bits(value):
    return struct.unpack('<I', struct.pack('<f', float(value)))[0]


def _grouped_operand_ok(ptr, ld, contiguous_extent):
    return ptr % 16 == 0 and ld % 4 == 0 and contiguous_extent % 4 == 0


def _gemm_grouped_table(specs, device):
    """(device table, rows, tiles) for ak_gemm_f32_grouped.  specs: tuples (a_ptr, lda, b_ptr, ldb, c_ptr, ldc, M, N, K,
    transA, transB, alpha[, beta[, symmetric[, absmax_a, absmax_b, absmax_c]]]) of device addresses of float32 matrices
    with contiguous rows; C <- alpha * op(A) op(B) + beta * C; symmetric: only the lower tiles are computed, and
    mirrored; absmax_*: addresses of float words (0: none) holding the operands' largest magnitudes (pieces = 22) and
    receiving the result's."""
    rows, first = [], 0
    for spec in sorted(specs, key=lambda sp: -sp[8]):
        a, lda, b, ldb, c, ldc, M, N, K, tA, tB, alpha = spec[:12]
        beta = spec[12] if len(spec) > 12 else 0.0
        symmetric = bool(spec[13]) if len(spec) > 13 else False
        max_a, max_b, max_c = spec[14:17] if len(spec) > 16 else (0, 0, 0)
        if M <= 0 or N <= 0 or K <= 0:
            continue
        if symmetric and M != N:
            raise ValueError('a symmetric product is square')
        if not (_grouped_operand_ok(a, lda, M if tA else K) and _grouped_operand_ok(b, ldb, K if tB else N)):
            raise ValueError('grouped products need 16-byte aligned operands whose leading dimension and '
                             'contiguous extent are multiples of 4')
        if lda < (M if tA else K) or ldb < (K if tB else N) or ldc < N:
            raise ValueError('leading dimension smaller than the row length')
        rows.append((a, b, c, lda, ldb, ldc, M, N, K, int(bool(tA)) | (int(bool(tB)) << 1) | (int(symmetric) << 2),
                     _float_bits(alpha) | (_float_bits(beta) << 32), first, max_a, max_b, max_c, 0))
        first += ((M + 127) // 128) * ((N + 127) // 128)
    if not rows:
        return None, 0, 0
    return device_table(tuple(rows), device), len(rows), first


def _launch_gemm_grouped(table, count, tiles, pieces):
    if count:
        rc = _lib.load().ak_gemm_f32_grouped(int(pieces), ctypes.c_void_p(table.data_ptr()), count, tiles, _stream())
        _lib.check(rc, 'ak_gemm_f32_grouped')


def gemm_grouped_raw(specs, device, pieces=3):
    """One launch for many products C_i <- alpha_i * op(A_i) op(B_i) (specs as for _gemm_grouped_table)."""
    _launch_gemm_grouped(*_gemm_grouped_table(specs, device), pieces)


def absmax_grouped(vectors, device):
    """vectors: (address, elements, element stride, address of the float word that receives max |x|); one launch.  The
    words have to be zero before (the maxima are folded in with an atomic maximum)."""
    block = _lib.load().ak_absmax_block()
    rows, blocks = [], 0
    for ptr, n, stride, out in vectors:
        rows.append((ptr, n, stride, out, blocks))
        blocks += (n + block - 1) // block
    if rows:
        table = device_table(tuple(rows), device)
        _lib.check(_lib.load().ak_absmax_grouped(ctypes.c_void_p(table.data_ptr()), len(rows), blocks, _stream()),
                   'ak_absmax_grouped')


def gemm_grouped(problems, pieces=3):
    """problems: (A, B, C, transA, transB, alpha) with 2-D float32 tensors whose rows are contiguous;
    C <- alpha * op(A) @ op(B) for all of them in one launch."""
    if not problems:
        return
    specs = []
    for A, B, C, tA, tB, alpha in problems:
        _require_gpu(A, B, C)
        for t in (A, B, C):
            if t.dtype != torch.float32 or t.ndim != 2 or (t.stride(1) != 1 and t.shape[1] > 1):
                raise ValueError('operands have to be float32 matrices with contiguous rows')
        M, K = (A.shape[1], A.shape[0]) if tA else A.shape
        K2, N = (B.shape[1], B.shape[0]) if tB else B.shape
        if K != K2 or tuple(C.shape) != (M, N):
            raise ValueError('shapes do not match')
        specs.append((A.data_ptr(), A.stride(0), B.data_ptr(), B.stride(0), C.data_ptr(), C.stride(0), M, N, K,
                      tA, tB, alpha))
    gemm_grouped_raw(specs, problems[0][0].device, pieces)


def _channels_last_weight(g):
    """A 4-D gradient stored as [Cout][kh][kw][Cin] (and not at the same time as [Cout][Cin][kh][kw])."""
    return g.ndim == 4 and not g.is_contiguous() and g.is_contiguous(memory_format=torch.channels_last)


def kron_precond_groupable(B_inv, A_inv, grad_w, grad_b=None):
    """Whether kron_precond_grouped takes this module (else: kron_precond)."""
    small = [B_inv, A_inv] + ([grad_b] if grad_b is not None else [])
    if any(t is None or not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() for t in small):
        return False
    if grad_w is None or not grad_w.is_cuda or grad_w.dtype != torch.float32:
        return False
    if B_inv.ndim != 2 or A_inv.ndim != 2 or B_inv.shape[0] != B_inv.shape[1] or A_inv.shape[0] != A_inv.shape[1]:
        return False
    dB, dA = B_inv.shape[0], A_inv.shape[0]
    if grad_w.numel() != dB * dA or (grad_b is not None and grad_b.numel() != dB):
        return False
    if not grad_w.is_contiguous():
        if not _channels_last_weight(grad_w) or grad_w.shape[0] != dB or dA > _lib.load().ak_weight_layout_max_row():
            return False
    return dB % 4 == 0 and dA % 4 == 0 and all(t.data_ptr() % 16 == 0 for t in (B_inv, A_inv, grad_w))


HALF_PIECE_PRECONDITION = True     # grouped preconditioning on two fp16 pieces per element (3 matrix instructions per
                                   # product instead of the 6 of the bf16 three-piece split); False: three bf16 pieces


class KronPrecondPlan:
    """kron_precond for many modules in a handful of launches: all B_inv @ G, then all (.) @ A_inv, then all
    B_inv @ bias; channels-last convolution gradients are gathered into the contiguous layout before and
    scattered back after, one launch each.  items: (B_inv, A_inv, grad_w, grad_b or None), each accepted by
    kron_precond_groupable.  Construction does all host work (address tables, their upload); launch() only
    enqueues the kernels, so a caller can prepare while the device is still busy producing the operands.  The
    plan refers to the tensors by address: launch() is valid for as long as ``items`` are alive and unmoved."""

    def __init__(self, items, grad_scale=1.0, unit_items=()):
        """unit_items: (inv [F, 2, 2], grad_w [F], grad_b [F]) of the unit-wise modules (contiguous float32):
        one more launch applies all their 2 x 2 blocks."""
        self.items = list(items)
        self.unit_items = list(unit_items)
        self.grad_scale = float(grad_scale)
        self._units = None
        if self.unit_items:
            rows, blocks = [], 0
            for inv, gw, gb in self.unit_items:
                F = inv.shape[0]
                if any(t.dtype != torch.float32 or not t.is_contiguous() for t in (inv, gw, gb)) or \
                        gw.numel() != F or gb.numel() != F or tuple(inv.shape[1:]) != (2, 2):
                    raise ValueError('unit-wise items are float32 [F, 2, 2] blocks with [F] weight and bias gradients')
                rows.append((inv.data_ptr(), gw.data_ptr(), gb.data_ptr(), F, blocks))
                blocks += (F + 255) // 256
            self._units = (device_table(tuple(rows), self.unit_items[0][0].device), len(rows), blocks)
        if not self.items:
            return
        dev = self.items[0][0].device
        n_w = sum(it[2].numel() for it in self.items)
        n_cl = sum(it[2].numel() for it in self.items if not it[2].is_contiguous())
        n_b = sum(it[0].shape[0] for it in self.items if it[3] is not None)
        self._buf, _ = workspace(4 * (n_w + n_cl + n_b), dev)       # kept alive with the plan
        base = self._buf.data_ptr()
        first, second, layout, layout_rows, off = [], [], [], 0, 0
        for B_inv, A_inv, g, _ in self.items:
            dB, dA = B_inv.shape[0], A_inv.shape[0]
            t = base + 4 * off
            off += dB * dA
            g_ptr = g.data_ptr()
            if not g.is_contiguous():
                g_ptr = base + 4 * off
                off += dB * dA
                layout.append((g.data_ptr(), g_ptr, g.shape[1], g.shape[2] * g.shape[3], layout_rows))
                layout_rows += dB
            first.append((B_inv.data_ptr(), dB, g_ptr, dA, t, dA, dB, dA, dB, 0, 0, 1.0))
            # the inverses are symmetric: reading A_inv as its transpose makes both operands contiguous along k
            second.append((t, dA, A_inv.data_ptr(), dA, g_ptr, dA, dB, dA, dA, 0, 1, self.grad_scale))
        self._layout = (device_table(tuple(layout), dev), len(layout), layout_rows) if layout else None
        self._half = bool(HALF_PIECE_PRECONDITION)
        if self._half:
            # Operand ranges for the fp16 pieces, per module: the largest magnitude of B_inv and of A_inv is their largest
            # diagonal element (symmetric positive definite), that of the gradient is measured by one pass over it, that
            # of the intermediate B_inv G by the first product's own epilogue.
            block = _lib.load().ak_absmax_block()
            self._mx = torch.zeros(len(self.items), 4, dtype=torch.float32, device=dev)
            mx = self._mx.data_ptr()
            rows, blocks = [], 0
            for i, ((B_inv, A_inv, g, _), f1, f2) in enumerate(zip(self.items, first, second)):
                dB, dA = B_inv.shape[0], A_inv.shape[0]
                for ptr, n, stride, slot in ((B_inv.data_ptr(), dB, dB + 1, 0), (f1[2], dB * dA, 1, 1),
                                             (A_inv.data_ptr(), dA, dA + 1, 2)):
                    rows.append((ptr, n, stride, mx + 16 * i + 4 * slot, blocks))
                    blocks += (n + block - 1) // block
                first[i] = f1 + (0.0, False, mx + 16 * i, mx + 16 * i + 4, mx + 16 * i + 12)
                second[i] = f2 + (0.0, False, mx + 16 * i + 12, mx + 16 * i + 8, 0)
            self._absmax = (device_table(tuple(rows), dev), len(rows), blocks)
        self._first = _gemm_grouped_table(first, dev)
        self._second = _gemm_grouped_table(second, dev)
        rows, blocks, self._tmps, self._biases = [], 0, [], []
        flat = self._buf[:4 * (n_w + n_cl + n_b)].view(torch.float32)
        for B_inv, _, _, b in self.items:
            if b is None:
                continue
            dB = B_inv.shape[0]
            rows.append((B_inv.data_ptr(), b.data_ptr(), base + 4 * off, dB, blocks))
            self._tmps.append(flat[off:off + dB])
            self._biases.append(b.view(-1))
            blocks += (dB + 3) // 4
            off += dB
        self._gemv = (device_table(tuple(rows), dev), len(rows), blocks) if rows else None

    def _convert_layout(self, to_contiguous):
        if self._layout is not None:
            table, count, rows = self._layout
            rc = _lib.load().ak_weight_layout_grouped(ctypes.c_void_p(table.data_ptr()), count, rows, to_contiguous,
                                                      _stream())
            _lib.check(rc, 'ak_weight_layout_grouped')

    def launch(self):
        if self._units is not None:
            table, count, blocks = self._units
            rc = _lib.load().ak_unit_wise_mvp_grouped(ctypes.c_void_p(table.data_ptr()), count, blocks, self.grad_scale,
                                                      _stream())
            _lib.check(rc, 'ak_unit_wise_mvp_grouped')
        if not self.items:
            return
        self._convert_layout(1)
        # 22 to 24 mantissa bits: the terms of these sums cancel (entries of the inverses reach 1/damping), and what
        # a shorter split loses relative to the terms shows up magnified in the result
        if self._half:
            with _on_launch_stream():
                self._mx.zero_()
            table, count, blocks = self._absmax
            rc = _lib.load().ak_absmax_grouped(ctypes.c_void_p(table.data_ptr()), count, blocks, _stream())
            _lib.check(rc, 'ak_absmax_grouped')
            _launch_gemm_grouped(*self._first, 22)
            _launch_gemm_grouped(*self._second, 22)
        else:
            _launch_gemm_grouped(*self._first, 3)
            _launch_gemm_grouped(*self._second, 3)
        self._convert_layout(0)
        if self._gemv is not None:
            table, count, blocks = self._gemv
            rc = _lib.load().ak_gemv_f32_grouped(ctypes.c_void_p(table.data_ptr()), count, blocks, self.grad_scale,
                                                 _stream())
            _lib.check(rc, 'ak_gemv_f32_grouped')
            with _on_launch_stream():
                torch._foreach_copy_(self._biases, self._tmps)


def kron_precond_grouped(items, grad_scale=1.0):
    """In place, for all items: grad_w <- grad_scale * B_inv @ grad_w @ A_inv, grad_b <- grad_scale * B_inv @ grad_b."""
    KronPrecondPlan(items, grad_scale).launch()


# ------------------------------------------------------------------------------ Shampoo inverse root
ROOT_POLL_EVERY = 8      # Newton iterations enqueued between two reads of the convergence flags (0: never read them)


def inv_root_newton(S, p, ridge_eps, v0, out=None, max_power_iter=100, power_tol=1e-6, max_iter=100, tol=1e-6,
                    poll_every=None):
    """out[b] <- (S[b] + ridge_eps * lambda_max I)^(-1/p) for S = [batch, n, n] (or [n, n]); S keeps the
    ridge.  v0 = [batch, n] start vectors of the power iteration.  Returns (out, stats) with
    stats = [batch, 4] = (lambda_max, power iterations, newton iterations, final error) on the device.
    ``poll_every`` (default ROOT_POLL_EVERY): the Newton iterations are enqueued that many at a time and the host reads
    the convergence flags in between (one small device-to-host copy), so that nothing is launched for a batch that has
    converged; 0 enqueues all ``max_iter`` iterations without ever waiting (the kernels of converged matrices exit at
    once).  The results are the same either way."""
    _require_gpu(S, v0, out)
    single = S.ndim == 2
    S3 = S.unsqueeze(0) if single else S
    batch, n = S3.shape[0], S3.shape[1]
    if S3.dtype != torch.float32 or S3.shape[2] != n or S3.stride(2) != 1 or S3.stride(1) != n:
        raise ValueError('S has to be float32 [batch, n, n] with dense matrices')
    if n < 2:
        raise ValueError('n has to be >= 2 (the inverse root of a 1 x 1 statistic is defined as the identity)')
    v0 = v0.reshape(batch, n).to(torch.float32).contiguous()
    if out is None:
        out = torch.empty(batch, n, n, dtype=torch.float32, device=S.device)
    out3 = out.unsqueeze(0) if out.ndim == 2 else out
    if out3.dtype != torch.float32 or out3.shape != (batch, n, n) or out3.stride(2) != 1 or out3.stride(1) != n:
        raise ValueError('out has to be float32 [batch, n, n] with dense matrices')
    stats = torch.empty(batch, 4, dtype=torch.float32, device=S.device)
    lib = _lib.load()
    ws, ws_bytes, keep = _ws_args(_ws_need('ak_inv_root_ws_bytes', n, batch), S.device)
    strideS = S3.stride(0) if batch > 1 else n * n
    strideO = out3.stride(0) if batch > 1 else n * n
    poll = ROOT_POLL_EVERY if poll_every is None else int(poll_every)
    args = (ctypes.c_void_p(S3.data_ptr()), n, batch, strideS, int(p), float(ridge_eps), ctypes.c_void_p(v0.data_ptr()),
            int(max_power_iter), float(power_tol), int(max_iter), float(tol), ctypes.c_void_p(out3.data_ptr()), strideO,
            ctypes.c_void_p(stats.data_ptr()), ws, ws_bytes, _stream())
    if poll <= 0 or poll >= max_iter:
        _lib.check(lib.ak_inv_root_newton(*args), 'ak_inv_root_newton')
    else:
        off = lib.ak_inv_root_active_offset(n, batch)
        active = keep[off:off + 4 * batch].view(torch.int32)
        _lib.check(lib.ak_inv_root_newton_part(1, 0, *args), 'ak_inv_root_newton_part')
        done = 0
        while done < max_iter:
            with _on_launch_stream():
                if not bool(active.any().item()):      # waits for what has been enqueued so far
                    break
            chunk = min(poll, max_iter - done)
            _lib.check(lib.ak_inv_root_newton_part(2, chunk, *args), 'ak_inv_root_newton_part')
            done += chunk
        _lib.check(lib.ak_inv_root_newton_part(4, 0, *args), 'ak_inv_root_newton_part')
    return (out3[0] if single and out.ndim == 3 else out), stats
