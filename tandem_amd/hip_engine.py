"""The engine object tandem's own Group expects from a native plug-in, over libtandem_hip.so.

For a tandem maintainer: copy this file to `tandem/hip_engine.py`. It has the surface of the
pybind module the reference builds from tandem/csrc/engine.cpp:103-122 (`Engine(job, rank, size,
slots, slot_bytes, timeout, device)`, `connect`, `close`, the collectives, and a handle with
`wait()`, `done()`, `started`, `finished`), bound with ctypes, so tandem/comm.py only has to
import it where it imports its own native module. tandem_amd.comm.Group does not use this file:
it is the same binding grown into a whole Group.
"""

import ctypes
import os

import torch

LIB_PATH = os.environ.get("TANDEM_HIP_LIB", os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libtandem_hip.so"))
_L = ctypes.CDLL(LIB_PATH)
_VP, _PVP, _I64 = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int64
_PI64, _PD = ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_double)
_L.tdm_last_error.restype = ctypes.c_char_p
_L.tdm_engine_create.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _I64, ctypes.c_double, ctypes.c_int, _PVP]
_L.tdm_all_reduce.argtypes = [_VP, _VP, _I64, ctypes.c_int, ctypes.c_int, _VP, _PVP]
_L.tdm_reduce_scatter.argtypes = [_VP, _VP, _I64, ctypes.c_int, _PI64, ctypes.c_int, ctypes.c_int, _VP, _PVP]
_L.tdm_all_gather.argtypes = [_VP, _VP, _I64, ctypes.c_int, _PI64, ctypes.c_int, _VP, _PVP]
_L.tdm_broadcast.argtypes = [_VP, _VP, _I64, ctypes.c_int, ctypes.c_int, _VP, _PVP]
_L.tdm_sendrecv.argtypes = [_VP, _VP, _I64, ctypes.c_int, _VP, _I64, ctypes.c_int, ctypes.c_int, _VP, _PVP]
_L.tdm_barrier.argtypes = [_VP, _PVP]
_L.tdm_work_wait.argtypes = [_VP, _VP]
_L.tdm_work_times.argtypes = [_VP, _PD, _PD]
for _name in ("tdm_engine_connect", "tdm_engine_close", "tdm_engine_destroy", "tdm_work_done", "tdm_work_free"):
    getattr(_L, _name).argtypes = [_VP]

cuda = True  # what tandem/comm.py reads from the native module to know it can take GPU tensors
DTYPE = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.bfloat16: 3, torch.int64: 4, torch.int32: 5,
         torch.int16: 7, torch.int8: 8, torch.uint8: 9}
BYTES = 6  # tensors that are only copied (all_gather, broadcast, send/recv) may have any dtype: they travel as bytes
ERRORS = {1: ValueError, 2: RuntimeError, 3: TimeoutError}  # as tandem/csrc/engine.cpp:54-55 translates its exceptions


def _check(status):
    if status:
        raise ERRORS.get(status, RuntimeError)(_L.tdm_last_error().decode(errors="replace"))


def _stream(device):
    return _VP(torch.cuda.current_stream(device).cuda_stream)


def _flat(t):
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("the hip engine needs contiguous tensors in GPU memory")  # tandem/csrc/collectives.cpp:42-47
    return t.view(-1)


def _reduced(t):
    try:
        return DTYPE[t.dtype], t.numel()
    except KeyError:
        raise ValueError(f"the hip engine cannot reduce {t.dtype}") from None


def _copied(t, sizes=()):
    """(dtype code, element count, chunk sizes): in elements, or in bytes for a dtype the kernels do not know."""
    code = DTYPE.get(t.dtype)
    if code is not None:
        return code, t.numel(), list(sizes)
    es = t.element_size()
    return BYTES, t.numel() * es, [s * es for s in sizes]


def _sizes(sizes):
    return (_I64 * max(1, len(sizes)))(*sizes), len(sizes)


class Handle:
    """What tandem's _CppWork wraps (tandem/comm.py:84-107): wait() makes the caller's current
    stream wait for the collective, done() polls it, started / finished are its time stamps on
    time.perf_counter's clock. The C ABI has only the tensors' addresses, so the handle keeps
    the tensors alive; one that is dropped before anybody waited for it hands them to its
    engine, which lets go of them once the collective has run (the reference's engine holds
    its tensor until the job has run, tandem/csrc/collectives.cpp:314-324)."""

    def __init__(self, pointer, device, keep, engine=None):
        self._p, self._device, self._keep, self._engine, self._waited = pointer, device, keep, engine, False

    def wait(self):
        self._waited = True  # from here on the caller's stream is ordered behind the collective
        _check(_L.tdm_work_wait(self._p, _stream(self._device)))

    def done(self):
        return bool(_L.tdm_work_done(self._p))

    def _times(self):
        a, b = ctypes.c_double(), ctypes.c_double()
        _check(_L.tdm_work_times(self._p, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    started = property(lambda self: self._times()[0])
    finished = property(lambda self: self._times()[1])

    def __del__(self):
        p, self._p = getattr(self, "_p", None), None
        if not p:
            return
        try:
            e = getattr(self, "_engine", None)
            if e is not None and e._e and self._keep and not self._waited and not _L.tdm_work_done(p):
                e._orphans.append((p, self._keep))  # not run yet and nobody waited: the tensors must outlive it
                return
            _L.tdm_work_free(p)
        except Exception:  # the interpreter is going down and has taken the library first
            pass


class Engine:
    """Same constructor and methods as the pybind Engine (tandem/csrc/engine.cpp:109-122)."""

    def __init__(self, job, rank, size, slots, slot_bytes, timeout, device):
        self._e, self._device = _VP(), torch.device("cuda", device)
        self._orphans = []  # (work, tensors) of collectives whose handle was dropped before they had run
        _check(_L.tdm_engine_create(job.encode(), rank, size, slots, slot_bytes, float(timeout), device, ctypes.byref(self._e)))

    def connect(self):
        _check(_L.tdm_engine_connect(self._e))

    def close(self):
        e, self._e = self._e, None
        orphans, self._orphans = self._orphans, []
        if e:
            try:
                _check(_L.tdm_engine_close(e))  # runs what is queued and waits for the GPU
            finally:
                for p, _ in orphans:
                    _L.tdm_work_free(p)
                _L.tdm_engine_destroy(e)

    def _reap(self):
        """Lets go of the tensors of dropped collectives that have finished on the GPU."""
        still = []
        for p, keep in self._orphans:
            if _L.tdm_work_done(p):
                _L.tdm_work_free(p)
            else:
                still.append((p, keep))
        self._orphans = still

    def _start(self, call, *keep):
        if self._orphans:
            self._reap()
        out = _VP()
        _check(call(ctypes.byref(out)))
        return Handle(out, self._device, keep, self)

    def all_reduce(self, t, average):
        f = _flat(t)
        code, n = _reduced(f)
        return self._start(lambda o: _L.tdm_all_reduce(self._e, f.data_ptr(), n, code, int(average), _stream(self._device), o), f)

    def reduce_scatter(self, t, sizes, average):
        f = _flat(t)
        code, n = _reduced(f)
        arr, k = _sizes(list(sizes))
        return self._start(lambda o: _L.tdm_reduce_scatter(self._e, f.data_ptr(), n, code, arr, k, int(average), _stream(self._device), o), f)

    def all_gather(self, t, sizes):
        f = _flat(t)
        code, n, szs = _copied(f, sizes)
        arr, k = _sizes(szs)
        return self._start(lambda o: _L.tdm_all_gather(self._e, f.data_ptr(), n, code, arr, k, _stream(self._device), o), f)

    def broadcast(self, t, root):
        f = _flat(t)
        code, n, _ = _copied(f)
        return self._start(lambda o: _L.tdm_broadcast(self._e, f.data_ptr(), n, code, root, _stream(self._device), o), f)

    def send(self, t, dst):
        f = _flat(t)
        code, n, _ = _copied(f)
        return self._start(lambda o: _L.tdm_sendrecv(self._e, f.data_ptr(), n, dst, None, 0, -1, code, _stream(self._device), o), f)

    def recv(self, t, src):
        f = _flat(t)
        code, n, _ = _copied(f)
        return self._start(lambda o: _L.tdm_sendrecv(self._e, None, 0, -1, f.data_ptr(), n, src, code, _stream(self._device), o), f)

    def sendrecv(self, send, dst, recv, src):
        s, r = _flat(send), _flat(recv)
        code, n, _ = _copied(s)
        m = _copied(r)[1]
        return self._start(lambda o: _L.tdm_sendrecv(self._e, s.data_ptr(), n, dst, r.data_ptr(), m, src, code, _stream(self._device), o), s, r)

    def barrier(self):
        return self._start(lambda o: _L.tdm_barrier(self._e, o))
