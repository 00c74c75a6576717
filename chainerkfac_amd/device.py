"""Device-memory plumbing: torch-ROCm tensors carry the buffers, raw pointers go
to the C ABI.  Nothing here computes."""
import threading

import torch

from . import _lib


def require_gpu_tensor(t, name='array', dtype=torch.float32):
    if not isinstance(t, torch.Tensor):
        raise TypeError('{} must be a torch tensor on the GPU'.format(name))
    if not t.is_cuda:
        raise _lib.KfacHipError(
            '{} lives on {}; the K-FAC kernels only run on the GPU and there '
            'is no CPU fallback'.format(name, t.device))
    if dtype is not None and t.dtype != dtype:
        raise ValueError('{} must be {}, not {}'.format(name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError('{} must be C-contiguous'.format(name))
    return t


def ptr(t):
    return 0 if t is None else t.data_ptr()


def stream_handle(stream=None):
    """hipStream_t (as int) of ``stream`` or of torch's current stream."""
    if stream is None:
        # the raw handle without building a torch.cuda.Stream object (this is on the path of
        # every kernel launch)
        return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


class Workspace(object):
    """Grow-only scratch buffer handed to the C ABI as caller workspace."""

    def __init__(self):
        self._buf = None

    def get(self, nbytes, device):
        nbytes = max(int(nbytes), 256)
        if self._buf is None or self._buf.numel() < nbytes or self._buf.device != device:
            # wait for work that may still use the old buffer before dropping it
            if self._buf is not None:
                if torch.cuda.is_current_stream_capturing():
                    raise _lib.KfacHipError(
                        'a scratch buffer would have to grow ({} -> {} bytes) while a HIP graph is being '
                        'captured: run the same calls once before the capture'.format(self._buf.numel(), nbytes))
                torch.cuda.synchronize(self._buf.device)
            self._buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return self._buf


# Scratch buffers of work queued on the caller's own stream (no lane), by kind.
_default_workspaces = {}
# The lane whose work is being queued by this thread: (Lanes object, lane index) or None.
_queueing = threading.local()


def current_lane():
    """Index of the lane whose work is being queued, None on the caller's stream."""
    cur = getattr(_queueing, 'lane', None)
    return None if cur is None else cur[1]


def workspace(kind, nbytes, device):
    """Scratch buffer of ``kind`` for the lane being queued on (work on
    different lanes runs concurrently and must not share scratch memory; the
    lanes of different ``Lanes`` objects are different streams and have their
    own buffers)."""
    cur = getattr(_queueing, 'lane', None)
    table, key = (_default_workspaces, kind) if cur is None else (cur[0].workspaces, (kind, cur[1]))
    ws = table.get(key)
    if ws is None:
        ws = table[key] = Workspace()
    return ws.get(nbytes, device)


class Lanes(object):
    """Side streams for per-layer work that does not depend on other layers.

    The factor kernels of one layer (and later its preconditioning products) are
    often too small to fill the GPU and each waits for the previous one to drain
    when they share a stream.  ``run`` deals such work onto ``n`` streams in
    turn; every piece first waits for what the caller's stream has queued so far
    (its inputs), and ``join`` makes the caller's stream wait for all of it.
    With ``n`` = 0 everything runs on the caller's stream.  The scratch buffers
    of the work queued on a lane belong to this object.
    """

    def __init__(self, n=0):
        self.n = int(n)
        self.workspaces = {}
        self._streams = {}
        self._turn = 0
        self._busy = []

    def _pool(self, device):
        pool = self._streams.get(device)
        if pool is None or len(pool) < self.n:
            pool = self._streams[device] = (pool or []) + [
                torch.cuda.Stream(device=device) for _ in range(self.n - len(pool or []))]
        return pool

    def run(self, fn, tensors=()):
        """Calls ``fn()`` with the next lane as the current stream.  ``tensors``
        are the arrays it reads: their memory is kept from reuse until the lane
        has passed this point."""
        if self.n <= 0:
            return fn()
        main = torch.cuda.current_stream()
        pool = self._pool(main.device)
        index = self._turn % self.n
        lane = pool[index]
        self._turn += 1
        lane.wait_stream(main)
        outer = getattr(_queueing, 'lane', None)
        _queueing.lane = (self, index)
        torch.cuda.set_stream(lane)
        try:
            out = fn()
        finally:
            torch.cuda.set_stream(main)
            _queueing.lane = outer
        for t in tensors:
            if isinstance(t, torch.Tensor) and t.is_cuda:
                t.record_stream(lane)
        if lane not in self._busy:
            self._busy.append(lane)
        return out

    def skip(self):
        """Passes the turn on without queueing anything: for a piece of work that the caller
        keeps on its own stream this time, so that the pieces after it go to the lanes they go
        to when it does take one (a lane's scratch buffers keep the sizes its pieces need)."""
        if self.n > 0:
            self._turn += 1

    def join(self):
        # every phase deals its work the same way each time it runs (the scratch
        # buffers of a lane then keep their sizes, which a captured graph needs)
        self._turn = 0
        if not self._busy:
            return
        main = torch.cuda.current_stream()
        for lane in self._busy:
            main.wait_stream(lane)
        self._busy = []
