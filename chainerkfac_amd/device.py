"""Device-memory plumbing: torch-ROCm tensors carry the buffers, raw pointers go
to the C ABI.  Nothing here computes."""
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
        stream = torch.cuda.current_stream()
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
                torch.cuda.synchronize(self._buf.device)
            self._buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return self._buf


_default_workspaces = {}


def workspace(kind, nbytes, device):
    ws = _default_workspaces.get(kind)
    if ws is None:
        ws = _default_workspaces[kind] = Workspace()
    return ws.get(nbytes, device)
