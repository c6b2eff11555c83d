"""DeviceContext: the one in-order stream every reference GPU method takes as `ctx`.

Mirrors the subset of Mojo's gpu.host.DeviceContext that the rollout / update path uses
(enqueue_create_buffer, enqueue_memset, synchronize); buffers are torch tensors on the GPU.
"""
import ctypes as C

import torch

from . import _lib


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise _lib.MrlError("device buffer expected, got a %s tensor" % t.device)
    if not t.is_contiguous():
        raise _lib.MrlError("device buffers must be contiguous")
    return t.data_ptr()


class DeviceContext:
    def __init__(self, device="cuda:0", stream=None):
        if not torch.cuda.is_available():
            raise _lib.MrlError("no GPU visible: the MI355X path has no CPU fallback")
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.stream = stream if stream is not None else torch.cuda.current_stream(self.device)
        handle = C.c_void_p()
        _lib.call("mrl_ctx_create", C.c_void_p(self.stream.cuda_stream), C.byref(handle))
        self.handle = handle

    def enqueue_create_buffer(self, n, dtype=torch.float32):
        return torch.empty(n, dtype=dtype, device=self.device)

    def enqueue_memset(self, buf, value):
        with torch.cuda.stream(self.stream):
            buf.fill_(value)

    def synchronize(self):
        _lib.call("mrl_ctx_synchronize", self.handle)

    def workspace(self):
        """(mlp_floats, rollout_floats) that the context's two workspaces hold now."""
        import ctypes
        a, b = ctypes.c_uint64(0), ctypes.c_uint64(0)
        _lib.call("mrl_ctx_workspace", self.handle, ctypes.byref(a), ctypes.byref(b))
        return a.value, b.value

    def reserve(self, mlp_floats=0, rollout_floats=0):
        """Size the workspaces ahead, so that no later call has to drain the stream and allocate."""
        _lib.call("mrl_ctx_reserve", self.handle, int(mlp_floats), int(rollout_floats))

    def set_spin_limit(self, polls):
        """Bound on the polls of a wait at a kernel-internal wavefront barrier (0: the default).  A
        wait that gives up makes the next synchronize() raise; a tiny value exercises that path."""
        _lib.call("mrl_ctx_set_spin_limit", self.handle, int(polls))

    PHASES = ("policy_fwd", "sample_store", "env_step", "post_store", "collect")

    def profile_begin(self, max_marks=8192, sample_every=1):
        """Arm per-phase device timing (HIP events on this context's stream); with sample_every = k
        only every k-th rollout step carries events."""
        _lib.call("mrl_profile_sample_every", self.handle, sample_every)
        _lib.call("mrl_profile_begin", self.handle, max_marks)

    def profile_end(self):
        """Synchronise and return {phase: (total_ms, launches)}."""
        n = len(self.PHASES)
        ms = (C.c_double * n)()
        cnt = (C.c_int * n)()
        _lib.call("mrl_profile_end", self.handle, n, ms, cnt)
        return {p: (ms[i], cnt[i]) for i, p in enumerate(self.PHASES)}

    def close(self):
        if self.handle:
            _lib.call("mrl_ctx_destroy", self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
