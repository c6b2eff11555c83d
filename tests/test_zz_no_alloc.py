"""mrl_clip_grad_norm_static, the entry point that allocates nothing (its partial sums live in a
file-scope device array), against mrl_clip_grad_norm on the same gradients."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_clip_grad_norm_static_equals_clip_grad_norm(mrl, orc):
    ctx = mrl.DeviceContext("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(7)
    # two calls in a row on the shared scratch array, the second with a smaller input (fewer
    # partial sums than the first call left behind), then one that is not clipped at all
    for n, scale, max_norm in ((141_477, 0.05, 0.5), (3_001, 0.05, 0.5), (70_000, 1e-4, 0.5), (1, 3.0, 0.5)):
        print("case n", n, flush=True)
        grads = (torch.rand(n, device="cuda", generator=g) - 0.5) * 2 * scale
        a, b = grads.clone(), grads.clone()
        mrl.ppo.clip_grad_norm(ctx, a, max_norm)
        ctx.synchronize()
        # free device memory as the driver counts it (hipMemGetInfo): a hipMalloc or hipFree inside the
        # library would move it, which torch's own allocator statistics cannot see.  Warm state: every
        # tensor of this case exists already and nothing is created between the two readings.
        free_before, _ = torch.cuda.mem_get_info()
        mrl.ppo.clip_grad_norm_static(ctx, b, max_norm)
        ctx.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, "free device memory moved by %d bytes" % (free_before - free_after)
        assert torch.equal(a, b), "differs in %d places" % int((a != b).sum())
        want = grads.cpu().numpy().copy()
        orc.orc_clip_grad_norm(want, n, max_norm)
        np.testing.assert_allclose(b.cpu().numpy(), want, rtol=1e-5, atol=1e-9)
        clipped = float(np.sqrt((grads.cpu().numpy().astype(np.float64) ** 2).sum())) > max_norm
        assert clipped == (n > 1 and scale > 1e-3) or n == 1
    # Under HIP graph capture an allocation (or any synchronising call) fails the capture: the entry
    # point is captured on the context's stream and the graph is replayed on fresh copies of the
    # gradients, with eager work and synchronisations between the replays.
    n, max_norm = 141_477, 0.5
    src = (torch.rand(n, device="cuda", generator=g) - 0.5) * 0.1
    buf = src.clone()
    want = src.clone()
    mrl.ppo.clip_grad_norm(ctx, want, max_norm)
    ctx.synchronize()
    side = torch.cuda.Stream()                               # capture needs a stream other than the default one
    cctx = mrl.DeviceContext("cuda:0", stream=side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        mrl.ppo.clip_grad_norm_static(cctx, buf, max_norm)
    for rep in range(3):
        buf.copy_(src)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(buf, want), "graph replay %d differs in %d places" % (rep, int((buf != want).sum()))
        mrl.ppo.clip_grad_norm_static(ctx, src.clone(), 0.25)       # eager use of the same array in between
        ctx.synchronize()
    # empty input is a no-op, a size beyond the stated limit is refused with a message
    mrl.ppo.clip_grad_norm_static(ctx, torch.zeros(0, device="cuda"), 0.5)
    lib = mrl._lib.lib()
    rc = lib.mrl_clip_grad_norm_static(ctx.handle, ctypes.c_void_p(a.data_ptr()), mrl.ppo.CLIP_STATIC_MAX_N + 1,
                                       ctypes.c_float(0.5))
    assert rc == -1 and b"exceeds the limit" in lib.mrl_last_error()
    del graph
    cctx.close()
    ctx.close()
