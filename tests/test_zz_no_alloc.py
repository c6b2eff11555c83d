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
        before = torch.cuda.memory_allocated()
        mrl.ppo.clip_grad_norm_static(ctx, b, max_norm)
        ctx.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(a, b), "differs in %d places" % int((a != b).sum())
        want = grads.cpu().numpy().copy()
        orc.orc_clip_grad_norm(want, n, max_norm)
        np.testing.assert_allclose(b.cpu().numpy(), want, rtol=1e-5, atol=1e-9)
        clipped = float(np.sqrt((grads.cpu().numpy().astype(np.float64) ** 2).sum())) > max_norm
        assert clipped == (n > 1 and scale > 1e-3) or n == 1
    # empty input is a no-op, a size beyond the stated limit is refused with a message
    mrl.ppo.clip_grad_norm_static(ctx, torch.zeros(0, device="cuda"), 0.5)
    lib = mrl._lib.lib()
    rc = lib.mrl_clip_grad_norm_static(ctx.handle, ctypes.c_void_p(a.data_ptr()), mrl.ppo.CLIP_STATIC_MAX_N + 1,
                                       ctypes.c_float(0.5))
    assert rc == -1 and b"exceeds the limit" in lib.mrl_last_error()
    ctx.close()
