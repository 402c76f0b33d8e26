"""n2_composite_loss_static (scratch in a device array of the library, no allocation) against
n2_composite_loss_indexed (caller's workspace): bit-identical outputs, two calls in a row, the second smaller."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import dev, host, q16
from test_oracle_composite import make_rays

pytestmark = pytest.mark.gpu


def _call(static, numsteps, out, coords, target, cap, ray_counter=None):
    from neus2_amd import capi
    from neus2_amd.capi import check, ptr
    L = capi.lib()
    n_rays = numsteps.shape[0]
    cfg = capi.CompositeConfig(128.0, 0.01, 1.0, (C.c_float * 3)(0.3, 0.6, 0.9), n_rays)
    d_ns = dev(numsteps.astype(np.int32))
    d_out, d_coords, d_target = dev(q16(out), torch.float16), dev(coords), dev(target)
    counter = torch.zeros(1, dtype=torch.int32, device="cuda")
    cout = torch.zeros((cap, 7), dtype=torch.float32, device="cuda")
    dloss = torch.zeros((cap, 16), dtype=torch.float16, device="cuda")
    loss = torch.zeros(n_rays, dtype=torch.float32, device="cuda")
    index = torch.full((cap,), -1, dtype=torch.int32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [stream, C.byref(cfg), C.c_uint32(n_rays), ptr(ray_counter), ptr(d_ns), ptr(d_out), ptr(d_coords), ptr(d_target),
            C.c_uint32(cap), ptr(counter), ptr(cout), ptr(dloss), ptr(loss), ptr(index)]
    if static:
        # Everything the call needs exists before it: it must not change the device's free memory (hipMemGetInfo sees
        # allocations of any library, not only torch's allocator).  A first call on the device is let through beforehand:
        # it looks the scratch array's address up, which may load the code object.
        global _warm
        if not _warm:
            _warm = True
            rng = np.random.default_rng(1)
            _call(True, *make_rays(rng, 8, lo=1, hi=9), 256)   # buffers of its own: the call rewrites numsteps in place
        before_torch, (before_free, _) = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()
        check(L.n2_composite_loss_static(*args), "n2_composite_loss_static")
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before_torch
        assert torch.cuda.mem_get_info()[0] == before_free
    else:
        nbytes = int(L.n2_composite_workspace_bytes(C.c_uint32(max(n_rays, 1))))
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        check(L.n2_composite_loss_indexed(*args, ptr(ws), C.c_uint64(nbytes)), "n2_composite_loss_indexed")
    torch.cuda.synchronize()
    return dict(numsteps=host(d_ns), counter=host(counter), coords=host(cout), dloss=dloss.cpu().numpy().view(np.uint16),
                loss=host(loss), index=host(index))


_warm = False


def _same(a, b):
    for k in a:
        assert np.array_equal(a[k], b[k]), k


def test_static_scratch_matches_workspace_entry_point():
    rng = np.random.default_rng(11)
    # first call: 3000 rays; then 9000 (from 8192 rays on the rays' places come from a scan kernel, whose sums sit in the
    # scratch as well); then, right after it on the same GPU, 700 rays (the array keeps the earlier calls' rows)
    for n_rays, cap, sharp, hi in ((3000, 1 << 18, True, 150), (9000, 1 << 18, True, 40), (700, 1 << 14, False, 150)):
        numsteps, out, coords, target = make_rays(rng, n_rays, lo=1, hi=hi, sharp=sharp)
        ref = _call(False, numsteps, out, coords, target, cap)
        got = _call(True, numsteps, out, coords, target, cap)
        assert int(ref["counter"][0]) > 0
        _same(ref, got)
    # a live-ray counter below n_rays: slots of the dead rays are rewritten, not inherited
    numsteps, out, coords, target = make_rays(rng, 500, lo=2, hi=60)
    live = torch.tensor([100], dtype=torch.int32, device="cuda")
    _same(_call(False, numsteps, out, coords, target, 1 << 14, live), _call(True, numsteps, out, coords, target, 1 << 14, live))


def test_static_scratch_rejects_more_rays_than_it_holds():
    from neus2_amd import capi
    L = capi.lib()
    cfg = capi.CompositeConfig(128.0, 0.01, 1.0, (C.c_float * 3)(0, 0, 0), 1)
    counter = torch.zeros(1, dtype=torch.int32, device="cuda")
    rc = L.n2_composite_loss_static(None, C.byref(cfg), C.c_uint32(65537), None, None, None, None, None, C.c_uint32(8),
                                    capi.ptr(counter), None, None, None, None)
    assert rc == 1 and b"65536" in L.n2_last_error()
