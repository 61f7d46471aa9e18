"""mcn_bnorm_backward_static -- the entry point that allocates nothing (its partial sums live in a device array built
into the library) -- against mcn_bnorm_backward, which takes them in a workspace of the caller's: same bits on every
output, on two calls in a row that share the array, the second with a smaller input; moments given and from the
batch; shapes beyond the array's size rejected before anything is launched."""
import ctypes as C

import numpy as np
import pytest

from matconvnet_amd import workloads
from util import bits_equal

pytestmark = pytest.mark.gpu

CALLS = [(56, 56, 64, 8), (14, 14, 16, 3)]   # second call smaller: fewer channels and fewer partial sums per channel


def _inputs(capi, shape, seed):
    w = workloads.bnorm_case(seed=seed, H=shape[0], W=shape[1], C=shape[2], N=shape[3])
    return [capi.to_device(w[k]) for k in ("x", "g", "dy")]


@pytest.mark.parametrize("given", [False, True])
def test_static_scratch_entry_point_matches_the_workspace_one(capi, given):
    import torch
    L = capi.lib()
    for i, shape in enumerate(CALLS):
        H, W, Cc, N = shape
        assert L.mcn_bnorm_workspace_bytes(H, W, Cc, N) <= capi.BNORM_STATIC_SCRATCH_BYTES
        x, g, dy = _inputs(capi, shape, 40 + i)
        mom_in = None
        if given:
            mom_in = capi.to_device(np.asfortranarray(np.stack([np.linspace(-1, 1, Cc), np.linspace(0.5, 2, Cc)], axis=1), dtype=np.float32))
        want = capi.bnorm_backward(x, g, dy, 1e-4, moments=mom_in)
        out = (capi.empty(shape), capi.empty((Cc,)), capi.empty((Cc,)), mom_in if given else capi.empty((Cc, 2)))
        for t in out[:3]:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        # the call's defining property: device memory in use is the same before and after it (the first call on a device
        # also looks the array's address up, which allocates nothing either)
        free_before, _ = torch.cuda.mem_get_info()
        got = capi.bnorm_backward_static(x, g, dy, 1e-4, moments=mom_in, out=out)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, (shape, free_before - free_after)
        for name, a, b in zip(("dzdx", "dzdg", "dzdb", "moments"), got, want):
            assert bits_equal(capi.to_host(a), capi.to_host(b)), (shape, name)


def test_shapes_beyond_the_scratch_are_rejected(capi):
    L = capi.lib()
    H, W, Cc, N = 64, 64, 1024, 64      # one partial per plane: 65536 partials of 32 bytes = 2 MiB
    assert L.mcn_bnorm_workspace_bytes(H, W, Cc, N) > capi.BNORM_STATIC_SCRATCH_BYTES
    x, dy, dx = (capi.empty((H, W, Cc, N)) for _ in range(3))
    g, dg, db = (capi.empty((Cc,)) for _ in range(3))
    rc = L.mcn_bnorm_backward_static(capi.stream(), capi.ptr(dx), capi.ptr(dg), capi.ptr(db), None, capi.ptr(x), capi.ptr(g),
                                     capi.ptr(dy), H, W, Cc, N, 1e-4, 0)
    assert rc == capi.UNSUPPORTED
    assert b"scratch" in L.mcn_last_error_message()
