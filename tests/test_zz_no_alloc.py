"""trips_splat_forward_static: the forward on the library's own static workspace, for callers that cannot allocate.

Called through the C ABI twice in a row on one context, the second time with a smaller scene (so that whatever the
first call left in the shared array is still there), each result held against trips_splat_forward on a caller-owned
workspace: images, saved lists and point records bit for bit."""
import ctypes as C

import numpy as np
import pytest
import torch

from trips_amd import abi, scenes

pytestmark = pytest.mark.gpu


def _both(sc, desc):
    from tests.gpu_util import GpuRun
    run = GpuRun(sc, desc)
    want = run.forward()
    want_state = None
    if desc.train:
        want_state = [x for b in range(desc.num_views) for x in (*run.lists(b), *run.points(b))]
    # the same inputs through the entry point without a workspace argument
    images = run.ctx.alloc_images(desc, fill=float("nan"))
    saved = run.ctx.alloc_bytes(run.ctx.saved_size(desc)) if desc.train else None
    out = abi.TripsSplatOut()
    for l, im in enumerate(images):
        out.image[l] = im.data_ptr()
    out.saved = None if saved is None else C.c_void_p(saved.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream(run.ctx.device).cuda_stream)
    rc = run.ctx.lib.trips_splat_forward_static(run.ctx.ctx, C.byref(desc), C.byref(run.tin), C.byref(out), stream)
    assert rc == abi.TRIPS_OK, run.ctx.lib.trips_last_error_string()
    torch.cuda.synchronize()
    assert run.ctx.lib.trips_splat_check(run.ctx.ctx, None, stream) == abi.TRIPS_OK
    for l, (a, b) in enumerate(zip(images, want)):
        np.testing.assert_array_equal(a.cpu().numpy(), b, err_msg=f"layer {l}")
    if desc.train:
        run.saved = saved
        got_state = [x for b in range(desc.num_views) for x in (*run.lists(b), *run.points(b))]
        for a, b in zip(got_state, want_state):
            np.testing.assert_array_equal(a, b)
    return run


def test_static_workspace_forward_twice_then_smaller():
    big = scenes.tiny(n=20000, w=160, h=120, f=120.0, num_layers=5, list_depth=16, seed=77, views=2, radius=(0.004, 0.3))
    _both(big, abi.desc_for_scene(big))
    small = scenes.tiny(n=3000, w=64, h=48, f=60.0, num_layers=3, list_depth=8, seed=78)
    _both(small, abi.desc_for_scene(small))
    _both(small, abi.desc_for_scene(small, train=False))  # no saved state: counters and records live in the workspace


def test_static_workspace_rejects_scenes_beyond_its_size():
    from trips_amd.renderer import get_context
    ctx = get_context(0)
    sc = scenes.tiny(n=500, w=64, h=48, num_layers=3)
    d = abi.desc_for_scene(sc)
    d.num_points = 4_000_000  # worst-case list storage of 4 N L entries: far beyond 64 MiB; nothing is dereferenced
    assert ctx.workspace_size(d) > abi.TRIPS_STATIC_WORKSPACE_BYTES
    tin, out = abi.TripsSplatIn(), abi.TripsSplatOut()
    rc = ctx.lib.trips_splat_forward_static(ctx.ctx, C.byref(d), C.byref(tin), C.byref(out), None)
    assert rc == abi.TRIPS_ERR_WORKSPACE_SMALL
    assert b"static" in ctx.lib.trips_last_error_string()
