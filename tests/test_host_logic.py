"""Host-side behaviour of the C ABI that needs no GPU: argument checking and loud failure without a device."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk


def test_null_handles_are_rejected():
    lib = nk.lib()
    assert lib.nuka_world_step(None) == 2
    assert lib.nuka_world_step_n(None, 3) == 2
    assert lib.nuka_world_synchronize(None) == 2
    assert lib.nuka_world_dispatch_op(None, 0, 0) == 2
    view = nk.abi.BufferViewC()
    assert lib.nuka_world_get_buffer_view(None, 0, C.byref(view)) == 2
    out = C.c_void_p()
    cfg = nk.synthetic.config(1, 4)
    tdesc, keep = cfg.template.to_c()
    desc = nk.abi.world_desc(4, cfg.dt)
    assert lib.nuka_world_create_from_template(None, C.byref(tdesc), C.byref(desc), C.byref(out)) == 2
    assert lib.nuka_device_create(None, C.byref(out)) == 1


def test_device_creation_fails_loudly_without_a_gpu():
    import torch  # only to ask whether this machine has a GPU
    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(nk.NukaError) as info:
        nk.Device(0)
    assert "device" in str(info.value).lower()


def test_synthetic_configs_have_the_published_shapes():
    shapes = {1: (8, 7, 0), 2: (13, 18, 4), 3: (31, 36, 12), 5: (65, 64, 64)}
    for index, (links, dof, spheres) in shapes.items():
        cfg = nk.synthetic.config(index, 4)
        assert cfg.template.link_count == links and cfg.template.dof == dof
        assert sum(b["kind"] == nk.abi.SHAPE_SPHERE for b in cfg.template.bodies) == spheres
        state = cfg.state()
        assert state["q"].shape == (4, links) and state["base_pose"].shape == (4, 7)
        again = nk.synthetic.config(index, 4).state()
        assert all(np.array_equal(state[k], again[k]) for k in state)      # seeded: the same every time
    assert nk.synthetic.config(4, 8).template.dof == 36
