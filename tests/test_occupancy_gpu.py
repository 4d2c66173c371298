"""The block-level scheduler's occupancy model in gfx950 units against the runtime's own occupancy calculator, for
every kernel the model zoo is made of: workgroups per compute unit = min(4 SIMDs x min(8, 512 / registers rounded up to
8) waves / waves per workgroup, 160 KiB / LDS rounded up to 1280 bytes, 32) (reference counterpart: the budget
arithmetic of src/server/sm_resources.cpp:17-66, which charges regs x threads as CUDA allocates them)."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu


def model_blocks_per_cu(threads, regs, lds, caps):
    from paella_amd import _abi
    lib = ctypes.CDLL(os.path.join(_abi.LIB_DIR, "libllis_server.so"), mode=ctypes.RTLD_GLOBAL)
    lib.llis_sm_resources_blocks_per_cu.restype = ctypes.c_uint
    return lib.llis_sm_resources_blocks_per_cu(threads, regs, lds, caps.lds_bytes_per_cu, 32)


@pytest.fixture(scope="module")
def caps(cuda):
    from paella_amd import _abi
    c = _abi.DeviceCaps()
    _abi.check(_abi.hip().llis_hip_get_device_caps(ctypes.byref(c)))
    # the constants the model is written in
    assert c.wavefront_size == 64 and c.max_threads_per_cu == 4 * 8 * 64 and c.lds_bytes_per_cu == 160 * 1024
    return c


FAMILIES = [("dense", 256), ("dense_long", 512), ("pool", 256), ("gap", 256), ("eltwise", 256), ("copy", 256), ("softmax", 256),
            ("softmax_short", 256), ("lrn", 256)]


@pytest.mark.parametrize("family,block", FAMILIES)
def test_memory_bound_kernels(caps, family, block):
    from paella_amd import _abi
    lib = _abi.ops()
    regs, lds, got = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_int()
    _abi.check(lib.paella_kernel_vgprs(family.encode(), ctypes.byref(regs)))
    _abi.check(lib.paella_kernel_static_lds(family.encode(), ctypes.byref(lds)))
    _abi.check(lib.paella_kernel_occupancy(family.encode(), block, 0, ctypes.byref(got)))
    assert model_blocks_per_cu(block, regs.value, lds.value, caps) == got.value, (family, regs.value, lds.value)


def conv_variants():
    out = [(1, 0, 1, 1, 4, 0)]  # depthwise (block 256)
    for k_order in (0, 1):
        for mi, ni in ((1, 1), (1, 2), (2, 1), (2, 2)):
            for kw in (1, 2, 4, 8):
                out.append((0, 0, mi, ni, kw, k_order))
        for kw in (1, 2, 4, 8):
            out.append((0, 2, 1, 1, kw, k_order))
    for kw in (1, 2, 4, 8):
        out += [(0, 1, 1, 1, kw, 1), (0, 3, 1, 1, kw, 1)]
    return out


@pytest.mark.parametrize("kind,form,mi,ni,kw,k_order", conv_variants())
def test_conv_kernels_with_the_planner_lds(caps, kind, form, mi, ni, kw, k_order):
    """LDS as the planner sizes it: kw partial tiles of mi x ni x 16 registers x 64 lanes (none for one wave), and for the
    offset-table order a table that may be larger; both ends are tried."""
    from paella_amd import _abi
    lib = _abi.ops()
    block = 256 if kind == 1 else 64 * kw
    red = 0 if (kind == 1 or kw == 1) else kw * mi * ni * 16 * 64 * 4
    for lds in sorted({red, max(red, 40 * 1024)} if (kind == 0 and k_order == 0) else {red}):
        regs, static, got = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_int()
        _abi.check(lib.paella_conv_kernel_occupancy(kind, form, mi, ni, kw, k_order, lds, ctypes.byref(got), ctypes.byref(regs), ctypes.byref(static)))
        assert model_blocks_per_cu(block, regs.value, lds + static.value, caps) == got.value, (regs.value, lds, static.value)


def test_every_zoo_stage_reports_registers_and_fits_the_device(caps):
    """Stage dims carry the launched kernel's real register count, and the pooled budget admits every single stage of
    every zoo model on an idle device (a kernel that did not would wait for ever)."""
    from paella_amd import models
    for name in models.names():
        m = models.Exec(name, seed=1)
        try:
            for i in range(m.num_stages):
                d = m.stage_dims(i)
                assert 0 < d.vgprs <= 512 and 0 < d.block <= 1024
                per_cu = model_blocks_per_cu(d.block, d.vgprs, d.lds_bytes, caps)
                assert per_cu >= 1, (name, i, d.block, d.vgprs, d.lds_bytes)
                assert per_cu * caps.num_cus + 0 >= 1
        finally:
            m.close()
