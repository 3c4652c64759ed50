"""CPU-side checks of the shipped library: it loads, exports every symbol the
public header declares, and its pool logic behaves like DyNet's
AlignedMemoryPool (dynet/aligned-mem-pool.cc:8-91; scenario of
tests/test-mem.cc:36-48: an allocation larger than the pool forces growth).
No compute entry point is called here."""
import ctypes as C

import numpy as np
import pytest

from dynet_amd import lib
from dynet_amd.device import DyhipError, Pool, device_count


def test_library_exports_every_declared_symbol():
    names = lib.declared_symbols()
    assert len(names) > 60
    missing = [n for n in names if not hasattr(lib.cdll, n)]
    assert not missing, missing


def test_header_cites_the_reference_for_every_operator_group():
    text = open(lib.HEADER_PATH).read()
    for needle in ("dynet/nodes-lstm.cc", "dynet/matrix-multiply.h", "dynet/aligned-mem-pool", "dynet/gpu-ops.h",
                   "dynet/nodes-pickneglogsoftmax.cc", "dynet/param-nodes.cc", "dynet/expr.cc:248-253",
                   "dynet/training.cc:619-622"):
        assert needle in text, needle


def test_status_convention_and_last_error():
    p = C.c_void_p(None)
    st = lib.cdll.dyhip_pool_create_host(b"zero", C.c_size_t(0), C.c_size_t(0), C.byref(p))
    assert st == lib.ERR_INVALID_ARG
    assert "size 0" in lib.last_error()
    assert lib.cdll.dyhip_device_sync(C.c_void_p(None)) == lib.ERR_INVALID_ARG
    assert "null device" in lib.last_error()


def test_pool_rounds_to_alignment_and_bumps():
    pool = Pool.create_host("cpu pool", 1 << 20)
    try:
        a = pool.allocate(1)
        b = pool.allocate(33)
        c = pool.allocate(64)
        assert a % 32 == 0 and b - a == 32 and c - b == 64  # CPUAllocator alignment is 32
        assert pool.used() == 32 + 64 + 64
        assert pool.capacity() == 1 << 20 and pool.num_blocks() == 1
        pool.free()
        assert pool.used() == 0
        assert pool.allocate(8) == a  # bump allocator restarts at the base
    finally:
        pool.destroy()


def test_pool_memory_is_zero_filled_and_zero_allocated_clears_the_used_prefix():
    pool = Pool.create_host("cpu pool", 4096)
    try:
        p = pool.allocate(1024)
        buf = (C.c_ubyte * 1024).from_address(p)
        assert not any(buf)
        for k in range(1024):
            buf[k] = 0xAB
        pool.zero_allocated()
        assert not any(buf)
    finally:
        pool.destroy()


def test_pool_grows_in_expanding_units_and_consolidates_on_free():
    unit = 1 << 16
    pool = Pool.create_host("cpu pool", 4096, expanding_unit=unit)
    try:
        pool.allocate(4000)
        big = 3 * unit + 5  # does not fit: new block of ceil(n / unit) * unit bytes
        pool.allocate(big)
        assert pool.num_blocks() == 2
        assert pool.capacity() == 4096 + 4 * unit
        assert pool.used() == 4000 + 32 * ((big + 31) // 32) - 0 + (32 - 4000 % 32) % 32
        # checkpoints are refused once the pool has grown (aligned-mem-pool.cc:71-75)
        with pytest.raises(DyhipError) as e:
            pool.set_used(64)
        assert e.value.status == lib.ERR_INVALID_ARG
        pool.free()  # one block of the total capacity
        assert pool.num_blocks() == 1 and pool.capacity() == 4096 + 4 * unit and pool.used() == 0
        pool.allocate(big)  # now fits without growing
        assert pool.num_blocks() == 1
    finally:
        pool.destroy()


def test_pool_growth_scenario_of_test_mem():
    """tests/test-mem.cc:36-48: a 1024x1024 fp32 parameter (4 MiB) in a 1 MiB pool."""
    pool = Pool.create_host("param pool", 1 << 20)
    try:
        p = pool.allocate(1024 * 1024 * 4)
        assert p != 0 and pool.num_blocks() == 2
        assert pool.capacity() == (1 << 20) + (1 << 24)  # default expanding unit 1 << 24
        view = np.ctypeslib.as_array((C.c_float * (1024 * 1024)).from_address(p))
        assert float(view.sum()) == 0.0
    finally:
        pool.destroy()


def test_pool_set_used_checkpoint_and_revert():
    pool = Pool.create_host("cpu pool", 8192)
    try:
        pool.allocate(100)
        mark = pool.used()
        pool.allocate(500)
        pool.set_used(mark)  # Device::revert (dynet/devices.cc:68-80)
        assert pool.used() == mark
        with pytest.raises(DyhipError):
            pool.set_used(1 << 30)
    finally:
        pool.destroy()


def test_no_silent_cpu_fallback_without_a_gpu():
    if device_count() > 0:
        pytest.skip("a GPU is visible")
    from dynet_amd import Device

    with pytest.raises(DyhipError) as e:
        Device(0)
    assert e.value.status == lib.ERR_NO_DEVICE
