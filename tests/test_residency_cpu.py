"""Host logic of device mirrors and shared arrays that needs no GPU: the address
registry, the module aliasing of ``import appy.np_shared`` and the behaviour of
the array constructors on a machine without a device."""
import numpy as np
import pytest

from appy_amd import residency


def test_lookup_finds_views_by_address_containment():
    base = 1 << 40          # addresses are only compared, never dereferenced, until a launch
    m = residency.register(base, 4096, pinned=False)
    try:
        assert residency.active()
        assert residency.lookup(base, 4096) == (m, 0)
        assert residency.lookup(base + 100, 200) == (m, 100)
        assert residency.lookup(base + 4000, 97) is None          # runs past the end
        assert residency.lookup(base - 8, 16) is None
        assert residency.lookup(base + 8192, 8) is None
        assert residency.register(base, 4096, pinned=False) is m  # same range: same mirror
        with pytest.raises(ValueError):
            residency.register(base + 1024, 4096, pinned=False)   # partial overlap from above
        with pytest.raises(ValueError):
            residency.register(base - 1024, 2048, pinned=False)   # partial overlap from below
        m2 = residency.register(base + 4096, 64, pinned=False)    # adjacent is fine
        assert residency.lookup(base + 4096, 64) == (m2, 0)
        residency.unregister(base + 4096)
    finally:
        residency.unregister(base)
    assert residency.lookup(base, 8) is None


def test_resident_rejects_what_cannot_be_mirrored():
    with pytest.raises(TypeError):
        residency.resident([1.0, 2.0]).__enter__()
    with pytest.raises(ValueError):
        residency.sync_host(np.zeros((4, 4))[:, 1])
    residency.sync_host(np.zeros(4))      # not mirrored: nothing to do
    residency.invalidate(np.zeros(4))


def test_import_appy_np_shared_is_the_same_module_object():
    import appy
    import appy.np_shared as nps
    import appy_amd
    import appy_amd.np_shared as nps2

    assert appy is appy_amd and nps is nps2
    assert appy.resident is residency.resident and nps.resident is residency.resident
    import appy.residency as r2

    assert r2 is residency                # one registry, whatever name it was imported under


def test_shared_array_constructors_without_a_gpu():
    import appy.np_shared as nps
    from appy_amd.backends.hip import runtime as rt

    if rt.device_count() > 0:
        pytest.skip("a GPU is present: covered by the GPU tests")
    a = nps.empty((3, 4), dtype=np.float32)
    assert a.shape == (3, 4) and a.dtype == np.float32 and not nps.has_device_buffer(a)
    assert nps.zeros(5, dtype=np.int32).tolist() == [0] * 5
    c = nps.copy(np.arange(6).reshape(2, 3))
    assert np.array_equal(c, np.arange(6).reshape(2, 3))
    r = nps.randn(2, 3, dtype=np.float32)
    assert r.shape == (2, 3) and r.dtype == np.float32
    assert nps.empty_like(r, dtype=np.int64).dtype == np.int64
    with pytest.raises(KeyError):
        nps.get_device_buffer(a)
