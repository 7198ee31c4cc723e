"""The on-disk code-object cache on a device: an object the runtime refuses to load is dropped and recompiled."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_cached_object_the_runtime_refuses_is_recompiled(hip_backend_session, tmp_path, monkeypatch):
    """A well-formed cache file (header, checksum, AMDGPU ELF) that holds a code object for another target passes the
    file checks; hipModuleLoadData then refuses it, the file is deleted, the kernel compiled again, and it runs."""
    from descent_amd import hip_backend, kernel as K

    cache = tmp_path / "cache"
    cache.mkdir()
    monkeypatch.setenv("DSC_CACHE_DIR", str(cache))
    kernel = K.FillKernel(K.Literal.f32(3.5), 70001)  # a descriptor no other test compiles in this process
    hip_backend.codegen_compile(kernel, "gfx950")
    (ours,) = list(cache.iterdir())
    hip_backend.codegen_compile(kernel, "gfx942")
    (other,) = [f for f in cache.iterdir() if f != ours]
    good = ours.read_bytes()
    ours.write_bytes(other.read_bytes())

    be = hip_backend_session
    before = hip_backend.cache_stats()
    h = be.alloc(70001 * 4)
    be.launch(kernel, [h], 0)
    got = np.frombuffer(be.read(h, 0, 70001 * 4), np.float32)
    be.free(h)
    delta = tuple(a - b for a, b in zip(hip_backend.cache_stats(), before))
    assert delta == (1, 1, 1), delta  # read from the cache, refused by the runtime and dropped, compiled once
    assert np.all(got == 3.5)
    assert ours.read_bytes() == good
