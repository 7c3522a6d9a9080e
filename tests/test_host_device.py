"""Host-side pieces of the device layer that need no GPU: the disk cache behind Compiler.compile_cached
(/root/reference/jsgrad/runtime/allocator.ts:123-139, /root/reference/jsgrad/env/node.ts:89-122)."""
import os

import pytest

from denograd_amd import diskcache
from denograd_amd.device import CompileError, HIPCompiler


@pytest.fixture
def cache_db(tmp_path, monkeypatch):
    monkeypatch.setenv("CACHE_DB", str(tmp_path / "cache" / "jsgrad.db"))
    monkeypatch.delenv("DISABLE_COMPILER_CACHE", raising=False)
    monkeypatch.delenv("ASSERT_COMPILE", raising=False)
    return tmp_path / "cache" / "jsgrad.db"


def test_disk_cache_round_trip(cache_db):
    assert diskcache.disk_get("t", "k") is None            # no table yet: a miss, not an error
    diskcache.disk_put("t", "k", b"\x00\x01\xff")
    diskcache.disk_put("t", "k2", b"other")
    diskcache.disk_put("s", "k", "text value")
    assert diskcache.disk_get("t", "k") == b"\x00\x01\xff"
    assert diskcache.disk_get("t", "k2") == b"other"
    assert diskcache.disk_get("s", "k") == "text value"
    assert diskcache.disk_get("t", "absent") is None
    diskcache.disk_put("t", "k", b"again")                 # a second put replaces
    assert diskcache.disk_get("t", "k") == b"again"
    assert cache_db.exists()
    with pytest.raises(TypeError):
        diskcache.disk_put("t", "k", 3)


def test_cache_paths_follow_the_environment(monkeypatch):
    monkeypatch.delenv("CACHE_DB", raising=False)
    monkeypatch.setenv("CACHE_DIR", "/x/y")
    assert diskcache.cache_db() == "/x/y/jsgrad/jsgrad.db"
    monkeypatch.delenv("CACHE_DIR")
    monkeypatch.setenv("XDG_CACHE_HOME", "/z")
    assert diskcache.cache_dir() == "/z/jsgrad"


class CountingCompiler(HIPCompiler):
    def compile(self, src):
        self.compiles += 1
        return b"CODE:" + src.encode()


def test_compile_cached_survives_the_process_object(cache_db):
    a = CountingCompiler()
    assert a.compile_cached("k1") == b"CODE:k1" and a.compiles == 1
    assert a.compile_cached("k1") == b"CODE:k1" and a.compiles == 1
    b = CountingCompiler()                                  # stands for a later process: nothing in its dictionary
    assert b.compile_cached("k1") == b"CODE:k1" and b.compiles == 0
    assert b.compile_cached("k2") == b"CODE:k2" and b.compiles == 1
    other = CountingCompiler(cachekey="compile_hip_other")  # another key, another table
    assert other.compile_cached("k1") == b"CODE:k1" and other.compiles == 1


def test_compile_cache_table_follows_architecture_flags_and_compiler():
    """A code object made for another architecture, with other flags or by another compiler must never come back from the
    disk cache: each of the three is part of the table's name."""
    base = HIPCompiler().cachekey
    assert base.startswith("compile_hip_gfx950_")
    assert HIPCompiler(arch="gfx942").cachekey.startswith("compile_hip_gfx942_")

    class OtherFlags(HIPCompiler):
        FLAGS = HIPCompiler.FLAGS + ["-ffast-math"]
    assert OtherFlags().cachekey != base
    assert HIPCompiler(hipcc="/nonexistent/hipcc").cachekey != base      # no version line: another table, not an exception
    assert HIPCompiler().cachekey == base


def test_compile_cache_switches(cache_db, monkeypatch):
    CountingCompiler().compile_cached("k1")
    monkeypatch.setenv("ASSERT_COMPILE", "1")
    assert CountingCompiler().compile_cached("k1") == b"CODE:k1"
    with pytest.raises(RuntimeError, match="ASSERT_COMPILE"):
        CountingCompiler().compile_cached("never seen")
    monkeypatch.delenv("ASSERT_COMPILE")
    monkeypatch.setenv("DISABLE_COMPILER_CACHE", "1")
    c = CountingCompiler()
    assert c.cachekey is None
    c.compile_cached("k1")
    assert c.compiles == 1                                  # the disk copy is not consulted


def test_hipcc_code_object_comes_back_from_disk(cache_db):
    src = 'extern "C" __global__ void E_3(float* data0, const float* data1, const int n) { int i = blockIdx.x*blockDim.x+threadIdx.x; if (i < n) data0[i] = data1[i]*2.0f; }'
    a = HIPCompiler()
    if not os.path.exists(a.hipcc):
        pytest.skip("no hipcc")
    image = a.compile_cached(src)
    assert (image[:4] == b"\x7fELF" or image.startswith(b"__CLANG_OFFLOAD_BUNDLE__")) and a.compiles == 1
    b = HIPCompiler()
    assert b.compile_cached(src) == image and b.compiles == 0
    with pytest.raises(CompileError):
        HIPCompiler().compile_cached("this is not HIP")
