"""The persistent kernel cache behind the C ABI: the cases of the reference's
sarek/framework/test/test_framework_cache.ml (directory, key, put/get, statistics), the
MD5 key pinned by RFC 1321's test suite and by hashlib, and, on a GPU, the compile path
using it."""
import ctypes as C
import hashlib
import os

import numpy as np
import pytest


@pytest.fixture()
def cache(hip, tmp_path, monkeypatch):
    monkeypatch.setenv("XDG_CACHE_HOME", str(tmp_path))
    hip.cache_reset_stats()
    return hip


def test_cache_dir_follows_the_reference_rule(hip, tmp_path, monkeypatch):
    # Framework_cache.get_cache_dir: $XDG_CACHE_HOME, else $HOME/.cache, then "spoc"
    monkeypatch.setenv("XDG_CACHE_HOME", str(tmp_path / "x"))
    os.makedirs(tmp_path / "x")
    d = hip.cache_dir()
    assert d == str(tmp_path / "x" / "spoc") and os.path.isdir(d)
    monkeypatch.delenv("XDG_CACHE_HOME")
    monkeypatch.setenv("HOME", str(tmp_path / "h"))
    os.makedirs(tmp_path / "h")
    d = hip.cache_dir()
    assert d == str(tmp_path / "h" / ".cache" / "spoc") and os.path.isdir(d)


RFC1321 = [
    ("", "d41d8cd98f00b204e9800998ecf8427e"),
    ("a", "0cc175b9c0f1b6a831c399e269772661"),
    ("abc", "900150983cd24fb0d6963f7d28e17f72"),
    ("message digest", "f96b697d7cb7938d525a2f31aaf161d0"),
    ("abcdefghijklmnopqrstuvwxyz", "c3fcd3d76192e4007dfb496cca67e13b"),
    ("ABCDEFGHIJKLMNOPQRSTUVWXYZabcdefghijklmnopqrstuvwxyz0123456789", "d174ab98d277d9f5a5611c2c9f419d9f"),
    ("1234567890" * 8, "57edf4a22be3c955ac49da2e2107b67a"),
]


@pytest.mark.parametrize("text,digest", RFC1321)
def test_key_is_md5_of_the_concatenation(hip, text, digest):
    # compute_key = Digest.to_hex (Digest.string (dev_name ^ driver_version ^ source))
    assert hip.cache_compute_key("", "", text) == digest
    third = len(text) // 3
    assert hip.cache_compute_key(text[:third], text[third:2 * third], text[2 * third:]) == digest


def test_key_matches_hashlib_across_block_boundaries(hip):
    rng = np.random.default_rng(3)
    for n in [55, 56, 57, 63, 64, 65, 119, 120, 128, 1000, 4097]:
        s = "".join(chr(c) for c in rng.integers(32, 127, n))
        assert hip.cache_compute_key("Device1", "1.0", s) == hashlib.md5(("Device11.0" + s).encode()).hexdigest()
    k1 = hip.cache_compute_key("Device1", "1.0", "code1")
    k2 = hip.cache_compute_key("Device1", "1.0", "code2")
    assert len(k1) == 32 and k1 != k2                      # test_compute_key(_different)


def test_put_get_and_persistence(cache):
    cache.cache_put("test_key_12345", b"test binary data\x00\x01\xff")
    assert cache.cache_get("test_key_12345") == b"test binary data\x00\x01\xff"
    assert cache.cache_get("nonexistent_key_67890") is None
    # the entry is a file named by the key under the cache directory
    assert open(os.path.join(cache.cache_dir(), "test_key_12345"), "rb").read().startswith(b"test binary")
    big = bytes(range(256)) * 1024                          # larger than the binding's first buffer
    cache.cache_put("big", big)
    assert cache.cache_get("big") == big
    cache.cache_put("empty", b"")
    assert cache.cache_get("empty") == b""


def test_statistics(cache):
    assert cache.cache_stats() == dict(hits=0, misses=0, puts=0, errors=0)
    cache.cache_put("rate_test", b"data")
    cache.cache_get("rate_test")
    cache.cache_get("rate_test")
    cache.cache_get("nonexistent_rate")
    st = cache.cache_stats()
    assert st == dict(hits=2, misses=1, puts=1, errors=0)   # hit rate 2/3, as in test_hit_rate
    cache.cache_reset_stats()
    assert cache.cache_stats()["hits"] == 0


def test_bad_keys_and_io_errors_are_counted_not_raised(cache, tmp_path):
    cache.cache_put("../escape", b"x")                       # not a plain file name
    assert not os.path.exists(tmp_path / "escape")
    assert cache.cache_get("a/b") is None
    assert cache.cache_stats()["errors"] == 2
    os.chmod(cache.cache_dir(), 0o500)
    try:
        if os.geteuid() != 0:                                # root ignores directory permissions
            cache.cache_put("k", b"v")
            assert cache.cache_stats()["errors"] == 3
    finally:
        os.chmod(cache.cache_dir(), 0o700)


KERNEL = r'''
extern "C" __global__ void scale2(float* x, int n) {
  int i = threadIdx.x + blockIdx.x * blockDim.x;
  if (i < n) x[i] = 2.0f * x[i] + 1.0f;
}
'''


@pytest.mark.gpu
def test_compile_goes_through_the_disk_cache(hip, torch_cuda, tmp_path, monkeypatch):
    torch = torch_cuda
    monkeypatch.setenv("XDG_CACHE_HOME", str(tmp_path))
    hip.check(hip.lib.sarek_hip_kernel_clear_cache())
    hip.cache_reset_stats()
    x = torch.arange(1000, dtype=torch.float32, device="cuda")

    def run():
        hip.run_source(KERNEL, "scale2", (256, 1, 1), (4, 1, 1), [("buf", x), ("i32", 1000)])
        hip.check(hip.lib.sarek_hip_device_synchronize())

    run()                                                    # compiled, stored
    assert hip.cache_stats() == dict(hits=0, misses=1, puts=1, errors=0)
    files = os.listdir(hip.cache_dir())
    assert len(files) == 1 and len(files[0]) == 32
    run()                                                    # in-memory cache: disk untouched
    assert hip.cache_stats() == dict(hits=0, misses=1, puts=1, errors=0)
    hip.check(hip.lib.sarek_hip_kernel_clear_cache())
    run()                                                    # code object read back from disk
    assert hip.cache_stats() == dict(hits=1, misses=1, puts=1, errors=0)
    exp = torch.arange(1000, dtype=torch.float32)
    for _ in range(3):
        exp = 2 * exp + 1
    assert torch.equal(x.cpu(), exp)
    # a damaged entry is counted, recompiled and replaced
    path = os.path.join(hip.cache_dir(), files[0])
    open(path, "wb").write(b"not a code object")
    hip.check(hip.lib.sarek_hip_kernel_clear_cache())
    run()
    st = hip.cache_stats()
    assert st["errors"] == 1 and st["puts"] == 2 and os.path.getsize(path) > 1000
