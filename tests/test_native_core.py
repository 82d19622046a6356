"""The native cache core (tempura_amd/csrc/host/cache_core.cpp) under the address and undefined-behaviour
sanitizers: a C++ driver (tests/native/cache_core_driver.cpp) runs random orders of requests against it and
checks the core's invariants after every operation.  Host code only; no GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("clang++")
    if not cxx:
        pytest.skip("no C++ compiler")
    exe = str(tmp_path_factory.mktemp("native") / "cache_core_driver")
    cmd = [cxx, "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           os.path.join(ROOT, "tests", "native", "cache_core_driver.cpp"),
           os.path.join(ROOT, "tempura_amd", "csrc", "host", "cache_core.cpp"), "-o", exe]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0 and "sanitize" in p.stderr:
        pytest.skip("the compiler has no sanitizer runtime here")
    assert p.returncode == 0, p.stderr[-2000:]
    return exe


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_orders_under_sanitizers(driver, seed):
    # (the harness may preload a library of its own; ASan wants to come first in the list)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    p = subprocess.run([driver, str(seed)], capture_output=True, text=True, timeout=120, env=env)
    assert p.returncode == 0, (p.stdout + p.stderr)[-2000:]
    assert p.stdout.startswith("ok seed")


def test_truncate_refused_where_a_window_gave_pages_back():
    from tempura_amd.cache import CacheManager
    from tempura_amd.parts import CacheSpec
    m = CacheManager([CacheSpec("full", 2, 16), CacheSpec("window", 2, 16, window=24)], page_size=8, num_pages=[32, 8],
                     max_requests=1)
    m.add("a")
    for _ in range(10):
        m.reserve("a", 10)
        m.commit("a", 10)
    free = m.free_pages()
    with pytest.raises(ValueError):
        m.truncate("a", 60)            # the window group no longer holds positions 37..59
    assert m.free_pages() == free and m.num_tokens("a") == 100
    m.truncate("a", 98)                # still inside what the window holds
    assert m.num_tokens("a") == 98
    m.check()
