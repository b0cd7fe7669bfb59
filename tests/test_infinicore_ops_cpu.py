"""The framework-side adaptor library without a GPU: its LRU cache (compiled as a host program), its exports,
and what it answers on the CPU device (where InfiniOP has no paged operators, as in the reference)."""
import ctypes
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CACHE_HEADER_DIR = ROOT / "infinicore_amd" / "csrc" / "infinicore"

LRU_PROGRAM = r"""
#include "lru_cache.h"
#include <cstdio>
#include <memory>
using namespace infinicore_amd;
static int alive = 0;
struct Counted { Counted() { ++alive; } ~Counted() { --alive; } };
int main() {
    // capacity, refresh on get, eviction from the least recently used end
    LruCache<int, int> c(2);
    c.put(1, 10); c.put(2, 20);
    std::printf("get1=%d\n", c.get(1).value_or(-1));          // refreshes 1: 2 is now the oldest
    c.put(3, 30);                                               // evicts 2
    std::printf("has1=%d has2=%d has3=%d size=%zu\n", c.contains(1), c.contains(2), c.contains(3), c.size());
    const bool found2 = c.get(2).has_value();
    std::printf("miss2=%d hits=%llu misses=%llu\n", found2, (unsigned long long)c.hits(), (unsigned long long)c.misses());
    c.put(1, 11);                                               // overwrite keeps the size, refreshes 1
    c.put(4, 40);                                               // evicts 3
    std::printf("v1=%d has3=%d has4=%d size=%zu\n", c.get(1).value_or(-1), c.contains(3), c.contains(4), c.size());
    c.setCapacity(1);                                           // keeps the most recent one: 1
    std::printf("after_shrink has1=%d has4=%d size=%zu\n", c.contains(1), c.contains(4), c.size());
    c.setCapacity(0);                                           // unbounded
    for (int i = 100; i < 400; ++i) c.put(i, i);
    std::printf("unbounded size=%zu\n", c.size());
    c.clear();
    std::printf("cleared size=%zu\n", c.size());
    // values are released on eviction, on overwrite and on clear, but live on in other owners
    {
        LruCache<int, std::shared_ptr<Counted>> s(2);
        auto held = std::make_shared<Counted>();
        s.put(1, held); s.put(2, std::make_shared<Counted>()); s.put(3, std::make_shared<Counted>());
        std::printf("alive_after_evicting_held=%d\n", alive);  // 1 evicted from the cache but still held: 3
        held.reset();
        std::printf("alive_after_release=%d\n", alive);        // 2
        s.put(3, std::make_shared<Counted>());
        std::printf("alive_after_overwrite=%d\n", alive);      // 2
        s.clear();
        std::printf("alive_after_clear=%d\n", alive);          // 0
    }
    // keys: metadata words compared in full; NULL strides and spelled-out contiguous strides are one key
    size_t shape[3] = {4, 32, 128};
    ptrdiff_t contiguous[3] = {4096, 128, 1}, padded[3] = {8192, 128, 1};
    MetaKey a, b, d, e;
    a.addTensor(19, 3, shape, nullptr); b.addTensor(19, 3, shape, contiguous); d.addTensor(19, 3, shape, padded);
    e.addTensor(12, 3, shape, nullptr);
    std::printf("same=%d padded_differs=%d dtype_differs=%d hash_same=%d\n", a == b, !(a == d), !(a == e), a.hash() == b.hash());
    // two argument lists whose ranks differ must not spell the same words: (rank 3 [4, 32, 128]) + (rank 1 [7])
    // against (rank 2 [4, 32]) + (rank 2 ...) built so that the concatenated extents and strides coincide
    {
        size_t s3[3] = {2, 3, 1}, s1[1] = {1};
        size_t s2a[2] = {2, 3}, s2b[2] = {1, 1};
        ptrdiff_t t3[3] = {3, 1, 1}, t1[1] = {1};
        ptrdiff_t t2a[2] = {3, 1}, t2b[2] = {1, 1};
        MetaKey x, y;
        x.addTensor(19, 3, s3, t3); x.addTensor(19, 1, s1, t1);
        y.addTensor(19, 2, s2a, t2a); y.addTensor(19, 2, s2b, t2b);
        std::printf("ranks_differ=%d\n", !(x == y));
    }
    // the reference's fold: seed ^= hash(v) + 0x9e3779b9 + (seed << 6) + (seed >> 2), starting from 0
    MetaKey k; k.add(7); k.add(9);
    size_t seed = 0;
    for (long long v : {7LL, 9LL}) seed ^= std::hash<int64_t>{}(v) + 0x9e3779b9 + (seed << 6) + (seed >> 2);
    std::printf("fold=%d\n", k.hash() == seed);
    return 0;
}
"""


def test_lru_cache_and_metadata_key(tmp_path):
    src, exe = tmp_path / "lru.cc", tmp_path / "lru"
    src.write_text(LRU_PROGRAM)
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", str(CACHE_HEADER_DIR), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()
    assert out == [
        "get1=10",
        "has1=1 has2=0 has3=1 size=2",
        "miss2=0 hits=1 misses=1",
        "v1=11 has3=0 has4=1 size=2",
        "after_shrink has1=1 has4=0 size=1",
        "unbounded size=301",
        "cleared size=0",
        "alive_after_evicting_held=3",
        "alive_after_release=2",
        "alive_after_overwrite=2",
        "alive_after_clear=0",
        "same=1 padded_differs=1 dtype_differs=1 hash_same=1",
        "ranks_differ=1",
        "fold=1",
    ]


@pytest.fixture(scope="module")
def core(lib):
    from infinicore_amd import libinfinicore_ops

    return libinfinicore_ops


def host_view(core, lib, shape, dtype):
    n = len(shape)
    arr = (ctypes.c_size_t * n)(*shape)
    v = core.TensorView(None, dtype, n, ctypes.cast(arr, ctypes.POINTER(ctypes.c_size_t)), None)
    v._keep = arr
    return v


def test_on_the_cpu_device_the_operators_are_not_supported_and_nothing_is_cached(core, lib):
    L = core.LIBINFINICORE_OPS
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    core.cache_clear()
    q = host_view(core, lib, (2, 8, 128), lib.InfiniDtype.F16)
    kc = host_view(core, lib, (4, 8, 16, 128), lib.InfiniDtype.F16)
    bt = host_view(core, lib, (2, 2), lib.InfiniDtype.I64)
    sl = host_view(core, lib, (2,), lib.InfiniDtype.I64)
    plan = ctypes.c_void_p(0xDEAD)
    r = ctypes.byref
    status = L.infinicoreOpPlanPagedAttention(r(plan), r(q), r(q), r(kc), r(kc), r(bt), r(sl), None, 0.5)
    assert status == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED and not plan.value  # reset to NULL on failure
    assert L.infinicoreOpPagedAttention(r(q), r(q), r(kc), r(kc), r(bt), r(sl), None, 0.5, None) == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    assert L.infinicoreOpPlanPagedCaching(r(plan), r(kc), r(kc), r(q), r(q), r(sl)) == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    assert L.infinicoreOpPlanKVCaching(r(plan), r(kc), r(kc), r(kc), r(kc), r(sl)) == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    assert L.infinicoreOpPlanPagedAttentionPrefill(r(plan), r(q), r(q), r(kc), r(kc), r(bt), r(sl), r(sl), None, 0.5) == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    entries, hits, misses = core.cache_stats(core.OpKind.PAGED_ATTENTION)
    assert (entries, hits, misses) == (0, 0, 2)  # two look-ups, nothing stored for a descriptor that was refused
    core.cache_clear()


def test_null_arguments(core, lib):
    L = core.LIBINFINICORE_OPS
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    q = host_view(core, lib, (2, 8, 128), lib.InfiniDtype.F16)
    r = ctypes.byref
    plan = ctypes.c_void_p()
    NULL = lib.InfiniStatus.NULL_POINTER
    assert L.infinicoreOpPlanPagedAttention(None, r(q), r(q), r(q), r(q), r(q), r(q), None, 1.0) == NULL
    assert L.infinicoreOpPlanPagedAttention(r(plan), None, r(q), r(q), r(q), r(q), r(q), None, 1.0) == NULL
    assert L.infinicoreOpPlanPagedCaching(r(plan), r(q), r(q), r(q), r(q), None) == NULL
    no_shape = core.TensorView(None, lib.InfiniDtype.F16, 3, None, None)
    assert L.infinicoreOpPagedAttention(r(no_shape), r(q), r(q), r(q), r(q), r(q), None, 1.0, None) == NULL
    assert L.infinicoreOpRun(None, None) == NULL
    assert L.infinicoreOpCleanup(None) == NULL and L.infinicoreOpCleanup(r(plan)) == NULL
    assert L.infinicoreOpPlannedWorkspaceSize(None, None) == NULL
    assert L.infinicoreOpCacheStats(99, None, None, None) == lib.InfiniStatus.BAD_PARAM
    assert L.infinicoreOpCacheSetCapacity(100) == 0
