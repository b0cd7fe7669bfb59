"""GPU parity of infiniopKVCaching (through the C ABI): bit-exact against the CPU oracle."""
import numpy as np
import pytest
import torch

from capi import create_kv_caching, run_kv_caching

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def bits(t):
    t = t.contiguous().cpu()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def normal(rng, shape, dtype):
    return torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).to(dtype)


def strided(t, strides):
    """The same values as ``t`` in storage with the given element strides."""
    span = 1 + sum((n - 1) * s for n, s in zip(t.shape, strides))
    buf = torch.full((span,), 7.0, dtype=t.dtype, device=t.device)
    view = torch.as_strided(buf, t.shape, strides)
    view.copy_(t)
    return view


def check(gpu_handle, oracle, k_cache, v_cache, k, v, past, what):
    print("case", what, tuple(k_cache.shape), tuple(k.shape), k.dtype, k_cache.stride(), flush=True)
    on = lambda t: strided(t.to(DEV), t.stride()) if not t.is_contiguous() else t.to(DEV)  # noqa: E731
    kd, vd = on(k_cache), on(v_cache)
    run_kv_caching(gpu_handle, kd, vd, on(k), on(v), past.to(DEV))
    k_want, v_want = oracle.kv_caching(k_cache.clone(memory_format=torch.preserve_format), v_cache.clone(memory_format=torch.preserve_format), k, v, past)
    assert torch.equal(bits(kd), bits(k_want)), what
    assert torch.equal(bits(vd), bits(v_want)), what


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "shape,strides",
    [
        # test/infiniop/kv_caching.py:35-43
        ((1, 1, 8, 1), None),
        ((1, 8, 32, 32), None),
        ((8, 8, 64, 32), None),
        ((1, 32, 8, 64), (32768, 1024, 64, 1)),
        ((4, 8, 32, 16), (65536, 8192, 256, 16)),
        ((8, 16, 64, 128), (8388608, 524288, 8192, 1)),
        ((1, 2, 2304, 128), (589824, 294912, 128, 1)),
    ],
)
def test_reference_test_shapes(gpu_handle, oracle, dtype, shape, strides):
    rng = np.random.default_rng([*shape, 1])
    B, H, S, D = shape
    n = int(rng.integers(1, S)) if S > 1 else 1
    k_cache, v_cache = normal(rng, shape, dtype), normal(rng, shape, dtype)
    if strides is not None:
        k_cache, v_cache = strided(k_cache, strides), strided(v_cache, strides)
    k, v = normal(rng, (B, H, n, D), dtype), normal(rng, (B, H, n, D), dtype)
    past = torch.from_numpy(rng.integers(0, S - n + 1, B))
    check(gpu_handle, oracle, k_cache, v_cache, k, v, past, f"ref{shape}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_step_one_token_per_sequence(gpu_handle, oracle, dtype):
    """The shape the operator has in a decode loop: one new token for each of 32 sequences."""
    rng = np.random.default_rng(11)
    k_cache, v_cache = normal(rng, (32, 8, 512, 128), dtype), normal(rng, (32, 8, 512, 128), dtype)
    k, v = normal(rng, (32, 8, 1, 128), dtype), normal(rng, (32, 8, 1, 128), dtype)
    past = torch.from_numpy(rng.integers(0, 512, 32))
    check(gpu_handle, oracle, k_cache, v_cache, k, v, past, "decode step")


def test_int32_lengths_and_odd_sizes(gpu_handle, oracle):
    rng = np.random.default_rng(12)
    k_cache, v_cache = normal(rng, (3, 5, 37, 72), torch.float16), normal(rng, (3, 5, 37, 72), torch.float16)
    k, v = normal(rng, (3, 5, 7, 72), torch.float16), normal(rng, (3, 5, 7, 72), torch.float16)
    past = torch.tensor([0, 30, 11], dtype=torch.int32)
    check(gpu_handle, oracle, k_cache, v_cache, k, v, past, "i32")


def test_every_dimension_strided(gpu_handle, oracle):
    """Caches stored [batch, position, head, dim] and viewed [batch, head, position, dim]; new tensors that are
    every other column of wider ones."""
    rng = np.random.default_rng(13)
    B, H, S, D, n = 3, 4, 20, 24, 6
    k_cache = normal(rng, (B, S, H, D), torch.bfloat16).permute(0, 2, 1, 3)
    v_cache = normal(rng, (B, S, H, D), torch.bfloat16).permute(0, 2, 1, 3)
    k = normal(rng, (B, H, n, 2 * D), torch.bfloat16)[..., ::2]
    v = normal(rng, (B, H, n, 2 * D), torch.bfloat16)[..., ::2]
    check(gpu_handle, oracle, k_cache, v_cache, k, v, torch.tensor([0, 14, 7]), "strided")


def test_unaligned_bases_take_narrower_units(gpu_handle, oracle):
    rng = np.random.default_rng(14)
    B, H, S, D, n = 2, 2, 16, 64, 3
    pool = torch.zeros(2 * B * H * S * D + 8, dtype=torch.float16, device=DEV)
    kd = pool[1:1 + B * H * S * D].view(B, H, S, D)              # 2 bytes off a 16-byte boundary
    vd = pool[B * H * S * D + 4:2 * B * H * S * D + 4].view(B, H, S, D)  # 8 bytes off
    k, v = normal(rng, (B, H, n, D), torch.float16), normal(rng, (B, H, n, D), torch.float16)
    past = torch.tensor([5, 13])
    run_kv_caching(gpu_handle, kd, vd, k.to(DEV), v.to(DEV), past.to(DEV))
    want_k, want_v = oracle.kv_caching(torch.zeros(B, H, S, D, dtype=torch.float16), torch.zeros(B, H, S, D, dtype=torch.float16), k, v, past)
    assert torch.equal(bits(kd), bits(want_k)) and torch.equal(bits(vd), bits(want_v))
    assert pool[0] == 0 and pool[-1] == 0


def test_positions_outside_the_cache_are_dropped(gpu_handle):
    """past + s beyond the cache (an out-of-bounds write in the reference) and negative lengths write nothing."""
    rng = np.random.default_rng(15)
    B, H, S, D, n = 3, 2, 8, 16, 4
    k_cache = torch.full((B, H, S, D), 3.0, dtype=torch.float32)
    v_cache = torch.full((B, H, S, D), 4.0, dtype=torch.float32)
    k, v = normal(rng, (B, H, n, D), torch.float32), normal(rng, (B, H, n, D), torch.float32)
    past = torch.tensor([6, -2, 100])
    kd, vd = k_cache.to(DEV), v_cache.to(DEV)
    guard = torch.full((1024,), 9.0, device=DEV)
    run_kv_caching(gpu_handle, kd, vd, k.to(DEV), v.to(DEV), past.to(DEV))
    want_k, want_v = k_cache.clone(), v_cache.clone()
    want_k[0, :, 6:8], want_v[0, :, 6:8] = k[0, :, :2], v[0, :, :2]
    want_k[1, :, 0:2], want_v[1, :, 0:2] = k[1, :, 2:], v[1, :, 2:]
    assert torch.equal(kd.cpu(), want_k) and torch.equal(vd.cpu(), want_v)
    assert bool((guard == 9.0).all())


def test_many_appends_build_the_same_cache_as_one(gpu_handle, oracle):
    """Token by token (the decode loop) equals one append of the whole run."""
    rng = np.random.default_rng(16)
    B, H, S, D, n = 4, 8, 48, 128, 20
    k, v = normal(rng, (B, H, n, D), torch.bfloat16), normal(rng, (B, H, n, D), torch.bfloat16)
    start = torch.tensor([0, 5, 28, 13])
    once_k, once_v = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=DEV), torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=DEV)
    run_kv_caching(gpu_handle, once_k, once_v, k.to(DEV), v.to(DEV), start.to(DEV))
    step_k, step_v = torch.zeros_like(once_k), torch.zeros_like(once_v)
    kd, vd = k.to(DEV), v.to(DEV)
    for t in range(n):
        run_kv_caching(gpu_handle, step_k, step_v, kd[:, :, t:t + 1], vd[:, :, t:t + 1], (start + t).to(DEV))
    assert torch.equal(bits(step_k), bits(once_k)) and torch.equal(bits(step_v), bits(once_v))
    want_k, _ = oracle.kv_caching(torch.zeros(B, H, S, D, dtype=torch.bfloat16), torch.zeros(B, H, S, D, dtype=torch.bfloat16), k, v, start)
    assert torch.equal(bits(once_k), bits(want_k))


def test_python_operator(gpu_handle, oracle):
    from infinicore_amd import ops

    rng = np.random.default_rng(17)
    k_cache, v_cache = normal(rng, (2, 4, 32, 64), torch.float16), normal(rng, (2, 4, 32, 64), torch.float16)
    k, v = normal(rng, (2, 4, 3, 64), torch.float16), normal(rng, (2, 4, 3, 64), torch.float16)
    past = torch.tensor([4, 29])
    kd, vd = ops.kv_caching(k_cache.to(DEV), v_cache.to(DEV), k.to(DEV), v.to(DEV), past.to(DEV))
    torch.cuda.synchronize()
    want_k, want_v = oracle.kv_caching(k_cache.clone(), v_cache.clone(), k, v, past)
    assert torch.equal(bits(kd), bits(want_k)) and torch.equal(bits(vd), bits(want_v))


def test_empty_operands_and_null_pointers(gpu_handle):
    k_cache = torch.zeros(2, 2, 8, 16, dtype=torch.float16, device=DEV)
    empty = torch.zeros(2, 2, 0, 16, dtype=torch.float16, device=DEV)
    past = torch.zeros(2, dtype=torch.int64, device=DEV)
    run_kv_caching(gpu_handle, k_cache, k_cache.clone(), empty, empty, past)  # nothing to do: succeeds
    from ctypes import c_void_p

    from infinicore_amd import libinfiniop as L

    new = torch.zeros(2, 2, 1, 16, dtype=torch.float16, device=DEV)
    status, op = create_kv_caching(gpu_handle, k_cache, k_cache, new, new, past)
    assert status == 0
    assert L.LIBINFINIOP.infiniopKVCaching(op, c_void_p(0), 0, c_void_p(k_cache.data_ptr()), c_void_p(0),
                                           c_void_p(new.data_ptr()), c_void_p(new.data_ptr()), c_void_p(past.data_ptr()),
                                           c_void_p(0)) == L.InfiniStatus.NULL_POINTER
    L.check_error(L.LIBINFINIOP.infiniopDestroyKVCachingDescriptor(op))
