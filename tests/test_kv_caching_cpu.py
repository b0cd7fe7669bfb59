"""kv_caching on a CPU-only host: create-time validation through the C ABI (one case per status-returning
check of the reference's src/infiniop/ops/kv_caching/info.h) and pinning of the oracle's append function
against numpy assignment, the closed form of the operator."""
import ctypes

import numpy as np
import pytest
import torch

F16, BF16, F32, I64, I32, U32, F64 = 12, 19, 13, 6, 5, 9, 14
OK, NULLP, BAD_DTYPE, BAD_SHAPE = 0, 4, 10, 11


def specs(B=4, H=8, S=64, s=5, D=32, dtype=F16, past=I64):
    cache, new = ((B, H, S, D), None, dtype), ((B, H, s, D), None, dtype)
    return {"k_cache": cache, "v_cache": cache, "k": new, "v": new, "past": ((B,), None, past)}


def mutate(sp, name, shape=None, strides=None, dtype=None):
    out = dict(sp)
    old = sp[name]
    out[name] = (shape or old[0], strides if strides is not None else old[1], dtype or old[2])
    return out


def create(lib, handle, sp):
    descs = [lib.create_tensor_descriptor(*sp[n]) for n in ("k_cache", "v_cache", "k", "v", "past")]
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreateKVCachingDescriptor(handle, ctypes.byref(op), *descs)
    for d in descs:
        lib.destroy_tensor_descriptor(d)
    return status, op


CASES = [
    # line numbers are src/infiniop/ops/kv_caching/info.h
    ("valid f16 / i64", OK, lambda s: s),
    ("valid bf16 (:37)", OK, lambda s: specs(dtype=BF16)),
    ("valid f32 (:37)", OK, lambda s: specs(dtype=F32)),
    ("valid i32 lengths (:39)", OK, lambda s: specs(past=I32)),
    ("valid strided caches (test/infiniop/kv_caching.py:39)", OK,
     lambda s: mutate(mutate(specs(B=1, H=32, S=8, s=3, D=64), "k_cache", strides=(32768, 1024, 64, 1)), "v_cache", strides=(32768, 1024, 64, 1))),
    ("cache dtype f64 (:37)", BAD_DTYPE, lambda s: specs(dtype=F64)),
    ("lengths dtype u32 (:39)", BAD_DTYPE, lambda s: specs(past=U32)),
    ("new keys of another dtype", BAD_DTYPE, lambda s: mutate(s, "k", dtype=BF16)),
    ("value cache of another dtype", BAD_DTYPE, lambda s: mutate(s, "v_cache", dtype=F32)),
    ("cache rank 3 (:41)", BAD_SHAPE, lambda s: mutate(mutate(s, "k_cache", shape=(4, 8, 2048)), "v_cache", shape=(4, 8, 2048))),
    ("new keys rank 3 (:41)", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(4, 8, 160)), "v", shape=(4, 8, 160))),
    ("caches differ in shape (:48)", BAD_SHAPE, lambda s: mutate(s, "v_cache", shape=(4, 8, 32, 32))),
    ("new keys and values differ in shape (:49)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(4, 8, 4, 32))),
    ("batch differs between caches and new tensors", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(2, 8, 5, 32)), "v", shape=(2, 8, 5, 32))),
    ("heads differ between caches and new tensors", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(4, 4, 5, 32)), "v", shape=(4, 4, 5, 32))),
    ("head size differs between caches and new tensors", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(4, 8, 5, 16)), "v", shape=(4, 8, 5, 16))),
    ("lengths rank 2", BAD_SHAPE, lambda s: mutate(s, "past", shape=(4, 1))),
    ("one length too few", BAD_SHAPE, lambda s: mutate(s, "past", shape=(3,))),
    ("lengths strided", BAD_SHAPE, lambda s: mutate(s, "past", strides=(2,))),
]


@pytest.mark.parametrize("what,expected,change", CASES, ids=[c[0] for c in CASES])
def test_kv_caching_validation(lib, host_amd_handle, what, expected, change):
    status, op = create(lib, host_amd_handle, change(specs()))
    assert status == expected, what
    if status == OK:
        size = ctypes.c_size_t(99)
        assert lib.LIBINFINIOP.infiniopGetKVCachingWorkspaceSize(op, ctypes.byref(size)) == OK
        assert size.value == 0
        assert lib.LIBINFINIOP.infiniopDestroyKVCachingDescriptor(op) == OK


def test_kv_caching_null_arguments(lib, host_amd_handle):
    sp = specs()
    t = lib.create_tensor_descriptor(*sp["k_cache"])
    op = lib.infiniopOperatorDescriptor_t()
    null = lib.infiniopTensorDescriptor_t()
    assert lib.LIBINFINIOP.infiniopCreateKVCachingDescriptor(host_amd_handle, ctypes.byref(op), t, t, t, t, null) == NULLP
    assert lib.LIBINFINIOP.infiniopCreateKVCachingDescriptor(None, ctypes.byref(op), t, t, t, t, t) == NULLP
    assert lib.LIBINFINIOP.infiniopGetKVCachingWorkspaceSize(None, ctypes.byref(ctypes.c_size_t())) == NULLP
    assert lib.LIBINFINIOP.infiniopDestroyKVCachingDescriptor(None) == NULLP
    lib.destroy_tensor_descriptor(t)


def test_kv_caching_rejects_a_cpu_handle(lib):
    handle = ctypes.pointer(lib.Handle(lib.InfiniDevice.CPU, 0))
    status, _ = create(lib, handle, specs())
    assert status == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED  # as the reference's switch (operator.cc:33-57)


# ---- the oracle against numpy assignment -------------------------------------------------------------

def numpy_model(k_cache, v_cache, k, v, past):
    kc, vc = k_cache.copy(), v_cache.copy()
    n = k.shape[2]
    for b in range(k.shape[0]):
        kc[b, :, past[b]:past[b] + n, :] = k[b]
        vc[b, :, past[b]:past[b] + n, :] = v[b]
    return kc, vc


@pytest.mark.parametrize("np_dtype,torch_view", [(np.uint16, torch.int16), (np.uint32, torch.int32)])
@pytest.mark.parametrize("B,H,S,D", [(1, 1, 8, 1), (1, 8, 32, 32), (8, 8, 64, 32), (4, 8, 32, 16)])  # test/infiniop/kv_caching.py:35-43
def test_oracle_kv_caching_is_numpy_assignment(oracle, np_dtype, torch_view, B, H, S, D):
    """Random bit patterns (NaN payloads included, so a conversion anywhere would show), every byte of the
    caches compared, positions nobody writes keep their sentinel."""
    rng = np.random.default_rng([B, H, S, D])
    n = int(rng.integers(1, S)) if S > 1 else 1
    info = np.iinfo(np_dtype)
    k_cache = rng.integers(0, info.max, (B, H, S, D), dtype=np_dtype)
    v_cache = rng.integers(0, info.max, (B, H, S, D), dtype=np_dtype)
    k = rng.integers(0, info.max, (B, H, n, D), dtype=np_dtype)
    v = rng.integers(0, info.max, (B, H, n, D), dtype=np_dtype)
    past = rng.integers(0, S - n + 1, B)
    want_k, want_v = numpy_model(k_cache, v_cache, k, v, past)
    signed = np.int16 if np_dtype == np.uint16 else np.int32
    tk, tv = (torch.from_numpy(x.view(signed).copy()) for x in (k_cache, v_cache))
    got_k, got_v = oracle.kv_caching(tk, tv, torch.from_numpy(k.view(signed).copy()), torch.from_numpy(v.view(signed).copy()),
                                     torch.from_numpy(past))
    assert np.array_equal(got_k.numpy().view(np_dtype), want_k)
    assert np.array_equal(got_v.numpy().view(np_dtype), want_v)


def test_oracle_kv_caching_strided_operands(oracle):
    """Every dimension strided: caches that are slices of wider pools with the head and position dims
    swapped in storage, new tensors with a strided innermost dimension."""
    rng = np.random.default_rng(5)
    B, H, S, D, n = 3, 4, 20, 8, 6
    k_pool = torch.from_numpy(rng.standard_normal((B, S + 3, H, D + 2), dtype=np.float32))
    v_pool = torch.from_numpy(rng.standard_normal((B, S + 3, H, D + 2), dtype=np.float32))
    k_cache = k_pool[:, :S, :, :D].permute(0, 2, 1, 3)
    v_cache = v_pool[:, :S, :, :D].permute(0, 2, 1, 3)
    k = torch.from_numpy(rng.standard_normal((B, H, n, 2 * D), dtype=np.float32))[..., ::2]
    v = torch.from_numpy(rng.standard_normal((B, H, n, 2 * D), dtype=np.float32))[..., ::2]
    past = torch.tensor([0, 14, 7])
    want_k, want_v = numpy_model(k_cache.numpy(), v_cache.numpy(), k.numpy(), v.numpy(), past.numpy())
    pool_before = k_pool.clone()
    oracle.kv_caching(k_cache, v_cache, k, v, past)
    assert np.array_equal(k_cache.numpy(), want_k) and np.array_equal(v_cache.numpy(), want_v)
    assert torch.equal(k_pool[:, S:], pool_before[:, S:]) and torch.equal(k_pool[..., D:], pool_before[..., D:])


def test_oracle_kv_caching_matches_the_reference_tests_torch_function(oracle):
    rng = np.random.default_rng(6)
    k_cache = torch.from_numpy(rng.standard_normal((8, 16, 64, 128), dtype=np.float32)).to(torch.bfloat16)
    v_cache = torch.from_numpy(rng.standard_normal((8, 16, 64, 128), dtype=np.float32)).to(torch.bfloat16)
    k = torch.from_numpy(rng.standard_normal((8, 16, 9, 128), dtype=np.float32)).to(torch.bfloat16)
    v = torch.from_numpy(rng.standard_normal((8, 16, 9, 128), dtype=np.float32)).to(torch.bfloat16)
    past = torch.from_numpy(rng.integers(0, 64 - 9, 8))
    want_k, want_v = oracle.torch_reference_kv_caching(k_cache.clone(), v_cache.clone(), k, v, past)
    got_k, got_v = oracle.kv_caching(k_cache.clone(), v_cache.clone(), k, v, past)
    assert torch.equal(got_k.view(torch.int16), want_k.view(torch.int16))
    assert torch.equal(got_v.view(torch.int16), want_v.view(torch.int16))


def test_oracle_kv_caching_reports_positions_outside_the_cache(oracle):
    k_cache, v_cache = torch.zeros(2, 1, 4, 2), torch.zeros(2, 1, 4, 2)
    k, v = torch.ones(2, 1, 2, 2), torch.ones(2, 1, 2, 2)
    with pytest.raises(ValueError):
        oracle.kv_caching(k_cache, v_cache, k, v, torch.tensor([0, 3]))
