"""The fused rotary-embedding + paged_caching operator on a CPU-only host: create-time validation through the C
ABI (the checks of the reference's RoPE, src/infiniop/ops/rope/rope.h:72-160, and of paged_caching) and pinning of
the oracle function by closed forms, by a torch formulation that shares no code with it, and by its bit-equality
with the (separately pinned) plain scatter when the rotation is the identity."""
import ctypes
import math

import numpy as np
import pytest
import torch

F16, BF16, F32, F64, I64, I32, U8, U64 = 12, 19, 13, 14, 6, 5, 7, 10
OK, NULLP, BAD_DTYPE, BAD_SHAPE, BAD_STRIDES = 0, 4, 10, 11, 12
J, NEOX = 0, 1


def specs(ntok=6, H=4, D=64, Dv=64, bs=16, NB=8, table_len=100, dtype=F16, pos=I64):
    return {
        "k_cache": ((NB, H, bs, D), None, dtype), "v_cache": ((NB, H, bs, Dv), None, dtype),
        "k": ((ntok, H, D), None, dtype), "v": ((ntok, H, Dv), None, dtype),
        "slots": ((ntok,), None, I64), "pos": ((ntok,), None, pos),
        "sin": ((table_len, D // 2), None, dtype), "cos": ((table_len, D // 2), None, dtype),
    }


def mutate(sp, name, shape=None, strides=None, dtype=None):
    out = dict(sp)
    old = sp[name]
    out[name] = (shape or old[0], strides if strides is not None else old[1], dtype or old[2])
    return out


def create(lib, handle, sp, algo=NEOX, drop=None):
    names = ("k_cache", "v_cache", "k", "v", "slots", "pos", "sin", "cos")
    descs = [None if n == drop else lib.create_tensor_descriptor(*sp[n]) for n in names]
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreateRoPEPagedCachingDescriptor(handle, ctypes.byref(op), *descs, algo)
    for d in descs:
        if d is not None:
            lib.destroy_tensor_descriptor(d)
    return status, op


CASES = [
    # rope.h = src/infiniop/ops/rope/rope.h, info.h = src/infiniop/ops/paged_caching/info.h
    ("valid f16", OK, lambda s: s),
    ("valid bf16", OK, lambda s: specs(dtype=BF16)),
    ("valid f32", OK, lambda s: specs(dtype=F32)),
    ("valid i32 positions (rope.h:89)", OK, lambda s: specs(pos=I32)),
    ("valid u8 positions (rope.h:89)", OK, lambda s: specs(pos=U8)),
    ("valid u64 positions (rope.h:89)", OK, lambda s: specs(pos=U64)),
    ("f64 is no pool dtype (info.h:43)", BAD_DTYPE, lambda s: specs(dtype=F64)),
    ("sin of another dtype (rope.h:86)", BAD_DTYPE, lambda s: mutate(s, "sin", dtype=BF16)),
    ("cos of another dtype (rope.h:86)", BAD_DTYPE, lambda s: mutate(s, "cos", dtype=F32)),
    ("positions not integer (rope.h:89)", BAD_DTYPE, lambda s: mutate(s, "pos", dtype=F32)),
    ("slots not i64 (info.h:47)", BAD_DTYPE, lambda s: mutate(s, "slots", dtype=I32)),
    ("positions rank 2 (rope.h:99)", BAD_SHAPE, lambda s: mutate(s, "pos", shape=(6, 1))),
    ("one position too few (rope.h:141)", BAD_SHAPE, lambda s: mutate(s, "pos", shape=(5,))),
    ("sin rank 1 (rope.h:102)", BAD_SHAPE, lambda s: mutate(s, "sin", shape=(3200,))),
    ("tables differ in length (rope.h:143)", BAD_SHAPE, lambda s: mutate(s, "cos", shape=(99, 32))),
    ("tables not half a head wide (rope.h:146)", BAD_SHAPE, lambda s: mutate(mutate(s, "sin", shape=(100, 64)), "cos", shape=(100, 64))),
    ("k rank 2 (info.h:52)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(6, 256))),
    ("k and v differ in tokens (info.h:69)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(5, 4, 64))),
    ("pool head count differs (info.h:77)", BAD_SHAPE, lambda s: mutate(s, "k_cache", shape=(8, 2, 16, 64))),
    ("k last stride 2 (rope.h:152)", BAD_STRIDES, lambda s: mutate(s, "k", strides=(512, 128, 2))),
    ("sin padded rows (rope.h:159)", BAD_STRIDES, lambda s: mutate(s, "sin", strides=(40, 1))),
    ("positions strided", BAD_STRIDES, lambda s: mutate(s, "pos", strides=(2,))),
    # heads of a token must follow one another (the kernel finds head h at h * head_size; rope/cuda/kernel.cuh:29-31
    # would honour a head stride, the scatter of paged_caching/cuda/kernel.cuh:70-78 does not)
    ("k heads padded inside a token", BAD_STRIDES, lambda s: mutate(s, "k", strides=(4 * 80, 80, 1))),
    ("v heads interleaved with another tensor", BAD_STRIDES, lambda s: mutate(s, "v", strides=(4 * 128, 128, 1))),
    ("valid: k and v as column slices of one projection output (token stride only)", OK,
     lambda s: mutate(mutate(s, "k", strides=(3 * 256, 64, 1)), "v", strides=(3 * 256, 64, 1))),
    ("valid: one KV head, any head stride", OK,
     lambda s: mutate(mutate(mutate(mutate(s, "k", shape=(6, 1, 64), strides=(640, 80, 1)), "v", shape=(6, 1, 64)),
                             "k_cache", shape=(8, 1, 16, 64)), "v_cache", shape=(8, 1, 16, 64))),
]


@pytest.mark.parametrize("what,expected,change", CASES, ids=[c[0] for c in CASES])
def test_validation(lib, host_amd_handle, what, expected, change):
    status, op = create(lib, host_amd_handle, change(specs()))
    assert status == expected, what
    if status == OK:
        size = ctypes.c_size_t(7)
        lib.check_error(lib.LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
        assert size.value == 0
        lib.check_error(lib.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))


def test_null_operands_and_unknown_algorithm(lib, host_amd_handle):
    for missing in ("pos", "sin", "cos", "k", "slots"):
        status, _ = create(lib, host_amd_handle, specs(), drop=missing)
        assert status == NULLP, missing
    status, _ = create(lib, host_amd_handle, specs(), algo=2)  # rope.h:80: algo < COUNT, else NULL_POINTER
    assert status == NULLP
    assert lib.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(None) == NULLP


def test_cpu_device_is_not_supported(lib):
    handle = ctypes.pointer(lib.Handle(lib.InfiniDevice.CPU, 0))
    status, _ = create(lib, handle, specs())
    assert status == 5


# ---- the variant that rotates the query in the same launch -----------------------------------------------

def qk_specs(Hq=12, **kw):
    sp = specs(**kw)
    ntok, D, dtype = sp["k"][0][0], sp["k"][0][2], sp["k"][2]
    sp["q"] = ((ntok, Hq, D), None, dtype)
    sp["q_out"] = ((ntok, Hq, D), None, dtype)
    return sp


def create_qk(lib, handle, sp, algo=NEOX, drop=None):
    names = ("q_out", "q", "k_cache", "v_cache", "k", "v", "slots", "pos", "sin", "cos")
    descs = [None if n == drop else lib.create_tensor_descriptor(*sp[n]) for n in names]
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreateRoPEQKPagedCachingDescriptor(handle, ctypes.byref(op), *descs, algo)
    for d in descs:
        if d is not None:
            lib.destroy_tensor_descriptor(d)
    return status, op


QK_CASES = [
    ("valid", OK, lambda s: s),
    ("valid: q a slice of a fused projection (token stride wider than its heads)", OK,
     lambda s: mutate(s, "q", strides=(12 * 64 + 2 * 4 * 64, 64, 1))),
    ("valid: q_out with padded heads", OK, lambda s: mutate(s, "q_out", strides=(12 * 80, 80, 1))),
    ("q of another dtype (rope.h:84)", BAD_DTYPE, lambda s: mutate(s, "q", dtype=BF16)),
    ("q_out of another dtype (rope.h:84)", BAD_DTYPE, lambda s: mutate(s, "q_out", dtype=F32)),
    ("q rank 2 (rope.h:99)", BAD_SHAPE, lambda s: mutate(s, "q", shape=(6, 12 * 64))),
    ("q with another token count", BAD_SHAPE, lambda s: mutate(s, "q", shape=(5, 12, 64))),
    ("q with another head size", BAD_SHAPE, lambda s: mutate(s, "q", shape=(6, 12, 128))),
    ("q_out with another head count (rope.h:109)", BAD_SHAPE, lambda s: mutate(s, "q_out", shape=(6, 8, 64))),
    ("q last stride 2 (rope.h:152)", BAD_STRIDES, lambda s: mutate(s, "q", strides=(12 * 128, 128, 2))),
    ("q_out last stride 2 (rope.h:152)", BAD_STRIDES, lambda s: mutate(s, "q_out", strides=(12 * 128, 128, 2))),
    ("the scatter's checks still apply: slots not i64 (info.h:47)", BAD_DTYPE, lambda s: mutate(s, "slots", dtype=I32)),
    ("the table checks still apply (rope.h:143)", BAD_SHAPE, lambda s: mutate(s, "cos", shape=(99, 32))),
]


@pytest.mark.parametrize("what,expected,change", QK_CASES, ids=[c[0] for c in QK_CASES])
def test_validation_with_query(lib, host_amd_handle, what, expected, change):
    status, op = create_qk(lib, host_amd_handle, change(qk_specs()))
    assert status == expected, what
    if status == OK:
        size = ctypes.c_size_t(7)
        lib.check_error(lib.LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
        assert size.value == 0
        lib.check_error(lib.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))


def test_query_operands_must_be_given_and_each_descriptor_runs_with_its_own_entry_point(lib, host_amd_handle):
    for missing in ("q", "q_out", "k", "pos"):
        status, _ = create_qk(lib, host_amd_handle, qk_specs(), drop=missing)
        assert status == NULLP, missing
    BAD_PARAM = 3
    nil = ctypes.c_void_p(0)
    status, with_q = create_qk(lib, host_amd_handle, qk_specs())
    assert status == OK
    assert lib.LIBINFINIOP.infiniopRoPEPagedCaching(with_q, nil, 0, *([nil] * 8), nil) == BAD_PARAM
    status, without_q = create(lib, host_amd_handle, specs())
    assert status == OK
    assert lib.LIBINFINIOP.infiniopRoPEQKPagedCaching(without_q, nil, 0, *([nil] * 10), nil) == BAD_PARAM
    assert lib.LIBINFINIOP.infiniopRoPEQKPagedCaching(None, nil, 0, *([nil] * 10), nil) == NULLP
    for op in (with_q, without_q):
        lib.check_error(lib.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))


def test_extents_the_kernel_cannot_count_are_refused_before_any_gpu_call(lib, host_amd_handle):
    """Heads, row steps and workgroups are counted in 32 bits: a descriptor beyond that (metadata only, nothing of
    that size exists) is answered BAD_TENSOR_SHAPE at run time, before any device call."""
    sp = qk_specs(Hq=(1 << 31) - 2, ntok=1, H=4, D=2, Dv=2, bs=1, NB=1)
    status, op = create_qk(lib, host_amd_handle, sp)
    assert status == OK
    somewhere = ctypes.c_void_p(4096)  # never dereferenced
    assert lib.LIBINFINIOP.infiniopRoPEQKPagedCaching(op, None, 0, *([somewhere] * 10), None) == BAD_SHAPE
    lib.check_error(lib.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))


# ---- the oracle function ------------------------------------------------------------------------------------

def tables(table_len, D, dtype, theta=10000.0):
    """sin / cos tables as the reference's test builds them (test/infiniop/rope.py:124-131)."""
    freqs = 1.0 / (theta ** (torch.arange(0, D, 2).float() / D))
    angles = torch.outer(torch.arange(table_len).float(), freqs)
    return torch.sin(angles).to(dtype), torch.cos(angles).to(dtype)


def make_case(dtype, ntok=37, H=3, D=64, Dv=64, bs=16, NB=12, table_len=300, seed=0):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((ntok, H, D), generator=g).to(dtype)
    v = torch.randn((ntok, H, Dv), generator=g).to(dtype)
    slots = torch.randperm(NB * bs, generator=g)[:ntok].to(torch.int64)
    slots[::7] = -1
    pos = torch.randint(0, table_len, (ntok,), generator=g)
    sin, cos = tables(table_len, D, dtype)
    k_cache = torch.full((NB, H, bs, D), 7.0, dtype=dtype)
    v_cache = torch.full((NB, H, bs, Dv), -3.0, dtype=dtype)
    return k_cache, v_cache, k, v, slots, pos, sin, cos


@pytest.mark.parametrize("neox", [False, True], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_oracle_equals_torch_rotation_then_numpy_scatter_bit_for_bit(oracle, dtype, neox):
    """Independent statement: the rotation as torch tensor operations in fp32 (separate multiplications and
    additions, one cast), then numpy fancy assignment into the pools."""
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(dtype, seed=3)
    want_k, want_v = k_cache.clone(), v_cache.clone()
    rotated = oracle.torch_reference_rope(k, pos, sin, cos, neox)
    live = slots >= 0
    want_k[slots[live] // 16, :, slots[live] % 16] = rotated[live]
    want_v[slots[live] // 16, :, slots[live] % 16] = v[live]
    oracle.rope_paged_caching(k_cache, v_cache, k, v, slots, pos, sin, cos, neox)
    view = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(k_cache.view(view), want_k.view(view))
    assert torch.equal(v_cache.view(view), want_v.view(view))


@pytest.mark.parametrize("neox", [False, True], ids=["gpt_j", "gpt_neox"])
def test_oracle_with_identity_rotation_is_the_plain_scatter(oracle, neox):
    """sin = 0, cos = 1: the fused function must leave exactly what paged_caching leaves."""
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(torch.bfloat16, seed=5)
    sin, cos = torch.zeros_like(sin), torch.ones_like(cos)
    plain_k, plain_v = k_cache.clone(), v_cache.clone()
    oracle.paged_caching(plain_k, plain_v, k, v, slots)
    oracle.rope_paged_caching(k_cache, v_cache, k, v, slots, pos, sin, cos, neox)
    assert torch.equal(k_cache.view(torch.int16), plain_k.view(torch.int16))
    assert torch.equal(v_cache.view(torch.int16), plain_v.view(torch.int16))


def test_oracle_position_zero_is_the_identity_and_pairs_are_where_the_algorithm_says(oracle):
    """Row 0 of real tables is sin 0 / cos 1. A vector with a single 1 rotates into its pair partner only:
    element a of pair (a, b) at angle t gives (cos t) at a and (sin t) at b."""
    D, H, dtype = 16, 1, torch.float32
    sin, cos = tables(50, D, dtype)
    for neox in (False, True):
        for j in range(D // 2):
            a, b = (j, j + D // 2) if neox else (2 * j, 2 * j + 1)
            k = torch.zeros((2, H, D), dtype=dtype)
            k[:, 0, a] = 1.0
            v = torch.zeros((2, H, D), dtype=dtype)
            k_cache = torch.zeros((1, H, 16, D), dtype=dtype)
            v_cache = torch.zeros_like(k_cache)
            pos = torch.tensor([0, 9])
            oracle.rope_paged_caching(k_cache, v_cache, k, v, torch.tensor([3, 5]), pos, sin, cos, neox)
            assert torch.equal(k_cache[0, 0, 3], k[0, 0])  # position 0: untouched
            want = torch.zeros(D)
            want[a], want[b] = cos[9, j], sin[9, j]
            assert torch.equal(k_cache[0, 0, 5], want), (neox, j)


@pytest.mark.parametrize("neox", [False, True], ids=["gpt_j", "gpt_neox"])
def test_oracle_rotation_preserves_pair_norms_and_the_opposite_angle_undoes_it(oracle, neox):
    """fp32 with exact-enough tables: |(y_a, y_b)| = |(x_a, x_b)| for every pair, and rotating the result by
    the opposite angle (sin negated) returns the input, both to fp32 rounding."""
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(torch.float32, ntok=20, seed=9)
    slots = torch.arange(20)
    oracle.rope_paged_caching(k_cache, v_cache, k, v, slots, pos, sin, cos, neox)
    rotated = k_cache[slots // 16, :, slots % 16]
    half = k.shape[-1] // 2
    pairs = (lambda t: (t[..., :half], t[..., half:])) if neox else (lambda t: (t[..., 0::2], t[..., 1::2]))
    (xa, xb), (ya, yb) = pairs(k), pairs(rotated)
    assert torch.allclose(xa ** 2 + xb ** 2, ya ** 2 + yb ** 2, rtol=1e-5, atol=1e-6)
    back_k, back_v = torch.zeros_like(k_cache), torch.zeros_like(v_cache)
    oracle.rope_paged_caching(back_k, back_v, rotated.contiguous(), v, slots, pos, -sin, cos, neox)
    assert torch.allclose(back_k[slots // 16, :, slots % 16], k, rtol=1e-5, atol=1e-6)


def test_oracle_against_float64_rotation(oracle):
    """Closed form in float64 from the angles themselves (not from the rounded tables' fp32 products)."""
    dtype, D, table_len = torch.float32, 32, 64
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(dtype, ntok=16, H=2, D=D, Dv=D, table_len=table_len, seed=11)
    slots = torch.arange(16)
    oracle.rope_paged_caching(k_cache, v_cache, k, v, slots, pos, sin, cos, True)
    got = k_cache[slots // 16, :, slots % 16].double()
    freqs = 1.0 / (10000.0 ** (torch.arange(0, D, 2).double() / D))
    ang = pos.double()[:, None] * freqs[None]
    x1, x2 = k[..., :D // 2].double(), k[..., D // 2:].double()
    want = torch.cat([x1 * ang.cos()[:, None] - x2 * ang.sin()[:, None], x1 * ang.sin()[:, None] + x2 * ang.cos()[:, None]], dim=-1)
    assert torch.allclose(got, want, rtol=0, atol=3e-5)  # fp32 tables of angles up to 63 rad: ~1e-6 * |x| each


def test_oracle_clamps_positions_and_skips_padding(oracle):
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(torch.float16, ntok=8, table_len=10, seed=13)
    slots = torch.tensor([0, 1, -1, 3, 4, -5, 6, 7])
    far = torch.tensor([0, 9, 3, 12, -4, 2, 10 ** 12, 5])
    near = far.clamp(0, 9)
    a_k, a_v, b_k, b_v = k_cache.clone(), v_cache.clone(), k_cache.clone(), v_cache.clone()
    oracle.rope_paged_caching(a_k, a_v, k, v, slots, far, sin, cos, False)
    oracle.rope_paged_caching(b_k, b_v, k, v, slots, near, sin, cos, False)
    assert torch.equal(a_k.view(torch.int16), b_k.view(torch.int16))
    assert torch.all(a_k[0, :, 2] == 7) and torch.all(a_k[0, :, 5] == 7)  # padding tokens left their slots alone


# ---- the rotation on its own (what the fused operator applies to the query) -------------------------------

@pytest.mark.parametrize("neox", [False, True], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_rope_oracle_equals_the_torch_rotation_bit_for_bit(oracle, dtype, neox):
    g = torch.Generator().manual_seed(21)
    x = torch.randn((19, 5, 64), generator=g).to(dtype)
    pos = torch.randint(0, 200, (19,), generator=g)
    sin, cos = tables(200, 64, dtype)
    got = oracle.rope(x, pos, sin, cos, neox)
    want = oracle.torch_reference_rope(x, pos, sin, cos, neox)
    view = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(got.view(view), want.view(view))


@pytest.mark.parametrize("neox", [False, True], ids=["gpt_j", "gpt_neox"])
def test_rope_oracle_strided_in_place_and_consistent_with_the_fused_function(oracle, neox):
    """q as a slice of a fused projection output, rotated in place; and rotating k with this function and then
    scattering it with the (separately pinned) plain scatter leaves exactly what the fused function leaves."""
    k_cache, v_cache, k, v, slots, pos, sin, cos = make_case(torch.bfloat16, seed=23)
    ntok, H, D = k.shape
    fused = torch.randn((ntok, 7 * D + 2 * H * D)).to(torch.bfloat16)
    q = fused[:, :7 * D].view(ntok, 7, D)
    assert not q.is_contiguous()
    want = oracle.torch_reference_rope(q.clone(), pos, sin, cos, neox)
    untouched = fused[:, 7 * D:].clone()
    oracle.rope(q, pos, sin, cos, neox, out=q)
    assert torch.equal(q.contiguous().view(torch.int16), want.view(torch.int16))
    assert torch.equal(fused[:, 7 * D:], untouched)
    two_k, two_v = k_cache.clone(), v_cache.clone()
    oracle.paged_caching(two_k, two_v, oracle.rope(k, pos, sin, cos, neox), v, slots)
    oracle.rope_paged_caching(k_cache, v_cache, k, v, slots, pos, sin, cos, neox)
    assert torch.equal(k_cache.view(torch.int16), two_k.view(torch.int16))
    assert torch.equal(v_cache.view(torch.int16), two_v.view(torch.int16))


def test_rope_oracle_clamps_positions(oracle):
    g = torch.Generator().manual_seed(25)
    x = torch.randn((6, 2, 32), generator=g).to(torch.float16)
    sin, cos = tables(10, 32, torch.float16)
    far = torch.tensor([0, 9, 12, -4, 10 ** 12, 5])
    assert torch.equal(oracle.rope(x, far, sin, cos, True).view(torch.int16),
                       oracle.rope(x, far.clamp(0, 9), sin, cos, True).view(torch.int16))
