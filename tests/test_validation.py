"""Create-time validation of both operators: one case per status-returning check of the reference's
info.h files, run through the C ABI with a host-only AMD handle (descriptor creation is pure host
code, so none of this needs a GPU)."""
import ctypes

import pytest

F16, BF16, F32, I64, I32, U32, U8 = 12, 19, 13, 6, 5, 9, 7
OK, NULLP, BAD_DTYPE, BAD_SHAPE, BAD_STRIDES, NO_WS = 0, 4, 10, 11, 12, 13


class Spec:
    """shape / strides (None = packed) / dtype of one operand."""

    def __init__(self, shape, dtype, strides=None):
        self.shape, self.dtype, self.strides = tuple(shape), dtype, strides


def attention_specs(B=4, H=8, Hkv=8, D=128, Dv=None, bs=16, NB=64, maxb=16, dtype=F16, idx=I64):
    Dv = Dv or D
    return {
        "out": Spec((B, H, Dv), dtype), "q": Spec((B, H, D), dtype),
        "k": Spec((NB, Hkv, bs, D), dtype), "v": Spec((NB, Hkv, bs, Dv), dtype),
        "bt": Spec((B, maxb), idx), "lens": Spec((B,), idx), "alibi": None,
    }


def create_attention(lib, handle, specs, scale=0.0884):
    order = ["out", "q", "k", "v", "bt", "lens"]
    descs = [lib.create_tensor_descriptor(specs[n].shape, specs[n].strides, specs[n].dtype) for n in order]
    alibi = specs.get("alibi")
    alibi_desc = lib.create_tensor_descriptor(alibi.shape, alibi.strides, alibi.dtype) if alibi else None
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreatePagedAttentionDescriptor(handle, ctypes.byref(op), *descs, alibi_desc, scale)
    for d in descs:
        lib.destroy_tensor_descriptor(d)
    if alibi_desc:
        lib.destroy_tensor_descriptor(alibi_desc)
    return status, op


def mutate(specs, name, **kw):
    s = specs[name]
    specs[name] = Spec(kw.get("shape", s.shape), kw.get("dtype", s.dtype), kw.get("strides", s.strides))
    return specs


ATTENTION_CASES = [
    # (what, expected status, mutation) - line numbers are src/infiniop/ops/paged_attention/info.h
    ("valid", OK, lambda s: s),
    ("q dtype f32 (:52)", BAD_DTYPE, lambda s: mutate(s, "q", dtype=F32)),
    ("out dtype differs (:53)", BAD_DTYPE, lambda s: mutate(s, "out", dtype=BF16)),
    ("k dtype differs (:53)", BAD_DTYPE, lambda s: mutate(s, "k", dtype=BF16)),
    ("v dtype differs (:53)", BAD_DTYPE, lambda s: mutate(s, "v", dtype=BF16)),
    ("q rank 2 (:57)", BAD_SHAPE, lambda s: mutate(s, "q", shape=(4, 1024))),
    ("out rank 4 (:57)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(4, 8, 1, 128))),
    ("k rank 3 (:60)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(64, 8, 2048))),
    ("v rank 5 (:60)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(64, 8, 16, 128, 1))),
    ("table rank 1 (:63)", BAD_SHAPE, lambda s: mutate(s, "bt", shape=(64,))),
    ("lens rank 2 (:63)", BAD_SHAPE, lambda s: mutate(s, "lens", shape=(4, 1))),
    ("q last stride 2 (:67)", BAD_STRIDES, lambda s: mutate(s, "q", strides=(2048, 256, 2))),
    ("out last stride 2 (:68)", BAD_STRIDES, lambda s: mutate(s, "out", strides=(2048, 256, 2))),
    ("k last stride 2 (:69)", BAD_STRIDES, lambda s: mutate(s, "k", strides=(32768, 4096, 256, 2))),
    ("v last stride 2 (:70)", BAD_STRIDES, lambda s: mutate(s, "v", strides=(32768, 4096, 256, 2))),
    ("table dtype f32 (:76)", BAD_DTYPE, lambda s: mutate(s, "bt", dtype=F32)),
    ("lens dtype u8 (:77)", BAD_DTYPE, lambda s: mutate(s, "lens", dtype=U8)),
    ("index dtypes differ (:86)", BAD_DTYPE, lambda s: mutate(s, "lens", dtype=I32)),
    ("table inner stride 2 (:95)", BAD_STRIDES, lambda s: mutate(s, "bt", strides=(32, 2))),
    ("lens stride 2 (:96)", BAD_STRIDES, lambda s: mutate(s, "lens", strides=(2,))),
    ("alibi dtype f16 (:99)", BAD_DTYPE, lambda s: {**s, "alibi": Spec((8,), F16)}),
    ("alibi rank 2 (:102)", BAD_SHAPE, lambda s: {**s, "alibi": Spec((8, 1), F32)}),
    ("alibi stride 2 (:105)", BAD_STRIDES, lambda s: {**s, "alibi": Spec((8,), F32, (2,))}),
    ("alibi valid", OK, lambda s: {**s, "alibi": Spec((8,), F32)}),
    ("heads not a multiple of kv heads (:131)", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(64, 3, 16, 128)), "v", shape=(64, 3, 16, 128))),
    ("k head size differs (:135)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(64, 8, 16, 64))),
    ("v pool size differs (:138)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(32, 8, 16, 128))),
    ("v page size differs (:138)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(64, 8, 32, 128))),
    ("value size differs, not MLA (:141)", BAD_SHAPE, lambda s: mutate(mutate(s, "v", shape=(64, 8, 16, 64)), "out", shape=(4, 8, 64))),
    ("out shape differs (:145)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(4, 8, 64))),
    ("out batch differs (:145)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(5, 8, 128))),
    ("lens length differs (:149)", BAD_SHAPE, lambda s: mutate(s, "lens", shape=(5,))),
    ("table has fewer rows than sequences (stricter than the reference)", BAD_SHAPE, lambda s: mutate(s, "bt", shape=(3, 16))),
    ("alibi shorter than heads (stricter than the reference)", BAD_SHAPE, lambda s: {**s, "alibi": Spec((4,), F32)}),
]


@pytest.mark.parametrize("what,expected,change", ATTENTION_CASES, ids=[c[0] for c in ATTENTION_CASES])
def test_paged_attention_validation(lib, host_amd_handle, what, expected, change):
    status, op = create_attention(lib, host_amd_handle, change(attention_specs()))
    assert status == expected, what
    if status == OK:
        assert lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op) == OK


@pytest.mark.parametrize("head_size,ok", [(64, True), (128, True), (192, True), (256, True), (576, True), (32, False), (96, False), (512, False)])
def test_paged_attention_head_sizes(lib, host_amd_handle, head_size, ok):
    status, op = create_attention(lib, host_amd_handle, attention_specs(D=head_size))  # info.h:127
    assert status == (OK if ok else BAD_SHAPE)
    if ok:
        lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op)


def test_paged_attention_mla_value_size(lib, host_amd_handle):
    status, op = create_attention(lib, host_amd_handle, attention_specs(H=16, Hkv=1, D=576, Dv=512))  # info.h:116,141
    assert status == OK
    lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op)


@pytest.mark.parametrize("idx", [I64, I32, U32])
def test_paged_attention_index_dtypes(lib, host_amd_handle, idx):
    status, op = create_attention(lib, host_amd_handle, attention_specs(idx=idx))
    assert status == OK
    lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op)


def test_paged_attention_descriptor_owns_its_metadata_and_reports_device(lib, host_amd_handle):
    status, op = create_attention(lib, host_amd_handle, attention_specs(B=32, H=32, Hkv=8, maxb=256))
    assert status == OK  # tensor descriptors are already destroyed at this point
    assert op.contents.device_type == lib.InfiniDevice.AMD and op.contents.device_id == 0
    dev, idx = ctypes.c_int(-1), ctypes.c_int(-1)
    assert lib.LIBINFINIOP.infiniopGetDescriptorDeviceType(op, ctypes.byref(dev)) == OK and dev.value == lib.InfiniDevice.AMD
    assert lib.LIBINFINIOP.infiniopGetDescriptorDeviceId(op, ctypes.byref(idx)) == OK and idx.value == 0
    size = ctypes.c_size_t(0)
    assert lib.LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, ctypes.byref(size)) == OK
    assert 0 < size.value < (1 << 30)  # long sequences need room for partial results, bounded
    assert lib.LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, None) == NULLP
    # running with a short or missing workspace is refused before anything is launched
    # (reference: nvidia/paged_attention_nvidia.cu:216-226)
    args = [ctypes.c_void_p(0)] * 7
    assert lib.LIBINFINIOP.infiniopPagedAttention(op, ctypes.c_void_p(0), 0, *args, None) == NO_WS
    assert lib.LIBINFINIOP.infiniopPagedAttention(op, ctypes.c_void_p(0), size.value, *args, None) == NO_WS
    assert lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op) == OK
    assert lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(None) == NULLP


def test_paged_attention_shapes_beyond_one_launch_are_refused_at_creation(lib, host_amd_handle):
    """Sequences and heads sit on the y / z axes of some launches (limit 65535 each): larger batches are
    answered with BAD_TENSOR_SHAPE when the descriptor is made, not with a failed launch later."""
    status, op = create_attention(lib, host_amd_handle, attention_specs(B=65535, NB=4, maxb=2))
    assert status == OK
    lib.check_error(lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    status, _ = create_attention(lib, host_amd_handle, attention_specs(B=65536, NB=4, maxb=2))
    assert status == BAD_SHAPE


def test_paged_attention_workspace_is_sized_for_the_planned_schedule(lib, host_amd_handle):
    """The Llama-3-8B batch-32 decode shape: (128 pieces + 32 sequences) rows of partial results, 2.7 MB - less
    than the 8 * B * H * (D + 2) * 4 = 4.26 MB of the reference's nvidia backend."""
    specs = attention_specs(B=32, H=32, Hkv=8, NB=5400, maxb=256, dtype=BF16)
    status, op = create_attention(lib, host_amd_handle, specs)
    assert status == OK
    size = ctypes.c_size_t(0)
    lib.check_error(lib.LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, ctypes.byref(size)))
    assert 2_600_000 < size.value < 2_720_000  # incl. 32 KB of first-tile entries
    lib.check_error(lib.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


def test_paged_attention_null_arguments(lib, host_amd_handle):
    t = lib.create_tensor_descriptor((4, 8, 128), None, F16)
    op = lib.infiniopOperatorDescriptor_t()
    L = lib.LIBINFINIOP
    assert L.infiniopCreatePagedAttentionDescriptor(None, ctypes.byref(op), t, t, t, t, t, t, None, 1.0) == NULLP
    assert L.infiniopCreatePagedAttentionDescriptor(host_amd_handle, None, t, t, t, t, t, t, None, 1.0) == NULLP
    assert L.infiniopCreatePagedAttentionDescriptor(host_amd_handle, ctypes.byref(op), None, t, t, t, t, t, None, 1.0) == NULLP
    lib.destroy_tensor_descriptor(t)


# ---------------------------------------------------------------------------------------------------


def caching_specs(ntok=32, Hkv=8, D=128, Dv=None, bs=16, NB=64, dtype=BF16):
    Dv = Dv or D
    return {
        "k_cache": Spec((NB, Hkv, bs, D), dtype), "v_cache": Spec((NB, Hkv, bs, Dv), dtype),
        "k": Spec((ntok, Hkv, D), dtype), "v": Spec((ntok, Hkv, Dv), dtype), "slots": Spec((ntok,), I64),
    }


def create_caching(lib, handle, specs):
    order = ["k_cache", "v_cache", "k", "v", "slots"]
    descs = [lib.create_tensor_descriptor(specs[n].shape, specs[n].strides, specs[n].dtype) for n in order]
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreatePagedCachingDescriptor(handle, ctypes.byref(op), *descs)
    for d in descs:
        lib.destroy_tensor_descriptor(d)
    return status, op


CACHING_CASES = [
    # line numbers are src/infiniop/ops/paged_caching/info.h
    ("valid bf16", OK, lambda s: s),
    ("valid f32 (:43)", OK, lambda s: caching_specs(dtype=F32)),
    ("valid f16", OK, lambda s: caching_specs(dtype=F16)),
    ("valid MLA sizes 576/512", OK, lambda s: caching_specs(Hkv=1, D=576, Dv=512)),
    ("valid permuted cache strides", OK, lambda s: mutate(mutate(s, "k_cache", strides=(16384, 128, 1024, 1)), "v_cache", strides=(16384, 128, 1024, 1))),
    ("k dtype i64 (:43)", BAD_DTYPE, lambda s: mutate(s, "k", dtype=I64)),
    ("v dtype differs (:44)", BAD_DTYPE, lambda s: mutate(s, "v", dtype=F16)),
    ("cache dtype differs (:44)", BAD_DTYPE, lambda s: mutate(s, "k_cache", dtype=F16)),
    ("slot dtype i32 (:47)", BAD_DTYPE, lambda s: mutate(s, "slots", dtype=I32)),
    ("k rank 2 (:52)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(32, 1024))),
    ("cache rank 3 (:52)", BAD_SHAPE, lambda s: mutate(s, "k_cache", shape=(64, 8, 2048))),
    ("slots rank 2 (:52)", BAD_SHAPE, lambda s: mutate(s, "slots", shape=(32, 1))),
    ("k tokens differ from slots (:69)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(31, 8, 128))),
    ("v heads differ (:69)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(32, 4, 128))),
    ("v pool differs (:75)", BAD_SHAPE, lambda s: mutate(s, "v_cache", shape=(32, 8, 16, 128))),
    ("v page size differs (:75)", BAD_SHAPE, lambda s: mutate(s, "v_cache", shape=(64, 8, 32, 128))),
    ("cache heads differ (:78)", BAD_SHAPE, lambda s: mutate(mutate(s, "k_cache", shape=(64, 4, 16, 128)), "v_cache", shape=(64, 4, 16, 128))),
    ("cache head size differs (:78)", BAD_SHAPE, lambda s: mutate(s, "k_cache", shape=(64, 8, 16, 64))),
    ("v cache value size differs (:78)", BAD_SHAPE, lambda s: mutate(s, "v_cache", shape=(64, 8, 16, 64))),
]


@pytest.mark.parametrize("what,expected,change", CACHING_CASES, ids=[c[0] for c in CACHING_CASES])
def test_paged_caching_validation(lib, host_amd_handle, what, expected, change):
    status, op = create_caching(lib, host_amd_handle, change(caching_specs()))
    assert status == expected, what
    if status == OK:
        size = ctypes.c_size_t(99)
        assert lib.LIBINFINIOP.infiniopGetPagedCachingWorkspaceSize(op, ctypes.byref(size)) == OK
        assert size.value == 0  # reference: nvidia/paged_caching_nvidia.cu:47-49
        assert lib.LIBINFINIOP.infiniopDestroyPagedCachingDescriptor(op) == OK


def test_tensor_descriptor_default_strides_are_packed(lib, host_amd_handle):
    """NULL strides mean C-contiguous (reference src/infiniop/tensor_descriptor.cc:12-21): a cache given
    without strides must validate like one given with explicit packed strides."""
    s = caching_specs()
    s = mutate(s, "k_cache", strides=(8 * 16 * 128, 16 * 128, 128, 1))
    status, op = create_caching(lib, host_amd_handle, s)
    assert status == OK
    lib.LIBINFINIOP.infiniopDestroyPagedCachingDescriptor(op)
    assert lib.LIBINFINIOP.infiniopCreateTensorDescriptor(None, 1, None, None, F16) == NULLP


def test_paged_caching_refuses_extents_its_kernel_cannot_count_before_any_gpu_call(lib, host_amd_handle):
    """The scatter kernel counts heads, row units and workgroups in 32 bits: a descriptor beyond that (descriptors are
    metadata, nothing of that size exists) is answered BAD_TENSOR_SHAPE at run time, before any device call."""
    big = 1 << 31
    s = {"k_cache": Spec((1, big, 1, 2), BF16), "v_cache": Spec((1, big, 1, 2), BF16),
         "k": Spec((1, big, 2), BF16), "v": Spec((1, big, 2), BF16), "slots": Spec((1,), I64)}
    status, op = create_caching(lib, host_amd_handle, s)
    assert status == OK
    somewhere = ctypes.c_void_p(4096)  # never dereferenced
    assert lib.LIBINFINIOP.infiniopPagedCaching(op, None, 0, *([somewhere] * 5), None) == BAD_SHAPE
    assert lib.LIBINFINIOP.infiniopDestroyPagedCachingDescriptor(op) == OK
