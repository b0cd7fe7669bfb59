"""Create-time validation of paged_attention_prefill: one case per status-returning check of the
reference's src/infiniop/ops/paged_attention_prefill/info.h, run through the C ABI with a host-only
AMD handle (descriptor creation is pure host code, so none of this needs a GPU)."""
import ctypes

import pytest

from test_validation import BAD_DTYPE, BAD_SHAPE, BAD_STRIDES, BF16, F16, F32, I32, I64, NULLP, OK, U8, U32, Spec, mutate

BAD_PARAM = 3


def prefill_specs(T=40, B=4, H=8, Hkv=8, D=128, Dv=None, bs=16, NB=64, maxb=16, dtype=F16, idx=I64):
    Dv = Dv or D
    return {
        "out": Spec((T, H, Dv), dtype), "q": Spec((T, H, D), dtype),
        "k": Spec((NB, Hkv, bs, D), dtype), "v": Spec((NB, Hkv, bs, Dv), dtype),
        "bt": Spec((B, maxb), idx), "lens": Spec((B,), idx), "cum": Spec((B + 1,), idx), "alibi": None,
    }


def create_prefill(lib, handle, specs, scale=0.0884):
    order = ["out", "q", "k", "v", "bt", "lens", "cum"]
    descs = [lib.create_tensor_descriptor(specs[n].shape, specs[n].strides, specs[n].dtype) for n in order]
    alibi = specs.get("alibi")
    alibi_desc = lib.create_tensor_descriptor(alibi.shape, alibi.strides, alibi.dtype) if alibi else None
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreatePagedAttentionPrefillDescriptor(handle, ctypes.byref(op), *descs, alibi_desc,
                                                                           scale)
    for d in descs:
        lib.destroy_tensor_descriptor(d)
    if alibi_desc:
        lib.destroy_tensor_descriptor(alibi_desc)
    return status, op


CASES = [
    # (what, expected status, mutation) - line numbers are src/infiniop/ops/paged_attention_prefill/info.h
    ("valid", OK, lambda s: s),
    ("q dtype f32 (:56)", BAD_DTYPE, lambda s: mutate(s, "q", dtype=F32)),
    ("out dtype differs (:57)", BAD_DTYPE, lambda s: mutate(s, "out", dtype=BF16)),
    ("k dtype differs (:57)", BAD_DTYPE, lambda s: mutate(s, "k", dtype=BF16)),
    ("v dtype differs (:57)", BAD_DTYPE, lambda s: mutate(s, "v", dtype=BF16)),
    ("q rank 2 (:62)", BAD_SHAPE, lambda s: mutate(s, "q", shape=(40, 1024))),
    ("out rank 4 (:62)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(40, 8, 1, 128))),
    ("k rank 3 (:66)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(64, 8, 2048))),
    ("v rank 5 (:66)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(64, 8, 16, 128, 1))),
    ("table rank 1 (:69)", BAD_SHAPE, lambda s: mutate(s, "bt", shape=(64,))),
    ("lens rank 2 (:69)", BAD_SHAPE, lambda s: mutate(s, "lens", shape=(4, 1))),
    ("cum rank 2 (:69)", BAD_SHAPE, lambda s: mutate(s, "cum", shape=(5, 1))),
    ("q last stride 2 (:73)", BAD_STRIDES, lambda s: mutate(s, "q", strides=(2048, 256, 2))),
    ("out last stride 2 (:74)", BAD_STRIDES, lambda s: mutate(s, "out", strides=(2048, 256, 2))),
    ("k last stride 2 (:75)", BAD_STRIDES, lambda s: mutate(s, "k", strides=(32768, 4096, 256, 2))),
    ("v last stride 2 (:76)", BAD_STRIDES, lambda s: mutate(s, "v", strides=(32768, 4096, 256, 2))),
    ("table dtype f32 (:80)", BAD_DTYPE, lambda s: mutate(s, "bt", dtype=F32)),
    ("lens dtype u8 (:86)", BAD_DTYPE, lambda s: mutate(s, "lens", dtype=U8)),
    ("cum dtype f32 (:90)", BAD_DTYPE, lambda s: mutate(s, "cum", dtype=F32)),
    ("lens index dtype differs from the table's (stricter than the reference)", BAD_DTYPE, lambda s: mutate(s, "lens", dtype=I32)),
    ("cum index dtype differs from the table's (stricter than the reference)", BAD_DTYPE, lambda s: mutate(s, "cum", dtype=U32)),
    ("table inner stride 2 (:94)", BAD_STRIDES, lambda s: mutate(s, "bt", strides=(32, 2))),
    ("lens stride 2 (stricter than the reference)", BAD_STRIDES, lambda s: mutate(s, "lens", strides=(2,))),
    ("cum stride 2 (stricter than the reference)", BAD_STRIDES, lambda s: mutate(s, "cum", strides=(2,))),
    ("alibi dtype f16 (:97)", BAD_DTYPE, lambda s: {**s, "alibi": Spec((8,), F16)}),
    ("alibi rank 2 (:100)", BAD_SHAPE, lambda s: {**s, "alibi": Spec((8, 1), F32)}),
    ("alibi stride 2 (:103)", BAD_STRIDES, lambda s: {**s, "alibi": Spec((8,), F32, (2,))}),
    ("alibi valid", OK, lambda s: {**s, "alibi": Spec((8,), F32)}),
    ("heads not a multiple of kv heads (:123)", BAD_SHAPE, lambda s: mutate(mutate(s, "k", shape=(64, 3, 16, 128)), "v", shape=(64, 3, 16, 128))),
    ("k head size differs (:129)", BAD_SHAPE, lambda s: mutate(s, "k", shape=(64, 8, 16, 64))),
    ("v pool size differs (:132)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(32, 8, 16, 128))),
    ("v page size differs (:132)", BAD_SHAPE, lambda s: mutate(s, "v", shape=(64, 8, 32, 128))),
    ("value size differs, not MLA (:135)", BAD_SHAPE, lambda s: mutate(mutate(s, "v", shape=(64, 8, 16, 64)), "out", shape=(40, 8, 64))),
    ("out width differs (:139)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(40, 8, 64))),
    ("out rows differ (:139)", BAD_SHAPE, lambda s: mutate(s, "out", shape=(41, 8, 128))),
    ("cum length is not num_seqs + 1 (:144)", BAD_PARAM, lambda s: mutate(s, "cum", shape=(4,))),
    ("table has fewer rows than sequences (stricter than the reference)", BAD_SHAPE, lambda s: mutate(s, "bt", shape=(3, 16))),
    ("alibi shorter than heads (stricter than the reference)", BAD_SHAPE, lambda s: {**s, "alibi": Spec((4,), F32)}),
]


@pytest.mark.parametrize("what,expected,change", CASES, ids=[c[0] for c in CASES])
def test_prefill_validation(lib, host_amd_handle, what, expected, change):
    status, op = create_prefill(lib, host_amd_handle, change(prefill_specs()))
    assert status == expected, what
    if status == OK:
        size = ctypes.c_size_t(99)
        assert lib.LIBINFINIOP.infiniopGetPagedAttentionPrefillWorkspaceSize(op, ctypes.byref(size)) == OK
        assert size.value == 0  # softmax state stays in registers; nothing is staged in device memory
        assert lib.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op) == OK


@pytest.mark.parametrize("head_size,ok", [(64, True), (128, True), (192, True), (256, True), (576, True), (32, False), (96, False), (512, False)])
def test_prefill_head_sizes(lib, host_amd_handle, head_size, ok):
    status, op = create_prefill(lib, host_amd_handle, prefill_specs(D=head_size))  # info.h:120
    assert status == (OK if ok else BAD_SHAPE)
    if ok:
        lib.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op)


def test_prefill_mla_value_size(lib, host_amd_handle):
    status, op = create_prefill(lib, host_amd_handle, prefill_specs(H=16, Hkv=1, D=576, Dv=512))  # info.h:113,135
    assert status == OK
    lib.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op)


@pytest.mark.parametrize("idx", [I64, I32, U32])
def test_prefill_index_dtypes(lib, host_amd_handle, idx):
    status, op = create_prefill(lib, host_amd_handle, prefill_specs(idx=idx))
    assert status == OK
    lib.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op)


def test_prefill_null_arguments_and_device(lib, host_amd_handle):
    t = lib.create_tensor_descriptor((4, 8, 128), None, F16)
    op = lib.infiniopOperatorDescriptor_t()
    L = lib.LIBINFINIOP
    assert L.infiniopCreatePagedAttentionPrefillDescriptor(None, ctypes.byref(op), t, t, t, t, t, t, t, None, 1.0) == NULLP
    assert L.infiniopCreatePagedAttentionPrefillDescriptor(host_amd_handle, None, t, t, t, t, t, t, t, None, 1.0) == NULLP
    assert L.infiniopCreatePagedAttentionPrefillDescriptor(host_amd_handle, ctypes.byref(op), t, t, t, t, t, t, None, None, 1.0) == NULLP
    lib.destroy_tensor_descriptor(t)
    assert L.infiniopGetPagedAttentionPrefillWorkspaceSize(None, None) == NULLP
    assert L.infiniopDestroyPagedAttentionPrefillDescriptor(None) == NULLP
    status, op = create_prefill(lib, host_amd_handle, prefill_specs())
    assert status == OK and op.contents.device_type == lib.InfiniDevice.AMD
    # data pointers are checked before anything is launched
    args = [ctypes.c_void_p(0)] * 8
    assert L.infiniopPagedAttentionPrefill(op, ctypes.c_void_p(0), 0, *args, None) == NULLP
    assert L.infiniopDestroyPagedAttentionPrefillDescriptor(op) == OK


def test_prefill_has_no_cpu_backend(lib):
    """As in the reference (src/infiniop/ops/paged_attention_prefill/operator.cc:36-70 has no CPU case)."""
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    handle = lib.create_handle()
    t = lib.create_tensor_descriptor((2, 4, 128), None, F16)
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreatePagedAttentionPrefillDescriptor(handle, ctypes.byref(op), t, t, t, t, t, t, t, None, 1.0)
    assert status == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    lib.destroy_tensor_descriptor(t)
    lib.destroy_handle(handle)
