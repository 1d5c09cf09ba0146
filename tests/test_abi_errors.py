"""Argument validation of the C ABI: every rejected call returns its error code before anything is launched,
so these run without a GPU (the pointers are never dereferenced)."""
import ctypes

import pytest

from mercury_artifact_amd import _native as N

OK, EINVAL, EDTYPE, EHEADDIM, EALIGN, EUNSUPPORTED = 0, -1, -2, -3, -4, -6
P = 0x10000           # a non-NULL, 16-byte aligned "pointer"


@pytest.fixture(scope="module")
def lib():
    return N.lib()


def _fwd(lib, q=P, k=P, v=P, out=P, lse=P, B=1, Sq=64, Sc=64, Hq=2, Hkv=2, D=128,
         strides=None, scale=0.1, mask=0, dtype=0, descales=(None, None, None)):
    if strides is None:
        strides = [Sq * Hq * D, Hq * D, D, Sc * Hkv * D, Hkv * D, D, Sc * Hkv * D, Hkv * D, D, Sq * Hq * D, Hq * D, D]
    return lib.mhip_attn_fwd_block(q, k, v, out, lse, B, Sq, Sc, Hq, Hkv, D, *strides, scale, mask, dtype,
                                   *descales, None)


def test_forward_rejects(lib):
    for bad in (0, 4, 100, 136, 256):
        assert _fwd(lib, D=bad) == EHEADDIM
    assert _fwd(lib, D=72, dtype=1) == EHEADDIM                 # e4m3: multiples of 16
    big64 = 1 << 19                                             # D = 64: spans of one (batch, head) stay below 1 GiB
    assert _fwd(lib, D=64, Sc=1024, strides=[64 * 128, 128, 64, 1024 * big64, big64, 64, 1024 * big64, big64, 64,
                                             64 * 128, 128, 64]) == EUNSUPPORTED
    assert _fwd(lib, Hq=3, Hkv=2) == EINVAL
    assert _fwd(lib, Sq=-1) == EINVAL
    assert _fwd(lib, scale=0.0) == EINVAL
    assert _fwd(lib, scale=float("inf")) == EINVAL
    assert _fwd(lib, scale=float("nan")) == EINVAL
    assert _fwd(lib, mask=2) == EINVAL
    assert _fwd(lib, dtype=7) == EDTYPE
    assert _fwd(lib, q=None) == EINVAL
    assert _fwd(lib, k=None) == EINVAL
    assert _fwd(lib, q=P + 8) == EALIGN
    s = [64 * 2 * 128, 2 * 128, 128] * 4
    s[1] += 4                                   # a row stride that breaks 16-byte alignment
    assert _fwd(lib, strides=s) == EALIGN
    big = 1 << 20                               # rows 2 MiB apart: 2048 of them span 4 GiB
    assert _fwd(lib, Sc=2048, strides=[64 * 256, 256, 128, 2048 * big, big, 128, 2048 * big, big, 128,
                                       64 * 256, 256, 128]) == EUNSUPPORTED
    assert _fwd(lib, dtype=1, descales=(P, P + 2, P)) == EALIGN    # descales are pointers to device floats
    # nothing to do: accepted without touching the pointers
    assert _fwd(lib, B=0) == OK
    assert _fwd(lib, Sq=0) == OK
    assert lib.mhip_error_string(EHEADDIM).startswith(b"head dimension")


def test_backward_rejects(lib):
    def bwd(B=1, Sq=64, Sc=64, Hq=2, Hkv=2, D=128, scale=0.1, mask=0, dq=P, ws=P, strides=None, dq_acc=None):
        if strides is None:
            strides = [Sq * Hq * D, Hq * D, D, Sc * Hkv * D, Hkv * D, D, Sc * Hkv * D, Hkv * D, D,
                       Sq * Hq * D, Hq * D, D, Sq * Hq * D, Hq * D, D]
        return lib.mhip_attn_bwd_block(P, P, P, P, P, P, dq, P, P, dq_acc, B, Sq, Sc, Hq, Hkv, D, *strides,
                                       scale, mask, 0, ws, None)

    for bad in (0, 4, 100, 136, 256):
        assert bwd(D=bad) == EHEADDIM
    assert bwd(Hq=5, Hkv=2) == EINVAL
    assert bwd(scale=-1.0) == EINVAL
    assert bwd(mask=3) == EINVAL
    assert bwd(dq=None) == EINVAL
    assert bwd(ws=None) == EINVAL
    assert bwd(dq=P + 4) == EALIGN
    assert bwd(strides=[64 * 256, 257, 128, 64 * 256, 256, 128, 64 * 256, 256, 128] + [64 * 256, 256, 128] * 2) == EALIGN
    assert bwd(strides=[64 * 256, 256, 128] * 3 + [64 * 256, 260, 128, 64 * 256, 256, 128]) == EALIGN     # dq rows
    assert bwd(Sq=4096, strides=[1 << 33, 1 << 21, 128, 64 * 256, 256, 128, 64 * 256, 256, 128]
               + [4096 * 256, 256, 128] * 2) == EUNSUPPORTED
    assert bwd(B=0) == OK
    assert lib.mhip_attn_bwd_workspace_bytes(2, 100, 64, 4, 2, 128) >= 2 * 2 * 4 * 100 * 4


def test_elementwise_rejects(lib):
    assert lib.mhip_flash_reduce(P, P, None, 8, 128, None) == EINVAL
    assert lib.mhip_flash_reduce(P, P + 4, P, 8, 128, None) == EALIGN
    assert lib.mhip_flash_reduce(P, P, P, -1, 128, None) == EINVAL
    assert lib.mhip_flash_reduce(P, P, P, 0, 128, None) == OK
    two = (ctypes.c_void_p * 2)(P, P)
    sb2 = (ctypes.c_int64 * 2)(8 * 4 * 128, 8 * 4 * 128)

    def many(outs=two, lses=two, sb=sb2, begin=None, n=2, fo=P, fl=P, D=128, st=(128 * 4, 128), B=1):
        return lib.mhip_lse_merge_many(outs, lses, sb, begin, n, fo, fl, B, 8, 4, D, *st, None)

    assert many(n=0) == EINVAL and many(n=65) == EINVAL
    assert many(fo=None) == EINVAL and many(outs=None) == EINVAL and many(sb=None) == EINVAL
    assert many(outs=(ctypes.c_void_p * 2)(P, None)) == EINVAL
    assert many(begin=(ctypes.c_int * 2)(0, 9)) == EINVAL and many(begin=(ctypes.c_int * 2)(-1, 0)) == EINVAL
    assert many(outs=(ctypes.c_void_p * 2)(P, P + 8)) == EALIGN
    assert many(st=(128 * 4 + 4, 128)) == EALIGN
    assert many(sb=(ctypes.c_int64 * 2)(4096, 4100)) == EALIGN
    assert many(D=44) == EUNSUPPORTED and many(D=264) == EUNSUPPORTED      # multiples of 8 up to 256
    assert many(B=0) == OK
    assert lib.mhip_tree_merge(P, None, P, 8, 128, 0, None) == EINVAL
    assert lib.mhip_tree_merge(P + 8, P, P, 8, 128, 1, None) == EALIGN
    assert lib.mhip_tree_merge(P, P, P, 0, 128, 1, None) == OK
    # overlapping operands: dst == src is the in-place form of the tree merge, any other overlap is refused;
    # the flat packed kernels take no overlap at all
    assert lib.mhip_tree_merge(P, P, P + 16, 8, 128, 1, None) == EINVAL
    assert lib.mhip_tree_merge(P + 16, P, P, 8, 128, 0, None) == EINVAL
    assert lib.mhip_flash_reduce(P, P + 0x100000, P, 8, 128, None) == EINVAL
    assert lib.mhip_flash_reduce(P + 0x100000, P, P + 16, 8, 128, None) == EINVAL
    assert lib.mhip_pack_reduce(P, P, P, P + 32, 1, 8, 2, 128, None) == EINVAL
    assert lib.mhip_pack_reduce(None, P, P, None, 1, 8, 2, 128, None) == EINVAL
    assert lib.mhip_pack_reduce(P + 4, P, P, P, 1, 8, 2, 128, None) == EALIGN
    assert lib.mhip_pack_reduce(None, P, P, P, 0, 8, 2, 128, None) == OK
    assert lib.mhip_grad_accumulate(None, P, None, 16, None) == EINVAL
    assert lib.mhip_grad_accumulate(None, P + 2, P, 16, None) == EALIGN
    assert lib.mhip_grad_accumulate(None, P, P, 0, None) == OK
    assert lib.mhip_unpack(P, None, P, 1, 8, 2, 128, None) == EINVAL
    assert lib.mhip_unpack(P, P + 8, P, 1, 8, 2, 128, None) == EALIGN
    assert lib.mhip_unpack(P, P, P, 1, 8, 2, 100, None) == EUNSUPPORTED
    assert lib.mhip_unpack(P, P, P, 0, 8, 2, 128, None) == OK
    assert lib.mhip_quantize_e4m3(P, 1, 64, P, P, P, None) == EDTYPE
    assert lib.mhip_quantize_e4m3(P, 2, -1, P, P, P, None) == EINVAL
    assert lib.mhip_quantize_e4m3(P, 2, 64, P, None, P, None) == EINVAL
    assert lib.mhip_quantize_e4m3(None, 2, 64, P, P, P, None) == EINVAL
    assert lib.mhip_quantize_e4m3(P + 4, 2, 64, P, P, P, None) == EALIGN
