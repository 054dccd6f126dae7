"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and rejects
bad arguments with status codes before anything is launched (no GPU needed for any of this)."""
import ctypes
import os
import re

import pytest

from flexsae_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flexsae_amd.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(flexsae_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/flexsae_amd.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "python binding table and header disagree"
    assert lib.flexsae_abi_version() == _lib.ABI_VERSION


def test_header_constants_match_binding():
    text = open(HEADER).read()
    for name, value in (("FLEXSAE_ERR_INVALID_ARGUMENT", _lib.ERR_INVALID_ARGUMENT),
                        ("FLEXSAE_ERR_UNSUPPORTED", _lib.ERR_UNSUPPORTED),
                        ("FLEXSAE_ERR_WORKSPACE", _lib.ERR_WORKSPACE),
                        ("FLEXSAE_ERR_LAUNCH", _lib.ERR_LAUNCH),
                        ("FLEXSAE_ERR_ALIGNMENT", _lib.ERR_ALIGNMENT),
                        ("FLEXSAE_ERR_SCRATCH_LIMIT", _lib.ERR_SCRATCH_LIMIT),
                        ("FLEXSAE_BF16", _lib.BF16), ("FLEXSAE_F16", _lib.F16),
                        ("FLEXSAE_ABI_VERSION", _lib.ABI_VERSION)):
        m = re.search(rf"{name}\s*=?\s*(-?\d+)", text)
        assert m and int(m.group(1)) == value, name


def test_status_strings():
    for code in (0, -1, -2, -3, -4, -5, -6, -99):
        assert isinstance(_lib.status_string(code), str) and _lib.status_string(code)


FAKE = ctypes.c_void_p(0x10000)  # never dereferenced: validation fails first
NULL = ctypes.c_void_p(0)


def _shape(B=4, K=8, F=16, D=64, wd=0, vd=0, bd=0, td=0):
    return _lib.Shape(B, K, F, D, wd, vd, bd, td)


def test_workspace_queries():
    lib = _lib.load()
    assert lib.flexsae_fwd_workspace_bytes(ctypes.byref(_shape())) >= 4 * 4
    assert lib.flexsae_fwd_workspace_bytes(ctypes.byref(_shape(B=4096, D=2304))) % 256 == 0
    assert lib.flexsae_fwd_workspace_bytes(ctypes.byref(_shape(B=0))) == 0
    assert lib.flexsae_csr_workspace_bytes(4, 8, 16) >= 16 * 4
    assert lib.flexsae_csr_workspace_bytes(0, 8, 16) == 0


@pytest.mark.parametrize("entry", ["flexsae_hier_fwd", "flexsae_topk_fwd"])
def test_forward_rejects_bad_arguments(entry):
    lib = _lib.load()
    fn = getattr(lib, entry)

    def call(shape, ptrs=None, ws=FAKE, ws_bytes=1 << 20):
        p = ptrs or [FAKE] * 7
        return fn(ctypes.byref(shape), *p, ws, ws_bytes, NULL, NULL)

    assert call(_shape(B=0)) == _lib.ERR_INVALID_ARGUMENT
    assert call(_shape(K=-1)) == _lib.ERR_INVALID_ARGUMENT
    assert call(_shape(wd=7)) == _lib.ERR_INVALID_ARGUMENT
    assert call(_shape(F=1 << 31)) == _lib.ERR_UNSUPPORTED
    assert call(_shape(B=1 << 20, K=1 << 12)) == _lib.ERR_UNSUPPORTED
    for i in range(7):
        ptrs = [FAKE] * 7
        ptrs[i] = NULL
        assert call(_shape(), ptrs) == _lib.ERR_INVALID_ARGUMENT
    odd = [FAKE] * 7
    odd[1] = ctypes.c_void_p(0x10001)  # weight not aligned to its element
    assert call(_shape(), odd) == _lib.ERR_ALIGNMENT
    assert call(_shape(), ws=NULL) == _lib.ERR_WORKSPACE
    assert call(_shape(), ws_bytes=8) == _lib.ERR_WORKSPACE
    assert call(_shape(), ws=ctypes.c_void_p(0x10010)) == _lib.ERR_WORKSPACE


def test_backward_and_csr_reject_bad_arguments():
    lib = _lib.load()
    sh = _shape()
    ok = [FAKE] * 8
    atomic = lib.flexsae_hier_bwd_atomic
    assert atomic(ctypes.byref(_shape(D=0)), *ok, 0, NULL, NULL) == _lib.ERR_INVALID_ARGUMENT
    for i in range(8):
        ptrs = [FAKE] * 8
        ptrs[i] = NULL
        assert atomic(ctypes.byref(sh), *ptrs, 0, NULL, NULL) == _lib.ERR_INVALID_ARGUMENT

    def seg(shape, ptrs=None, ws=FAKE, ws_bytes=1 << 30, dw_dtype=0):
        a = ptrs or [FAKE] * 8
        return lib.flexsae_hier_bwd(ctypes.byref(shape), *a[:6], dw_dtype, a[6], a[7], ws, ws_bytes, 0, NULL, NULL)

    assert seg(_shape(K=0)) == _lib.ERR_INVALID_ARGUMENT
    assert seg(sh, dw_dtype=5) == _lib.ERR_INVALID_ARGUMENT
    for i in range(8):
        ptrs = [FAKE] * 8
        ptrs[i] = NULL
        assert seg(sh, ptrs) == _lib.ERR_INVALID_ARGUMENT
    assert seg(sh, ws=NULL) == _lib.ERR_WORKSPACE
    assert seg(sh, ws_bytes=64) == _lib.ERR_WORKSPACE
    need_min = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), 0)
    need_all = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(sh), 1 << 30)
    assert 0 < need_min <= need_all and need_min % 256 == 0
    assert lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(_shape(B=-1)), 0) == 0
    assert lib.flexsae_csr_build(NULL, 4, 8, 16, FAKE, FAKE, FAKE, 1 << 20, NULL, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert lib.flexsae_csr_build(FAKE, 4, 8, 16, FAKE, FAKE, FAKE, 4, NULL, NULL) == _lib.ERR_WORKSPACE
    assert lib.flexsae_csr_build(FAKE, 1 << 20, 1 << 12, 16, FAKE, FAKE, FAKE, 1 << 20, NULL, NULL) == _lib.ERR_UNSUPPORTED
    # (shape, begin, map, indices or NULL, weight, vals, resid, grad_out, dW, dW_dtype, dvals, dbias, ws, bytes, flags, stream)
    assert lib.flexsae_topk_bwd(ctypes.byref(sh), FAKE, FAKE, NULL, FAKE, FAKE, FAKE, FAKE, FAKE, 9, FAKE, FAKE, FAKE,
                                1 << 20, 0, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert lib.flexsae_topk_bwd(ctypes.byref(sh), FAKE, NULL, NULL, FAKE, FAKE, FAKE, FAKE, FAKE, 0, FAKE, FAKE, FAKE,
                                1 << 20, 0, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert lib.flexsae_topk_bwd(ctypes.byref(sh), FAKE, FAKE, ctypes.c_void_p(0x10004), FAKE, FAKE, FAKE, FAKE, FAKE, 0,
                                FAKE, FAKE, FAKE, 1 << 20, 0, NULL) == _lib.ERR_ALIGNMENT
    assert lib.flexsae_topk_bwd(ctypes.byref(sh), FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 0, FAKE, FAKE, NULL,
                                1 << 20, 0, NULL) == _lib.ERR_WORKSPACE
    assert lib.flexsae_topk_bwd_workspace_bytes(ctypes.byref(sh), 0) >= 64 * 4
    assert (lib.flexsae_topk_bwd_workspace_bytes(ctypes.byref(sh), 1 << 30)
            >= lib.flexsae_topk_bwd_workspace_bytes(ctypes.byref(sh), 0))
    assert lib.flexsae_cast_from_f32(NULL, 1, FAKE, 10, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert lib.flexsae_cast_from_f32(FAKE, 1, FAKE, -1, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert lib.flexsae_cast_from_f32(FAKE, 1, FAKE, 0, NULL) == _lib.OK


def test_static_forward_rejects_bad_arguments_before_touching_the_gpu():
    lib = _lib.load()
    fn = lib.flexsae_hier_fwd_static
    args = [FAKE] * 7
    assert fn(ctypes.byref(_shape(B=0)), *args, NULL, NULL) == _lib.ERR_INVALID_ARGUMENT
    assert fn(ctypes.byref(_shape(F=1 << 31)), *args, NULL, NULL) == _lib.ERR_UNSUPPORTED
    # B * ceil(D/64) * 4 bytes of loss partials beyond the static array
    assert fn(ctypes.byref(_shape(B=70000, K=1, D=4096)), *args, NULL, NULL) == _lib.ERR_SCRATCH_LIMIT
    m = re.search(r"FLEXSAE_STATIC_SCRATCH_BYTES\s*\((\d+)u\s*<<\s*(\d+)\)", open(HEADER).read())
    assert m and (int(m.group(1)) << int(m.group(2))) == 16 << 20
