"""The C-ABI library loads without a GPU and exports every symbol ``include/agmi.h`` declares."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "agmi.h")
LIB = os.path.join(ROOT, "autograd_amd", "libagmi.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(agmi_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is not built; run `make -C autograd_amd/csrc`")
    return ctypes.CDLL(LIB)


def test_header_declares_entry_points():
    names = declared_symbols()
    assert "agmi_elementwise" in names and "agmi_gemm" in names and len(names) >= 10


def test_every_declared_symbol_is_exported(lib):
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_the_header():
    from autograd_amd import _lib

    assert sorted(_lib.EXPORTS) == declared_symbols()
    L = _lib.lib()
    assert L.agmi_version() >= 100
    assert _lib.AgmiArray.strides.size == 8 * 8  # AGMI_MAX_DIMS int64 strides


def test_op_codes_match_header():
    from autograd_amd import _lib

    text = open(HEADER).read()
    body = re.search(r"typedef enum agmi_op \{(.*?)\} agmi_op;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    value = -1
    for item in body.split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            name, v = [s.strip() for s in item.split("=")]
            value = int(v)
        else:
            name, value = item, value + 1
        py = name.replace("AGMI_OP_", "")
        assert getattr(_lib.Op, py) == value, (name, value)


def test_argument_errors_are_reported_without_a_gpu(lib):
    # argument validation happens on the host before any launch
    lib.agmi_last_error.restype = ctypes.c_char_p
    rc = lib.agmi_fill(0, None, ctypes.c_int64(16), ctypes.c_double(0.0), None)
    assert rc == -1 and b"fill" in lib.agmi_last_error()
    rc = lib.agmi_gemm(0, ctypes.c_int64(1), ctypes.c_int64(-1), ctypes.c_int64(1), ctypes.c_int64(1),
                       ctypes.c_double(1.0), None, ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_int64(0), None,
                       ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_double(0.0), None,
                       ctypes.c_int64(1), ctypes.c_int64(0), None, ctypes.c_size_t(0), None)
    assert rc == -1
    i64, c_int = ctypes.c_int64, ctypes.c_int
    # the copy-shaped index entry points: empty extents are a no-op, everything else is checked before the launch
    for name, args in (("agmi_cumsum", (i64(2), i64(0), i64(3))), ("agmi_reverse", (i64(0), i64(4), i64(3)))):
        assert getattr(lib, name)(0, None, *args, None, None) == 0
    assert lib.agmi_triangle(0, None, i64(1), i64(0), i64(5), i64(0), c_int(1), None, None) == 0
    for name, args in (("agmi_cumsum", (i64(2), i64(4), i64(3))), ("agmi_reverse", (i64(2), i64(4), i64(3)))):
        assert getattr(lib, name)(0, None, *args, None, None) == -1 and b"null" in lib.agmi_last_error()
        assert getattr(lib, name)(0, None, i64(-1), i64(4), i64(3), None, None) == -1 and b"negative" in lib.agmi_last_error()
    assert lib.agmi_triangle(0, None, i64(1), i64(3), i64(5), i64(0), c_int(1), None, None) == -1
    buf = (ctypes.c_double * 8)()
    for name, args in (("agmi_cumsum", (i64(1), i64(8), i64(1))), ("agmi_reverse", (i64(1), i64(8), i64(1)))):
        assert getattr(lib, name)(7, buf, *args, buf, None) == -1 and b"floating" in lib.agmi_last_error()
    assert lib.agmi_triangle(7, buf, i64(1), i64(2), i64(4), i64(0), c_int(0), buf, None) == -1
    assert lib.agmi_sort_rows(0, None, i64(0), i64(5), None, None, None, None) == 0
    assert lib.agmi_sort_rows(1, buf, i64(1), i64(8), None, None, None, None) == -1 and b"no result" in lib.agmi_last_error()
    assert lib.agmi_sort_rows(1, buf, i64(1), i64(70000), buf, None, None, None) == -2 and b"65536" in lib.agmi_last_error()
    assert lib.agmi_sort_rows(7, buf, i64(1), i64(8), buf, None, None, None) == -1 and b"floating" in lib.agmi_last_error()


def test_the_source_of_a_specialised_program_compiles_for_gfx950():
    """``agmi_program_source``: the straight-line kernel a recurring program is compiled to, here for a program with
    one-rule, two-rule and long functors, a mask, a row sum and two outputs.  The run-time compiler needs no GPU, so
    this checks on the CPU that the text the library generates (and the headers it carries inside) compiles for
    gfx950 with the library's own flags."""
    from autograd_amd import _lib
    from autograd_amd._lib import Op

    def W(op, dst, a=0, b=0, c=0, d=0):
        return op | dst << 8 | a << 12 | b << 16 | c << 20 | d << 24

    words = [W(Op.MUL, 2, 0, 1), W(Op.EXP, 3, 2), W(Op.MUL_ADD, 4, 3, 0, 15), W(_lib.PROGRAM_MASK, 5, 4, 0, 3),
             W(_lib.PROGRAM_ROWSUM, 6, 5), W(Op.TANH, 7, 6), W(Op.POW, 8, 7, 14), W(Op.SUB_MUL, 9, 8, 0, 1),
             W(Op.LSE_VJP, 10, 9, 0, 1, 2), W(_lib.PROGRAM_STORE, 10, 10, 0), W(_lib.PROGRAM_STORE, 7, 7, 1)]
    try:
        rtc = ctypes.CDLL("libhiprtc.so")
    except OSError:
        rtc = ctypes.CDLL("/opt/rocm/lib/libhiprtc.so")
    for code, name in ((0, "float"), (1, "double")):
        source = _lib.program_source(code, 2, 2, words, 16, row_sums=True)
        assert f"typedef {name} T;" in source and "FLseVjp<T>::apply" in source and "row_values" in source
        assert source.count("// instruction") == len(words)
        prog = ctypes.c_void_p()
        assert rtc.hiprtcCreateProgram(ctypes.byref(prog), source.encode(), b"agmi_specialized.hip", 0, None, None) == 0
        options = [o.encode() for o in ("--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
                                        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")]
        rc = rtc.hiprtcCompileProgram(prog, len(options), (ctypes.c_char_p * len(options))(*options))
        n = ctypes.c_size_t()
        rtc.hiprtcGetProgramLogSize(prog, ctypes.byref(n))
        log = ctypes.create_string_buffer(n.value + 1)
        rtc.hiprtcGetProgramLog(prog, log)
        assert rc == 0, log.value.decode()[:2000]
        rtc.hiprtcGetCodeSize(prog, ctypes.byref(n))
        assert n.value > 1000
        rtc.hiprtcDestroyProgram(ctypes.byref(prog))
    with pytest.raises(_lib.AgmiError, match="unknown op"):
        _lib.program_source(0, 1, 0, [W(200, 1, 0)], 16)


def test_device_path_fails_loudly_without_gpu():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import autograd_amd.numpy as np

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        np.ones((2, 2))
