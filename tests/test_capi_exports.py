"""The C-ABI library loads on a machine without a GPU and exports every symbol include/born_rocm.h
declares; the ctypes binding covers exactly that set.  No compute call is made here."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    src = open(os.path.join(ROOT, "include", "born_rocm.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(born_rocm_\w+)\s*\(", src)))


def test_header_symbols_are_exported():
    from born_amd import _capi
    assert os.path.exists(_capi.LIB_PATH), "build the library first: python -m born_amd.build"
    lib = ctypes.CDLL(_capi.LIB_PATH)
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/born_rocm.h but not exported"
    assert sorted(_capi.SYMBOLS) == names


def test_last_error_is_thread_local_string():
    from born_amd import _capi
    msg = _capi.lib().born_rocm_last_error()
    assert isinstance(msg, bytes)


def test_argument_checks_need_no_gpu():
    # pure host-side validation paths return before any HIP call
    from born_amd import _capi
    L = _capi.lib()
    assert L.born_rocm_sampler_create(None, 0, 10, None) == _capi.ERR_ARGUMENT
    assert b"null output" in L.born_rocm_last_error()
    assert L.born_rocm_sampler_set_path(None, 0) == _capi.ERR_ARGUMENT
    assert L.born_rocm_sampler_set_step(None, 0) == _capi.ERR_ARGUMENT
    assert L.born_rocm_sampler_get_step(None, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_expneg(None, None, 0, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_sampler_destroy(None) == _capi.OK


def test_product_package_never_touches_the_oracle():
    # the product path must not import, link or execute anything under oracle/
    pkg = os.path.join(ROOT, "born_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f


def test_broadcast_shape_rule_on_the_host():
    # born_rocm_broadcast_shape is pure host logic (tensor.BroadcastShapes, internal/tensor/shape.go:83-118):
    # checked here against numpy's rule, with the reference's message for incompatible shapes
    import numpy as np
    from born_amd import _capi
    L = _capi.lib()

    def arr(shape):
        return (ctypes.c_int64 * max(len(shape), 1))(*shape)

    cases = [((2, 3), (2, 3)), ((3, 1), (4,)), ((2, 3), (1,)), ((2, 1, 4), (5, 1)), ((), (2, 3)), ((7,), ()), ((1, 1, 6), (6,)),
             ((3, 1, 2, 1), (4, 1, 5))]
    for a, b in cases:
        nd = max(len(a), len(b))
        out = (ctypes.c_int64 * max(nd, 1))()
        assert L.born_rocm_broadcast_shape(arr(a), len(a), arr(b), len(b), out) == _capi.OK, (a, b)
        assert tuple(out[i] for i in range(nd)) == np.broadcast_shapes(a, b), (a, b)
    out = (ctypes.c_int64 * 2)()
    assert L.born_rocm_broadcast_shape(arr((2, 3)), 2, arr((4,)), 1, out) == _capi.ERR_ARGUMENT
    assert L.born_rocm_last_error() == b"broadcast: shapes not compatible for broadcasting: [2 3] vs [4] (dimension 1: 3 vs 4)"
    assert L.born_rocm_broadcast_shape(arr((2, 0)), 2, arr((4,)), 1, out) == _capi.ERR_ARGUMENT      # empty extent
    assert L.born_rocm_broadcast_shape(arr((1,) * 9), 9, arr((4,)), 1, out) == _capi.ERR_ARGUMENT    # too many dimensions


def test_producer_and_backend_argument_checks_need_no_gpu():
    from born_amd import _capi
    L = _capi.lib()
    one = (ctypes.c_int64 * 1)(4)
    assert L.born_rocm_linear(None, 1, 1, 1, None, 1, 1, None, None, 1, None) == _capi.ERR_ARGUMENT
    assert b"linear: null pointer" in L.born_rocm_last_error()
    buf = ctypes.create_string_buffer(64)                 # never dereferenced: the checks below fail first
    p = ctypes.addressof(buf)
    assert L.born_rocm_matmul(p, p, p, 2, 0, 2, 2, 2, 2, None) == _capi.ERR_ARGUMENT
    assert b"matmul: shape" in L.born_rocm_last_error()
    assert L.born_rocm_matmul(p, p, p, 2, 2, 2, 1, 2, 2, None) == _capi.ERR_ARGUMENT
    assert b"row pitch" in L.born_rocm_last_error()
    assert L.born_rocm_add(None, one, 1, None, one, 1, None, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_transpose(p, (ctypes.c_int64 * 2)(2, 3), 2, (ctypes.c_int32 * 2)(0, 0), p, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_last_error() == b"transpose: duplicate axis 0"
    assert L.born_rocm_transpose(p, (ctypes.c_int64 * 2)(2, 3), 2, (ctypes.c_int32 * 2)(0, 2), p, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_last_error() == b"transpose: invalid axis 2 for 2D tensor"
    assert L.born_rocm_reshape(p, (ctypes.c_int64 * 2)(2, 3), 2, (ctypes.c_int64 * 2)(4, 2), 2, p, None) == _capi.ERR_ARGUMENT
    assert L.born_rocm_last_error() == b"reshape: incompatible shapes: [2 3] -> [4 2] (different number of elements)"
    assert L.born_rocm_spec_verify_bonus(None, None, 0, None, 0, None, 0, 1, 1, 1, None, None, None, None, None, None) == _capi.ERR_ARGUMENT


def test_struct_layouts_of_the_binding_match_the_header(tmp_path):
    # the two structs that cross the boundary: sizes and member offsets as the C compiler lays them out, against the
    # ctypes mirrors (and the C++ wrapper compiles against the same header)
    import subprocess
    from born_amd import _capi
    structs = {"born_sampler_config": _capi.SamplerConfigC, "born_sampler_row_configs": _capi.RowConfigsC}
    lines = []
    for name, cls in structs.items():
        lines.append(f'printf("{name} %zu\\n", sizeof({name}));')
        for field, _ in cls._fields_:
            lines.append(f'printf("{name}.{field} %zu\\n", offsetof({name}, {field}));')
    src = tmp_path / "layout.c"
    src.write_text('#include <stddef.h>\n#include <stdio.h>\n#include "born_rocm.h"\nint main(void) {\n' + "\n".join(lines) +
                   "\nreturn 0;\n}\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = dict(line.split() for line in subprocess.check_output([str(exe)], text=True).splitlines())
    for name, cls in structs.items():
        assert int(got[name]) == ctypes.sizeof(cls), name
        for field, _ in cls._fields_:
            assert int(got[f"{name}.{field}"]) == getattr(cls, field).offset, (name, field)
    # every member of the header's structs is mirrored (no field left out at the end)
    hdr = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "born_rocm.h")).read(), flags=re.S)
    for name, cls in structs.items():
        body = re.search(r"typedef struct " + name + r" \{(.*?)\} " + name + ";", hdr, flags=re.S).group(1)
        members = re.findall(r"(\w+)\s*;", body)
        assert members == [f for f, _ in cls._fields_], (name, members)
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), "-x", "c++",
                           os.path.join(ROOT, "include", "born_rocm.hpp")], stderr=subprocess.DEVNULL)
