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
