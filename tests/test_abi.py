"""CPU-side checks of the drop-in boundary: the shared library loads without a GPU and exports
every entry point include/mi355_tensor.h declares; host-side argument checks that need no device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import mi355tensor as mt
    if not os.path.exists(mt.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return mt.lib()


def test_every_declared_symbol_is_exported(lib):
    import mi355tensor as mt
    names = mt.exported_symbols()
    assert len(names) >= 45
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_header_cites_the_reference_for_every_op():
    header = open(os.path.join(ROOT, "include", "mi355_tensor.h")).read()
    for decl in re.findall(r"^int (mt_[a-z0-9_]+)\(", header, re.M):
        if decl in ("mt_init", "mt_malloc", "mt_free", "mt_copy_h2d", "mt_copy_d2h", "mt_copy_d2d", "mt_synchronize", "mt_set_stream", "mt_set_option", "mt_get_info"):
            continue
        pos = header.index("int " + decl + "(")
        # the comment attached to the declaration: from the end of the previous declaration to the end of this one (a
        # group of declarations under one comment, such as the two norm-folding calls, shares that comment)
        end = header.index(";", pos)
        end = header.find("\n", end) if header.find("\n", end) >= 0 else len(header)
        start = pos
        while True:
            prev = header.rfind(";", 0, start)
            start = prev if prev >= 0 else 0
            block = header[start:end]
            if "/*" in block or prev < 0:
                break
        attached = header[start:end]
        # a citation of the function it replaces, or the statement that the reference has no such function
        assert re.search(r"(cuda|cpu|netlayer)/[a-z_.]+:\d+|:\d{3,4}|[Nn]o counterpart in the reference", attached), decl


def test_python_binding_covers_the_header():
    import mi355tensor as mt
    src = open(os.path.join(ROOT, "cuda-cnn-gan-vae_amd", "mi355tensor.py")).read()
    unbound = [n for n in mt.exported_symbols() if '"%s"' % n not in src and n not in ("mt_last_error", "mt_get_stream")]
    assert not unbound, unbound


def test_last_error_is_a_string(lib):
    lib.mt_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.mt_last_error(), bytes)
