"""The C-ABI library loads without a GPU and exports every entry point include/*.h declares."""
import ctypes
import glob
import os
import re

from rustane_amd import hipdec

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = open(h).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(hipdec_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(hipdec._LIB_PATH)
    decl = declared_symbols()
    assert len(decl) >= 19
    for name in sorted(decl):
        assert hasattr(lib, name), "libhipdecode.so does not export %s" % name
    assert decl == set(hipdec.EXPORTS), decl ^ set(hipdec.EXPORTS)


def test_create_rejects_bad_arguments_without_touching_a_gpu():
    lib = hipdec.load_library()
    out = ctypes.c_void_p()
    assert lib.hipdec_create(None, None, 0, None, None, ctypes.byref(out)) == hipdec.ERR_ARG
    assert not out.value
    assert b"null" in lib.hipdec_last_error(None)
    assert lib.hipdec_len(None) == 0
    assert lib.hipdec_set_len(None, 3) == hipdec.ERR_ARG
