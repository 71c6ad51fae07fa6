"""``load_ext('_ext', names)`` as the reference offers it (DFA3D/dfa3D/ext_loader.py:25-29):
returns the module holding the native entry points after checking that each name exists.
Here that module is ``dfa3D._ext``, a ctypes front end of libdfa3d_hip.so."""
import importlib


def load_ext(name, funcs):
    ext = importlib.import_module("dfa3D." + name)
    for fun in funcs:
        assert hasattr(ext, fun), f"{fun} miss in module {name}"
    # fail here, not at the first call, if the HIP library has not been built
    from . import _lib
    _lib.lib()
    return ext


def check_ops_exist():
    import os
    from . import _lib
    return os.path.exists(_lib.LIB_PATH)
