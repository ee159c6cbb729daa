"""TEST INFRASTRUCTURE: loader for the reference's own CPU extension modules
built by oracle/build_ref.py into oracle/_ref/.  `available()` is False when
they have not been built (the recipe needs the reference checkout)."""
import importlib.util
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_DIR = os.path.join(_HERE, "_ref")
_cache = {}


def available(name="_mapped_convolution"):
    return os.path.exists(os.path.join(_DIR, name + ".so"))


def module(name):
    """Import oracle/_ref/<name>.so (e.g. '_mapped_convolution')."""
    if name not in _cache:
        import torch  # noqa: F401  (the modules link against libtorch)
        path = os.path.join(_DIR, name + ".so")
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _cache[name] = mod
    return _cache[name]
