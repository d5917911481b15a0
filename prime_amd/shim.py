"""Make the reference's import paths resolve to this package for the compression path.

The reference imports the path as ``zeroband.C.compression``, ``zeroband.C.collectives`` and
``zeroband.collectives`` (src/zeroband/diloco.py:6,59, src/zeroband/collectives.py:38,
scripts/all_reduce.py:6, tests/test_c/test_compression.py:6, tests/test_c/test_collectives.py:3-5).  ``install()`` puts
this package's modules under those names in ``sys.modules``, so such imports, left as they
are, reach the HIP kernels:

    import prime_amd.shim; prime_amd.shim.install()
    from zeroband.C.compression import uniform_8bit_quantize          # prime_amd.C.compression
    from zeroband.collectives import Compression, all_reduce          # prime_amd.collectives

Only these modules are provided.  If a real ``zeroband`` package is importable it is kept and
the three submodules are replaced inside it; otherwise an empty ``zeroband`` namespace is
created to hold them.
"""
from __future__ import annotations

import importlib
import sys
import types

_TARGETS = {
    "zeroband.C.compression": "prime_amd.C.compression",
    "zeroband.C.collectives": "prime_amd.C.collectives",
    "zeroband.collectives": "prime_amd.collectives",
}


def _package(name: str) -> types.ModuleType:
    """The module ``name`` if it can be imported, else a fresh namespace registered under it."""
    if name in sys.modules:
        return sys.modules[name]
    try:
        return importlib.import_module(name)
    except Exception:
        mod = types.ModuleType(name)
        mod.__path__ = []           # mark as a package so that submodule imports consult sys.modules
        sys.modules[name] = mod
        return mod


def install() -> None:
    """Register the drop-in modules under the reference's names (idempotent)."""
    root = _package("zeroband")
    c_pkg = _package("zeroband.C")
    setattr(root, "C", c_pkg)
    for alias, target in _TARGETS.items():
        mod = importlib.import_module(target)
        sys.modules[alias] = mod
        parent, _, leaf = alias.rpartition(".")
        setattr(sys.modules[parent], leaf, mod)
    # zeroband.config.Compression is what the call site passes (src/zeroband/config.py:10-12); a real
    # zeroband.config, if importable, already defines an enum with the same value strings
    if "zeroband.config" not in sys.modules:
        try:
            importlib.import_module("zeroband.config")
        except Exception:
            cfg = importlib.import_module("prime_amd.config")
            sys.modules["zeroband.config"] = cfg
            setattr(root, "config", cfg)


def uninstall() -> None:
    """Remove what ``install`` registered."""
    for alias in list(_TARGETS) + ["zeroband.config", "zeroband.C", "zeroband"]:
        mod = sys.modules.get(alias)
        if mod is not None and (getattr(mod, "__name__", "").startswith("prime_amd") or not getattr(mod, "__file__", None)):
            del sys.modules[alias]
