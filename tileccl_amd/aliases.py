"""The reference's import names for this package.

Every caller of the reference starts with ``import tileccl``, ``from tileccl_v2 import ...`` or
``from tileccl.memory.symmetric_heap import SymmetricHeap`` (``/root/reference/README.md:128,141-145``,
``tests/test_gemm_allscatter_smoke.py:9,20``, ``examples/benchmark_patterns.py:19-26``).  After

    import tileccl_amd
    tileccl_amd.install_aliases()

those statements resolve to this package: ``tileccl`` and any ``tileccl.<x>`` is ``tileccl_amd``
resp. ``tileccl_amd.<x>``, ``tileccl_v2`` and any ``tileccl_v2.<x>`` is ``tileccl_amd.v2`` resp.
``tileccl_amd.v2.<x>``.  An alias is the very module object of the real name, so classes imported
under either name are the same classes.  Nothing is aliased until the call, and the call refuses to
shadow a ``tileccl`` / ``tileccl_v2`` that is really installed unless ``force=True``.
"""

from __future__ import annotations

import importlib
import importlib.abc
import importlib.machinery
import importlib.util
import sys

_ROOTS = {"tileccl": "tileccl_amd", "tileccl_v2": "tileccl_amd.v2"}
# Parts of this package that have no counterpart under the reference's names.
_PRIVATE = ("tileccl_amd.csrc", "tileccl_amd.aliases", "tileccl_amd.v2.calibrate", "tileccl_amd.v2.fused")


def real_name(alias: str) -> str | None:
    """``tileccl.ops`` -> ``tileccl_amd.ops``, ``tileccl_v2.wg`` -> ``tileccl_amd.v2.wg``; None for other names."""
    root, _, rest = alias.partition(".")
    if root not in _ROOTS:
        return None
    if root == "tileccl" and rest.split(".")[0] == "v2":
        return None  # the reference has no tileccl.v2
    name = _ROOTS[root] + ("." + rest if rest else "")
    if any(name == p or name.startswith(p + ".") for p in _PRIVATE):
        return None
    return name


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    """Resolves an aliased name to the module of its real name (imported on demand)."""

    def find_spec(self, fullname, path=None, target=None):
        if fullname.partition(".")[0] not in _ROOTS:
            return None
        # Names under the aliased roots are answered here and nowhere else: left to the path finder, a name
        # without a counterpart would be looked up in this package's directories and loaded a second time.
        name = real_name(fullname)
        try:
            found = name is not None and importlib.util.find_spec(name) is not None
        except ModuleNotFoundError:
            found = False
        if not found:
            raise ModuleNotFoundError(f"No module named {fullname!r}", name=fullname)
        return importlib.machinery.ModuleSpec(fullname, self, is_package=None)

    def create_module(self, spec):
        return importlib.import_module(real_name(spec.name))

    def exec_module(self, module):  # already executed under its real name
        pass


_finder: _AliasFinder | None = None


def _installed_elsewhere(root: str) -> bool:
    for finder in sys.meta_path:
        if isinstance(finder, _AliasFinder):
            continue
        try:
            spec = finder.find_spec(root, None) if hasattr(finder, "find_spec") else None
        except (ImportError, AttributeError, ValueError):
            spec = None
        if spec is not None:
            return True
    return False


def install_aliases(force: bool = False) -> None:
    """Make ``tileccl`` / ``tileccl_v2`` (and their submodules) importable as aliases of this package.

    Raises ``ImportError`` if a distribution of that name is importable already (``force=True``
    shadows it for this process).  Calling it twice is harmless.
    """
    global _finder
    if _finder is not None:
        return
    for root in _ROOTS:
        loaded = sys.modules.get(root)
        if loaded is not None and loaded is not sys.modules.get(_ROOTS[root]) and not force:
            raise ImportError(f"a module named {root!r} is already imported from {getattr(loaded, '__file__', '?')}; "
                              f"pass force=True to replace it with tileccl_amd")
        if loaded is None and not force and _installed_elsewhere(root):
            raise ImportError(f"a package named {root!r} is installed; pass force=True to shadow it with tileccl_amd")
    _finder = _AliasFinder()
    sys.meta_path.insert(0, _finder)
    for root, name in _ROOTS.items():
        if force:
            for key in [k for k in sys.modules if k == root or k.startswith(root + ".")]:
                del sys.modules[key]
        sys.modules[root] = importlib.import_module(name)
    # Submodules that are loaded already get their alias at once (an `import tileccl.ops` would find it
    # through the finder as well; attribute access `tileccl.ops` works either way).
    for key, module in list(sys.modules.items()):
        for root, name in _ROOTS.items():
            if key.startswith(name + "."):
                alias = root + key[len(name):]
                if real_name(alias) == key:
                    sys.modules.setdefault(alias, module)


def remove_aliases() -> None:
    """Undo ``install_aliases`` (used by the tests)."""
    global _finder
    if _finder is None:
        return
    sys.meta_path.remove(_finder)
    _finder = None
    for key in [k for k in sys.modules if k.split(".")[0] in _ROOTS]:
        del sys.modules[key]
