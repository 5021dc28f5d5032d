"""MI355X PJRT plugin: Python side.

`initialize()` is what JAX's plugin discovery calls (entry-point group
`jax_plugins`); it locates `libpjrt_plugin_mi355x.so` and registers it under the
platform name "mi355x", so `JAX_PLATFORMS=mi355x` runs jitted programs through
the library's PJRT C API.  It mirrors the reference's
src/jax_plugins/mps/__init__.py:94-148 (library search with an environment
override, `xla_bridge.register_plugin(name, priority=500, library_path=...)`),
minus the macOS checks and the monkey-patches.

Everything else in this package drives the same library without JAX:
`pjrt.py` (ctypes client for the C API), `shlo/` (StableHLO emitter),
`programs/` (the benchmark programs), `runner.py`.
"""
from __future__ import annotations

import os
import subprocess
import warnings
from importlib import metadata
from pathlib import Path

PLATFORM_NAME = "mi355x"
LIB_NAME = "libpjrt_plugin_mi355x.so"
# jaxlib release line whose PJRT C API (0.72) and StableHLO bytecode version the library was written against: the one
# the reference pins (src/jax_plugins/mps/__init__.py:8-10)
BUILT_FOR_JAXLIB = (0, 10)
_PKG_DIR = Path(os.path.dirname(os.path.abspath(__file__)))


class Mi355xPluginError(RuntimeError):
    pass


def _candidate_libraries():
    yield _PKG_DIR / LIB_NAME
    yield _PKG_DIR / "lib" / LIB_NAME
    yield Path("/usr/local/lib") / LIB_NAME


def find_library() -> str | None:
    """Path of the plugin library, or None.  `MI355X_PJRT_LIBRARY_PATH` wins over the search next to this
    package and must then name an existing file (same precedence as the reference's MPS_LIBRARY_PATH,
    src/jax_plugins/mps/__init__.py:37-61)."""
    override = os.environ.get("MI355X_PJRT_LIBRARY_PATH")
    if override is None:
        return next((str(c) for c in _candidate_libraries() if c.exists()), None)
    if not Path(override).is_file():
        raise Mi355xPluginError(f"MI355X_PJRT_LIBRARY_PATH={override!r} names no file")
    return override


def check_jaxlib_version() -> None:
    """Warn when the installed jaxlib is of another major.minor line than the one the library was written against
    (the PJRT function table and the bytecode version both move with it); never fails initialisation.  Mirrors
    src/jax_plugins/mps/__init__.py:63-91."""
    try:
        installed = metadata.version("jaxlib")
        major, minor = (int(x) for x in installed.split(".")[:2])
    except (metadata.PackageNotFoundError, ValueError):
        return
    if (major, minor) != BUILT_FOR_JAXLIB:
        want = "%d.%d" % BUILT_FOR_JAXLIB
        warnings.warn(f"the {PLATFORM_NAME} plugin was written against jaxlib {want}.x but jaxlib {installed} is installed: "
                      f"the PJRT function table or the StableHLO bytecode version may differ "
                      f"(consider jaxlib>={want}.0,<{BUILT_FOR_JAXLIB[0]}.{BUILT_FOR_JAXLIB[1] + 1})", stacklevel=3)


def _register(xla_bridge, library_path: str) -> None:
    try:
        xla_bridge.register_plugin(PLATFORM_NAME, priority=500, library_path=library_path, options=None)
    except Exception as e:   # a second initialize() in one process finds the platform registered already
        text = str(e)
        if "ALREADY_EXISTS" in text and PLATFORM_NAME in text.lower():
            return
        raise Mi355xPluginError(f"jax refused the {PLATFORM_NAME} plugin at {library_path}: {e}") from e


def initialize() -> None:
    """Entry point of the `jax_plugins` group: make `JAX_PLATFORMS=mi355x` resolve to this library.

    Needs jax with `xla_bridge.register_plugin`; anything missing raises Mi355xPluginError so that jax's
    plugin discovery reports it instead of silently running elsewhere."""
    check_jaxlib_version()
    library_path = find_library()
    if library_path is None:
        raise Mi355xPluginError(f"{LIB_NAME} is neither next to {_PKG_DIR} nor named by MI355X_PJRT_LIBRARY_PATH; "
                                "build it with __graft_entry__.build()")
    try:
        import jax
        from jax._src import xla_bridge
    except ImportError as e:
        raise Mi355xPluginError(f"jax is not importable here ({e}); the plugin can still be driven through jax_mps_amd.pjrt") from e
    register = getattr(xla_bridge, "register_plugin", None)
    if register is None:
        raise Mi355xPluginError(f"jax {getattr(jax, '__version__', '?')} predates xla_bridge.register_plugin; a newer jax is needed")
    # the front end reads the stablehlo dialect; with shardy on, jax would emit sdy ops instead
    # (reference: src/jax_plugins/mps/__init__.py:120-131)
    try:
        jax.config.update("jax_use_shardy_partitioner", False)
    except (AttributeError, KeyError, ValueError):
        pass
    _register(xla_bridge, library_path)


def build_library(force: bool = True, jobs: int = 8) -> str:
    """Compile csrc/ into the plugin library and the ahead-of-time kernel compiler (gfx950)."""
    cmd = ["make", "-C", str(_PKG_DIR / "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise Mi355xPluginError("building the plugin failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return str(_PKG_DIR / LIB_NAME)


def aot_compile(mlir_paths, quiet: bool = True, env: dict | None = None) -> str:
    """Cross-compile the fused kernels of StableHLO text files into the kernel cache (no GPU needed).
    `env` adds compile switches (the MI355X_* variables the planner reads at every compile)."""
    tool = _PKG_DIR / "mi355x-aot"
    r = subprocess.run([str(tool)] + [str(p) for p in mlir_paths], capture_output=True, text=True,
                       env={**os.environ, **(env or {})})
    if r.returncode != 0:
        raise Mi355xPluginError("ahead-of-time kernel compilation failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return r.stdout
