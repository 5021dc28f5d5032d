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
from pathlib import Path

PLATFORM_NAME = "mi355x"
LIB_NAME = "libpjrt_plugin_mi355x.so"
_PKG_DIR = Path(os.path.dirname(os.path.abspath(__file__)))


class Mi355xPluginError(RuntimeError):
    pass


def find_library() -> str | None:
    """Environment override first, then next to this package (reference: __init__.py:37-61)."""
    env = os.environ.get("MI355X_PJRT_LIBRARY_PATH")
    if env is not None:
        if Path(env).exists():
            return env
        raise Mi355xPluginError(f"MI355X_PJRT_LIBRARY_PATH is set to '{env}', but the file does not exist.")
    for cand in (_PKG_DIR / LIB_NAME, _PKG_DIR / "lib" / LIB_NAME, Path("/usr/local/lib") / LIB_NAME):
        if cand.exists():
            return str(cand)
    return None


def initialize() -> None:
    """Register the plugin with JAX (raises Mi355xPluginError when that is impossible)."""
    library_path = find_library()
    if library_path is None:
        raise Mi355xPluginError(f"Could not find {LIB_NAME} next to {_PKG_DIR}; set MI355X_PJRT_LIBRARY_PATH or build the library.")
    try:
        from jax._src import xla_bridge as xb
    except ImportError as e:
        raise Mi355xPluginError(f"Failed to import JAX xla_bridge: {e}") from e
    if not hasattr(xb, "register_plugin"):
        raise Mi355xPluginError("JAX version does not support register_plugin API.")
    try:
        import jax
        # the front end reads StableHLO, not the sdy dialect (reference: __init__.py:120-131)
        jax.config.update("jax_use_shardy_partitioner", False)
    except Exception:
        pass
    try:
        xb.register_plugin(PLATFORM_NAME, priority=500, library_path=library_path, options=None)
    except Exception as e:
        if not ("ALREADY_EXISTS" in str(e) and PLATFORM_NAME in str(e).lower()):
            raise Mi355xPluginError(f"Failed to register the {PLATFORM_NAME} plugin with JAX: {e}") from e


def build_library(force: bool = True, jobs: int = 8) -> str:
    """Compile csrc/ into the plugin library and the ahead-of-time kernel compiler (gfx950)."""
    cmd = ["make", "-C", str(_PKG_DIR / "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise Mi355xPluginError("building the plugin failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return str(_PKG_DIR / LIB_NAME)


def aot_compile(mlir_paths, quiet: bool = True) -> str:
    """Cross-compile the fused kernels of StableHLO text files into the kernel cache (no GPU needed)."""
    tool = _PKG_DIR / "mi355x-aot"
    r = subprocess.run([str(tool)] + [str(p) for p in mlir_paths], capture_output=True, text=True)
    if r.returncode != 0:
        raise Mi355xPluginError("ahead-of-time kernel compilation failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return r.stdout
