"""The JAX registration hook (`jax_mps_amd.initialize`, the entry point of the `jax_plugins` group) driven without
jax: a stand-in `jax` / `jax._src.xla_bridge` pair in `sys.modules` records what the hook asks of it.  Mirrors what
the reference's hook does (src/jax_plugins/mps/__init__.py:94-148): library search with an environment override,
shardy switched off, `register_plugin(name, priority=500, library_path=..., options=None)`, a second registration
tolerated, anything else reported as the plugin's own error; and its jaxlib version guard (:63-91)."""
import sys
import types
import warnings

import pytest

import jax_mps_amd


class _Bridge(types.ModuleType):
    def __init__(self, fail_with=None, has_register=True):
        super().__init__("jax._src.xla_bridge")
        self.calls = []
        self.fail_with = fail_with
        if has_register:
            self.register_plugin = self._register_plugin

    def _register_plugin(self, name, *, priority=400, library_path=None, options=None, c_api=None):
        if any(c["name"] == name for c in self.calls):
            raise RuntimeError(f"ALREADY_EXISTS: PJRT_Api already exists for device type {name}")
        if self.fail_with:
            raise RuntimeError(self.fail_with)
        self.calls.append(dict(name=name, priority=priority, library_path=library_path, options=options))


@pytest.fixture
def fake_jax(monkeypatch):
    def install(**kw):
        bridge = _Bridge(**kw)
        jax = types.ModuleType("jax")
        jax.__version__ = "0.10.0"
        updates = []
        jax.config = types.SimpleNamespace(update=lambda k, v: updates.append((k, v)))
        src = types.ModuleType("jax._src")
        src.xla_bridge = bridge
        jax._src = src
        monkeypatch.setitem(sys.modules, "jax", jax)
        monkeypatch.setitem(sys.modules, "jax._src", src)
        monkeypatch.setitem(sys.modules, "jax._src.xla_bridge", bridge)
        bridge.config_updates = updates
        return bridge
    monkeypatch.delenv("MI355X_PJRT_LIBRARY_PATH", raising=False)
    return install


def test_initialize_registers_the_built_library(fake_jax):
    bridge = fake_jax()
    jax_mps_amd.initialize()
    lib = jax_mps_amd.find_library()
    assert lib and lib.endswith(jax_mps_amd.LIB_NAME)
    assert bridge.calls == [dict(name="mi355x", priority=500, library_path=lib, options=None)]
    assert ("jax_use_shardy_partitioner", False) in bridge.config_updates


def test_second_initialize_is_tolerated(fake_jax):
    bridge = fake_jax()
    jax_mps_amd.initialize()
    jax_mps_amd.initialize()          # the bridge raises ALREADY_EXISTS for mi355x: not an error
    assert len(bridge.calls) == 1


def test_other_registration_failures_are_reported(fake_jax):
    fake_jax(fail_with="INVALID_ARGUMENT: struct_size mismatch")
    with pytest.raises(jax_mps_amd.Mi355xPluginError, match="struct_size mismatch"):
        jax_mps_amd.initialize()


def test_bridge_without_register_plugin(fake_jax):
    fake_jax(has_register=False)
    with pytest.raises(jax_mps_amd.Mi355xPluginError, match="register_plugin"):
        jax_mps_amd.initialize()


def test_environment_override(fake_jax, monkeypatch, tmp_path):
    bridge = fake_jax()
    other = tmp_path / "elsewhere.so"
    other.write_bytes(b"")
    monkeypatch.setenv("MI355X_PJRT_LIBRARY_PATH", str(other))
    jax_mps_amd.initialize()
    assert bridge.calls[0]["library_path"] == str(other)
    monkeypatch.setenv("MI355X_PJRT_LIBRARY_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(jax_mps_amd.Mi355xPluginError, match="names no file"):
        jax_mps_amd.initialize()


def test_missing_library_is_an_error(fake_jax, monkeypatch):
    fake_jax()
    monkeypatch.setattr(jax_mps_amd, "_candidate_libraries", lambda: iter(()))
    with pytest.raises(jax_mps_amd.Mi355xPluginError, match="build it"):
        jax_mps_amd.initialize()


def test_missing_jax_is_an_error(monkeypatch):
    monkeypatch.setitem(sys.modules, "jax", None)       # makes `import jax` raise ImportError
    with pytest.raises(jax_mps_amd.Mi355xPluginError, match="jax is not importable"):
        jax_mps_amd.initialize()


@pytest.mark.parametrize("installed, warns", [("0.10.3", False), ("0.9.1", True), ("0.11.0", True), ("garbage", False), (None, False)])
def test_jaxlib_version_guard(monkeypatch, installed, warns):
    def version(name):
        assert name == "jaxlib"
        if installed is None:
            raise jax_mps_amd.metadata.PackageNotFoundError(name)
        return installed
    monkeypatch.setattr(jax_mps_amd.metadata, "version", version)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        jax_mps_amd.check_jaxlib_version()
    assert bool(caught) == warns
    if warns:
        assert "jaxlib 0.10.x" in str(caught[0].message) and installed in str(caught[0].message)
