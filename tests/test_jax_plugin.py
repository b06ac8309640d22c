"""The JAX entry point without JAX: stand-in `jax._src.xla_bridge` / `jaxlib.xla_client` modules
record what `initialize()` registers.  Restates the contract of the reference's
python/jax_plugins/metalhlo/__init__.py:13-69 (name, priority, path override, idempotence,
METALHLO_PYTHON default)."""
import os
import sys
import types

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "metalhlo_amd", "lib", "libPJRTMetalHLO.so")


@pytest.fixture()
def fake_jax(monkeypatch):
    calls, state = [], {"loaded": False}
    jax, src, xb = types.ModuleType("jax"), types.ModuleType("jax._src"), types.ModuleType("jax._src.xla_bridge")
    jaxlib, xc = types.ModuleType("jaxlib"), types.ModuleType("jaxlib.xla_client")

    def register_plugin(name, priority=400, library_path=None, options=None):
        calls.append(dict(name=name, priority=priority, library_path=library_path, options=options))
        state["loaded"] = True
    xb.register_plugin = register_plugin
    xc.pjrt_plugin_loaded = lambda name: state["loaded"] and name == "metalhlo"
    jax._src, src.xla_bridge, jaxlib.xla_client = src, xb, xc
    for name, mod in (("jax", jax), ("jax._src", src), ("jax._src.xla_bridge", xb), ("jaxlib", jaxlib), ("jaxlib.xla_client", xc)):
        monkeypatch.setitem(sys.modules, name, mod)
    monkeypatch.delenv("METALHLO_PLUGIN_PATH", raising=False)
    monkeypatch.delenv("METALHLO_PYTHON", raising=False)
    return calls


def test_registers_the_built_library_once(fake_jax):
    from metalhlo_amd import jax_plugin
    assert os.path.isfile(PLUGIN), "plugin not built"
    jax_plugin.initialize()
    jax_plugin.initialize()                        # already loaded: no second registration
    assert fake_jax == [dict(name="metalhlo", priority=500, library_path=os.path.realpath(PLUGIN), options=None)]
    assert os.environ["METALHLO_PYTHON"] == sys.executable


def test_path_override_and_missing_library(fake_jax, monkeypatch, tmp_path):
    from metalhlo_amd import jax_plugin
    other = tmp_path / "libPJRTMetalHLO.so"
    other.write_bytes(b"")
    monkeypatch.setenv("METALHLO_PLUGIN_PATH", str(other))
    monkeypatch.setenv("METALHLO_PYTHON", "/usr/bin/python3")      # an explicit choice is kept
    jax_plugin.initialize()
    assert fake_jax[0]["library_path"] == os.path.realpath(str(other))
    assert os.environ["METALHLO_PYTHON"] == "/usr/bin/python3"
    monkeypatch.setattr(jax_plugin, "library_candidates", lambda: [str(tmp_path / "nowhere.so")])
    sys.modules["jaxlib.xla_client"].pjrt_plugin_loaded = lambda name: False
    with pytest.raises(RuntimeError, match="Could not find libPJRTMetalHLO.so"):
        jax_plugin.initialize()


def test_the_library_it_registers_exports_the_pjrt_entry_point():
    import ctypes
    from metalhlo_amd import jax_plugin
    lib = ctypes.CDLL(jax_plugin.find_library())
    assert hasattr(lib, "GetPjrtApi")
