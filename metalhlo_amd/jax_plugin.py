"""JAX entry point for the PJRT plugin: `initialize()` registers libPJRTMetalHLO.so as the
"metalhlo" backend, as the reference's python/jax_plugins/metalhlo/__init__.py:13-69 does for
its dylib -- same backend name and priority (500), same METALHLO_PLUGIN_PATH override, same
METALHLO_PYTHON default (the interpreter the plugin starts to turn MLIR bytecode into text must
be the one that has jaxlib), and a second call is a no-op once the plugin is loaded.

JAX finds it through the `jax_plugins` entry-point group:

    [project.entry-points.'jax_plugins']
    metalhlo = "metalhlo_amd.jax_plugin"

or call `metalhlo_amd.jax_plugin.initialize()` before the first JAX computation.  jax and jaxlib
are imported inside `initialize()` only: importing this module needs neither.
"""
import os
import sys

PLUGIN_NAME = "metalhlo"
PRIORITY = 500
LIBRARY = "libPJRTMetalHLO.so"


def library_candidates():
    """Where the shared library is looked for, in order: METALHLO_PLUGIN_PATH, next to this
    module (a packaged copy), the in-tree build output."""
    here = os.path.dirname(os.path.abspath(__file__))
    out = [os.path.join(here, LIBRARY), os.path.join(here, "lib", LIBRARY)]
    env = os.environ.get("METALHLO_PLUGIN_PATH")
    if env:
        out.insert(0, env)
    return out


def find_library():
    for path in library_candidates():
        real = os.path.realpath(path)
        if os.path.isfile(real):
            return real
    raise RuntimeError(
        f"Could not find {LIBRARY}. Build it with `python -c \"import __graft_entry__ as g; g.build()\"` "
        "or set METALHLO_PLUGIN_PATH to its location.")


def initialize():
    """Registers the plugin with JAX's PJRT backend system."""
    import jax._src.xla_bridge as xb
    import jaxlib.xla_client as xla_client

    os.environ.setdefault("METALHLO_PYTHON", sys.executable)
    loaded = getattr(xla_client, "pjrt_plugin_loaded", None)
    if loaded is not None and loaded(PLUGIN_NAME):      # registering twice is an ALREADY_EXISTS error in recent JAX
        return
    xb.register_plugin(PLUGIN_NAME, priority=PRIORITY, library_path=find_library(), options=None)
