"""PJRT plugin on the GPU: host <-> device round trips, events, compile + execute, serialize ->
deserialize -> execute, a fused kernel through the plugin, asynchronous transfers in flight
(tests/pjrt/pjrt_driver.cpp, gpu mode); once more with METALHLO_PJRT_SYNC_TRANSFERS=1, where
every transfer completes inside its call."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "metalhlo_amd", "lib", "libPJRTMetalHLO.so")
DRIVER = os.path.join(ROOT, "tests", "pjrt", "pjrt_driver")

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("sync,graph", [("0", "0"), ("1", "0"), ("0", "1")], ids=["async", "sync", "async+graph"])
def test_driver_gpu_cases(sync, graph):
    """The third run replays executions as HIP graphs (captured on the stream the transfer thread's
    copies also use) while transfers are asynchronous; its last case executes while a second
    thread uploads and downloads on the same client, and two threads execute two programs on the one
    client while graphs are captured."""
    assert os.path.exists(PLUGIN) and os.path.exists(DRIVER), "plugin / driver not built"
    env = dict(os.environ, METALHLO_PJRT_SYNC_TRANSFERS=sync, METALHLO_HIP_GRAPH=graph)
    r = subprocess.run([DRIVER, PLUGIN, "gpu"], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    for case in ("table", "errors", "platform", "compile", "round_trip", "execute", "async_transfers",
                 "execute_while_transferring", "two_programs_two_threads", "all"):
        assert f"ok {case}\n" in r.stdout, r.stdout
    print(r.stdout)
