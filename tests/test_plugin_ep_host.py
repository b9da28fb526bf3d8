"""CPU-side checks of the plugin execution provider: the library loads, exports the two entry points ONNX Runtime
looks up, and answers the factory-level queries that need no GPU."""
import ctypes
import subprocess

import pytest

from ep_host import host

pytestmark = pytest.mark.skipif(not host.available(), reason="plugin EP or host shim not built "
                                                             "(needs the ONNX Runtime C API headers)")


def test_plugin_exports_entry_points():
    out = subprocess.run(["nm", "-D", "--defined-only", str(host.PLUGIN)], capture_output=True, text=True, check=True)
    exported = {l.split()[-1] for l in out.stdout.splitlines() if " T " in l}
    assert exported == {"CreateEpFactories", "ReleaseEpFactory"}
    lib = ctypes.CDLL(str(host.PLUGIN))
    assert lib.CreateEpFactories and lib.ReleaseEpFactory


def test_factory_identity():
    info = host.probe_factory(offer_amd_gpu=False)
    assert info["name"] == "Mi355xExecutionProvider"
    assert info["vendor"] == "AMD" and info["vendor_id"] == 0x1002
    assert info["stream_aware"] is True
    # a CPU and an NVIDIA GPU are never claimed
    assert info["num_ep_devices"] == 0


def test_factory_offers_only_visible_gpus():
    import torch
    info = host.probe_factory(offer_amd_gpu=True)
    assert info["num_ep_devices"] == (1 if torch.cuda.is_available() else 0)
