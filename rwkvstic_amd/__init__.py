"""MI355X-native FASTQUANT RWKV-4 forward path.

``RWKV(path)`` / ``RWKVMaster`` mirror the reference's user API, ``HipRWKV`` its inner model,
``ops`` its three native operators; everything runs in ``librwkv_hip.so`` (C ABI: include/rwkv_hip.h).
Submodules are imported on first use so that ``import rwkvstic_amd`` stays light.
"""

__all__ = ["RWKV", "RWKVMaster", "HipRWKV"]


def __getattr__(name):
    if name in ("RWKV", "RWKVMaster"):
        from . import master
        return getattr(master, name)
    if name == "HipRWKV":
        from .model import HipRWKV
        return HipRWKV
    raise AttributeError(name)
