"""Device registry (counterpart of the reference's device.py:5-29).

`Device.get_allocator(name)` / `Device.get_backend(name)` hand out per-name
singletons; an unknown name raises ValueError.  The package ships exactly one
device, "hip".  It has no CPU execution path: if the native extension is not
built or no gfx950 GPU is visible, asking for "hip" raises.  Other devices can
be plugged in with `Device.register` (the test-suite registers its numpy oracle
as "cpu" that way).
"""
from __future__ import annotations

_hip_ctx = None


def hip_context():
    """The process-wide hip_ext.HipContext (device 0), created on first use."""
    global _hip_ctx
    if _hip_ctx is None:
        try:
            from . import hip_ext
        except ImportError as exc:
            raise RuntimeError(
                "autograd_amd.hip_ext is not built: run `python -m autograd_amd.build` "
                "(there is no CPU fallback for the 'hip' device)") from exc
        _hip_ctx = hip_ext.HipContext(0)
    return _hip_ctx


class Device:
    _allocators = {}
    _backends = {}
    _factories = {}

    @classmethod
    def register(cls, device_name, allocator_factory, backend_factory):
        cls._factories[device_name] = (allocator_factory, backend_factory)
        cls._allocators.pop(device_name, None)
        cls._backends.pop(device_name, None)

    @classmethod
    def get_allocator(cls, device_name):
        if device_name not in cls._allocators:
            if device_name == "hip":
                from .storage import HipAllocator
                cls._allocators[device_name] = HipAllocator()
            elif device_name in cls._factories:
                cls._allocators[device_name] = cls._factories[device_name][0]()
            else:
                raise ValueError(f"Unknown device: {device_name}")
        return cls._allocators[device_name]

    @classmethod
    def get_backend(cls, device_name):
        if device_name not in cls._backends:
            if device_name == "hip":
                from .backend import HipBackend
                cls._backends[device_name] = HipBackend()
            elif device_name in cls._factories:
                cls._backends[device_name] = cls._factories[device_name][1]()
            else:
                raise ValueError(f"Unknown device: {device_name}")
        return cls._backends[device_name]
