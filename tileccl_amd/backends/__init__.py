from tileccl_amd.backends.hip import DeviceProperties, HIPBackend, get_backend

__all__ = ["DeviceProperties", "HIPBackend", "get_backend"]
