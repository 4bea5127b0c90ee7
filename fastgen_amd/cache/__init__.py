from .manager import RELEASED, CacheManager, OutOfPages, OutOfSlots

__all__ = ["RELEASED", "CacheManager", "OutOfPages", "OutOfSlots", "CacheStorage", "CacheGroup", "group_entries"]


def __getattr__(name):  # the storage needs torch tensors on a device; the manager does not
    if name in ("CacheStorage", "CacheGroup", "group_entries"):
        from . import storage

        return getattr(storage, name)
    raise AttributeError(name)
