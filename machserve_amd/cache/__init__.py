from .pool import BlockPool, CacheError, OutOfPages, SlotPool
from .manager import CacheManager, GroupSpec, KVBinding, StateBinding, group_name
from .device import DeviceCache

__all__ = ["BlockPool", "CacheError", "OutOfPages", "SlotPool", "CacheManager", "GroupSpec", "KVBinding",
           "StateBinding", "group_name", "DeviceCache"]
