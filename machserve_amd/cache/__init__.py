"""The cache: pools of page ids and of state slots, the manager that sorts layers into groups and hands out
pages, and the device memory behind them.

The pools and the manager's bookkeeping are the native host runtime's (``csrc/host/cache.hpp``).  ``BlockPool``
follows the reference's allocator (``crates/mach-model/src/paged_kv.rs:229-289``): a LIFO free list over a bump
pointer, with a bitmap of live pages so that freeing a page twice, or one that was never handed out, fails at
once.  ``SlotPool`` hands out indices into the per-request arrays of fixed size, lowest free index first.
``OutOfPages`` (a ``CacheError``) says that a request's next tokens do not fit: the scheduler decides who gives
pages back.
"""
from ..kernels.build import ensure_host_module

_host = ensure_host_module()
BlockPool, SlotPool, CacheCore = _host.BlockPool, _host.SlotPool, _host.CacheCore
CacheError, OutOfPages = _host.CacheError, _host.OutOfPages

from .manager import CacheManager, GroupSpec, KVBinding, StateBinding, group_name, pages_by_need  # noqa: E402
from .device import DeviceCache  # noqa: E402

__all__ = ["BlockPool", "CacheCore", "CacheError", "OutOfPages", "SlotPool", "CacheManager", "GroupSpec", "KVBinding",
           "StateBinding", "group_name", "pages_by_need", "DeviceCache"]
