"""Pools of page ids and of state slots, from the native host runtime (``csrc/host/cache.hpp``).

``BlockPool`` follows the reference's allocator (``crates/mach-model/src/paged_kv.rs:229-289``):
a LIFO free list over a bump pointer, with a bitmap of live pages so that freeing a page
twice, or one that was never handed out, fails at once.  ``SlotPool`` hands out indices into
the per-request arrays of fixed size, lowest free index first.  ``OutOfPages`` (a
``CacheError``) says that a request's next tokens do not fit: the scheduler decides who gives
pages back.
"""
from __future__ import annotations

from ..kernels.build import ensure_host_module

_host = ensure_host_module()
BlockPool = _host.BlockPool
SlotPool = _host.SlotPool
CacheError = _host.CacheError
OutOfPages = _host.OutOfPages
CacheCore = _host.CacheCore
