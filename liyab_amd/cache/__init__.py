"""Paged key/value cache, block tables and per-request state slots."""

from .pages import UNMAPPED, CacheGroup, CacheManager, KVSpec, PagePool, StateSpec  # noqa: F401
from .storage import CacheStorage, LayerCache  # noqa: F401
