"""Errors of the cache manager."""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was taken."""


class NoFreeSlot(RuntimeError):
    """Every request slot is in use."""
