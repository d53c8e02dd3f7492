from .diffcache import DiffCache

__all__ = ["DiffCache"]
