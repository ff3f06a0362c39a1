"""The host runtime in C++ (csrc/host): the cache manager's bookkeeping and the scheduler's
decisions. `native.library()` builds it with the host compiler at first use and loads it."""
from .native import HostLibraryError, build, library

__all__ = ["HostLibraryError", "build", "library"]
