from .library import KernelError, KernelLibraryError

__all__ = ["KernelError", "KernelLibraryError"]
