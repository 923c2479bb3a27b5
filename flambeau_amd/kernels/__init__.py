from .library import KernelError, load
