from .lib import KernelError, KernelLibraryError
