from . import library, ops
from .ops import KernelError
from .library import KernelLibraryError
