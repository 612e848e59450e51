from . import ops
from .library import library, loaded_path, KernelLibraryError
from .ops import KernelArgumentError
