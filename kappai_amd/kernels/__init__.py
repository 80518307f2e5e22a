"""Hand-written HIP kernels for gfx950 and their Python faces."""
from . import ops, profile, tuning
from .lib import (KernelBuildError, KernelLaunchError, LIBRARIES, build_all, compile_library,
                  library)

__all__ = ["ops", "profile", "tuning", "KernelBuildError", "KernelLaunchError", "LIBRARIES", "build_all",
           "compile_library", "library"]
